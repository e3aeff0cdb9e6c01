"""Registry entry of the Llama-style W4A8KV4 family: it runs through the static-batch decode engine
(qserve_amd.decode.DecodeEngine, checkpoints through qserve_amd.loader.load_llama_w4a8), not through the paged engine."""
from ..serving.registry import register_model


@register_model("LlamaForCausalLM", engine="static-batch")
@register_model("llama_w4a8", engine="static-batch")
class LlamaW4A8:
    @staticmethod
    def engine_class():
        from ..decode import DecodeEngine       # (needs libqserve_amd.so: imported on use only)
        return DecodeEngine
