"""Paged serving engine: model registry and configuration, checkpoint loading, a paged cache with sequence slots, a
continuous-batching scheduler (prompt portions beside single decoded tokens), sampling, and the command line.

    from qserve_amd.serving import Engine
    eng = Engine.from_pretrained(model_dir, dtype="bfloat16", max_tokens=4096)
    out = eng.generate([[1, 2, 3]], max_new=16)

Models register themselves by the `architecture` name of their config.json (qserve_amd/models).
"""
from .engine import Engine, SamplingParams  # noqa: F401
from .registry import register_model, resolve_model  # noqa: F401
