"""Vekalorn: a decoder-only model of latent-attention layers with mixture-of-experts feed-forwards.

config.json: {architecture, width, vocab, norm: {eps}, layers: [{type, mixer: {...}, mlp: {...} | null}]}.
Layer: x += layer_norm_1(mixer(x)); x += layer_norm_2(ff(x)) - the norms sit on the sublayers' OUTPUTS, the sublayers read
the residual stream itself (float; rounded to the storage type where it enters a matrix product).
Mixers (qserve_amd.layers.latent_attention.LatentAttention):
  latent_attention    no positions, sliding window `mask.size`
  latent_attention_2  rotated part of `rot_dim` dimensions (rotary table from `rot`), causal, sigmoid output gate
Feed-forward: qserve_amd.layers.moe.GroupedTopKMoE.  Output: layer norm, then the `head` matrix.
Tensor names: embed, head, final.norm, l<i>.norm1/2, l<i>.mix.{dq, dq.norm, uq, dkv, dkv.norm, uk, uv, o[, g]},
l<i>.mlp.{router, e<k>.up, e<k>.down}.
"""
import torch

from ..layers.latent_attention import LatentAttention
from ..layers.moe import GroupedTopKMoE
from ..layers.ops import linear
from ..layers.rotary import RotaryTable
from ..serving.registry import register_model

MIXERS = ("latent_attention", "latent_attention_2")


@register_model("Vekalorn")
class Vekalorn:
    def __init__(self, ops, width, vocab, eps, embed, head, final_norm, layers):
        self.ops, self.width, self.vocab, self.eps = ops, width, vocab, eps
        self.embed, self.head, self.final_norm, self.layers = embed, head, final_norm, layers
        self.cache_rows = [L["mixer"].row_width for L in layers]
        self.rotaries = list({id(L["mixer"].rotary): L["mixer"].rotary for L in layers if L["mixer"].rotary is not None}.values())

    def reserve_positions(self, n):
        """Make every rotary table cover positions [0, n)."""
        for r in self.rotaries:
            r.reserve(n)

    def graph_signature(self):
        """What a captured step holds by address and must find unchanged at replay."""
        return tuple(r.table.data_ptr() for r in self.rotaries)

    @classmethod
    def from_config(cls, config, weights, ops, device, dtype, page=64):
        D, V, eps = int(config["width"]), int(config["vocab"]), float(config["norm"]["eps"])

        def w(name):
            if name not in weights:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            return weights[name].to(device=device, dtype=dtype).contiguous()

        rotaries, layers = {}, []
        for i, spec in enumerate(config["layers"]):
            kind, m, p = spec["type"], spec["mixer"], f"l{i}.mix."
            if kind not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            wm = {k: w(p + n) for k, n in (("dq", "dq"), ("dq_norm", "dq.norm"), ("uq", "uq"), ("dkv", "dkv"),
                                           ("dkv_norm", "dkv.norm"), ("uk", "uk"), ("uv", "uv"), ("o", "o"))}
            common = dict(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
                          q_rank=int(m["q_rank"]), scale=float(m["scale"]), eps=eps, page=page)
            if kind == "latent_attention":
                window = int(m["mask"]["size"]) if m.get("mask") else None
                mixer = LatentAttention(ops, weights=wm, window=window, **common)
            else:
                rot = m["rot"]
                rt = RotaryTable(int(rot["dims"]), float(rot["base"]), rot.get("scaling"), device)
                rt = rotaries.setdefault(rt.key(), rt)                   # layers with the same constants share one table
                wm["g"] = w(p + "g")
                mixer = LatentAttention(ops, weights=wm, rot_dim=int(m["rot_dim"]), rotary=rt, gated=True, **common)
            L = {"mixer": mixer, "norm1": w(f"l{i}.norm1"), "ff": None}
            mlp = spec.get("mlp")
            if mlp:
                if mlp.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                r, q = mlp["router"], f"l{i}.mlp."
                E, g = int(r["experts"]), r.get("groups") or {}
                L["ff"] = GroupedTopKMoE(ops, router=w(q + "router"), up=[w(f"{q}e{e}.up") for e in range(E)],
                                         down=[w(f"{q}e{e}.down") for e in range(E)], top_k=int(r["top"]),
                                         groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))))
                if L["ff"].up.size(1) != int(mlp["expert"]["ff"]):
                    raise ValueError(f"layer {i}: expert tensors do not have ff = {mlp['expert']['ff']}")
                L["norm2"] = w(f"l{i}.norm2")
            layers.append(L)
        embed, head = w("embed"), w("head")
        if embed.shape != (V, D) or head.shape != (V, D):
            raise ValueError("embed / head do not have the shape [vocab, width] of the config")
        return cls(ops, D, V, eps, embed, head, w("final.norm"), layers)

    def forward(self, batch, pools, tap=None):
        """-> the float residual stream [T, width] after the last layer; tap(i, x) is called after every layer (tests)."""
        ops = self.ops
        x, h = ops.embed(batch.tokens, self.embed)
        for i, L in enumerate(self.layers):
            h = ops.add_layer_norm(x, L["mixer"](h, batch, pools[i]), L["norm1"], self.eps)
            if L["ff"] is not None:
                h = ops.add_layer_norm(x, L["ff"](h), L["norm2"], self.eps)
            if tap is not None:
                tap(i, x)
        return x

    def logits(self, x, rows):
        return linear(self.ops.layer_norm_rows(x, rows, self.final_norm, self.eps), self.head).float()
