"""Mumelix: a decoder-only model of recurrent and attention mixers on several residual streams.

config.json: {architecture, width, vocab, streams, embedding: {scale}, norm: {eps}, loop: {start, stop, times} | absent,
layers: [{type, mixer: {...}, mlp: {kind: dense | moe, ...} | null}]}.

* Residual: `streams` copies of the embedding output (float).  A sublayer reads u = sum_s in[s] x_s, and all streams are
  rewritten at once, x_t <- sum_s mix[s, t] x_s + out[t] y (tensors l<i>.hc1.* for the mixer, l<i>.hc2.* for the feed-forward).
  The output is computed from the sum of the streams.
* Norm: tanh(alpha u) w + b, no statistics (tensors <name>, <name>.b, <name>.alpha).
* The mixer's input is moved towards the previous token's (before that move; zeros before the first): h + (h' - h) shift.
* Mixers: `gla` (qserve_amd.layers.recurrent.GatedLinearAttention); `parallel` = attention with rotated keys and values
  (qserve_amd.layers.softmax_attention.RotatedValueAttention) beside a gated delta rule (GatedDeltaRule), joined by ParallelMixer.
* Feed-forward: dense gated units or a top-k mixture of them (qserve_amd.layers.moe).
* `loop` repeats a block of consecutive layers: the layer order is [0, start) + [start, stop) x times + [stop, n).  A repeated
  layer shares its weights between its runs, never its cache pools or states (`run_slices`).
"""
import torch

from ..layers.moe import GatedFeedForward, TopKGatedMoE
from ..layers.ops import linear
from ..layers.recurrent import GatedDeltaRule, GatedLinearAttention, ParallelMixer
from ..layers.rotary import RotaryTable
from ..layers.softmax_attention import RotatedValueAttention
from ..serving.cache import StateSpec
from ..serving.registry import register_model


@register_model("Mumelix")
class Mumelix:
    def __init__(self, ops, width, vocab, streams, scale, embed, head, final_norm, layers, order, rotaries):
        self.ops, self.width, self.vocab, self.streams, self.scale = ops, width, vocab, streams, scale
        self.embed, self.head, self.final_norm, self.layers, self.order, self.rotaries = embed, head, final_norm, layers, order, rotaries
        # every layer RUN gets its own pools and states: [token-shift input | the mixer's]
        self.cache_rows, self.state_specs, self.run_slices = [], [], []
        for i in order:
            m = layers[i]["mixer"]
            p0, s0 = len(self.cache_rows), len(self.state_specs)
            self.cache_rows += m.cache_rows
            self.state_specs += [StateSpec((width,), copies=2)] + m.state_specs
            self.run_slices.append((p0, len(self.cache_rows), s0, len(self.state_specs)))

    def reserve_positions(self, n):
        for r in self.rotaries:
            r.reserve(n)

    def graph_signature(self):
        return tuple(r.table.data_ptr() for r in self.rotaries)

    @classmethod
    def from_config(cls, config, weights, ops, device, dtype, page=64):
        D, V, eps = int(config["width"]), int(config["vocab"]), float(config["norm"]["eps"])
        S = int(config.get("streams", 1))

        def w(name, as_float=False):
            if name not in weights:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            return weights[name].to(device=device, dtype=torch.float32 if as_float else dtype).contiguous()

        def norm(name):
            return (w(name), w(name + ".b"), float(weights[name + ".alpha"].float()))

        tables = {}

        def table(dims, base, scaling):
            t = RotaryTable(int(dims), float(base), scaling, device)
            return tables.setdefault(t.key(), t)

        layers = []
        for i, spec in enumerate(config["layers"]):
            kind, m, p = spec["type"], spec["mixer"], f"l{i}.mix."
            if kind == "gla":
                names = ("q", "k", "v", "g", "o", "norm", "a1", "a2")
                wm = dict({k: w(p + k) for k in names}, a2_b=w(p + "a2.b"))
                mixer = GatedLinearAttention(ops, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), tau=float(m["tau"]),
                                             eps=eps, weights=wm)
            elif kind == "parallel":
                a, b = m["left"], m["right"]
                rot = a["rot"]
                left = RotatedValueAttention(
                    ops, heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]), vdim=int(a["vdim"]), scale=float(a["scale"]),
                    rot_n=int(rot["dims"]), rope_k=table(rot["dims"], rot["base"], rot.get("scaling")),
                    rope_v=table(a["vdim"], rot["base"], None), weights={k: w(p + "left." + k) for k in ("q", "k", "v", "o")}, page=page)
                q = p + "right."
                wm = {k: w(q + k) for k in ("q", "k", "v", "b", "A_log", "norm", "a1", "a2", "dt_bias", "g1", "g2", "o")}
                wm.update(q_conv=w(q + "q.conv"), k_conv=w(q + "k.conv"), v_conv=w(q + "v.conv"))
                right = GatedDeltaRule(ops, heads=int(b["heads"]), kv_heads=int(b["kv_heads"]), dim=int(b["dim"]), vdim=int(b["vdim"]),
                                       taps=int(b["conv"]), eps=eps, weights=wm)
                mixer = ParallelMixer(ops, left, right, w(p + "left.out"), w(p + "right.out"), eps)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            L = {"mixer": mixer, "norm1": norm(f"l{i}.norm1"), "shift": w(f"l{i}.shift"), "ff": None,
                 "hc1": tuple(w(f"l{i}.hc1.{k}", True) for k in ("in", "mix", "out"))}
            mlp = spec.get("mlp")
            if mlp:
                q = f"l{i}.mlp."
                if mlp["kind"] == "dense":
                    L["ff"] = GatedFeedForward(ops, gate=w(q + "gate"), up=w(q + "up"), down=w(q + "down"))
                    ff = L["ff"].w_down.size(1)
                    want = int(mlp["ff"])
                elif mlp["kind"] == "moe":
                    E = int(mlp["router"]["experts"])
                    L["ff"] = TopKGatedMoE(ops, router=w(q + "router"), bias=w(q + "router.b"), gate=[w(f"{q}e{e}.gate") for e in range(E)],
                                           up=[w(f"{q}e{e}.up") for e in range(E)], down=[w(f"{q}e{e}.down") for e in range(E)],
                                           top_k=int(mlp["router"]["top"]))
                    ff, want = L["ff"].down.size(2), int(mlp["expert"]["ff"])
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                if ff != want:
                    raise ValueError(f"layer {i}: feed-forward tensors do not have ff = {want}")
                L["norm2"] = norm(f"l{i}.norm2")
                L["hc2"] = tuple(w(f"l{i}.hc2.{k}", True) for k in ("in", "mix", "out"))
            for k in ("hc1", "hc2"):
                if k in L and (L[k][0].shape != (S,) or L[k][1].shape != (S, S) or L[k][2].shape != (S,)):
                    raise ValueError(f"layer {i}: {k} tensors do not fit {S} streams")
            layers.append(L)
        n, loop = len(layers), config.get("loop")
        order = list(range(n))
        if loop:
            a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
            if not 0 <= a <= b <= n or times < 1:
                raise ValueError(f"loop {loop} over {n} layers")
            order = list(range(a)) + list(range(a, b)) * times + list(range(b, n))
        embed, head = w("embed"), w("head")
        if embed.shape != (V, D) or head.shape != (V, D):
            raise ValueError("embed / head do not have the shape [vocab, width] of the config")
        return cls(ops, D, V, S, float(config["embedding"]["scale"]), embed, head, norm("final.norm"), layers, order,
                   list(tables.values()))

    def forward(self, batch, pools, states=None, tap=None):
        """-> the float residual streams [T, streams, width] after the last layer run; tap(run, sum of streams) after every run."""
        ops = self.ops
        x = ops.embed_streams(batch.tokens, self.embed, self.scale, self.streams)
        for run, i in enumerate(self.order):
            L = self.layers[i]
            p0, p1, s0, s1 = self.run_slices[run]
            w_in, w_mix, w_out = L["hc1"]
            h = ops.hc_read(x, w_in, L["norm1"], L["shift"], batch, states[s0])
            y = L["mixer"](h, batch, pools[p0:p1], states[s0 + 1:s1])
            if L["ff"] is None:
                ops.hc_write(x, y, w_mix, w_out)
            else:                                               # the feed-forward's input comes out of the mixer's stream rewrite
                h = ops.hc_write(x, y, w_mix, w_out, then_read=(L["hc2"][0], L["norm2"]))
                ops.hc_write(x, L["ff"](h), L["hc2"][1], L["hc2"][2])
            if tap is not None:
                tap(run, x.sum(1))
        return x

    def logits(self, x, rows):
        return linear(self.ops.dyt_sum_rows(x, rows, self.final_norm), self.head).float()
