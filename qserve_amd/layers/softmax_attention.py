"""Causal grouped-query softmax attention over a paged cache, with rotated keys AND rotated values.

q (H heads), k, v (G heads; query head h reads key / value head h // (H / G)) come from one product.  The first `rot_n`
dimensions of every q and k head turn with the position (halves layout, table `rope_k`); every value turns over all its
`vdim` dimensions by its own position (table `rope_v`) and is cached so; a head's output at position i is turned back by
-i, so that the sum carries the RELATIVE rotation i - j of each value.  score = q . k * scale, softmax over j <= i.

Cache: per key / value head one pool of rows [v (vdim) | k (dim)].  The attention itself is the paged row-attention kernel of
the latent layers (qserve_amd.layers.latent_attention): a query [0 (vdim) | q * scale] against such rows scores q . k, and
the softmax-weighted sum of the rows' first vdim elements is the output; one launch serves all key / value heads.
"""
import torch

from .ops import linear


class RotatedValueAttention:
    def __init__(self, ops, *, heads, kv_heads, dim, vdim, scale, rot_n, rope_k, rope_v, weights, page=64):
        """weights: q [H dim, D], k [G dim, D], v [G vdim, D], o [D, H vdim]."""
        if heads % kv_heads or vdim % 2 or rot_n % 2 or rot_n > dim:
            raise ValueError(f"attention: {heads} heads over {kv_heads}, vdim {vdim}, {rot_n} rotated of {dim}")
        self.ops, self.H, self.G, self.dim, self.vdim, self.scale, self.page = ops, heads, kv_heads, dim, vdim, float(scale), page
        self.rot_n, self.rope_k, self.rope_v = rot_n, rope_k, rope_v
        w = weights
        D = w["q"].size(1)
        for k, shp in {"q": (heads * dim, D), "k": (kv_heads * dim, D), "v": (kv_heads * vdim, D), "o": (D, heads * vdim)}.items():
            if tuple(w[k].shape) != shp:
                raise ValueError(f"attention weight {k}: shape {tuple(w[k].shape)}, expected {shp}")
        self.w_in, self.w_o = torch.cat([w["q"], w["k"], w["v"]], dim=0).contiguous(), w["o"].contiguous()
        self.cache_rows, self.state_specs = [(kv_heads, vdim + dim)], []

    def __call__(self, h, batch, pools, states):
        ops, T, H, G = self.ops, h.size(0), self.H, self.G
        pool = pools[0]                                                    # [G, rows, vdim + dim]
        n = batch.max_pos + 1
        proj = linear(h, self.w_in)
        qf = ops.attention_prep(proj, 0, H * self.dim, (H + G) * self.dim, H, G, self.dim, self.vdim, self.rot_n,
                                self.rope_k.reserve(n), self.rope_v.reserve(n), self.scale, pool, batch)
        o = ops.latent_attention(qf, pool, batch, None, self.vdim, self.page, q_first=self.vdim)      # head h reads pool h // (H / G)
        ops.rotate_heads(o, self.rope_v.table, batch.pos, -1.0)
        return linear(o.view(T, H * self.vdim), self.w_o)
