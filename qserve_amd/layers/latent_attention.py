"""Attention through low-rank latents over a paged cache of latent rows.

Per token: the query goes down to a latent (RMS-normed) and up to H heads of `dim` (+ `rot_dim` rotated) dimensions; keys and
values come from ONE shared latent row c (RMS-normed, `kv_rank` values) per token, k_h = W_uk,h c and v_h = W_uv,h c, plus an
optional rotated key part of `rot_dim` values shared by all heads.  Only [c | rotated key part] is cached.

The layer never materialises per-head keys or values: with q'_h = W_uk,h^T q_h the score q_h . k_h equals q'_h . c, and
sum_j p_j v_h,j = W_uv,h (sum_j p_j c_j), so attention runs directly on the cached rows and its cost per cached byte grows
with the number of heads.  Options, all parameters: a sliding window (a query at position i sees i - window < j <= i), a
rotary table for the rotated part (first `rot_n` of its dimensions), a sigmoid output gate computed from the layer input.
"""
import torch

from .ops import linear


class LatentAttention:
    def __init__(self, ops, *, heads, dim, vdim, kv_rank, q_rank, scale, eps, weights, rot_dim=0, rotary=None, window=None,
                 gated=False, page=64):
        """weights: dict with dq [q_rank, D], dq_norm, uq [H (dim + rot_dim), q_rank], dkv [kv_rank + rot_dim, D], dkv_norm,
        uk [H dim, kv_rank], uv [H vdim, kv_rank], o [D, H vdim] and, if gated, g [H vdim, D]."""
        self.ops, self.H, self.dim, self.vdim, self.rank, self.q_rank = ops, heads, dim, vdim, kv_rank, q_rank
        self.rot_dim, self.rotary, self.window, self.gated = rot_dim, rotary, window, gated
        self.scale, self.eps, self.page = float(scale), float(eps), page
        self.rot_n = rotary.dims if rotary is not None else 0
        if self.rot_n > rot_dim:
            raise ValueError(f"{self.rot_n} rotated dimensions in a rotated part of {rot_dim}")
        w = weights
        D = w["dq"].size(1)
        self.row_width = kv_rank + rot_dim
        expect = {"dq": (q_rank, D), "dq_norm": (q_rank,), "uq": (heads * (dim + rot_dim), q_rank),
                  "dkv": (kv_rank + rot_dim, D), "dkv_norm": (kv_rank,), "uk": (heads * dim, kv_rank),
                  "uv": (heads * vdim, kv_rank), "o": (D, heads * vdim)}
        if gated:
            expect["g"] = (heads * vdim, D)
        for k, shp in expect.items():
            if tuple(w[k].shape) != shp:
                raise ValueError(f"latent attention weight {k}: shape {tuple(w[k].shape)}, expected {shp}")
        # one product for everything that reads the layer input: [query latent | key-value latent + rotated key | gate]
        self.w_down = torch.cat([w["dq"], w["dkv"]] + ([w["g"]] if gated else []), dim=0).contiguous()
        self.q_off, self.kv_off, self.g_off = 0, q_rank, q_rank + kv_rank + rot_dim
        self.dq_norm, self.dkv_norm, self.w_uq, self.w_o = w["dq_norm"], w["dkv_norm"], w["uq"], w["o"]
        self.w_uk = w["uk"].view(heads, dim, kv_rank).contiguous()                     # q'_h = q_h @ w_uk[h]
        self.w_uv_t = w["uv"].view(heads, vdim, kv_rank).transpose(1, 2).contiguous()  # o_h = (sum p c) @ w_uv_t[h]

    def __call__(self, h, batch, pool):
        """h [T, D] (storage type) -> mixer output [T, D]; writes this step's rows into `pool` ([rows, row_width])."""
        ops, T, H = self.ops, h.size(0), self.H
        rope = self.rotary.reserve(batch.max_pos + 1) if self.rot_n else None
        down = linear(h, self.w_down)
        cq = ops.latent_prep(down, self.q_off, self.q_rank, self.dq_norm, self.kv_off, self.rank, self.dkv_norm, self.rot_dim,
                             self.rot_n, rope, pool, batch.slot, batch.pos, self.eps)
        q = linear(cq, self.w_uq)                                                   # [T, H (dim + rot_dim)]
        qn = q.view(T, H, self.dim + self.rot_dim)[..., :self.dim].transpose(0, 1)  # [H, T, dim] (strided view)
        q_abs = torch.bmm(qn, self.w_uk)                                            # [H, T, rank]
        qf = ops.latent_query(q, q_abs, rope, batch.pos, self.scale, H, self.dim, self.rot_dim, self.rot_n, self.rank)
        o_lat = ops.latent_attention(qf, pool, batch, self.window, self.rank, self.page)
        o = torch.bmm(o_lat.transpose(0, 1), self.w_uv_t).transpose(0, 1).reshape(T, H * self.vdim)
        if self.gated:
            ops.sigmoid_gate(o, down[:, self.g_off:self.g_off + H * self.vdim])
        return linear(o, self.w_o)
