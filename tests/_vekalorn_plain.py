"""Plain, slow restatement of the Vekalorn design in float64 torch on the CPU: the oracle of the serving tests.

One function per mechanism, whole sequences only (no cache, no batching, no paging): every token attends by an explicit
mask over explicit per-head keys and values.  Shares no code with qserve_amd; the weights are passed as a dict
name -> tensor and the configuration as the parsed config.json dict.
"""
import math

import torch

F = torch.float64


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def yarn_tables(rot, positions):
    """cos / sin [T, dims/2] of the scaled rotary embedding; rot = {"base", "dims", optional "scaling"}."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def corr(t):
            return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

        lo = max(math.floor(corr(float(sc["fast"]))), 0)
        hi = min(math.ceil(corr(float(sc["slow"]))), dims - 1)
        ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=F)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    a = positions.to(F)[:, None] * f[None, :]
    return torch.cos(a) * mag, torch.sin(a) * mag


def rotate_interleaved(x, cos, sin):
    """x [T, ..., dims]; pairs (2i, 2i+1)."""
    u, v = x[..., 0::2], x[..., 1::2]
    while cos.dim() < u.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    out = torch.empty_like(x)
    out[..., 0::2] = u * cos - v * sin
    out[..., 1::2] = v * cos + u * sin
    return out


def masked_softmax_attention(q, k, v, scale, window):
    """q, k [T, H, d], v [T, H, dv]; causal; window = None or the number of visible positions (itself included)."""
    T = q.shape[0]
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & (i - j < window)
    s = s.masked_fill(~ok[None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    return torch.einsum("hij,jhd->ihd", p, v)


def latent_attention(h, W, pre, m, eps):
    """The mixer without positions: windowed, no gate."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    cq = rms_norm(h @ W[pre + "dq"].T, W[pre + "dq.norm"], eps)
    q = (cq @ W[pre + "uq"].T).view(T, H, d)
    c = rms_norm(h @ W[pre + "dkv"].T, W[pre + "dkv.norm"], eps)
    k = (c @ W[pre + "uk"].T).view(T, H, d)
    v = (c @ W[pre + "uv"].T).view(T, H, dv)
    window = m["mask"]["size"] if m.get("mask") else None
    o = masked_softmax_attention(q, k, v, m["scale"], window)
    return o.reshape(T, H * dv) @ W[pre + "o"].T


def latent_attention_2(h, W, pre, m, eps):
    """The mixer with a rotated part shared over the heads, causal, with an output gate."""
    T = h.shape[0]
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_norm(h @ W[pre + "dq"].T, W[pre + "dq.norm"], eps)
    q = (cq @ W[pre + "uq"].T).view(T, H, d + dr)
    kv = h @ W[pre + "dkv"].T
    c = rms_norm(kv[:, :r], W[pre + "dkv.norm"], eps)
    kr = kv[:, r:]
    cos, sin = yarn_tables(m["rot"], torch.arange(T))
    nrot = int(m["rot"]["dims"])
    qr = q[..., d:].clone()
    qr[..., :nrot] = rotate_interleaved(qr[..., :nrot], cos, sin)
    kr = kr.clone()
    kr[..., :nrot] = rotate_interleaved(kr[..., :nrot], cos, sin)
    k = torch.cat([(c @ W[pre + "uk"].T).view(T, H, d), kr[:, None, :].expand(T, H, dr)], dim=-1)
    qq = torch.cat([q[..., :d], qr], dim=-1)
    v = (c @ W[pre + "uv"].T).view(T, H, dv)
    o = masked_softmax_attention(qq, k, v, m["scale"], None).reshape(T, H * dv)
    o = o * torch.sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def route(h, Wr, r):
    """-> (indices [T, top], weights [T, top]) of the grouped top-k router."""
    s = torch.softmax(h @ Wr.T, dim=-1)
    T, E = s.shape
    g = r.get("groups")
    allowed = torch.ones_like(s, dtype=torch.bool)
    if g:
        G, keep = int(g["count"]), int(g["keep"])
        gs = s.view(T, G, E // G).max(-1).values
        top_g = gs.topk(keep, dim=-1).indices
        gm = torch.zeros(T, G, dtype=torch.bool)
        gm.scatter_(1, top_g, True)
        allowed = gm[:, :, None].expand(T, G, E // G).reshape(T, E)
    idx = s.masked_fill(~allowed, -1.0).topk(int(r["top"]), dim=-1).indices
    return idx, s.gather(1, idx)


def moe(h, W, pre, mlp):
    idx, wt = route(h, W[pre + "router"], mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wt[t]):
            a = torch.relu(W[f"{pre}e{e}.up"] @ h[t]) ** 2
            out[t] += w * (W[f"{pre}e{e}.down"] @ a)
    return out


MIXERS = {"latent_attention": latent_attention, "latent_attention_2": latent_attention_2}


def forward(cfg, W, tokens, return_layers=False):
    """tokens: list of ints -> logits [T, vocab] (float64); optionally also the residual stream after every layer."""
    W = {k: (v.to(F) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    trace = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + layer_norm(MIXERS[L["type"]](x, W, p + "mix.", L["mixer"], eps), W[p + "norm1"], eps)
        if L.get("mlp"):
            x = x + layer_norm(moe(x, W, p + "mlp.", L["mlp"]), W[p + "norm2"], eps)
        trace.append(x.clone())
    logits = layer_norm(x, W["final.norm"], eps) @ W["head"].T
    return (logits, torch.stack(trace)) if return_layers else logits


def random_weights(cfg, seed=0, dtype=torch.bfloat16, scale=1.0):
    """Random tensors with the design's names and shapes (dict name -> tensor), for tests."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * (s * scale / math.sqrt(i))).to(dtype)

    def vec(n):
        return (1.0 + 0.1 * torch.randn(n, generator=g)).to(dtype)

    W = {"embed": (torch.randn(V, D, generator=g)).to(dtype), "final.norm": vec(D), "head": mat(V, D)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, d, dv, r, qr = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        dr = m.get("rot_dim", 0) if L["type"] == "latent_attention_2" else 0
        W[p + "norm1"], W[p + "norm2"] = vec(D), vec(D)
        W[p + "mix.dq"], W[p + "mix.dq.norm"] = mat(qr, D), vec(qr)
        W[p + "mix.uq"] = mat(H * (d + dr), qr, 2.0)
        W[p + "mix.dkv"], W[p + "mix.dkv.norm"] = mat(r + dr, D, 2.0), vec(r)
        W[p + "mix.uk"], W[p + "mix.uv"] = mat(H * d, r, 2.0), mat(H * dv, r)
        if L["type"] == "latent_attention_2":
            W[p + "mix.g"] = mat(H * dv, D)
        W[p + "mix.o"] = mat(D, H * dv)
        if L.get("mlp"):
            E, ff = L["mlp"]["router"]["experts"], L["mlp"]["expert"]["ff"]
            for e in range(E):
                W[f"{p}mlp.e{e}.up"], W[f"{p}mlp.e{e}.down"] = mat(ff, D), mat(D, ff)
            W[p + "mlp.router"] = mat(E, D, 3.0)
    return W
