"""Plain, slow float64 statement of the Mumelix design: one function per mechanism, written from its equations, sharing no code
with qserve_amd.  Whole sequences only: no cache, no state hand-over, no batching - every token of a sequence is computed in
one go from the first, which is what the engine's cuts, batches and reused pages must reproduce.

Notation: h [T, D] the input of a sublayer, W["name"] the checkpoint tensors (float64 here), `p` a tensor-name prefix.
"""
import math

import torch

F64 = torch.float64


def silu(z):
    return z * torch.sigmoid(z)


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def dyt(x, W, name):
    """tanh(alpha x) * w + b; no statistics."""
    return torch.tanh(W[name + ".alpha"] * x) * W[name] + W[name + ".b"]


def token_shift(h, mu):
    """Every token is moved towards its predecessor (zeros before the first) by the per-channel amounts mu."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    return h + (prev - h) * mu


# ---- rotations ------------------------------------------------------------------------------------------------------------

def rotary_frequencies(dims, base, scaling=None):
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling:
        factor, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        out = []
        for fi in f:
            wavelength = 2.0 * math.pi / fi
            if wavelength < orig / hi:
                out.append(fi)
            elif wavelength > orig / lo:
                out.append(fi / factor)
            else:
                s = (orig / wavelength - lo) / (hi - lo)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = out
    return torch.tensor(f, dtype=F64)


def rotate_halves(x, pos, freq, n, sign=1.0):
    """x [T, heads, d]: among the first n dimensions, i is paired with i + n / 2 and the pair turns by sign * pos * freq[i]."""
    a = sign * pos.to(F64)[:, None, None] * freq[None, None, :]
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., :n // 2], x[..., n // 2:n]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., n:]], dim=-1)


# ---- mixers ---------------------------------------------------------------------------------------------------------------

def softmax_attention(h, W, p, m):
    """Causal grouped-query softmax attention with partly rotated queries / keys and fully rotated values."""
    T = h.size(0)
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    pos = torch.arange(T)
    q = (h @ W[p + "q"].T).view(T, H, d)
    k = (h @ W[p + "k"].T).view(T, G, d)
    v = (h @ W[p + "v"].T).view(T, G, dv)
    fk = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    fv = rotary_frequencies(dv, rot["base"])
    q, k = rotate_halves(q, pos, fk, rot["dims"]), rotate_halves(k, pos, fk, rot["dims"])
    v = rotate_halves(v, pos, fv, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        for hh in range(H):
            g = hh // (H // G)
            s = (k[:i + 1, g] @ q[i, hh]) * m["scale"]
            w = torch.softmax(s, dim=0)
            out[i, hh] = w @ v[:i + 1, g]
    out = rotate_halves(out, pos, fv, dv, sign=-1.0)
    return out.reshape(T, H * dv) @ W[p + "o"].T


def causal_conv(x, w):
    """x [T, C], w [C, taps]: y[t, c] = sum_j w[c, taps - 1 - j] x[t - j, c], zeros before the start."""
    T, taps = x.size(0), w.size(1)
    y = torch.zeros_like(x)
    for j in range(taps):
        if j < T:
            y[j:] += x[:T - j] * w[:, taps - 1 - j]
    return y


def gated_delta_rule(h, W, p, m, eps):
    T = h.size(0)
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ W[p + "q"].T, W[p + "q.conv"])).view(T, G, d)
    k = silu(causal_conv(h @ W[p + "k"].T, W[p + "k.conv"])).view(T, G, d)
    v = silu(causal_conv(h @ W[p + "v"].T, W[p + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W[p + "b"].T)                                            # [T, H]
    dt = torch.nn.functional.softplus((h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]).view(T, H, d)
    decay = torch.exp(-torch.exp(W[p + "A_log"])[None, :, None] * dt)                 # [T, H, d]
    gate = torch.sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(T):
            S = decay[t, hh][:, None] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hh] = S.T @ q[t, g]
    o = rms(o, eps) * W[p + "norm"] * gate
    return o.reshape(T, H * dv) @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    left = softmax_attention(h, W, p + "left.", m["left"])
    right = gated_delta_rule(h, W, p + "right.", m["right"], eps)
    return 0.5 * (rms(left, eps) * W[p + "left.out"] + rms(right, eps) * W[p + "right.out"])


def gated_linear_attention(h, W, p, m, eps):
    T = h.size(0)
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / m["tau"])).view(T, H, d)
    o = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(T):
            S = alpha[t, hh][:, None] * S + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S.T @ q[t, hh]
    o = (rms(o, eps) * W[p + "norm"]).reshape(T, H * dv) * silu(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


MIXERS = {"gla": gated_linear_attention, "parallel": parallel_mixer}


# ---- feed-forwards --------------------------------------------------------------------------------------------------------

def gated_ff(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(h, W, p, r):
    """-> (chosen experts [T, top], weights [T, top]): the largest logits, softmax over the chosen logits only."""
    z = h @ W[p + "router"].T + W[p + "router.b"]
    top = z.topk(r["top"], dim=-1)
    return top.indices, torch.softmax(top.values, dim=-1)


def moe(h, W, p, mlp):
    idx, wt = route(h, W, p, mlp["router"])
    y = torch.zeros_like(h)
    for t in range(h.size(0)):
        for j in range(idx.size(1)):
            y[t] += wt[t, j] * gated_ff(h[t:t + 1], W, f"{p}e{int(idx[t, j])}.")[0]
    return y


def feed_forward(h, W, p, mlp):
    return gated_ff(h, W, p) if mlp["kind"] == "dense" else moe(h, W, p, mlp)


# ---- the model --------------------------------------------------------------------------------------------------------------

def layer_order(cfg):
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg, W, tokens, return_layers=False):
    """-> logits [T, vocab] (float64) and, if asked, the sum of the streams after every layer run."""
    W = {k: v.to(F64) if v.is_floating_point() else v for k, v in W.items()}
    eps, S = float(cfg["norm"]["eps"]), int(cfg.get("streams", 1))
    x0 = W["embed"][torch.tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    xs = [x0.clone() for _ in range(S)]
    seen = []
    for i in layer_order(cfg):
        spec, p = cfg["layers"][i], f"l{i}."
        for q in (1, 2):
            if q == 2 and not spec.get("mlp"):
                continue
            hc = p + f"hc{q}."
            u = sum(W[hc + "in"][s] * xs[s] for s in range(S))
            h = dyt(u, W, p + f"norm{q}")
            if q == 1:
                h = token_shift(h, W[p + "shift"])
                y = MIXERS[spec["type"]](h, W, p + "mix.", spec["mixer"], eps)
            else:
                y = feed_forward(h, W, p + "mlp.", spec["mlp"])
            xs = [sum(W[hc + "mix"][s, t] * xs[s] for s in range(S)) + W[hc + "out"][t] * y for t in range(S)]
        seen.append(sum(xs))
    logits = dyt(sum(xs), W, "final.norm") @ W["head"].T
    return (logits, seen) if return_layers else logits


# ---- random checkpoints for tests ------------------------------------------------------------------------------------------

def random_weights(cfg, seed=0):
    """A checkpoint of the config's shapes: bfloat16-representable values (both storage types then see the same numbers),
    scaled so that activations stay of order one and every mechanism carries weight in the result."""
    g = torch.Generator().manual_seed(seed)
    D, V, S = int(cfg["width"]), int(cfg["vocab"]), int(cfg.get("streams", 1))

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * (s / math.sqrt(i))).bfloat16().double()

    def vec(n, mean=0.0, s=1.0):
        return (torch.randn(n, generator=g) * s + mean).bfloat16().double()

    W = {"embed": (torch.randn(V, D, generator=g) * 0.5).bfloat16().double(), "head": mat(V, D)}

    def norm(name):
        W[name], W[name + ".b"] = vec(D, 1.0, 0.2), vec(D, 0.0, 0.1)
        W[name + ".alpha"] = (torch.rand((), generator=g) * 0.5 + 0.4).bfloat16().double()

    norm("final.norm")
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        norm(p + "norm1")
        W[p + "shift"] = torch.rand(D, generator=g).bfloat16().double()
        for q in (1, 2):
            W[p + f"hc{q}.in"] = (vec(S, 0.0, 0.3) + 1.0 / S).bfloat16().double()
            W[p + f"hc{q}.out"] = vec(S, 0.8, 0.3)
            W[p + f"hc{q}.mix"] = (torch.eye(S, dtype=F64) * 0.8 + torch.randn(S, S, generator=g).double() * 0.15).bfloat16().double()
        if spec["type"] == "gla":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            r = max(2, D // 8)
            W.update({p + "mix.q": mat(H * d, D, 2.0), p + "mix.k": mat(H * d, D, 2.0), p + "mix.v": mat(H * dv, D), p + "mix.g": mat(H * dv, D),
                      p + "mix.o": mat(D, H * dv), p + "mix.norm": vec(dv, 1.0, 0.2), p + "mix.a1": mat(r, D), p + "mix.a2": mat(H * d, r, 2.0),
                      p + "mix.a2.b": vec(H * d, 3.0, 1.5)})
        else:
            a, b = m["left"], m["right"]
            q = p + "mix.left."
            W.update({q + "q": mat(a["heads"] * a["dim"], D, 2.0), q + "k": mat(a["kv_heads"] * a["dim"], D, 2.0),
                      q + "v": mat(a["kv_heads"] * a["vdim"], D), q + "o": mat(D, a["heads"] * a["vdim"]), q + "out": vec(D, 1.0, 0.2)})
            q, r = p + "mix.right.", max(2, D // 8)
            H, G, d, dv, taps = b["heads"], b["kv_heads"], b["dim"], b["vdim"], b["conv"]
            W.update({q + "q": mat(G * d, D, 2.0), q + "k": mat(G * d, D, 2.0), q + "v": mat(H * dv, D, 2.0),
                      q + "q.conv": mat(G * d, taps, 1.5), q + "k.conv": mat(G * d, taps, 1.5), q + "v.conv": mat(H * dv, taps, 1.5),
                      q + "b": mat(H, D, 2.0), q + "A_log": vec(H, -1.0, 0.7), q + "norm": vec(dv, 1.0, 0.2), q + "a1": mat(r, D),
                      q + "a2": mat(H * d, r, 2.0), q + "dt_bias": vec(H * d, -1.0, 1.0), q + "g1": mat(r, D), q + "g2": mat(H * dv, r, 2.0),
                      q + "o": mat(D, H * dv), q + "out": vec(D, 1.0, 0.2)})
        mlp = spec.get("mlp")
        if mlp:
            norm(p + "norm2")
            q = p + "mlp."
            if mlp["kind"] == "dense":
                ff = mlp["ff"]
                W.update({q + "gate": mat(ff, D), q + "up": mat(ff, D), q + "down": mat(D, ff)})
            else:
                E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
                W[q + "router"], W[q + "router.b"] = mat(E, D, 2.0), vec(E, 0.0, 0.5)
                for e in range(E):
                    W.update({f"{q}e{e}.gate": mat(ff, D, 1.5), f"{q}e{e}.up": mat(ff, D, 1.5), f"{q}e{e}.down": mat(D, ff, 1.5)})
    return W
