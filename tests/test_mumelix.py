"""The Mumelix model and its mechanisms through the serving engine against the plain float64 oracle (tests/_mumelix_plain.py).

Every test runs with the unfused tensor-op backend on the CPU (host logic: state rows, runs, loops over layers, the layers'
composition) and, marked `gpu`, with the HIP kernels.  Configurations and weights are made here: small, random, sizes unlike
each other so that a mixed-up dimension shows; where random weights would hide a fault (one key among hundreds, a state that
is lost, a stale slot) the weights or inputs are made so that it shows.
"""
import math

import pytest
import torch

import _mumelix_plain as P
from qserve_amd.layers.ops import make_ops
from qserve_amd.layers.rotary import RotaryTable
from qserve_amd.models.mumelix import Mumelix
from qserve_amd.serving import Engine, SamplingParams
from qserve_amd.serving.cache import CacheFull

BACKENDS = [pytest.param("unfused", id="unfused-cpu"), pytest.param("hip", marks=pytest.mark.gpu, id="hip")]


@pytest.fixture(params=BACKENDS)
def backend(request):
    if request.param == "hip" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return request.param


def device_of(backend):
    return "cuda:0" if backend == "hip" else "cpu"


BANDS = {"factor": 3.0, "low": 1.0, "high": 4.0, "original": 40}


def gla(heads=3, dim=8, vdim=12, tau=4.0, mlp=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": mlp}


def par(heads=4, kv_heads=2, dim=12, vdim=8, rot_dims=8, scaling=BANDS, base=200.0, scale=None,
        r_heads=4, r_kv=2, r_dim=6, r_vdim=10, taps=3, mlp=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = scaling
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot,
            "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    right = {"heads": r_heads, "kv_heads": r_kv, "dim": r_dim, "vdim": r_vdim, "conv": taps}
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def dense(ff=28):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=9):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def make_config(layers, width=40, vocab=53, streams=2, loop=None, eps=1e-5, scale=3.0):
    cfg = {"architecture": "Mumelix", "width": width, "vocab": vocab, "streams": streams, "embedding": {"scale": scale},
           "norm": {"eps": eps}, "layers": layers}
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


def standard_config():
    return make_config([gla(mlp=dense()), par(mlp=moe()), gla(heads=2, dim=5, vdim=7, tau=9.0, mlp=moe(experts=3, top=1, ff=6)),
                        par(heads=2, kv_heads=1, dim=6, vdim=6, rot_dims=6, scaling=None, r_heads=2, r_kv=2, r_dim=9, r_vdim=4, taps=4)],
                       loop=(1, 3, 2))


def f32(W):
    return {k: (v.float() if v.is_floating_point() else v) for k, v in W.items()}


def build_engine(cfg, W, backend, dtype="float32", max_tokens=1024, max_seqs=4, **kw):
    return Engine(Mumelix, cfg, W, dtype=dtype, device=device_of(backend), max_tokens=max_tokens, max_seqs=max_seqs,
                  backend=backend, **kw)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def run_schedule(eng, seqs, steps):
    """seqs: {name: tokens}; steps: [[(name, count), ...]] -> {name: logits [len, vocab]}; a sequence is closed after its last token."""
    at, slots, got = {k: 0 for k in seqs}, {}, {k: [] for k in seqs}
    for step in steps:
        items, want, n = [], [], 0
        for name, count in step:
            if name not in slots:
                slots[name] = eng.open_sequence()
            items.append((slots[name], seqs[name][at[name]:at[name] + count]))
            want += range(n, n + count)
            n += count
        logits = eng.execute(items, want).double().cpu()
        n = 0
        for name, count in step:
            got[name].append(logits[n:n + count])
            n += count
            at[name] += count
            if at[name] == len(seqs[name]):
                eng.close_sequence(slots.pop(name))
    return {k: torch.cat(v) for k, v in got.items() if v}


def assert_close(got, ref, tol, what=""):
    err = (got - ref).abs().max().item()
    scale = max(1.0, ref.abs().max().item())
    assert err <= tol * scale, f"{what}: max error {err:.3e} (allowed {tol * scale:.3e})"


F32_TOL = 2e-4      # float32 runs of a whole model against float64 (a fault shows at 1e-2 and above)


# ---- mechanisms alone ---------------------------------------------------------------------------------------------------------

def test_band_scaled_rotary_table():
    for dims, base, sc in ((8, 200.0, BANDS), (6, 50.0, None), (16, 1000.0, {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64})):
        t = RotaryTable(dims, base, sc, positions=4).reserve(300)
        f = P.rotary_frequencies(dims, base, sc)
        a = torch.arange(300, dtype=torch.float64)[:, None] * f[None, :]
        assert_close(t[:300, 0].double(), torch.cos(a), 1e-7)
        assert_close(t[:300, 1].double(), torch.sin(a), 1e-7)
    plain, scaled = P.rotary_frequencies(16, 1000.0), P.rotary_frequencies(16, 1000.0, {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64})
    ratio = scaled / plain                                 # all three bands occur: kept, divided by the factor, blended
    assert ratio.max() == 1.0 and abs(ratio.min() - 0.125) < 1e-12 and ((ratio > 0.126) & (ratio < 0.999)).any()


def _one_layer_engine(layer, backend, width=24, streams=2, seed=3, max_tokens=256, max_seqs=3):
    cfg = make_config([layer], width=width, streams=streams)
    W = P.random_weights(cfg, seed=seed)
    return cfg, W, build_engine(cfg, f32(W), backend, max_tokens=max_tokens, max_seqs=max_seqs)


def _mixer_alone(backend, layer, T, splits, seed=3, width=24, tol=2e-5):
    """One mixer through its layer object, the engine's cache and state, the tokens cut at `splits`, against the oracle."""
    cfg, W, eng = _one_layer_engine(layer, backend, width=width, seed=seed)
    dev = eng.device
    mixer = eng.model.layers[0]["mixer"]
    p0, p1, s0, s1 = eng.model.run_slices[0]
    g = torch.Generator().manual_seed(seed + 100)
    h = torch.randn(T, width, generator=g).bfloat16().float()
    ref = P.MIXERS[layer["type"]](h.double(), {k: v.double() for k, v in W.items()}, "l0.mix.", layer["mixer"], cfg["norm"]["eps"])
    slot = eng.open_sequence()
    outs, lo = [], 0
    for hi in list(splits) + [T]:
        b = eng.layout([(slot, [0] * (hi - lo))])
        outs.append(mixer(h[lo:hi].to(dev), b, eng.cache.pools[p0:p1], eng.cache.states[s0 + 1:s1]).double().cpu())
        lo = hi
    assert_close(torch.cat(outs), ref, tol, f"{layer['type']} cut at {splits}")


def test_gated_linear_attention_alone(backend):
    _mixer_alone(backend, gla(), 40, [])
    _mixer_alone(backend, gla(), 40, [1, 3, 17, 18, 39])
    _mixer_alone(backend, gla(heads=1, dim=40, vdim=70, tau=1.0), 21, [2, 4])         # a column split over several lanes, two column blocks
    _mixer_alone(backend, gla(heads=5, dim=3, vdim=2, tau=30.0), 9, [8])
    _mixer_alone(backend, gla(), 120, [15, 31, 48, 81])             # runs of 15, 16, 17, 33, 39 tokens: the kernel stages 16 at a time


def test_parallel_mixer_alone(backend):
    _mixer_alone(backend, par(), 45, [])
    _mixer_alone(backend, par(), 45, [1, 2, 4, 20, 44])                               # runs shorter than the convolution
    _mixer_alone(backend, par(taps=1, r_kv=1, kv_heads=4, rot_dims=12), 14, [5])     # no history; one q/k head for all; every dimension turns
    _mixer_alone(backend, par(taps=6, r_heads=3, r_kv=3, r_dim=20, r_vdim=3, heads=1, kv_heads=1, dim=4, vdim=2, rot_dims=2), 30, [3, 4, 6, 13])
    _mixer_alone(backend, par(), 150, [63, 64, 65, 129])                              # page borders
    _mixer_alone(backend, par(r_dim=40, r_vdim=70), 120, [15, 31, 48, 81])            # staging chunk edges; columns over two blocks


def test_stream_norm_and_token_shift(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(0)
    for S, D in ((1, 7), (2, 40), (3, 300)):
        cfg = make_config([gla()], width=D, streams=S)
        W = P.random_weights(cfg, seed=S)
        eng = build_engine(cfg, f32(W), backend, max_tokens=128, max_seqs=2)
        L = eng.model.layers[0]
        x = torch.randn(11, S, D, generator=g) * 2
        u = sum(W["l0.hc1.in"][s] * x[:, s].double() for s in range(S))
        ref = P.token_shift(P.dyt(u, W, "l0.norm1"), W["l0.shift"])
        slot = eng.open_sequence()
        got, lo = [], 0
        for hi in (1, 2, 7, 11):
            b = eng.layout([(slot, [0] * (hi - lo))])
            got.append(ops.hc_read(x[lo:hi].contiguous().to(dev), L["hc1"][0], L["norm1"], L["shift"], b, eng.cache.states[0]).double().cpu())
            lo = hi
        assert_close(torch.cat(got), ref, 2e-6, f"read with shift, {S} streams")
        got = ops.hc_read(x.to(dev), L["hc1"][0], L["norm1"]).double().cpu()
        assert_close(got, P.dyt(u, W, "l0.norm1"), 2e-6, "read without shift")
        y = torch.randn(11, D, generator=g)
        xd = x.clone().to(dev)
        ops.hc_write(xd, y.to(dev), L["hc1"][1], L["hc1"][2])
        ref = torch.stack([sum(W["l0.hc1.mix"][s, t] * x[:, s].double() for s in range(S)) + W["l0.hc1.out"][t] * y.double()
                           for t in range(S)], dim=1)
        assert_close(xd.double().cpu(), ref, 2e-6, "stream rewrite")
        rows = torch.tensor([10, 0, 4], dtype=torch.int32)
        out = ops.dyt_sum_rows(xd, rows.to(dev), eng.model.final_norm).double().cpu()
        assert_close(out, P.dyt(ref.sum(1)[rows.long()], W, "final.norm"), 3e-6, "final norm")


def test_router_and_gated_experts_alone(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(11)
    for E, top, ff, D, T in ((5, 2, 9, 40, 33), (3, 1, 6, 20, 7), (12, 3, 24, 72, 33), (4, 4, 10, 36, 2), (6, 2, 16, 64, 90)):
        h = torch.randn(T, D, generator=g)
        W = {"p.router": torch.randn(E, D, generator=g).double() * 0.6, "p.router.b": torch.randn(E, generator=g).double() * 2}
        gate, up, down = [], [], []
        for e in range(E):
            gate.append(torch.randn(ff, D, generator=g) / math.sqrt(D))
            up.append(torch.randn(ff, D, generator=g) / math.sqrt(D))
            down.append(torch.randn(D, ff, generator=g) / math.sqrt(ff))
            W[f"p.e{e}.gate"], W[f"p.e{e}.up"], W[f"p.e{e}.down"] = gate[-1].double(), up[-1].double(), down[-1].double()
        from qserve_amd.layers.moe import TopKGatedMoE
        layer = TopKGatedMoE(ops, router=W["p.router"].float().to(dev), bias=W["p.router.b"].float().to(dev), gate=[t.to(dev) for t in gate],
                             up=[t.to(dev) for t in up], down=[t.to(dev) for t in down], top_k=top)
        idx, wt = ops.moe_route(h.to(dev), layer.router, top, 1, 1, bias=layer.bias, renorm=True)
        ridx, rwt = P.route(h.double(), W, "p.", {"top": top})
        order = idx.cpu().long().argsort(dim=1), ridx.argsort(dim=1)
        assert torch.equal(idx.cpu().long().gather(1, order[0]), ridx.gather(1, order[1])), f"experts chosen, E={E}"
        assert_close(wt.cpu().double().gather(1, order[0]), rwt.gather(1, order[1]), 2e-6)
        assert_close(wt.sum(1).cpu().double(), torch.ones(T, dtype=torch.float64), 1e-6, "weights of the chosen sum to one")
        ref = P.moe(h.double(), W, "p.", {"router": {"top": top}})
        assert_close(layer(h.to(dev)).double().cpu(), ref, 1e-5, f"gated experts E={E}")
        if backend == "hip":                                  # per-token kernels and expert-sorted products
            for above in (0, 10 ** 9):
                ops.moe_sorted_above = above
                assert_close(layer(h.to(dev)).double().cpu(), ref, 1e-5, f"gated experts E={E}, sorted above {above}")
            del ops.moe_sorted_above


def test_the_bias_changes_the_choice(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    h = torch.zeros(1, 8)
    h[0, 0] = 1.0
    Wr = torch.zeros(4, 8)
    Wr[:, 0] = torch.tensor([1.0, 2.0, 3.0, 0.0])
    bias = torch.tensor([0.0, 0.0, -5.0, 2.5])
    idx, wt = ops.moe_route(h.to(dev), Wr.to(dev), 2, 1, 1, bias=bias.to(dev), renorm=True)      # logits 1, 2, -2, 2.5
    assert sorted(idx[0].tolist()) == [1, 3]
    w = dict(zip(idx[0].tolist(), wt[0].tolist()))
    assert abs(w[3] - 1.0 / (1.0 + math.exp(-0.5))) < 1e-6


def test_dense_feed_forward_alone(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    from qserve_amd.layers.moe import GatedFeedForward
    g = torch.Generator().manual_seed(2)
    h, W = torch.randn(9, 24, generator=g), {k: torch.randn(s, generator=g).double() / 4 for k, s in
                                               (("p.gate", (14, 24)), ("p.up", (14, 24)), ("p.down", (24, 14)))}
    layer = GatedFeedForward(ops, gate=W["p.gate"].float().to(dev), up=W["p.up"].float().to(dev), down=W["p.down"].float().to(dev))
    assert_close(layer(h.to(dev)).double().cpu(), P.gated_ff(h.double(), W, "p."), 1e-5)


# ---- faults that random weights would hide ---------------------------------------------------------------------------------------

def _selector_attention(backend, L, spike, dtype, as_prompt):
    """Attention alone with selector weights: the layer input IS [q | k | v].  All keys are small but the one at `spike`, which is
    large in a dimension that does not turn; the last queries point there.  -> (layer output, oracle) for the last positions."""
    m = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 6, "rot": {"base": 100.0, "dims": 4}, "scale": 1.0}
    D = 2 * 8 + 8 + 6
    eye = torch.eye(D, dtype=torch.float64)
    W = {"p.q": eye[:16], "p.k": eye[16:24], "p.v": eye[24:30], "p.o": eye[:, :12].contiguous()}      # (o: the heads' outputs as they are)
    g = torch.Generator().manual_seed(spike * 7 + L)
    h = (torch.randn(L, D, generator=g) * 0.05).bfloat16().double()
    h[:, 24:30] = torch.randn(L, 6, generator=g).bfloat16().double()
    h[spike, 16 + 7] = 6.0
    h[:, 7] = 2.0
    h[:, 8 + 7] = 2.0
    ref = P.softmax_attention(h[:, :], W, "p.", m)
    from qserve_amd.layers.softmax_attention import RotatedValueAttention
    from qserve_amd.serving.cache import PagedCache
    from qserve_amd.serving.engine import StepBatch
    dev = device_of(backend)
    ops = make_ops(backend, dtype, dev)
    page, npages = 64, (L + 63) // 64
    cache = PagedCache([(1, 14)], npages + 3, 2, dtype, dev, page=page)
    perm = torch.randperm(npages + 3, generator=g).tolist()
    cache.free_pages = perm                                               # pages out of order, not the first ones
    cache.admit()
    slot = cache.admit()
    rk, rv = RotaryTable(4, 100.0, None, dev), RotaryTable(6, 100.0, None, dev)
    layer = RotatedValueAttention(ops, heads=2, kv_heads=1, dim=8, vdim=6, scale=1.0, rot_n=4, rope_k=rk, rope_v=rv,
                                  weights={k[2:]: v.to(dtype).to(dev) for k, v in W.items()})
    nq = 3 if as_prompt else 1
    out = None
    for lo, hi in ((0, L - nq), (L - nq, L)):
        rows = cache.extend(slot, hi - lo)
        b = StepBatch(tokens=None, seq=torch.full((hi - lo,), slot, dtype=torch.int32, device=dev),
                      pos=torch.arange(lo, hi, dtype=torch.int32, device=dev), slot=torch.tensor(rows, dtype=torch.int64, device=dev),
                      block_table=cache.block_table(), max_pos=hi - 1, n_tokens=hi - lo, items=[(slot, 0, hi - lo)])
        out = layer(h[lo:hi].to(dtype).to(dev), b, cache.pools, [])
    return out.double().cpu(), ref[L - nq:], h


STORAGE = [pytest.param(torch.float32, 2e-5, id="float32"), pytest.param(torch.bfloat16, 3e-2, id="bfloat16")]


@pytest.mark.parametrize("dtype,tol", STORAGE)
@pytest.mark.parametrize("as_prompt", [False, True], ids=["decoded", "prompt"])
def test_far_keys_and_page_borders_stand_out(backend, as_prompt, dtype, tol):
    L = 330
    for spike in (0, 1, 63, 64, 65, 127, 128, 255, 256, L - 4, L - 1):
        out, ref, h = _selector_attention(backend, L, spike, dtype, as_prompt)
        if spike < L - 3:
            # the far key carries the result: the output is its value, turned by the distance; leaving it out would show
            far = P.rotate_halves(h[spike:spike + 1, None, 24:30], torch.tensor([L - 1 - spike]), P.rotary_frequencies(6, 100.0), 6, -1.0)
            assert (ref[-1, :6] - far[0, 0]).abs().max() < 0.05
        assert_close(out, ref, tol, f"spike at {spike}")


def test_a_far_write_stays_in_the_recurrent_state(backend):
    """Decays close to one and one early token with a large key and value: hundreds of tokens later the read-out is still that
    token's.  Cut into steps, so a state that is dropped, zeroed or taken from another slot shows."""
    for layer in (gla(heads=2, dim=8, vdim=6, tau=64.0), par(r_heads=2, r_kv=1, r_dim=8, r_vdim=6)):
        cfg, W, eng = _one_layer_engine(layer, backend, width=24, seed=5, max_tokens=512)
        p = "l0.mix." if layer["type"] == "gla" else "l0.mix.right."
        if layer["type"] == "gla":
            W[p + "a2.b"] = torch.full_like(W[p + "a2.b"], 9.0)              # sigmoid(9 + small)^(1 / 64): a decay of 1 - 2e-6
            W[p + "a2"] *= 0.1
        else:
            W[p + "dt_bias"] = torch.full_like(W[p + "dt_bias"], -12.0)      # softplus(-12): a decay of 1 - 6e-6 per token
            W[p + "a2"] *= 0.1
            W[p + "b"] = torch.zeros_like(W[p + "b"])                       # the write strength follows input channel 0 alone:
            W[p + "b"][:, 0] = 10.0                                          # ... beta = sigmoid(+-10)
        eng = build_engine(cfg, f32(W), backend, max_tokens=512, max_seqs=3)
        mixer = eng.model.layers[0]["mixer"]
        mixer = mixer if layer["type"] == "gla" else mixer.right
        T = 300
        g = torch.Generator().manual_seed(1)
        h = (torch.randn(T, 24, generator=g) * 0.02).bfloat16().float()
        h[3] = torch.randn(24, generator=g).bfloat16().float() * 3.0
        if layer["type"] == "parallel":          # unit keys: a later write would wipe an earlier one, so only token 3 writes at all
            h[:, 0], h[3, 0] = -1.0, 1.0
        fn = P.gated_linear_attention if layer["type"] == "gla" else P.gated_delta_rule
        m = layer["mixer"] if layer["type"] == "gla" else layer["mixer"]["right"]
        ref = fn(h.double(), {k: v.double() for k, v in W.items()}, p, m, cfg["norm"]["eps"])
        quiet = h.clone()
        quiet[3] = h[4]
        without = fn(quiet.double(), {k: v.double() for k, v in W.items()}, p, m, cfg["norm"]["eps"])
        assert (ref[-1] - without[-1]).abs().max() > 0.05 * ref[-1].abs().max()   # the far token still decides the last output
        eng.open_sequence()                                                   # the test's sequence does not sit in slot 0
        slot = eng.open_sequence()
        p0, p1, s0, s1 = eng.model.run_slices[0]
        states = eng.cache.states[s0 + 1:s1] if layer["type"] == "gla" else eng.cache.states[s0 + 1 + len(eng.model.layers[0]["mixer"].left.state_specs):s1]
        for s in eng.cache.states:
            s.fill_(7.0)                                                      # stale state everywhere: a new sequence must not read it
        outs, lo = [], 0
        for hi in (2, 5, 64, 65, 200, 299, 300):
            b = eng.layout([(slot, [0] * (hi - lo))])
            outs.append(mixer(h[lo:hi].to(eng.device), b, [], states).double().cpu())
            lo = hi
        assert_close(torch.cat(outs), ref, 5e-5, f"{layer['type']}: far write")


# ---- whole model through the engine --------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def std():
    cfg = standard_config()
    W = P.random_weights(cfg, seed=1)
    seqs = {"a": tokens_for(cfg, 150, 1), "b": tokens_for(cfg, 37, 2), "c": tokens_for(cfg, 1, 3), "d": tokens_for(cfg, 81, 4)}
    ref = {k: P.forward(cfg, W, v) for k, v in seqs.items()}
    return cfg, W, seqs, ref


def test_layer_runs_one_by_one(backend, std):
    cfg, W, seqs, _ = std
    eng = build_engine(cfg, f32(W), backend)
    _, ref_layers = P.forward(cfg, W, seqs["b"], return_layers=True)
    assert len(ref_layers) == 6 and eng.model.order == [0, 1, 2, 1, 2, 3]
    slot = eng.open_sequence()
    b = eng.layout([(slot, seqs["b"])])
    seen = []
    eng.model.forward(b, eng.cache.pools, states=eng.cache.states, tap=lambda i, x: seen.append(x.double().cpu().clone()))
    assert len(seen) == 6
    for i, x in enumerate(seen):
        assert_close(x, ref_layers[i], F32_TOL, f"sum of the streams after layer run {i}")


def test_whole_prompts(backend, std):
    cfg, W, seqs, ref = std
    eng = build_engine(cfg, f32(W), backend)
    for k in seqs:
        got = run_schedule(eng, seqs, [[(k, len(seqs[k]))]])
        assert_close(got[k], ref[k], F32_TOL, f"whole prompt {k}")


def test_prefill_then_token_by_token(backend, std):
    cfg, W, seqs, ref = std
    eng = build_engine(cfg, f32(W), backend)
    for k, first in (("a", 60), ("b", 1), ("d", 64)):
        n = len(seqs[k])
        got = run_schedule(eng, seqs, [[(k, first)]] + [[(k, 1)]] * (n - first))
        assert_close(got[k], ref[k], F32_TOL, f"{k}: {first} tokens, then one by one")


def test_portions_of_several_sizes(backend, std):
    cfg, W, seqs, ref = std
    eng = build_engine(cfg, f32(W), backend)
    for sizes in ([2] * 75, [64, 64, 22], [63, 2, 2, 61, 22], [3, 1, 1, 2, 5, 7, 45, 64, 1, 19, 2], [149, 1]):
        assert sum(sizes) == 150
        got = run_schedule(eng, seqs, [[("a", s)] for s in sizes])
        assert_close(got["a"], ref["a"], F32_TOL, f"portions {sizes[:6]}...")


def test_unequal_batches_match_each_alone(backend, std):
    cfg, W, seqs, ref = std
    eng = build_engine(cfg, f32(W), backend)
    steps = [[("a", 29), ("b", 2), ("c", 1)],
             [("a", 64), ("b", 1), ("d", 17)],
             [("b", 30), ("d", 1), ("a", 2)],
             [("d", 63), ("a", 1), ("b", 1)]]
    steps += [[("a", 1), ("b", 1)]] * 3 + [[("a", 1)]] * 51
    got = run_schedule(eng, seqs, steps)
    for k in seqs:
        assert_close(got[k], ref[k], F32_TOL, f"mixed batch, sequence {k}")


def test_a_sequence_left_out_of_steps_goes_on_later(backend, std):
    cfg, W, seqs, ref = std
    eng = build_engine(cfg, f32(W), backend)
    steps = [[("b", 10), ("d", 3)], [("d", 2)], [("d", 1)], [("b", 1), ("d", 1)], [("d", 70)], [("b", 26), ("d", 4)]]
    got = run_schedule(eng, seqs, steps)
    for k in ("b", "d"):
        assert_close(got[k], ref[k], F32_TOL, f"sequence {k}")


def test_pages_slots_and_states_are_used_again(backend, std):
    cfg, W, seqs, ref = std
    eng = build_engine(cfg, f32(W), backend, max_tokens=256, max_seqs=2)          # 4 pages, 2 slots: a (3 pages) + one more
    assert eng.cache.num_pages == 4
    seen_pages = []
    for rnd in range(3):
        order = [("a", "b"), ("d", "b"), ("b", "a")][rnd]
        steps = [[(order[0], 30), (order[1], 5)], [(order[0], len(seqs[order[0]]) - 30), (order[1], len(seqs[order[1]]) - 5)]]
        got = run_schedule(eng, seqs, steps)
        for k in order:
            assert_close(got[k], ref[k], F32_TOL, f"round {rnd}, sequence {k}")
        assert len(eng.cache.free_pages) == 4 and len(eng.cache.free_slots) == 2
        seen_pages.append(tuple(eng.cache.free_pages))
        assert any(float(s.abs().max()) > 0 for s in eng.cache.states)            # the slots' states are left as they were: stale
    assert len(set(seen_pages)) > 1
    s0, s1 = eng.open_sequence(), eng.open_sequence()
    with pytest.raises(CacheFull):
        eng.open_sequence()
    eng.close_sequence(s0)
    eng.close_sequence(s1)


def test_first_tokens_and_single_token_sequences(backend, std):
    cfg, W, seqs, ref = std
    eng = build_engine(cfg, f32(W), backend)
    got = run_schedule(eng, seqs, [[("c", 1)]])
    assert_close(got["c"], ref["c"], F32_TOL)
    got = run_schedule(eng, seqs, [[("b", 1)], [("b", 1)], [("b", 2)], [("b", 33)]])
    assert_close(got["b"][:4], ref["b"][:4], F32_TOL, "first tokens")


def test_long_decoding(backend):
    cfg = make_config([par(mlp=dense(12)), gla(mlp=None)], width=32, vocab=29, streams=3, loop=(0, 2, 2))
    W = P.random_weights(cfg, seed=9)
    toks = tokens_for(cfg, 210, 5)
    ref = P.forward(cfg, W, toks)
    eng = build_engine(cfg, f32(W), backend, max_tokens=256, max_seqs=1)
    got = run_schedule(eng, {"s": toks}, [[("s", 3)]] + [[("s", 1)]] * 207)
    assert_close(got["s"], ref, F32_TOL, "207 decoded tokens")


@pytest.mark.parametrize("variant", range(4))
def test_other_sizes(backend, variant):
    layers, kw = [
        ([gla(heads=1, dim=2, vdim=2, tau=1.0, mlp=moe(experts=2, top=2, ff=1))], dict(width=8, vocab=5, streams=1, eps=1e-3)),
        ([par(heads=6, kv_heads=3, dim=16, vdim=24, rot_dims=16, r_heads=6, r_kv=2, r_dim=20, r_vdim=24, taps=2, mlp=moe(experts=9, top=5, ff=33)),
          gla(heads=4, dim=32, vdim=16, tau=2.0, mlp=dense(100)), gla(heads=2, dim=16, vdim=48, mlp=None)],
         dict(width=96, vocab=200, streams=4, loop=(1, 2, 3), scale=0.5)),
        ([par(heads=2, kv_heads=2, dim=6, vdim=64, rot_dims=2, base=10.0, r_heads=1, r_kv=1, r_dim=70, r_vdim=5, taps=5, mlp=None)] * 2,
         dict(width=40, vocab=33, streams=2, eps=1e-6, loop=(0, 1, 1))),
        ([gla(mlp=dense(8)), par(mlp=moe(experts=3, top=3)), gla(mlp=None)], dict(width=48, vocab=61, streams=2, loop=(0, 3, 2))),
    ][variant]
    cfg = make_config(layers, **kw)
    W = P.random_weights(cfg, seed=20 + variant)
    toks = tokens_for(cfg, 75, variant)
    ref = P.forward(cfg, W, toks)
    eng = build_engine(cfg, f32(W), backend)
    got = run_schedule(eng, {"s": toks}, [[("s", 40)], [("s", 30)]] + [[("s", 1)]] * 5)
    assert_close(got["s"], ref, F32_TOL, f"sizes variant {variant}")


def test_bfloat16_storage_stays_near_the_oracle(backend, std):
    cfg, W, seqs, ref = std
    eng = build_engine(cfg, {k: v.bfloat16() for k, v in W.items()}, backend, dtype="bfloat16")
    got = run_schedule(eng, seqs, [[("a", 70), ("b", 37)], [("a", 80)]])
    for k in ("a", "b"):
        d = got[k] - ref[k]
        rel = (d - d.mean(-1, keepdim=True)).pow(2).mean().sqrt() / ref[k].std()
        assert rel < 0.1, f"bfloat16 run of {k}: relative error {rel:.3f}"
    got2 = run_schedule(eng, seqs, [[("a", 3)], [("a", 147)]])                      # cut differently: the same up to rounding
    rel = (got2["a"] - got["a"]).pow(2).mean().sqrt() / ref["a"].std()
    assert rel < 0.1


# ---- generation through the engine's own entry point and scheduler ---------------------------------------------------------------

def oracle_greedy(cfg, W, prompt, n):
    toks, margins = list(prompt), []
    for _ in range(n):
        lg = P.forward(cfg, W, toks)[-1]
        top2 = lg.topk(2).values
        margins.append(float(top2[0] - top2[1]))
        toks.append(int(lg.argmax()))
    return toks[len(prompt):], margins


def test_greedy_generation_through_the_scheduler(backend, std):
    cfg, W, _, _ = std
    prompts = [tokens_for(cfg, n, 40 + n) for n in (5, 70, 1, 33, 12, 64)]
    eng = build_engine(cfg, f32(W), backend, max_tokens=512, max_seqs=3, max_batch_tokens=48, prefill_chunk=20)
    outs = eng.generate(prompts, SamplingParams(max_new=6))
    assert not eng.has_work() and len(eng.cache.free_pages) == eng.cache.num_pages and len(eng.cache.free_slots) == 3
    for p, o in zip(prompts, outs):
        ref, margins = oracle_greedy(cfg, W, p, 6)
        for i, (a, b) in enumerate(zip(o, ref)):
            if a != b:
                assert margins[i] < 1e-3, f"prompt of {len(p)}: token {i} is {a}, oracle {b} (margin {margins[i]:.2e})"
                break
        else:
            assert len(o) == 6


def test_registry_and_checkpoint_directory(tmp_path, backend, std):
    import json

    from safetensors.torch import save_file

    from qserve_amd.serving import registry
    assert registry.architectures()["Mumelix"] == "paged"
    cfg, W, seqs, ref = std
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.bfloat16().contiguous() for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    eng = Engine.from_pretrained(str(tmp_path), dtype="float32", device=device_of(backend), max_tokens=128, backend=backend)
    got = run_schedule(eng, seqs, [[("b", 37)]])
    assert_close(got["b"], ref["b"], F32_TOL)
    bad = dict(cfg, layers=[dict(cfg["layers"][0], type="unknown")])
    with pytest.raises(ValueError):
        Mumelix.from_config(bad, f32(W), make_ops("unfused", torch.float32, "cpu"), "cpu", torch.float32)


# ---- GPU only: decode steps from a hipGraph advance the recurrent state once ----------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_from_a_graph_match_eager_steps(dtype, std):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    cfg, W, seqs, ref = std
    Wd = f32(W) if dtype == "float32" else {k: v.bfloat16() for k, v in W.items()}
    tol = 2e-5 if dtype == "float32" else 3e-2
    engines = [build_engine(cfg, Wd, "hip", dtype=dtype, decode_graphs=g) for g in (False, True)]
    steps = [[("a", 100), ("b", 20)]] + [[("a", 1), ("b", 1)]] * 6 + [[("d", 30)]] + [[("a", 1), ("b", 1), ("d", 1)]] * 5 + \
            [[("b", 6), ("a", 1)]] + [[("a", 1), ("d", 1)]] * 8
    got = [run_schedule(e, seqs, steps) for e in engines]
    assert any(v is not False for v in engines[1]._graphs.values()), "no step was captured"
    for k in got[0]:
        assert_close(got[1][k], got[0][k], tol, f"graph against eager, sequence {k}")
        if dtype == "float32":
            assert_close(got[1][k], ref[k][:got[0][k].shape[0]], F32_TOL, f"graph against the oracle, sequence {k}")


@pytest.mark.gpu
@pytest.mark.parametrize("E,top,ff,D,T", [(6, 3, 24, 40, 33), (16, 4, 136, 264, 64), (8, 2, 128, 192, 300), (3, 1, 64, 64, 70),
                                          (4, 4, 704, 1024, 150), (8, 8, 520, 2056, 3)])
def test_gated_expert_forms_agree_in_bfloat16(E, top, ff, D, T):
    """Per-token kernels, expert-major kernels, the grouped matrix-core kernel (widths that are multiples of its K step) and
    expert-sorted vendor products on the same bfloat16 inputs, against the float64 sum over the chosen gated experts."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from qserve_amd.layers.moe import _interleave
    dev = "cuda:0"
    g = torch.Generator().manual_seed(E * 100 + T)
    h = torch.randn(T, D, generator=g).bfloat16()
    gate = (torch.randn(E, ff, D, generator=g) / math.sqrt(D)).bfloat16()
    up = (torch.randn(E, ff, D, generator=g) / math.sqrt(D)).bfloat16()
    down = (torch.randn(E, D, ff, generator=g) / math.sqrt(ff)).bfloat16()
    idx = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).int()
    if T > 4:
        idx[:, 0] = idx[0, 0]                                            # one expert shared by many tokens, some experts unused
    wt = torch.rand(T, top, generator=g)
    ref = torch.zeros(T, D, dtype=torch.float64)
    for t in range(T):
        for k in range(top):
            e = int(idx[t, k])
            a = P.silu(gate[e].double() @ h[t].double()) * (up[e].double() @ h[t].double())
            ref[t] += wt[t, k].double() * (down[e].double() @ a)
    forms = {"per-token": dict(moe_token_slots=10 ** 9, moe_sorted_above=10 ** 9),
             "expert-major": dict(moe_token_slots=0, moe_expert_major_slots=10 ** 9),
             "expert-sorted, grouped kernel": dict(moe_token_slots=10 ** 9, moe_expert_major_slots=0, moe_sorted_above=0),
             "expert-sorted, vendor products": dict(moe_token_slots=10 ** 9, moe_expert_major_slots=0, moe_sorted_above=0,
                                                    moe_grouped_kernel=False)}
    w_in = _interleave(gate, up).to(dev)
    for name, knobs in forms.items():
        o = make_ops("hip", torch.bfloat16, dev)
        for k, v in knobs.items():
            setattr(o, k, v)
        y = o.moe_experts(h.to(dev), w_in, down.to(dev), idx.to(dev), wt.to(dev), act="swiglu").double().cpu()
        assert_close(y, ref, 2e-2, f"{name} form")


# ---- host logic alone ------------------------------------------------------------------------------------------------------------

def test_state_rows_swap_per_step_and_follow_the_slot():
    from qserve_amd.serving.cache import PagedCache, StateSpec
    cache = PagedCache([4, (3, 6)], num_pages=4, max_seqs=3, dtype=torch.float32, device="cpu", page=64,
                       states=[StateSpec((2, 5)), StateSpec((7,), copies=2)])
    assert cache.pools[0].shape == (256, 4) and cache.pools[1].shape == (3, 256, 6)
    assert cache.states[0].shape == (3, 2, 5) and cache.states[1].shape == (6, 7)
    a, b = cache.admit(), cache.admit()
    r1, w1 = cache.step_rows(b)
    r2, w2 = cache.step_rows(b)
    assert {r1, w1} == {2 * b, 2 * b + 1} and (r2, w2) == (w1, r1)          # the next step reads what this one wrote
    assert set(cache.step_rows(a)) == {2 * a, 2 * a + 1}
    cfg = make_config([gla()], width=8, vocab=11)
    eng = build_engine(cfg, f32(P.random_weights(cfg)), "unfused", max_tokens=128, max_seqs=2)
    s0, s1 = eng.open_sequence(), eng.open_sequence()
    batch = eng.layout([(s1, [1, 2, 3]), (s0, [4])])
    assert batch.run_off.tolist() == [0, 1, 2, 0] and batch.state_rd.tolist() == [-1] * 4          # both sequences start here
    assert batch.state_wr.tolist()[:2] == [-1, -1] and batch.state_wr.tolist()[2] in (2 * s1, 2 * s1 + 1)
    assert batch.runs().tolist() == [[s1, 0, 3, 0], [s0, 3, 1, 0]]
    nxt = eng.layout([(s1, [5, 6])])
    assert nxt.state_rd.tolist() == [batch.state_wr.tolist()[2]] * 2 and nxt.runs().tolist() == [[s1, 0, 2, 3]]
    with pytest.raises(ValueError):
        eng.layout([(s0, [1]), (s0, [2])])
