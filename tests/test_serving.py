"""The paged serving engine and the Vekalorn model against the plain float64 oracle (tests/_vekalorn_plain.py).

Every test runs twice: with the unfused tensor-op backend on the CPU (host logic: cache, scheduler, batching, the layers'
composition) and, marked `gpu`, with the HIP kernels.  Configurations and weights are made here (small, random, sizes unlike
each other so that a mixed-up dimension shows); where random weights would hide a fault the inputs are made so that it shows.
"""
import math

import pytest
import torch

import _vekalorn_plain as P
from qserve_amd.layers.ops import make_ops
from qserve_amd.layers.rotary import RotaryTable
from qserve_amd.models.vekalorn import Vekalorn
from qserve_amd.serving import Engine, SamplingParams
from qserve_amd.serving.cache import CacheFull, PagedCache
from qserve_amd.serving.engine import StepBatch
from qserve_amd.serving.scheduler import Request, Scheduler

BACKENDS = [pytest.param("unfused", id="unfused-cpu"), pytest.param("hip", marks=pytest.mark.gpu, id="hip")]


@pytest.fixture(params=BACKENDS)
def backend(request):
    if request.param == "hip" and not torch.cuda.is_available():
        pytest.skip("no GPU")
    return request.param


def device_of(backend):
    return "cuda:0" if backend == "hip" else "cpu"


SCALING = {"factor": 4.0, "original": 24, "fast": 8.0, "slow": 1.0}


def la(heads=2, dim=16, vdim=8, kv_rank=40, q_rank=24, window=5, scale=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if window:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m}


def la2(heads=3, dim=8, rot_dim=8, rot_dims=None, vdim=12, kv_rank=24, q_rank=20, scaling=SCALING, base=1000.0, scale=None):
    rot = {"base": base, "dims": rot_dims if rot_dims is not None else rot_dim}
    if scaling:
        rot["scaling"] = scaling
    return {"type": "latent_attention_2",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "rot": rot, "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim)}}


def moe(experts=6, groups=3, keep=2, top=3, ff=20):
    r = {"experts": experts, "top": top}
    if groups:
        r["groups"] = {"count": groups, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r}


def make_config(layers, width=48, vocab=61, eps=1e-5):
    return {"architecture": "Vekalorn", "width": width, "vocab": vocab, "norm": {"eps": eps},
            "layers": [dict(L, mlp=L.get("mlp")) for L in layers]}


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


def standard_config():
    return make_config([with_mlp(la2(), moe()), with_mlp(la(), moe(experts=4, groups=None, top=1, ff=12)),
                        with_mlp(la2(heads=1, dim=4, rot_dim=12, rot_dims=6, vdim=5, kv_rank=70, q_rank=9, scaling=None), None),
                        with_mlp(la(heads=5, dim=6, vdim=6, kv_rank=130, q_rank=7, window=70), moe(experts=8, groups=2, keep=1, top=4, ff=7))])


def build_engine(cfg, W, backend, dtype="float32", max_tokens=1024, max_seqs=4, **kw):
    return Engine(Vekalorn, cfg, W, dtype=dtype, device=device_of(backend), max_tokens=max_tokens, max_seqs=max_seqs,
                  backend=backend, **kw)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def run_schedule(eng, seqs, steps):
    """seqs: {name: tokens}; steps: [[(name, count), ...]] -> {name: logits [len, vocab]} (every position asked for).  A
    sequence is closed when its last token has run."""
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


F32_TOL = 1e-4      # whole-model float32 runs against float64: rounding through four layers and their norms (a fault shows at 1e-2 and above)


# ---- mechanisms alone -------------------------------------------------------------------------------------------------------------

def test_layer_norms(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(0)
    for D in (5, 48, 300):
        x = torch.randn(7, D, generator=g) * 3 + 1.5
        y = torch.randn(7, D, generator=g) * 2 - 4.0           # a large mean: a one-pass variance would lose digits
        w = torch.randn(D, generator=g)
        xd = x.clone().to(dev)
        h = ops.add_layer_norm(xd, y.to(dev), w.to(dev), 1e-5)
        ref = x.double() + P.layer_norm(y.double(), w.double(), 1e-5)
        assert_close(xd.double().cpu(), ref, 2e-6, f"add_layer_norm D={D}")
        assert_close(h.double().cpu(), ref, 2e-6)
        rows = torch.tensor([6, 0, 3], dtype=torch.int32)
        out = ops.layer_norm_rows(xd, rows.to(dev), w.to(dev), 1e-5)
        assert_close(out.double().cpu(), P.layer_norm(ref[rows.long()], w.double(), 1e-5), 3e-6, f"layer_norm_rows D={D}")


def test_rotary_table_matches_the_scaling_formula():
    for rot in ({"dims": 8, "base": 1000.0, "scaling": SCALING}, {"dims": 6, "base": 50.0},
                {"dims": 16, "base": 250.0, "scaling": {"factor": 2.0, "original": 10, "fast": 2.0, "slow": 0.5}}):
        t = RotaryTable(rot["dims"], rot["base"], rot.get("scaling"), positions=4).reserve(300)
        cos, sin = P.yarn_tables(rot, torch.arange(300))
        assert_close(t[:300, 0].double(), cos, 1e-7)
        assert_close(t[:300, 1].double(), sin, 1e-7)
    # a ramp that really ramps: some frequencies untouched, some divided by the factor, some in between
    r = RotaryTable(16, 250.0, {"factor": 2.0, "original": 10, "fast": 2.0, "slow": 0.5})
    plain = torch.tensor([250.0 ** (-2.0 * i / 16) for i in range(8)], dtype=torch.float64)
    ratio = r.freq / plain
    assert ratio.max() == 1.0 and ratio.min() == 0.5 and ((ratio > 0.5) & (ratio < 1.0)).any()


def _mixer_alone(backend, layer, T, splits):
    """One mixer through the layer object and a cache, the prompt cut at `splits`, against the oracle on the whole sequence."""
    cfg = make_config([layer])
    W = P.random_weights(cfg, seed=3)
    dev = device_of(backend)
    eng = build_engine(cfg, {k: v.float() for k, v in W.items()}, backend, max_tokens=256)
    mixer = eng.model.layers[0]["mixer"]
    g = torch.Generator().manual_seed(5)
    h = torch.randn(T, cfg["width"], generator=g).bfloat16().float()
    fn = P.MIXERS[layer["type"]]
    ref = fn(h.double(), {k: v.double() for k, v in W.items()}, "l0.mix.", layer["mixer"], cfg["norm"]["eps"])
    slot = eng.open_sequence()
    outs, lo = [], 0
    for hi in list(splits) + [T]:
        rows = eng.cache.extend(slot, hi - lo)
        b = StepBatch(tokens=None, seq=torch.full((hi - lo,), slot, dtype=torch.int32, device=dev),
                      pos=torch.arange(lo, hi, dtype=torch.int32, device=dev), slot=torch.tensor(rows, dtype=torch.int64, device=dev),
                      block_table=eng.cache.block_table(), max_pos=hi - 1, n_tokens=hi - lo, items=[(slot, 0, hi - lo)])
        outs.append(mixer(h[lo:hi].to(dev), b, eng.cache.pools[0]).double().cpu())
        lo = hi
    assert_close(torch.cat(outs), ref, F32_TOL, layer["type"])


def test_windowed_latent_attention_alone(backend):
    _mixer_alone(backend, la(window=5), 23, [])
    _mixer_alone(backend, la(window=5), 23, [2, 9, 10, 17])
    _mixer_alone(backend, la(window=1, heads=1), 9, [4])              # sees itself only
    _mixer_alone(backend, la(window=64, kv_rank=64), 150, [63, 64, 65, 129])


def test_rotary_gated_latent_attention_alone(backend):
    _mixer_alone(backend, la2(), 23, [])
    _mixer_alone(backend, la2(), 70, [1, 3, 64, 66])
    _mixer_alone(backend, la2(rot_dim=12, rot_dims=6, scaling=None), 19, [7])       # part of the rotated block passes unrotated
    _mixer_alone(backend, la2(heads=1, dim=4, rot_dim=2, vdim=3, kv_rank=5, q_rank=3), 11, [5])


def test_router_and_experts_alone(backend):
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    g = torch.Generator().manual_seed(11)
    for E, G, keep, top, ff, D in ((6, 3, 2, 3, 20, 40), (4, 1, 1, 1, 12, 40), (8, 2, 1, 4, 7, 36), (12, 4, 3, 4, 9, 40),
                                   (5, 5, 2, 2, 6, 20), (4, 2, 1, 2, 24, 72), (3, 1, 1, 2, 1032, 520)):
        T = 33
        h = torch.randn(T, D, generator=g)
        Wr = torch.randn(E, D, generator=g) * 0.6
        r = {"experts": E, "top": top, "groups": {"count": G, "keep": keep}}
        idx, wt = ops.moe_route(h.to(dev), Wr.to(dev).contiguous(), top, G, keep)
        ridx, rwt = P.route(h.double(), Wr.double(), r)
        order = idx.cpu().long().argsort(dim=1), ridx.argsort(dim=1)
        assert torch.equal(idx.cpu().long().gather(1, order[0]), ridx.gather(1, order[1])), f"experts chosen, E={E} G={G}"
        assert_close(wt.cpu().double().gather(1, order[0]), rwt.gather(1, order[1]), 2e-6)
        assert (wt.sum(1) < 1.0 + 1e-6).all()                 # scores as they are: not renormalised to one
        W = {"p.router": Wr.double()}
        ups, downs = [], []
        for e in range(E):
            ups.append(torch.randn(ff, D, generator=g) / math.sqrt(D))
            downs.append(torch.randn(D, ff, generator=g) / math.sqrt(ff))
            W[f"p.e{e}.up"], W[f"p.e{e}.down"] = ups[-1].double(), downs[-1].double()
        y = ops.moe_experts(h.to(dev), torch.stack(ups).to(dev), torch.stack(downs).to(dev), idx, wt)
        ref = P.moe(h.double(), W, "p.", {"router": r})
        assert_close(y.double().cpu(), ref, 1e-5, f"moe E={E}")
        if backend == "hip":                                  # both forms: per-token kernels and expert-sorted products
            for above in (0, 10 ** 9):
                ops.moe_sorted_above = above
                y = ops.moe_experts(h.to(dev), torch.stack(ups).to(dev), torch.stack(downs).to(dev), idx, wt)
                assert_close(y.double().cpu(), ref, 1e-5, f"moe E={E}, sorted above {above}")
            del ops.moe_sorted_above


def test_group_limit_changes_the_choice(backend):
    """Scores made so that the two best experts sit in one group and the third best in a group that is NOT kept."""
    dev = device_of(backend)
    ops = make_ops(backend, torch.float32, dev)
    z = torch.tensor([[3.0, 2.9, 0.0, 0.0, 2.8, 0.1, 1.0, 0.9]])       # groups of 2: maxima 3.0, 0.0, 2.8, 1.0
    h = torch.zeros(1, 8)
    h[0, 0] = 1.0
    Wr = torch.zeros(8, 8)
    Wr[:, 0] = z[0]
    idx, _ = ops.moe_route(h.to(dev), Wr.to(dev), 3, 4, 2)              # keep groups 0 and 2 -> experts 0, 1, 4
    assert sorted(idx[0].tolist()) == [0, 1, 4]
    idx, _ = ops.moe_route(h.to(dev), Wr.to(dev), 2, 4, 1)              # keep group 0 only
    assert sorted(idx[0].tolist()) == [0, 1]
    idx, _ = ops.moe_route(h.to(dev), Wr.to(dev), 4, 1, 1)              # no groups: plain top-4
    assert sorted(idx[0].tolist()) == [0, 1, 4, 6]


# ---- one score that stands out: far keys, page borders, window edges -----------------------------------------------------------

def _spike_case(ops, dev, rank, rot, page, L, spike, window, as_prompt):
    """(see below; inputs are bfloat16-representable so that both storage types see the same numbers)"""
    return _spike_case_impl(ops, dev, rank, rot, page, L, spike, window, as_prompt)


def _spike_case_impl(ops, dev, rank, rot, page, L, spike, window, as_prompt):
    """Cache of L rows of small noise; the row at `spike` carries a large value in `rank` direction 0 and the query (position
    L - 1) points there.  -> (weight the kernel gives, reference weight) of the spike row's contribution."""
    R = rank + rot
    g = torch.Generator().manual_seed(spike * 7 + L)
    npages = (L + page - 1) // page
    perm = torch.randperm(npages + 3, generator=g)[:npages]             # pages out of order, not the first ones
    pool = torch.zeros(((npages + 3) * page, R))
    rows = (torch.randn(L, R, generator=g) * 0.05).bfloat16().float()
    rows[spike, 0] = 6.0
    j = torch.arange(L)
    pool[perm[j // page] * page + j % page] = rows
    bt = torch.zeros((2, npages + 3), dtype=torch.int32)
    bt[1, :npages] = perm.int()
    nq = 3 if as_prompt else 1                                          # a prompt portion: the last 3 positions together
    qf = (torch.randn(nq, 2, R, generator=g) * 0.05).bfloat16().float()
    qf[:, :, 0] = 2.0
    pos = torch.arange(L - nq, L, dtype=torch.int32)
    b = StepBatch(tokens=None, seq=torch.ones(nq, dtype=torch.int32, device=dev), pos=pos.to(dev), slot=None, block_table=bt.to(dev),
                  max_pos=L - 1, n_tokens=nq, items=[(1, 0, nq)])
    out = ops.latent_attention(qf.to(dev), pool.to(dev).to(ops.dtype), b, window, rank, page)
    ref = torch.empty(nq, 2, rank, dtype=torch.float64)
    for t in range(nq):
        p = int(pos[t])
        lo = max(0, p - window + 1) if window else 0
        w = torch.softmax(qf[t].double() @ rows[lo:p + 1].double().T, dim=-1)
        ref[t] = w @ rows[lo:p + 1, :rank].double()
    return out.double().cpu(), ref


STORAGE = [pytest.param(torch.float32, 1e-5, id="float32"), pytest.param(torch.bfloat16, 2e-2, id="bfloat16")]


@pytest.mark.parametrize("dtype,tol", STORAGE)
@pytest.mark.parametrize("as_prompt", [False, True], ids=["decoded", "prompt"])
def test_far_keys_and_page_borders_stand_out(backend, as_prompt, dtype, tol):
    dev = device_of(backend)
    ops = make_ops(backend, dtype, dev)
    L = 700
    for spike in (0, 1, 63, 64, 65, 127, 128, 500, 639, 640, L - 4, L - 1):
        out, ref = _spike_case(ops, dev, 24, 8, 64, L, spike, 0, as_prompt)
        assert ref[-1, 0, 0] > 3.0                                      # the far key carries the result: leaving it out would show
        assert_close(out, ref, tol, f"spike at {spike}")


@pytest.mark.parametrize("dtype,tol", STORAGE)
@pytest.mark.parametrize("as_prompt", [False, True], ids=["decoded", "prompt"])
def test_window_edges_stand_out(backend, as_prompt, dtype, tol):
    dev = device_of(backend)
    ops = make_ops(backend, dtype, dev)
    for window, L in ((48, 210), (64, 200), (65, 200), (3, 130), (1, 70)):
        p = L - 1
        for spike, inside in ((p - window + 1, True), (p - window, False), (p - window - 1, False)):
            if spike < 0:
                continue
            out, ref = _spike_case(ops, dev, 16, 0, 64, L, spike, window, as_prompt)
            assert (ref[-1, 0, 0] > 3.0) == inside                      # just inside: it dominates; just outside: it is not seen
            assert_close(out, ref, tol, f"window {window}, spike at {spike}")


# ---- whole model through the engine --------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def std():
    cfg = standard_config()
    W = P.random_weights(cfg, seed=1)
    seqs = {"a": tokens_for(cfg, 150, 1), "b": tokens_for(cfg, 37, 2), "c": tokens_for(cfg, 1, 3), "d": tokens_for(cfg, 81, 4)}
    ref = {k: P.forward(cfg, W, v) for k, v in seqs.items()}
    return cfg, W, seqs, ref


def f32(W):
    return {k: (v.float() if v.is_floating_point() else v) for k, v in W.items()}


def test_layers_one_by_one(backend, std):
    cfg, W, seqs, _ = std
    eng = build_engine(cfg, f32(W), backend)
    _, ref_layers = P.forward(cfg, W, seqs["b"], return_layers=True)
    slot = eng.open_sequence()
    rows = eng.cache.extend(slot, len(seqs["b"]))
    dev = eng.device
    n = len(seqs["b"])
    b = StepBatch(tokens=torch.tensor(seqs["b"], dtype=torch.int32, device=dev), seq=torch.full((n,), slot, dtype=torch.int32, device=dev),
                  pos=torch.arange(n, dtype=torch.int32, device=dev), slot=torch.tensor(rows, dtype=torch.int64, device=dev),
                  block_table=eng.cache.block_table(), max_pos=n - 1, n_tokens=n, items=[(slot, 0, n)])
    seen = []
    eng.model.forward(b, eng.cache.pools, tap=lambda i, x: seen.append(x.double().cpu().clone()))
    assert len(seen) == len(cfg["layers"])
    for i, x in enumerate(seen):
        assert_close(x, ref_layers[i], F32_TOL, f"residual stream after layer {i}")


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


def test_pages_and_slots_are_used_again(backend, std):
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
    assert len(set(seen_pages)) > 1                                               # the free list's order really changed
    s0, s1 = eng.open_sequence(), eng.open_sequence()
    with pytest.raises(CacheFull):
        eng.open_sequence()
    eng.cache.extend(s0, 200)
    with pytest.raises(CacheFull):
        eng.cache.extend(s1, 65)
    eng.close_sequence(s0)
    eng.cache.extend(s1, 65)
    eng.close_sequence(s1)


def test_first_tokens_and_single_token_sequences(backend, std):
    cfg, W, seqs, ref = std
    eng = build_engine(cfg, f32(W), backend)
    got = run_schedule(eng, seqs, [[("c", 1)]])
    assert_close(got["c"], ref["c"], F32_TOL)
    got = run_schedule(eng, seqs, [[("b", 1)], [("b", 1)], [("b", 2)], [("b", 33)]])
    assert_close(got["b"][:4], ref["b"][:4], F32_TOL, "first tokens")


def test_long_decoding_across_pages_and_windows(backend):
    cfg = make_config([with_mlp(la(window=70, kv_rank=33), moe()), with_mlp(la2(), None)], width=32, vocab=29)
    W = P.random_weights(cfg, seed=9)
    toks = tokens_for(cfg, 210, 5)
    ref = P.forward(cfg, W, toks)
    eng = build_engine(cfg, f32(W), backend, max_tokens=256, max_seqs=1)
    got = run_schedule(eng, {"s": toks}, [[("s", 3)]] + [[("s", 1)]] * 207)
    assert_close(got["s"], ref, F32_TOL, "207 decoded tokens")


@pytest.mark.parametrize("variant", range(3))
def test_other_sizes(backend, variant):
    layers = [
        [with_mlp(la(heads=1, dim=2, vdim=1, kv_rank=3, q_rank=2, window=2), moe(experts=2, groups=2, keep=1, top=1, ff=1))],
        [with_mlp(la2(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=96, q_rank=64), moe(experts=9, groups=3, keep=3, top=5, ff=33)),
         with_mlp(la(heads=4, dim=32, vdim=40, kv_rank=200, q_rank=10, window=None), None)],
        [with_mlp(la2(heads=2, dim=6, rot_dim=64, rot_dims=64, vdim=6, kv_rank=260, q_rank=8, base=100.0), moe(experts=3, groups=1, keep=1, top=3))] * 3,
    ][variant]
    cfg = make_config(layers, width=[8, 96, 40][variant], vocab=[5, 200, 33][variant], eps=[1e-5, 1e-3, 1e-6][variant])
    W = P.random_weights(cfg, seed=20 + variant)
    toks = tokens_for(cfg, 75, variant)
    ref = P.forward(cfg, W, toks)
    eng = build_engine(cfg, f32(W), backend)
    got = run_schedule(eng, {"s": toks}, [[("s", 40)], [("s", 30)]] + [[("s", 1)]] * 5)
    assert_close(got["s"], ref, F32_TOL, f"sizes variant {variant}")


def test_bfloat16_storage_stays_near_the_oracle(backend, std):
    cfg, W, seqs, ref = std
    eng = build_engine(cfg, W, backend, dtype="bfloat16")
    got = run_schedule(eng, seqs, [[("a", 70), ("b", 37)], [("a", 80)]])
    for k in ("a", "b"):
        d = got[k] - ref[k]
        rel = (d - d.mean(-1, keepdim=True)).pow(2).mean().sqrt() / ref[k].std()
        assert rel < 0.15, f"bfloat16 run of {k}: relative error {rel:.3f}"
    # cut differently: the same logits up to rounding
    got2 = run_schedule(eng, seqs, [[("a", 3)], [("a", 147)]])
    rel = (got2["a"] - got["a"]).pow(2).mean().sqrt() / ref["a"].std()
    assert rel < 0.15


# ---- generation through the engine's own entry point and scheduler ---------------------------------------------------------------

def oracle_greedy(cfg, W, prompt, n):
    toks = list(prompt)
    margins = []
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


def test_sampling_is_seeded_and_truncated(backend, std):
    cfg, W, _, _ = std
    eng = build_engine(cfg, f32(W), backend, max_tokens=512)
    p = tokens_for(cfg, 9, 77)
    a = eng.generate([p], SamplingParams(max_new=8, temperature=0.9, top_k=5, top_p=0.9, seed=3))
    b = eng.generate([p], SamplingParams(max_new=8, temperature=0.9, top_k=5, top_p=0.9, seed=3))
    assert a == b and len(a[0]) == 8
    g = eng.generate([p], SamplingParams(max_new=4))
    k1 = eng.generate([p], SamplingParams(max_new=4, temperature=5.0, top_k=1, seed=1))
    assert g == k1                                                       # top-1 sampling is greedy whatever the temperature


# ---- host logic alone ------------------------------------------------------------------------------------------------------------

def test_scheduler_admission_and_budget():
    cache = PagedCache([4], num_pages=6, max_seqs=2, dtype=torch.float32, device="cpu", page=64)
    s = Scheduler(cache, max_batch_tokens=100, prefill_chunk=64)
    r1 = Request("r1", list(range(130)), SamplingParams(max_new=60))     # life 190 -> 3 pages
    r2 = Request("r2", list(range(100)), SamplingParams(max_new=100))    # life 200 -> 4 pages: does not fit beside r1
    r3 = Request("r3", list(range(10)), SamplingParams(max_new=10))      # 1 page, but behind r2 in the queue
    for r in (r1, r2, r3):
        s.add(r)
    w = s.schedule()
    assert [x.request.id for x in w] == ["r1"] and len(w[0].tokens) == 64 and not w[0].sample
    cache.extend(r1.slot, 64)
    r1.computed = 64
    w = s.schedule()
    assert len(w) == 1 and w[0].start == 64 and len(w[0].tokens) == 64    # r2 still waits: its pages are promised to r1
    cache.extend(r1.slot, 64)
    r1.computed = 128
    w = s.schedule()
    assert len(w[0].tokens) == 2 and w[0].sample
    s.finish(r1)
    w = s.schedule()
    assert [x.request.id for x in w] == ["r2", "r3"] and [len(x.tokens) for x in w] == [64, 10]
    with pytest.raises(ValueError):
        s.add(Request("big", list(range(400)), SamplingParams(max_new=1)))


def test_registry_knows_the_model_families():
    from qserve_amd.serving import registry
    a = registry.architectures()
    assert a["Vekalorn"] == "paged" and a["llama_w4a8"] == "static-batch"
    with pytest.raises(ValueError):
        registry.resolve_model({"architecture": "nothing"})
    cfg = standard_config()
    cfg["layers"][0]["type"] = "unknown_mixer"
    with pytest.raises(ValueError):
        Vekalorn.from_config(cfg, f32(P.random_weights(standard_config())), make_ops("unfused", torch.float32, "cpu"), "cpu",
                             torch.float32)


def test_checkpoint_directory_round_trip(tmp_path, backend, std):
    """config.json + model.safetensors on disk -> Engine.from_pretrained -> the same logits."""
    import json

    from safetensors.torch import save_file
    cfg, W, seqs, ref = std
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    eng = Engine.from_pretrained(str(tmp_path), dtype="float32", device=device_of(backend), max_tokens=128, backend=backend)
    got = run_schedule(eng, seqs, [[("b", 37)]])
    assert_close(got["b"], ref["b"], F32_TOL)


# ---- the two attention kernels against each other (GPU only) ------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("heads,rank,rot", [(1, 24, 8), (3, 96, 16), (6, 128, 0), (16, 192, 64), (40, 64, 32), (8, 512, 64)])
def test_matrix_core_attention_matches_the_wave_kernel(heads, rank, rot):
    """Prompt portions of several lengths and single decoded tokens of several sequences in ONE launch, with and without a
    window: the matrix-core kernel against the wave kernel on the same bfloat16 cache (they differ by the bfloat16 rounding
    of the query and of the probabilities only) and against a float64 softmax over the same rows."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev, page, R = "cuda:0", 64, rank + rot
    ops = make_ops("hip", torch.bfloat16, dev)
    g = torch.Generator().manual_seed(heads * 1000 + rank)
    runs = [(0, 0, 130), (1, 200, 1), (2, 63, 2), (3, 31, 33), (4, 500, 5), (5, 0, 1), (6, 64, 1)]      # (slot, start, tokens)
    npages = sum((s + n + page - 1) // page for _, s, n in runs)
    perm = torch.randperm(npages + 2, generator=g).int()
    pool = (torch.randn((npages + 2) * page, R, generator=g) * 0.5).bfloat16()
    bt = torch.zeros((len(runs), 16), dtype=torch.int32)
    used, seq, pos, items = 0, [], [], []
    for slot, start, n in runs:
        k = (start + n + page - 1) // page
        bt[slot, :k] = perm[used:used + k]
        used += k
        items.append((slot, len(seq), n))
        seq += [slot] * n
        pos += range(start, start + n)
    T = len(seq)
    qf = (torch.randn(T, heads, R, generator=g) * (2.0 / math.sqrt(R))).bfloat16().float()
    b = StepBatch(tokens=None, seq=torch.tensor(seq, dtype=torch.int32, device=dev), pos=torch.tensor(pos, dtype=torch.int32, device=dev),
                  slot=None, block_table=bt.to(dev), max_pos=max(pos), n_tokens=T, items=items)
    for window in (0, 7, 33, 64, 100):
        o_mfma = ops.latent_attention(qf.to(dev), pool.to(dev), b, window, rank, page, variant=0).double().cpu()
        o_wave = ops.latent_attention(qf.to(dev), pool.to(dev), b, window, rank, page, variant=1).double().cpu()
        ref = torch.empty(T, heads, rank, dtype=torch.float64)
        for t in range(T):
            lo = max(0, pos[t] - window + 1) if window else 0
            j = torch.arange(lo, pos[t] + 1)
            rows = pool[bt[seq[t], j // page].long() * page + j % page].double()
            ref[t] = torch.softmax(qf[t].double() @ rows.T, dim=-1) @ rows[:, :rank]
        assert_close(o_wave, ref, 5e-3, f"wave kernel, window {window}")
        assert_close(o_mfma, ref, 1e-2, f"matrix-core kernel, window {window}")
        for splits in (1, 3, 8):                                         # the keys of every tile cut over several workgroups
            o = ops.latent_attention(qf.to(dev), pool.to(dev), b, window, rank, page, key_splits=splits).double().cpu()
            assert_close(o, ref, 1e-2, f"matrix-core kernel, window {window}, {splits} key splits")


@pytest.mark.gpu
@pytest.mark.parametrize("E,top,ff,D,T", [(6, 3, 24, 40, 33), (16, 4, 136, 264, 64), (4, 2, 8, 520, 5), (8, 8, 1032, 2056, 3),
                                          (8, 2, 128, 192, 300), (3, 1, 64, 64, 70), (4, 4, 1408, 1024, 150)])
def test_expert_forms_agree_in_bfloat16(E, top, ff, D, T):
    """Per-token kernels, expert-major kernels, the grouped matrix-core kernel (widths that are multiples of 64) and
    expert-sorted vendor products on the same bfloat16 inputs, against the float64 sum over the chosen experts."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    dev = "cuda:0"
    ops = make_ops("hip", torch.bfloat16, dev)
    g = torch.Generator().manual_seed(E * 100 + T)
    h = torch.randn(T, D, generator=g).bfloat16()
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
            a = torch.relu(up[e].double() @ h[t].double()) ** 2
            ref[t] += wt[t, k].double() * (down[e].double() @ a)
    forms = {"per-token": dict(moe_token_slots=10 ** 9, moe_sorted_above=10 ** 9),
             "expert-major": dict(moe_token_slots=0, moe_expert_major_slots=10 ** 9),
             "expert-sorted, grouped kernel": dict(moe_token_slots=10 ** 9, moe_expert_major_slots=0, moe_sorted_above=0),
             "expert-sorted, vendor products": dict(moe_token_slots=10 ** 9, moe_expert_major_slots=0, moe_sorted_above=0,
                                                    moe_grouped_kernel=False)}
    for name, knobs in forms.items():
        o = make_ops("hip", torch.bfloat16, dev)
        for k, v in knobs.items():
            setattr(o, k, v)
        y = o.moe_experts(h.to(dev), up.to(dev), down.to(dev), idx.to(dev), wt.to(dev)).double().cpu()
        assert_close(y, ref, 2e-2, f"{name} form")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_from_a_graph_match_eager_steps(dtype, std):
    """Single-token steps replayed from a hipGraph against the same steps run eagerly: several replays of each graph with
    eager work (prompt portions, other batch sizes) between them, a sequence that ends and one that joins on its slot."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    cfg, W, seqs, ref = std
    Wd = f32(W) if dtype == "float32" else W
    tol = 2e-5 if dtype == "float32" else 3e-2
    engines = [build_engine(cfg, Wd, "hip", dtype=dtype, decode_graphs=g) for g in (False, True)]
    steps = [[("a", 100), ("b", 20)]] + [[("a", 1), ("b", 1)]] * 6 + [[("d", 30)]] + [[("a", 1), ("b", 1), ("d", 1)]] * 5 + \
            [[("b", 6), ("a", 1)]] + [[("a", 1), ("d", 1)]] * 8 + [[("c", 1)], [("a", 1), ("d", 1)], [("a", 1), ("d", 1)]]
    got = [run_schedule(e, seqs, steps) for e in engines]
    assert any(v is not False for v in engines[1]._graphs.values()), "no step was captured"
    assert len(engines[1]._graphs) >= 3
    for k in got[0]:
        assert_close(got[1][k], got[0][k], tol, f"graph against eager, sequence {k}")
        if dtype == "float32":
            assert_close(got[1][k], ref[k][:got[0][k].shape[0]], 3e-5, f"graph against the oracle, sequence {k}")
