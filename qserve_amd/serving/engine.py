"""The serving engine: a registered model + the paged cache + the scheduler + the sampler.

`Engine.step()` is the generation path: schedule -> `execute` -> sample -> book-keeping.  `execute` is the step function -
it lays the scheduled tokens out as one flat batch (token, sequence slot, position, cache row per token), runs the model
over it and returns float logits at the rows asked for.  Callers that bring their own tokens (a recorded trace, a test)
use `open_sequence` / `execute` / `close_sequence` directly and so drive the very same cache and kernels.
"""
import itertools
from dataclasses import dataclass, field

import torch

from ..layers.ops import make_ops
from . import registry
from .cache import PagedCache
from .sampler import SamplingParams, sample
from .scheduler import Request, Scheduler

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclass
class StepBatch:
    """One step's tokens as the kernels read them (device tensors unless noted)."""
    tokens: torch.Tensor        # int32 [T]
    seq: torch.Tensor           # int32 [T]  sequence slot (row of the block table)
    pos: torch.Tensor           # int32 [T]  position in its sequence
    slot: torch.Tensor          # int64 [T]  flat cache row the token's state is written to
    block_table: torch.Tensor   # int32 [slots, pages]
    max_pos: int                # host: largest position in the batch
    n_tokens: int
    items: list = None          # host: [(sequence slot, first flat token index, tokens)] - runs of consecutive positions
    run_off: torch.Tensor = None    # int32 [T]  index of the token within its run
    state_rd: torch.Tensor = None   # int32 [T]  two-copy state row the token's run reads (-1: the run starts its sequence)
    state_wr: torch.Tensor = None   # int32 [T]  two-copy state row to write, on the LAST token of a run (-1 elsewhere)
    _tiles: dict = field(default_factory=dict)
    _runs: torch.Tensor = None

    def runs(self):
        """int32 [n_runs, 4] = (sequence slot, first flat token index, tokens, position of the first token), on the device.
        The engine's layout brings it along with the other metadata; a batch made by hand gets it here (one synchronisation)."""
        if self._runs is None:
            pos = self.pos.tolist()
            rows = [(slot, first, n, pos[first]) for slot, first, n in self.items]
            self._runs = torch.tensor(rows, dtype=torch.int32).reshape(-1, 4).to(self.pos.device)
        return self._runs

    def tiles(self, tokens_per_tile):
        """Work tiles for kernels that serve a few consecutive tokens of one sequence per workgroup: int32 [n, 3] =
        (sequence slot, first flat token index, tokens <= tokens_per_tile), on the device; cached per size."""
        t = self._tiles.get(tokens_per_tile)
        if t is None:
            rows = [(slot, first + o, min(tokens_per_tile, n - o)) for slot, first, n in self.items
                    for o in range(0, n, tokens_per_tile)]
            t = torch.tensor(rows, dtype=torch.int32).reshape(-1, 3).to(self.tokens.device if self.tokens is not None else self.pos.device)
            self._tiles[tokens_per_tile] = t
        return t


class Engine:
    def __init__(self, model_cls, config, weights, dtype="bfloat16", device="cuda:0", max_tokens=4096, max_seqs=4,
                 backend="hip", max_batch_tokens=2048, prefill_chunk=512, page=64, decode_graphs=False):
        """decode_graphs: replay steps in which every sequence brings exactly one token from a hipGraph (captured per batch
        size and context bucket; the launch sequence of such a step has no host synchronisation).  Off unless asked for."""
        self.dtype = DTYPES[dtype] if isinstance(dtype, str) else dtype
        self.device = torch.device(device)
        if self.dtype == torch.float32 and self.device.type == "cuda":
            torch.backends.cuda.matmul.allow_tf32 = False          # float32 means float32 products
            torch.backends.cudnn.allow_tf32 = False
        self.ops = make_ops(backend, self.dtype, self.device)
        self.model = model_cls.from_config(config, weights, self.ops, self.device, self.dtype, page=page)
        self.cache = PagedCache(self.model.cache_rows, (int(max_tokens) + page - 1) // page, max_seqs, self.dtype, self.device,
                                page=page, states=getattr(self.model, "state_specs", ()))
        self.scheduler = Scheduler(self.cache, max_batch_tokens, prefill_chunk)
        self.requests = {}
        self._ids = itertools.count()
        self.decode_graphs = bool(decode_graphs) and backend == "hip"
        self._graphs = {}                      # key -> _DecodeGraph, or False where capture failed (that shape runs eagerly)

    @classmethod
    def from_pretrained(cls, model_dir, **kw):
        """model_dir: config.json + *.safetensors; the model class is chosen by the config's architecture."""
        from ..loader import iterate_checkpoint
        config = registry.read_config(model_dir)
        model_cls, kind = registry.resolve_model(config)
        if kind != "paged":
            raise ValueError(f"architecture {registry.architecture_of(config)!r} is served by the {kind} engine, not this one")
        return cls(model_cls, config, dict(iterate_checkpoint(model_dir)), **kw)

    # ---- the step function -------------------------------------------------------------------------------------------------
    def open_sequence(self):
        return self.cache.admit()

    def close_sequence(self, slot):
        self.cache.release(slot)

    def _layout_host(self, items):
        """Host side of a step's batch: extends the sequences' pages, swaps their two-copy states.  -> (meta int32 [6, T] =
        token, slot, position, index in run, state row to read, state row to write; flat cache rows; runs) or None."""
        toks, seq, pos, rows, runs, off, rd, wr = [], [], [], [], [], [], [], []
        V = self.model.vocab
        if len({slot for slot, t in items if len(t)}) != sum(1 for _, t in items if len(t)):
            raise ValueError("a sequence appears twice in one step")
        for slot, t in items:
            start, n = self.cache.length[slot], len(t)
            if any(not 0 <= int(v) < V for v in t):
                raise ValueError(f"token id outside the vocabulary of {V}")
            if not n:
                continue
            runs.append((slot, len(toks), n))
            rows += self.cache.extend(slot, n)
            toks += [int(v) for v in t]
            seq += [slot] * n
            pos += range(start, start + n)
            r, w = self.cache.step_rows(slot)
            off += range(n)
            rd += [r if start else -1] * n
            wr += [-1] * (n - 1) + [w]
        if not toks:
            return None
        return torch.tensor([toks, seq, pos, off, rd, wr], dtype=torch.int32), rows, runs

    def layout(self, items):
        """items: [(slot, tokens)] -> the StepBatch of these tokens on the device (None if there are none).  Part of `execute`;
        callers that run single layers use it directly."""
        host = self._layout_host(items)
        return None if host is None else self._to_device(*host)

    def _to_device(self, meta, rows, runs):
        dev = self.device
        max_pos, T = int(meta[2].max()), meta.size(1)
        runs4 = torch.tensor([(s, first, n, int(meta[2, first])) for s, first, n in runs], dtype=torch.int32)
        flat = torch.cat([meta.reshape(-1), runs4.reshape(-1)]).to(dev)      # (one host tensor, one copy)
        meta = flat[:6 * T].view(6, T)
        return StepBatch(tokens=meta[0], seq=meta[1], pos=meta[2], slot=torch.tensor(rows, dtype=torch.int64).to(dev),
                         block_table=self.cache.block_table(), max_pos=max_pos, n_tokens=T, items=runs,
                         run_off=meta[3], state_rd=meta[4], state_wr=meta[5], _runs=flat[6 * T:].view(-1, 4))

    @torch.no_grad()
    def execute(self, items, want):
        """items: [(slot, tokens)] - the next tokens of live sequences, all run as one batch; want: flat indices into the
        concatenated tokens.  -> float logits [len(want), vocab] (None if want is empty)."""
        host = self._layout_host(items)
        if host is None:
            return None
        if self.decode_graphs and all(n == 1 for _, _, n in host[2]):
            out = self._execute_graph(*host)
            if out is not None:
                return out[torch.tensor(list(want), dtype=torch.int64, device=self.device)] if want else None
        batch = self._to_device(*host)
        x = self._forward(batch)
        if not want:
            return None
        return self.model.logits(x, torch.tensor(list(want), dtype=torch.int32).to(self.device))

    def _forward(self, batch):
        if self.cache.states:
            return self.model.forward(batch, self.cache.pools, states=self.cache.states)
        return self.model.forward(batch, self.cache.pools)

    # ---- decode steps from a hipGraph ------------------------------------------------------------------------------------------
    GRAPH_BUCKET = 128                         # positions per context bucket (a graph freezes what is derived from max_pos)

    def _execute_graph(self, meta, rows, runs):
        """One token per sequence: fill the static inputs of the graph captured for (batch size, context bucket, model
        signature) and replay it.  -> float logits for every row, or None if this shape runs eagerly."""
        B, dev = meta.size(1), self.device
        bucket = int(meta[2].max()) // self.GRAPH_BUCKET
        sig = self.model.graph_signature() if hasattr(self.model, "graph_signature") else ()
        key = (B, bucket, sig)
        G = self._graphs.get(key)
        if G is False:
            return None
        slot = torch.tensor(rows, dtype=torch.int64)
        runs4 = torch.tensor([(s, first, n, int(meta[2, first])) for s, first, n in runs], dtype=torch.int32).reshape(-1, 4)
        if G is None:
            if len(self._graphs) >= 16:
                self._graphs.clear()
            batch = StepBatch(tokens=None, seq=None, pos=None, slot=slot.to(dev), block_table=self.cache.block_table(),
                              max_pos=(bucket + 1) * self.GRAPH_BUCKET - 1, n_tokens=B, items=list(runs))
            m = meta.to(dev)
            batch.tokens, batch.seq, batch.pos, batch.run_off, batch.state_rd, batch.state_wr = m[0], m[1], m[2], m[3], m[4], m[5]
            batch._runs = runs4.to(dev)
            G = {"meta": m, "batch": batch, "rows": torch.arange(B, dtype=torch.int32, device=dev)}
            if hasattr(self.model, "reserve_positions"):
                self.model.reserve_positions(batch.max_pos + 1)
                key = (B, bucket, self.model.graph_signature() if hasattr(self.model, "graph_signature") else ())
            try:
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                kept = [s.clone() for s in self.cache.states]      # a recurrent state must not advance twice: the warm-up's
                with torch.cuda.stream(side):                      # warm-up outside capture (allocator, lazy initialisation)
                    self.model.logits(self._forward(batch), G["rows"])
                torch.cuda.current_stream().wait_stream(side)
                for s, k in zip(self.cache.states, kept):          # ... step is taken back before the replay takes it
                    s.copy_(k)
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    G["logits"] = self.model.logits(self._forward(batch), G["rows"])
                G["graph"] = g
            except Exception:                                      # e.g. a launch sequence that synchronises: run eagerly
                torch.cuda.synchronize()
                self._graphs[key] = False
                return None
            self._graphs[key] = G
        batch = G["batch"]
        G["meta"].copy_(meta)
        batch.slot.copy_(slot)
        batch._runs.copy_(runs4)
        for tpb, t in batch._tiles.items():
            t.copy_(torch.tensor([(s, first, 1) for s, first, _ in runs], dtype=torch.int32).reshape(-1, 3))
        self.cache.block_table()
        G["graph"].replay()
        return G["logits"]

    # ---- generation ------------------------------------------------------------------------------------------------------------
    def add_request(self, prompt, params=None, request_id=None):
        params = params or SamplingParams()
        rid = request_id if request_id is not None else f"req{next(self._ids)}"
        r = Request(rid, [int(t) for t in prompt], params)
        if params.seed is not None:
            r.generator = torch.Generator(device=self.device).manual_seed(params.seed)
        self.scheduler.add(r)
        self.requests[rid] = r
        return rid

    def step(self):
        """Run one scheduled batch.  -> [(request id, new token, finished)] for the requests that got a token."""
        work = self.scheduler.schedule()
        if not work:
            return []
        want, at = [], 0
        for w in work:
            at += len(w.tokens)
            if w.sample:
                want.append(at - 1)
        logits = self.execute([(w.request.slot, w.tokens) for w in work], want)
        for w in work:
            w.request.computed += len(w.tokens)
        out = []
        if want:
            sampling = [w.request for w in work if w.sample]
            new = sample(logits, [r.params for r in sampling], [r.generator for r in sampling])
            for r, tok in zip(sampling, new):
                r.output.append(tok)
                done = len(r.output) >= r.params.max_new or (r.params.stop_token is not None and tok == r.params.stop_token)
                if done:
                    self.scheduler.finish(r)
                out.append((r.id, tok, done))
        return out

    def has_work(self):
        return bool(self.scheduler.waiting or self.scheduler.running)

    def generate(self, prompts, params=None, **kw):
        """prompts: lists of token ids -> lists of generated token ids (same order)."""
        if params is None:
            params = SamplingParams(**kw)
        ids = [self.add_request(p, params) for p in prompts]
        while self.has_work():
            if not self.step() and not self.scheduler.running:
                raise RuntimeError("the scheduler cannot place any waiting request")
        return [self.requests.pop(i).output for i in ids]
