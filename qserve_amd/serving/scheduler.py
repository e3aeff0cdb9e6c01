"""Continuous batching: which tokens of which requests run in the next step.

A step's batch mixes single decoded tokens of requests whose prompt is done with portions of prompts still being read.
Policy: decode tokens first (one per running request), then prompt portions in admission order up to `max_batch_tokens`
(a portion is at most `prefill_chunk` tokens and can end anywhere), then new requests are admitted while a slot is free
and the pages for their whole life (prompt + max_new) are not promised to others - so a running request never waits for
a page and nothing has to be preempted.
"""
from collections import deque
from dataclasses import dataclass, field

from .sampler import SamplingParams


@dataclass
class Request:
    id: str
    prompt: list
    params: SamplingParams = field(default_factory=SamplingParams)
    output: list = field(default_factory=list)
    slot: int = -1
    computed: int = 0                 # tokens whose state is in the cache
    finished: bool = False
    generator: object = None

    def tokens(self):
        return self.prompt + self.output

    def life(self):
        return len(self.prompt) + self.params.max_new


@dataclass
class Work:
    request: Request
    tokens: list                      # the tokens this step runs for the request
    start: int                        # position of the first of them
    sample: bool                      # the last of them ends the known sequence: sample what follows


class Scheduler:
    def __init__(self, cache, max_batch_tokens=2048, prefill_chunk=512):
        self.cache, self.max_batch_tokens, self.prefill_chunk = cache, int(max_batch_tokens), int(prefill_chunk)
        self.waiting, self.running = deque(), []

    def add(self, req):
        if req.life() > self.cache.num_pages * self.cache.page:
            raise ValueError(f"request {req.id}: {req.life()} tokens can never fit a cache of "
                             f"{self.cache.num_pages * self.cache.page}")
        if not req.prompt:
            raise ValueError(f"request {req.id}: empty prompt")
        self.waiting.append(req)

    def _promised(self):
        """Pages the running requests may still ask for."""
        c = self.cache
        return sum(c.pages_for(r.life()) - len(c.pages[r.slot]) for r in self.running)

    def _admit(self):
        c = self.cache
        while self.waiting and c.free_slots:
            r = self.waiting[0]
            if c.pages_for(r.life()) > len(c.free_pages) - self._promised():
                break
            self.waiting.popleft()
            r.slot = c.admit()
            self.running.append(r)

    def schedule(self):
        """-> list of Work for the next step (empty: nothing to do)."""
        self._admit()
        budget, work = self.max_batch_tokens, []
        for r in self.running:                                   # decoded tokens first
            known = r.tokens()
            if r.computed >= len(r.prompt) and budget > 0:
                work.append(Work(r, known[r.computed:], r.computed, True))
                budget -= len(known) - r.computed
        for r in self.running:                                   # then portions of prompts
            if r.computed < len(r.prompt) and budget > 0:
                n = min(len(r.prompt) - r.computed, self.prefill_chunk, budget)
                work.append(Work(r, r.prompt[r.computed:r.computed + n], r.computed, r.computed + n == len(r.prompt)))
                budget -= n
        return work

    def finish(self, req):
        req.finished = True
        self.running.remove(req)
        self.cache.release(req.slot)
        req.slot = -1
