"""Next-token sampling from float logits: greedy, or temperature with top-k / top-p truncation."""
from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class SamplingParams:
    max_new: int = 16
    temperature: float = 0.0          # 0: greedy
    top_k: int = 0                    # 0: no limit
    top_p: float = 1.0
    seed: Optional[int] = None
    stop_token: Optional[int] = None


def sample(logits, params, generators):
    """logits [R, V] float; params / generators: one per row -> list of R token ids."""
    out = torch.argmax(logits, dim=-1)
    if all(p.temperature <= 0.0 for p in params):
        return out.tolist()
    out = out.tolist()
    for r, p in enumerate(params):
        if p.temperature <= 0.0:
            continue
        z = logits[r] / p.temperature
        if p.top_k and p.top_k < z.numel():
            kth = torch.topk(z, p.top_k).values[-1]
            z = z.masked_fill(z < kth, float("-inf"))
        probs = torch.softmax(z, dim=-1)
        if p.top_p < 1.0:
            sp, si = torch.sort(probs, descending=True)
            keep = torch.cumsum(sp, 0) - sp < p.top_p          # always keeps the most likely token
            probs = torch.zeros_like(probs).scatter_(0, si[keep], sp[keep])
            probs = probs / probs.sum()
        out[r] = int(torch.multinomial(probs, 1, generator=generators[r]))
    return out
