"""Mixture of small feed-forward experts behind a grouped top-k router.

score = softmax(router . h) over all experts (float).  The experts form `groups` equal groups of neighbours; a group's score
is its largest expert score and only experts of the `keep` best groups are eligible (groups = keep = 1: a plain top-k
router).  The `top_k` eligible experts with the largest scores are used, weighted by those scores as they are (no
renormalisation).  Expert: down . act(up . h), act = relu(.)^2, no biases.
"""
import torch


class GroupedTopKMoE:
    def __init__(self, ops, *, router, up, down, top_k, groups=1, keep=1):
        """router [E, D]; up: list of E [ff, D]; down: list of E [D, ff] (stacked here into [E, ff, D] / [E, D, ff])."""
        self.ops = ops
        self.router = router.contiguous()
        self.up, self.down = torch.stack(list(up)).contiguous(), torch.stack(list(down)).contiguous()
        E, ff, D = self.up.shape
        self.top_k, self.groups, self.keep = int(top_k), int(groups), int(keep)
        if self.router.shape != (E, D) or self.down.shape != (E, D, ff):
            raise ValueError("mixture of experts: router / expert shapes do not fit each other")
        if E % self.groups or not 0 < self.keep <= self.groups or not 0 < self.top_k <= self.keep * (E // self.groups):
            raise ValueError(f"router: {E} experts, {self.groups} groups, keep {self.keep}, top {self.top_k}")

    def __call__(self, h):
        idx, wt = self.ops.moe_route(h, self.router, self.top_k, self.groups, self.keep)
        return self.ops.moe_experts(h, self.up, self.down, idx, wt)


def _interleave(gate, up):
    """[..., ff, D] gate and up rows -> [..., 2 ff, D] with row 2f = gate f and row 2f + 1 = up f, so that one product gives a
    gated unit's two halves as neighbours (qserve_amd.layers.ops `glu`)."""
    return torch.stack([gate, up], dim=-2).reshape(*gate.shape[:-2], 2 * gate.size(-2), gate.size(-1)).contiguous()


class GatedFeedForward:
    """Dense gated feed-forward: down . (silu(gate . h) * (up . h)), no biases."""

    def __init__(self, ops, *, gate, up, down):
        if gate.shape != up.shape or down.shape != (gate.size(1), gate.size(0)):
            raise ValueError("gated feed-forward: gate / up / down shapes do not fit each other")
        self.ops, self.w_in, self.w_down = ops, _interleave(gate, up), down.contiguous()

    def __call__(self, h):
        from .ops import linear
        return linear(self.ops.glu(linear(h, self.w_in)), self.w_down)


class TopKGatedMoE:
    """Mixture of gated experts behind a plain top-k router with a bias: logits z = router . h + bias (float); the `top_k`
    largest are chosen and weighted by the softmax over the chosen logits only.  Expert: down . (silu(gate . h) * (up . h))."""

    def __init__(self, ops, *, router, bias, gate, up, down, top_k):
        """router [E, D], bias [E]; gate / up: lists of E [ff, D]; down: list of E [D, ff]."""
        self.ops = ops
        self.router, self.bias = router.contiguous(), bias.contiguous()
        self.up = _interleave(torch.stack(list(gate)), torch.stack(list(up)))          # [E, 2 ff, D]
        self.down = torch.stack(list(down)).contiguous()
        E, ff2, D = self.up.shape
        self.top_k = int(top_k)
        if self.router.shape != (E, D) or self.bias.shape != (E,) or self.down.shape != (E, D, ff2 // 2):
            raise ValueError("mixture of experts: router / expert shapes do not fit each other")
        if not 0 < self.top_k <= E:
            raise ValueError(f"router: {E} experts, top {self.top_k}")

    def __call__(self, h):
        idx, wt = self.ops.moe_route(h, self.router, self.top_k, 1, 1, bias=self.bias, renorm=True)
        return self.ops.moe_experts(h, self.up, self.down, idx, wt, act="swiglu")
