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
