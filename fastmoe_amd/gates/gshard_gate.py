r"""GShard's balanced top-2 gate (fmoe/gates/gshard_gate.py)."""
import math

import torch
import torch.nn.functional as F

from .. import fmoe_cuda as fmoe_native
from .naive_gate import NaiveGate


def _histogram(idx, n_expert):
    r"""Entries of `idx` per expert (`-1` skipped), int32 on the device, by the
    library's histogram kernel: nothing is read back to the host, which keeps
    the gate inside a HIP graph."""
    count = torch.zeros(n_expert, dtype=torch.int32, device=idx.device)
    fmoe_native.expert_count(idx.contiguous(), count)
    return count


class GShardGate(NaiveGate):
    r"""Top-2 gate with a load-balance loss, a per-expert capacity of
    `ceil(rate * tokens) * 2 // experts` slots (rate = `capacity[0]` in
    training, `capacity[1]` in evaluation) and optional random dropping of the
    second expert when its weight is small."""

    def __init__(self, d_model, num_expert, world_size, topk=2,
                 capacity=(1.2, 2.4), random_routing=True, gate_bias=True):
        assert topk == 2, "topk should be 2 in gshard"
        super().__init__(d_model, num_expert, world_size, top_k=2, gate_bias=gate_bias)
        self.capacity = capacity
        self.random_routing = random_routing

    def forward(self, x):
        topk_idx, topk_val, logits = super().forward(x, return_all_scores=True)
        n_tok = logits.shape[0]
        top1 = topk_idx.view(-1, self.top_k)[:, 0]
        frac = _histogram(top1, self.tot_expert).to(torch.float) / n_tok
        prob = F.softmax(logits, dim=1).mean(dim=0)
        self.set_loss(torch.mean(frac * prob) * (self.num_expert ** 2))

        rate = self.capacity[0 if self.training else 1]
        cap = math.ceil(rate * x.shape[0]) * self.top_k // (self.world_size * self.num_expert)
        budget = torch.full((self.tot_expert,), cap, dtype=torch.int32,
                            device=topk_idx.device)
        topk_idx = fmoe_native.prune_gate_by_capacity(
            topk_idx.contiguous(), budget, self.num_expert, self.world_size)

        if self.random_routing:
            coin = torch.rand(logits.size(0), device=x.device)
            topk_idx[:, 1].masked_fill_(2 * topk_val[:, 1] < coin, -1)
        return topk_idx, topk_val
