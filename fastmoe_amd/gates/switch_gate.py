r"""Switch Transformer's top-1 gate (fmoe/gates/switch_gate.py)."""
import math

import torch
import torch.nn.functional as F

from .gshard_gate import _histogram
from .naive_gate import NaiveGate
from .utils import limit_by_capacity


class SwitchGate(NaiveGate):
    r"""Top-1 over an fp32 softmax (multiplicative-free jitter of
    +-`switch_eps` added to the logits in training), capacity
    `ceil(rate * tokens / experts)` per expert, and the Switch balance loss."""

    def __init__(self, d_model, num_expert, world_size, topk=1, switch_eps=.1,
                 capacity=(1.2, 2.4), gate_bias=True):
        assert topk == 1, "topk should be 1 in switch"
        super().__init__(d_model, num_expert, world_size, top_k=1, gate_bias=gate_bias)
        self.switch_eps = switch_eps
        self.capacity = capacity

    def forward(self, inp):
        score = self.gate(inp)
        if self.training:
            noise = torch.rand_like(score)
            score = score + (noise * 2 * self.switch_eps + 1.0 - self.switch_eps)
        score = F.softmax(score.float(), dim=-1)
        top1_score, top1_idx = torch.topk(score, k=1, dim=-1, largest=True)
        top1_score = top1_score.to(dtype=inp.dtype)

        rate = self.capacity[0 if self.training else 1]
        cap = math.ceil(rate * inp.shape[0] / self.num_expert)
        _lec, _gec, top1_idx = limit_by_capacity(top1_idx, self.num_expert,
                                                 self.world_size, cap)

        # per-expert counts of the slots that survived, and their total, stay on
        # the device (fmoe/gates/switch_gate.py:49-57 indexes with a mask, which
        # reads the number of survivors back to the host)
        count = _histogram(top1_idx, self.tot_expert).to(torch.float)
        n_kept = count.sum()
        frac = count / n_kept
        prob = score.sum(dim=0) / n_kept
        self.set_loss((frac * prob).sum() * self.tot_expert)
        return top1_idx, top1_score
