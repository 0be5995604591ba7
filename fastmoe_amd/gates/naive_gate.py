r"""Top-k of a linear layer (fmoe/gates/naive_gate.py)."""
import torch
import torch.nn as nn

from ..functions import topk_softmax
from .base_gate import BaseGate


class NaiveGate(BaseGate):
    r"""logits = Linear(d_model, experts); the k largest logits pick the experts
    and their softmax gives the combine weights.  Returns `(idx [..., k] int64,
    score [T, k])`, plus the full logits when `return_all_scores`."""

    def __init__(self, d_model, num_expert, world_size, top_k=2, gate_bias=True):
        super().__init__(num_expert, world_size)
        self.gate = nn.Linear(d_model, self.tot_expert, bias=gate_bias)
        self.top_k = top_k

    def forward(self, inp, return_all_scores=False):
        logits = self.gate(inp)
        top_idx, score = topk_softmax(logits, self.top_k)
        # idx keeps the leading dimensions of the input, score is [tokens, k]
        # (naive_gate.py:31-38: topk over dim -1, then view(-1, top_k) of the values)
        top_idx = top_idx.view(*logits.shape[:-1], self.top_k)
        # a zero loss so training loops can always call get_loss(); created on the
        # device (no host-to-device copy, so the forward can sit in a HIP graph)
        self.set_loss(torch.zeros(1, device=inp.device, requires_grad=True))
        if return_all_scores:
            return top_idx, score, logits
        return top_idx, score
