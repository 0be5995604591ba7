r"""The expert-parallel linear layer, mirroring fmoe/linear.py of the reference."""
from __future__ import annotations

import math

import torch
import torch.nn as nn
from torch.autograd import Function

from . import fmoe_cuda
from .functions import SegmentTable


def _segments(fwd_expert_count, device) -> torch.Tensor:
    if isinstance(fwd_expert_count, SegmentTable):
        return fwd_expert_count.seg_off
    return fmoe_cuda._seg_off_from_counts(fwd_expert_count, device)


class MOELinear(Function):
    r"""All experts' linear maps in one grouped GEMM; fmoe/linear.py:12-36.

    `fwd_expert_count` is the reference's host int64 tensor or a SegmentTable
    (device-side, no host round trip)."""

    @staticmethod
    def forward(ctx, global_input_buf, fwd_expert_count, weight, bias=None):
        x = global_input_buf.contiguous()
        seg_off = _segments(fwd_expert_count, x.device)
        out = fmoe_cuda.grouped_linear_fwd(x, seg_off, weight.contiguous(),
                                           None if bias is None else bias.contiguous())
        ctx.save_for_backward(x, seg_off, weight, bias)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        (x, seg_off, weight, bias) = ctx.saved_tensors
        need_dx, _, need_dw, need_db = ctx.needs_input_grad
        need_db = need_db and torch.is_tensor(bias)
        dx, dw, db = fmoe_cuda.grouped_linear_bwd(
            grad_out.contiguous(), x, seg_off, weight.contiguous(),
            need_bias=need_db, need_dx=need_dx, need_dw=need_dw)
        return dx, None, dw, db


class FMoELinear(nn.Module):
    r"""`num_expert` linear layers held as weight [E, out, in] and bias
    [E, out]; fmoe/linear.py:40-91."""

    def __init__(self, num_expert: int, in_feat: int, out_feat: int,
                 bias: bool = True, rank: int = 0):
        super().__init__()
        self.num_expert = num_expert
        self.in_feat = in_feat
        self.out_feat = out_feat
        self.rank = rank
        self.weight = nn.Parameter(torch.Tensor(num_expert, out_feat, in_feat))
        if bias:
            self.bias = nn.Parameter(torch.zeros(num_expert, out_feat))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()

    def forward(self, inp, fwd_expert_count):
        return MOELinear.apply(inp.type_as(self.weight), fwd_expert_count,
                               self.weight, self.bias)

    def extra_repr(self) -> str:
        return "num_expert={}, in_features={}, out_features={}, bias={}, rank={}".format(
            self.num_expert, self.in_feat, self.out_feat,
            self.bias is not None, self.rank)

    def reset_parameters(self):
        # same as torch.nn.Linear; the bias stays zero (fmoe/linear.py:86-91)
        torch.nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))
