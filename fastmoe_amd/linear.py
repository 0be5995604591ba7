r"""The expert-parallel linear layer, mirroring fmoe/linear.py of the reference."""
from __future__ import annotations

import math

import torch
import torch.nn as nn
from torch.autograd import Function

from . import fmoe_cuda
from .functions import SegmentTable, apply_activation


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


class MOELinearGelu(Function):
    r"""A grouped linear layer that returns its output twice: as it is (the
    pre-activations, the differentiable result) and through the exact GELU, written by
    the same output tiles where the library can (bf16 on the matrix cores).  The
    second result carries no gradient of its own: it is meant for MOEGeluLinear,
    whose backward returns the gradient with respect to the pre-activations."""

    @staticmethod
    def forward(ctx, global_input_buf, fwd_expert_count, weight, bias=None):
        x = global_input_buf.contiguous()
        seg_off = _segments(fwd_expert_count, x.device)
        pre, act = fmoe_cuda.grouped_linear_fwd(
            x, seg_off, weight.contiguous(), None if bias is None else bias.contiguous(),
            with_gelu=True)
        ctx.save_for_backward(x, seg_off, weight, bias)
        ctx.mark_non_differentiable(act)
        # (or autograd would fill a zero tensor of act's size for it at every backward)
        ctx.set_materialize_grads(False)
        return pre, act

    @staticmethod
    def backward(ctx, grad_pre, _grad_act):
        if grad_pre is None:
            return None, None, None, None
        (x, seg_off, weight, bias) = ctx.saved_tensors
        need_dx, _, need_dw, need_db = ctx.needs_input_grad
        need_db = need_db and torch.is_tensor(bias)
        dx, dw, db = fmoe_cuda.grouped_linear_bwd(
            grad_pre.contiguous(), x, seg_off, weight.contiguous(),
            need_bias=need_db, need_dx=need_dx, need_dw=need_dw)
        return dx, None, dw, db


class MOEGeluLinear(Function):
    r"""`linear(gelu(pre))` as one autograd node: the activation between the two
    expert layers and the second layer (fmoe/transformer.py:28-31 for
    torch.nn.GELU()).  Forward runs the activation kernel and the grouped GEMM;
    backward hands the saved pre-activations to the grouped backward, which
    applies gelu' to dX inside the GEMM epilogue (bf16) instead of writing
    dY W to memory for a separate activation kernel to read back."""

    @staticmethod
    def forward(ctx, pre, fwd_expert_count, weight, bias=None, act=None):
        pre = pre.contiguous()
        seg_off = _segments(fwd_expert_count, pre.device)
        if act is None:   # (MOELinearGelu hands over gelu(pre) with the pre-activations)
            act = fmoe_cuda.gelu_fwd(pre, seg_off[-1:])  # rows past the last segment are dead
        out = fmoe_cuda.grouped_linear_fwd(act, seg_off, weight.contiguous(),
                                           None if bias is None else bias.contiguous())
        ctx.save_for_backward(pre, act, seg_off, weight, bias)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        (pre, act, seg_off, weight, bias) = ctx.saved_tensors
        need_dx, _, need_dw, need_db = ctx.needs_input_grad[:4]
        need_db = need_db and torch.is_tensor(bias)
        dpre, dw, db = fmoe_cuda.grouped_linear_bwd(
            grad_out.contiguous(), act, seg_off, weight.contiguous(),
            need_bias=need_db, need_dx=need_dx, need_dw=need_dw, act_pre=pre)
        return dpre, None, dw, db, None


# --------------------------------------------------------------------------
# The same three nodes for experts kept as SEPARATE single-expert modules, the
# reference's layout (fmoe/transformer.py:51-55).  The kernels read every expert's
# weight through a table of pointers (cuda/parallel_linear.cuh:69-87 addresses the
# experts the same way), so no weight is copied; the weight and bias gradients of all
# experts are written into one array each and handed to autograd as per-expert views.
# --------------------------------------------------------------------------
class ParamTables:
    r"""Device pointer tables of per-expert parameter lists, rebuilt only when a
    parameter's storage has moved (optimizers update in place, so normally never)."""

    def __init__(self):
        self._key = {}
        self._table = {}

    def get(self, name: str, tensors):
        if tensors is None:
            return None
        key = tuple(t.data_ptr() for t in tensors)
        if self._key.get(name) != key:
            self._table[name] = fmoe_cuda.pointer_table([t.detach() for t in tensors])
            self._key[name] = key
        return self._table[name]


def _split_params(params, n_expert, has_bias):
    weights = params[:n_expert]
    biases = params[n_expert:2 * n_expert] if has_bias else None
    return weights, biases


def _list_grads(ctx, dw, db, n_expert, has_bias):
    r"""Per-expert views of the [E, ...] gradient arrays, in the order of the inputs."""
    need = ctx.needs_input_grad[ctx.n_fixed:]
    grads = [dw[i:i + 1] if dw is not None and need[i] else None for i in range(n_expert)]
    if has_bias:
        grads += [db[i:i + 1] if db is not None and need[n_expert + i] else None
                  for i in range(n_expert)]
    return grads


class MOELinearList(Function):
    r"""MOELinear over `n_expert` weights [1, out, in] (then `n_expert` biases [1, out]
    when `has_bias`) passed one by one behind the fixed arguments."""

    n_fixed = 6

    @staticmethod
    def forward(ctx, global_input_buf, fwd_expert_count, w_table, b_table, n_expert, has_bias,
                *params):
        x = global_input_buf.contiguous()
        seg_off = _segments(fwd_expert_count, x.device)
        out = fmoe_cuda.grouped_linear_fwd_ptrs(x, seg_off, w_table, b_table,
                                                params[0].shape[1])
        ctx.n_expert, ctx.has_bias, ctx.n_fixed = n_expert, has_bias, MOELinearList.n_fixed
        ctx.save_for_backward(x, seg_off, w_table, *params[:n_expert])
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, seg_off, w_table = ctx.saved_tensors[:3]
        need = ctx.needs_input_grad
        need_dw = any(need[ctx.n_fixed:ctx.n_fixed + ctx.n_expert])
        need_db = ctx.has_bias and any(need[ctx.n_fixed + ctx.n_expert:])
        dx, dw, db = fmoe_cuda.grouped_linear_bwd_ptrs(
            grad_out.contiguous(), x, seg_off, w_table, need_bias=need_db, need_dx=need[0],
            need_dw=need_dw)
        return (dx, None, None, None, None, None,
                *_list_grads(ctx, dw, db, ctx.n_expert, ctx.has_bias))


class MOELinearGeluList(Function):
    r"""MOELinearGelu over per-expert parameters (see MOELinearList)."""

    n_fixed = 6

    @staticmethod
    def forward(ctx, global_input_buf, fwd_expert_count, w_table, b_table, n_expert, has_bias,
                *params):
        x = global_input_buf.contiguous()
        seg_off = _segments(fwd_expert_count, x.device)
        pre, act = fmoe_cuda.grouped_linear_fwd_ptrs(x, seg_off, w_table, b_table,
                                                     params[0].shape[1], with_gelu=True)
        ctx.n_expert, ctx.has_bias, ctx.n_fixed = n_expert, has_bias, MOELinearGeluList.n_fixed
        ctx.save_for_backward(x, seg_off, w_table, *params[:n_expert])
        ctx.mark_non_differentiable(act)
        ctx.set_materialize_grads(False)
        return pre, act

    @staticmethod
    def backward(ctx, grad_pre, _grad_act):
        n_in = ctx.n_fixed + ctx.n_expert * (2 if ctx.has_bias else 1)
        if grad_pre is None:
            return (None,) * n_in
        x, seg_off, w_table = ctx.saved_tensors[:3]
        need = ctx.needs_input_grad
        need_dw = any(need[ctx.n_fixed:ctx.n_fixed + ctx.n_expert])
        need_db = ctx.has_bias and any(need[ctx.n_fixed + ctx.n_expert:])
        dx, dw, db = fmoe_cuda.grouped_linear_bwd_ptrs(
            grad_pre.contiguous(), x, seg_off, w_table, need_bias=need_db, need_dx=need[0],
            need_dw=need_dw)
        return (dx, None, None, None, None, None,
                *_list_grads(ctx, dw, db, ctx.n_expert, ctx.has_bias))


class MOEGeluLinearList(Function):
    r"""MOEGeluLinear over per-expert parameters (see MOELinearList); `act` is
    gelu(pre) from MOELinearGeluList, or None."""

    n_fixed = 7

    @staticmethod
    def forward(ctx, pre, fwd_expert_count, w_table, b_table, n_expert, has_bias, act, *params):
        pre = pre.contiguous()
        seg_off = _segments(fwd_expert_count, pre.device)
        if act is None:
            act = fmoe_cuda.gelu_fwd(pre, seg_off[-1:])
        out = fmoe_cuda.grouped_linear_fwd_ptrs(act, seg_off, w_table, b_table,
                                                params[0].shape[1])
        ctx.n_expert, ctx.has_bias, ctx.n_fixed = n_expert, has_bias, MOEGeluLinearList.n_fixed
        ctx.save_for_backward(pre, act, seg_off, w_table, *params[:n_expert])
        return out

    @staticmethod
    def backward(ctx, grad_out):
        pre, act, seg_off, w_table = ctx.saved_tensors[:4]
        need = ctx.needs_input_grad
        need_dw = any(need[ctx.n_fixed:ctx.n_fixed + ctx.n_expert])
        need_db = ctx.has_bias and any(need[ctx.n_fixed + ctx.n_expert:])
        dpre, dw, db = fmoe_cuda.grouped_linear_bwd_ptrs(
            grad_out.contiguous(), act, seg_off, w_table, need_bias=need_db, need_dx=need[0],
            need_dw=need_dw, act_pre=pre)
        return (dpre, None, None, None, None, None, None,
                *_list_grads(ctx, dw, db, ctx.n_expert, ctx.has_bias))


def linear_act_linear_list(activation, inp, fwd_expert_count, weights1, biases1, weights2,
                           biases2, tables: ParamTables):
    r"""`linear_act_linear` for experts kept as separate modules: `weights1[e]` is
    [1, hidden, in], `biases1[e]` [1, hidden] (or `biases1` None), likewise the second
    layer.  Nothing is concatenated."""
    n = len(weights1)
    x = inp.type_as(weights1[0])
    t_w1, t_b1 = tables.get("w1", weights1), tables.get("b1", biases1)
    t_w2, t_b2 = tables.get("w2", weights2), tables.get("b2", biases2)
    p1 = (*weights1, *(biases1 or ()))
    p2 = (*weights2, *(biases2 or ()))
    if is_exact_gelu(activation, x) and weights1[0].dtype == weights2[0].dtype:
        pre, act = MOELinearGeluList.apply(x, fwd_expert_count, t_w1, t_b1, n,
                                           biases1 is not None, *p1)
        return MOEGeluLinearList.apply(pre, fwd_expert_count, t_w2, t_b2, n,
                                       biases2 is not None, act, *p2)
    pre = MOELinearList.apply(x, fwd_expert_count, t_w1, t_b1, n, biases1 is not None, *p1)
    if is_exact_gelu(activation, pre) and pre.dtype == weights2[0].dtype:
        return MOEGeluLinearList.apply(pre, fwd_expert_count, t_w2, t_b2, n,
                                       biases2 is not None, None, *p2)
    live = fwd_expert_count.seg_off[-1:] if isinstance(fwd_expert_count, SegmentTable) else None
    h = apply_activation(activation, pre, live)
    return MOELinearList.apply(h.type_as(weights2[0]), fwd_expert_count, t_w2, t_b2, n,
                               biases2 is not None, *p2)


def is_exact_gelu(activation, x: torch.Tensor) -> bool:
    r"""Whether `activation(x)` is the erf GELU the library has kernels for."""
    return (type(activation) is torch.nn.GELU
            and getattr(activation, "approximate", "none") == "none" and x.is_cuda
            and x.dtype in (torch.float32, torch.float64, torch.float16, torch.bfloat16))


def act_linear(activation, pre, fwd_expert_count, weight, bias):
    r"""`linear(activation(pre))` over the experts' row segments."""
    if is_exact_gelu(activation, pre) and pre.dtype == weight.dtype:
        return MOEGeluLinear.apply(pre, fwd_expert_count, weight, bias)
    live = fwd_expert_count.seg_off[-1:] if isinstance(fwd_expert_count, SegmentTable) else None
    x = apply_activation(activation, pre, live)
    return MOELinear.apply(x.type_as(weight), fwd_expert_count, weight, bias)


def linear_act_linear(activation, inp, fwd_expert_count, weight1, bias1, weight2, bias2):
    r"""The reference's expert, `h4toh(activation(htoh4(inp)))` (fmoe/transformer.py:
    25-33), over the experts' row segments.  With torch.nn.GELU() the activation is
    written by the first layer's output tiles and differentiated inside the second
    layer's backward tiles."""
    x = inp.type_as(weight1)
    if is_exact_gelu(activation, x) and weight1.dtype == weight2.dtype:
        pre, act = MOELinearGelu.apply(x, fwd_expert_count, weight1, bias1)
        return MOEGeluLinear.apply(pre, fwd_expert_count, weight2, bias2, act)
    pre = MOELinear.apply(x, fwd_expert_count, weight1, bias1)
    return act_linear(activation, pre, fwd_expert_count, weight2, bias2)


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
