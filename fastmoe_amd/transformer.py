r"""The MoE feed-forward block of a Transformer, mirroring fmoe/transformer.py."""
from __future__ import annotations

import torch
import torch.nn as nn
from torch.autograd import Function

from . import fmoe_cuda
from .functions import SegmentTable
from .layers import FMoE
from .linear import (FMoELinear, MOELinear, ParamTables, act_linear, is_exact_gelu,
                     linear_act_linear, linear_act_linear_list)


def _watched(*modules) -> bool:
    r"""Whether anybody has hooks on one of `modules` that only a call of the module
    itself (forward hooks) or its own autograd nodes (backward hooks) would run."""
    return any(m is not None and isinstance(m, nn.Module) and
               (m._forward_hooks or m._forward_pre_hooks or m._backward_hooks or
                getattr(m, "_backward_pre_hooks", None))
               for m in modules)


class FusedExpertLayer(Function):
    r"""The whole dispatch of a layer of GELU expert MLPs as ONE autograd node:
    route -> scatter -> linear + GELU -> linear -> gather fused with the top-k
    combine (fmoe/layers.py:26-78,281-295 around fmoe/transformer.py:25-33), and the
    mirror image backwards.  The same kernels, in the same order, as the chain of
    FusedScatter / MOELinearGelu / MOEGeluLinear / FusedGatherCombine nodes; what
    it saves is host time (one node instead of four, no intermediate Python
    objects), which is all a small layer costs."""

    @staticmethod
    def forward(ctx, inp, gate_idx, score, w1, b1, w2, b2):
        top_k = gate_idx.shape[-1] if gate_idx.dim() >= 2 else 1
        n_tokens = inp.shape[0]
        with torch.no_grad():
            pos, _counts, seg_off, inv = fmoe_cuda.route(gate_idx.contiguous(), w1.shape[0])
        x = inp.contiguous()
        if 4 <= top_k <= 64:
            buf = fmoe_cuda.scatter_tokens(x, inv, top_k)
        else:
            buf = fmoe_cuda.local_scatter(x, pos, top_k, seg_off[-1:])
        pre, act = fmoe_cuda.grouped_linear_fwd(buf, seg_off, w1, b1, with_gelu=True)
        out_buf = fmoe_cuda.grouped_linear_fwd(act, seg_off, w2, b2)
        ctx.score_like = (score.shape, score.dtype)
        score = score.reshape(n_tokens, top_k).contiguous().to(out_buf.dtype)
        ctx.top_k, ctx.n_tokens = top_k, n_tokens
        ctx.has_bias = (b1 is not None, b2 is not None)
        ctx.save_for_backward(buf, pre, act, out_buf, score, seg_off, inv, w1, w2)
        return fmoe_cuda.gather_combine_fwd(out_buf, inv, score, n_tokens, top_k)

    @staticmethod
    def backward(ctx, grad_y):
        buf, pre, act, out_buf, score, seg_off, inv, w1, w2 = ctx.saved_tensors
        need = ctx.needs_input_grad
        d_out, dscore = fmoe_cuda.gather_combine_bwd(grad_y.contiguous(), out_buf, inv, score,
                                                     ctx.n_tokens, ctx.top_k)
        dpre, dw2, db2 = fmoe_cuda.grouped_linear_bwd(
            d_out, act, seg_off, w2, need_bias=need[6] and ctx.has_bias[1], need_dx=True,
            need_dw=need[5], act_pre=pre)
        dbuf, dw1, db1 = fmoe_cuda.grouped_linear_bwd(
            dpre, buf, seg_off, w1, need_bias=need[4] and ctx.has_bias[0], need_dx=need[0],
            need_dw=need[3])
        dx = fmoe_cuda.scatter_reduce(dbuf, inv, ctx.n_tokens, ctx.top_k) if need[0] else None
        dscore = dscore.reshape(ctx.score_like[0]).to(ctx.score_like[1]) if need[2] else None
        return dx, None, dscore, dw1, db1, dw2, db2


class _LinearView:
    r"""One expert of an FMoELinear as the reference's `experts[i].htoh4` would
    look: `weight` [1, out, in] and `bias` [1, out] are views of the fused
    parameters (gradients flow into them)."""

    def __init__(self, linear: FMoELinear, i: int):
        self.weight = linear.weight[i:i + 1]
        self.bias = None if linear.bias is None else linear.bias[i:i + 1]

    def __call__(self, inp, fwd_expert_count):
        return MOELinear.apply(inp.type_as(self.weight), fwd_expert_count, self.weight, self.bias)


class _ExpertView:
    r"""`experts[i]` of a fused `_Expert`: callable like the `_Expert(1, ...)` the
    reference keeps per expert (fmoe/transformer.py:51-55), backed by views."""

    def __init__(self, parent: "_Expert", i: int):
        self.htoh4 = _LinearView(parent.htoh4, i)
        self.h4toh = _LinearView(parent.h4toh, i)
        self.activation = parent.activation

    def __call__(self, inp, fwd_expert_count):
        return self.h4toh(self.activation(self.htoh4(inp, fwd_expert_count)), fwd_expert_count)

    def parameters(self):
        for lin in (self.htoh4, self.h4toh):
            yield lin.weight
            if lin.bias is not None:
                yield lin.bias


class _Expert(nn.Module):
    r"""`num_expert` two-layer MLPs held as two FMoELinear modules
    (fmoe/transformer.py:11-31).  Accepts host counts or a device-side
    SegmentTable as `fwd_expert_count`.  Indexing and iterating give per-expert
    views, so code written against the reference's list of single-expert modules
    (`layer.experts[i].htoh4.weight`) keeps working on the fused module."""

    accepts_segment_table = True

    def __init__(self, num_expert, d_model, d_hidden, activation, rank=0):
        super().__init__()
        self.htoh4 = FMoELinear(num_expert, d_model, d_hidden, bias=True, rank=rank)
        self.h4toh = FMoELinear(num_expert, d_hidden, d_model, bias=True, rank=rank)
        self.activation = activation

    def forward(self, inp, fwd_expert_count):
        if _watched(self.htoh4, self.h4toh, self.activation):
            # somebody watches the linear modules or the activation: call them as
            # modules, the way the reference does (fmoe/transformer.py:25-33)
            x = self.htoh4(inp, fwd_expert_count)
            if _watched(self.h4toh, self.activation):
                return self.h4toh(self.activation(x), fwd_expert_count)
            return act_linear(self.activation, x, fwd_expert_count, self.h4toh.weight,
                              self.h4toh.bias)
        # the activation is written by the first layer's output tiles, and its
        # backward runs inside the second layer's backward kernel
        return linear_act_linear(self.activation, inp, fwd_expert_count, self.htoh4.weight,
                                 self.htoh4.bias, self.h4toh.weight, self.h4toh.bias)

    def can_run_layer(self, inp, top_k) -> bool:
        r"""Whether the whole layer (dispatch included) can run as one autograd node:
        one 2-d GPU tensor in the parameters' dtype, the exact GELU between the two
        layers, and nobody watching the modules inside."""
        w1, w2 = self.htoh4.weight, self.h4toh.weight
        return (torch.is_tensor(inp) and inp.dim() == 2 and inp.is_cuda
                and inp.dtype == w1.dtype == w2.dtype and 1 <= top_k <= 64
                and is_exact_gelu(self.activation, inp)
                and not _watched(self, self.htoh4, self.h4toh, self.activation))

    def run_layer(self, inp, gate_idx, score):
        r"""`sum_j score[t, j] * expert_{gate_idx[t, j]}(inp[t])` over the live slots,
        as one autograd node (FusedExpertLayer)."""
        return FusedExpertLayer.apply(inp, gate_idx, score, self.htoh4.weight, self.htoh4.bias,
                                      self.h4toh.weight, self.h4toh.bias)

    def __len__(self):
        return self.htoh4.num_expert

    def __getitem__(self, i):
        n = len(self)
        if not -n <= i < n:
            raise IndexError(f"expert {i} of {n}")
        return _ExpertView(self, i % n)

    def __iter__(self):
        return (_ExpertView(self, i) for i in range(len(self)))

    # -- a list of such modules run as one --------------------------------------
    @staticmethod
    def can_run_list(experts) -> bool:
        r"""Whether `experts` (the reference's layout: one `_Expert(1, ...)` per
        expert) can run as ONE grouped call per layer on per-expert weight pointers:
        single-expert modules of one shape, dtype and device, and nobody watching them
        (hooks on a list module run only when that module is called, which the
        reference-shaped route does)."""
        first = experts[0] if len(experts) else None
        if not isinstance(first, _Expert):
            return False
        w1, w2 = first.htoh4.weight, first.h4toh.weight
        for e in experts:
            if not (isinstance(e, _Expert) and e.activation is first.activation
                    and e.htoh4.num_expert == 1 and e.h4toh.num_expert == 1
                    and e.htoh4.weight.shape == w1.shape and e.h4toh.weight.shape == w2.shape
                    and (e.htoh4.bias is None) == (first.htoh4.bias is None)
                    and (e.h4toh.bias is None) == (first.h4toh.bias is None)
                    and e.htoh4.weight.dtype == w1.dtype and e.h4toh.weight.dtype == w1.dtype
                    and e.htoh4.weight.device == w1.device
                    and e.h4toh.weight.device == w1.device
                    and e.htoh4.weight.is_cuda
                    and not _watched(e, e.htoh4, e.h4toh)):
                return False
        return not _watched(first.activation)

    @staticmethod
    def run_list(experts, inp, segments: SegmentTable):
        r"""The modules of `experts` applied to their row segments in two grouped
        GEMMs that read every expert's weight where it lies (tables of per-expert
        pointers, kept on the list and rebuilt only when a parameter's storage moves):
        no weight is copied and no count is read to the host."""
        tables = getattr(experts, "_fmoe_param_tables", None)
        if tables is None:
            tables = ParamTables()
            try:
                object.__setattr__(experts, "_fmoe_param_tables", tables)
            except Exception:   # a plain list: no place to keep them
                pass
        first = experts[0]

        def col(get):
            parts = [get(e) for e in experts]
            return None if parts[0] is None else parts

        return linear_act_linear_list(
            first.activation, inp, segments,
            col(lambda e: e.htoh4.weight), col(lambda e: e.htoh4.bias),
            col(lambda e: e.h4toh.weight), col(lambda e: e.h4toh.bias), tables)


class FMoETransformerMLP(FMoE):
    r"""A complete MoE MLP block (fmoe/transformer.py:34-66).

    * `activation`: the non-linearity between the two expert layers.
    * `d_hidden`: width of the hidden layer.
    * `fused` (this build): True keeps all experts in one `_Expert` whose
      weights are `[E, out, in]` tensors and runs the device-side dispatch;
      False builds `num_expert` single-expert modules as the reference does
      (state-dict keys `experts.<i>.htoh4.weight`); they still run as one
      grouped call per layer without a host read, the kernels reading each
      expert's weight through a pointer table (no copy).  Checkpoints in either
      layout load into either.
    """

    def __init__(self, num_expert=32, d_model=1024, d_hidden=4096,
                 activation=torch.nn.GELU(), expert_dp_comm="none", expert_rank=0,
                 fused=True, **kwargs):
        self._fused_layout = fused
        if fused:
            super().__init__(num_expert=num_expert, d_model=d_model, expert=None,
                             **kwargs)
            self.experts = _Expert(num_expert, d_model, d_hidden, activation,
                                   rank=expert_rank)
        else:
            def one_expert(d_model):
                return _Expert(1, d_model, d_hidden, activation, rank=0)
            super().__init__(num_expert=num_expert, d_model=d_model,
                             expert=one_expert, **kwargs)
        self.mark_parallel_comm(expert_dp_comm)

    def forward(self, inp: torch.Tensor):
        original_shape = inp.shape
        inp = inp.reshape(-1, self.d_model)
        output = super().forward(inp)
        return output.reshape(original_shape)

    # -- checkpoints written in the other expert layout -----------------------
    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        names = ("htoh4.weight", "htoh4.bias", "h4toh.weight", "h4toh.bias")
        ex = prefix + "experts."
        if self._fused_layout and (ex + "0." + names[0]) in state_dict:
            for n in names:
                parts = [state_dict.pop(f"{ex}{i}.{n}") for i in range(self.num_expert)]
                state_dict[ex + n] = torch.cat(parts, dim=0)
        elif not self._fused_layout and (ex + names[0]) in state_dict:
            for n in names:
                whole = state_dict.pop(ex + n)
                for i in range(self.num_expert):
                    state_dict[f"{ex}{i}.{n}"] = whole[i:i + 1].clone()
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)
