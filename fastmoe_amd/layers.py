r"""The MoE layer, mirroring fmoe/layers.py of the reference at world_size 1.

`FMoE` keeps the reference's constructor and hooks.  When the experts are one
fused module taking `(rows, fwd_expert_count)` -- this package's `_Expert` -- or
a list of such modules (the reference's layout of FMoETransformerMLP), the whole
dispatch stays on the device: route -> scatter -> grouped GEMMs -> gather fused
with the top-k combine, with no device-to-host copy.  Lists of arbitrary expert
modules take the reference's route, with ONE host read of the counts.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import _tree as tree
from .functions import (FusedGatherCombine, FusedScatter, MOEGather, MOEScatter,
                        RoutePlan, prepare_forward)
from .gates import NaiveGate


def mark_module_parallel_comm(module, comm):
    r"""Tags every parameter of `module` with the data-parallel group name
    (`'world'`, `'dp'`, `'none'`, `'gate'`); fmoe/layers.py:17-23."""
    for p in module.parameters():
        setattr(p, "dp_comm", comm)


def _fmoe_general_global_forward(inp, gate, expert_fn, num_expert, world_size,
                                 **kwargs):
    r"""Reference-shaped dispatch (fmoe/layers.py:26-78): count, scatter rows to
    expert order, run `expert_fn(rows, fwd_expert_count)`, gather the rows back
    to `[tokens * top_k, d]`.  Counts are handed to `expert_fn` on the host."""
    (pos, local_expert_count, global_expert_count, fwd_expert_count,
     fwd_batch_size) = prepare_forward(gate, num_expert, world_size)
    topk = gate.shape[1] if gate.dim() == 2 else 1
    tok = torch.div(pos, topk, rounding_mode="floor")

    x = tree.map_structure(
        lambda t: MOEScatter.apply(t, tok, local_expert_count, global_expert_count,
                                   fwd_batch_size, world_size), inp)
    x = expert_fn(x, fwd_expert_count)
    out_batch_size = tree.flatten(inp)[0].shape[0] * topk
    return tree.map_structure(
        lambda t: MOEGather.apply(t, pos, local_expert_count, global_expert_count,
                                  out_batch_size, world_size), x)


class FMoE(nn.Module):
    r"""A general MoE layer with an arbitrary module as the expert
    (fmoe/layers.py:87-312).

    * `num_expert`: experts on this worker; `world_size` must be 1 here.
    * `top_k`: experts per token.
    * `gate`: a gate class from `fastmoe_amd.gates`.
    * `expert`: a module class (called with `d_model`) or a list of them; when
      None the subclass assigns one fused module to `self.experts`.
    * `gate_hook(idx, score, None)`, `mask`, `mask_dict`, `gate_bias`,
      `slice_group` / `mp_group`, `moe_group`: as in the reference; the group
      arguments must stay None on one GPU.
    """

    def __init__(self, num_expert=32, d_model=1024, world_size=1, mp_group=None,
                 slice_group=None, moe_group=None, top_k=2, gate=NaiveGate,
                 expert=None, gate_hook=None, mask=None, mask_dict=None,
                 gate_bias=True):
        super().__init__()
        if world_size != 1 or mp_group is not None or slice_group is not None:
            raise NotImplementedError(
                "single-GPU build: world_size must be 1 and no slice/mp group")
        self.num_expert = num_expert
        self.d_model = d_model
        self.world_size = world_size
        self.slice_group = None
        self.slice_size = 1
        self.slice_rank = 0
        self.top_k = top_k
        if type(expert) is list:
            self.experts = nn.ModuleList([e(d_model) for e in expert])
            self.experts_fused = False
            self.num_expert = num_expert = len(expert)
        elif expert is not None:
            self.experts = nn.ModuleList([expert(d_model) for _ in range(num_expert)])
            self.experts_fused = False
        else:
            self.experts_fused = True
        if issubclass(gate, NaiveGate):
            self.gate = gate(d_model, num_expert, world_size, top_k, gate_bias=gate_bias)
        else:
            self.gate = gate(d_model, num_expert, world_size, top_k)
        self.gate_hook = gate_hook
        self.mask = mask
        self.mask_dict = mask_dict
        self.moe_group = moe_group

    # ------------------------------------------------------------- experts
    def expert_fn(self, inp, fwd_expert_count):
        r"""Runs the experts on expert-ordered rows: the fused module in one
        call, or each module of the list on its slice (fmoe/layers.py:164-180).
        Arbitrary modules need real slices, hence host counts: the caller
        (prepare_forward) has read them once."""
        if self.experts_fused:
            return self.experts(inp, fwd_expert_count)
        counts = fwd_expert_count
        if isinstance(counts, torch.Tensor):
            counts = counts.cpu().tolist()
        outputs, base = [], 0
        for i in range(self.num_expert):
            n = int(counts[i])
            outputs.append(self.experts[i](inp[base:base + n], torch.tensor([n])))
            base += n
        return torch.cat(outputs, dim=0)

    def expert_fn_single(self, inp, fwd_expert_count, idx):
        r"""One expert of a non-fused list (fmoe/layers.py:182-188)."""
        assert not self.experts_fused, "should not use fused experts"
        return self.experts[idx](inp, fwd_expert_count)

    def mark_parallel_comm(self, expert_dp_comm="none"):
        r"""Tags expert parameters with `expert_dp_comm` and the gate's with
        `'gate'` (fmoe/layers.py:190-203)."""
        if self.experts is not None:
            if isinstance(self.experts, list):
                for e in self.experts:
                    mark_module_parallel_comm(e, expert_dp_comm)
            else:
                mark_module_parallel_comm(self.experts, expert_dp_comm)
        mark_module_parallel_comm(self.gate, "gate")

    def _device_side_dispatch(self) -> bool:
        # the fused combine kernels keep a token's slots in the lanes of one wave
        if self.top_k > 64:
            return False
        if self.experts_fused:
            return getattr(self.experts, "accepts_segment_table", False)
        # a list of modules whose class knows how to run the whole list from a
        # device-side segment table (this package's _Expert does)
        can = getattr(type(self.experts[0]), "can_run_list", None) if len(self.experts) else None
        return can is not None and can(self.experts)

    def _run_experts(self, x, segments):
        if self.experts_fused:
            return self.experts(x, segments)
        return type(self.experts[0]).run_list(self.experts, x, segments)

    # ------------------------------------------------------------- forward
    def forward(self, moe_inp):
        r"""Gate, dispatch, experts, and the score-weighted sum of each token's
        top-k expert outputs (fmoe/layers.py:205-312)."""
        sizes = tree.flatten(tree.map_structure(lambda t: t.shape[0], moe_inp))
        assert all(s == sizes[0] for s in sizes), \
            "MoE inputs must have the same batch size"

        gate_top_k_idx, gate_score = self.gate(moe_inp)
        if self.gate_hook is not None:
            self.gate_hook(gate_top_k_idx, gate_score, None)

        masked = self.mask is not None and self.mask_dict is not None
        if self._device_side_dispatch():
            # no host copy anywhere: counts stay in the RoutePlan
            score = gate_score.reshape(-1, self.top_k)
            if masked:
                # masked tokens (fmoe/layers.py:240-251 deletes their rows, which
                # needs their number on the host) keep their place and lose their
                # slots instead: a slot of -1 is dropped by the routing kernels
                mask = self.mask.view(-1).to(gate_top_k_idx.device)
                gate_top_k_idx = torch.where((mask == 0).view(-1, 1),
                                             gate_top_k_idx.view(-1, self.top_k), -1)
            whole = getattr(self.experts, "can_run_layer", None) if self.experts_fused else None
            if whole is not None and whole(moe_inp, self.top_k):
                # dispatch, experts and combine as one autograd node (least host time)
                out = self.experts.run_layer(moe_inp, gate_top_k_idx, score)
            else:
                plan = RoutePlan(gate_top_k_idx, self.num_expert)
                x = tree.map_structure(lambda t: FusedScatter.apply(t, plan), moe_inp)
                x = tree.map_structure(lambda t: self._run_experts(t, plan.segments), x) \
                    if not self.experts_fused else self.experts(x, plan.segments)
                out = tree.map_structure(
                    lambda t: FusedGatherCombine.apply(t, score, plan), x)
            if masked:
                # a masked token's k slots all hold mask_dict[mask value] (zero if the
                # value has no entry), fmoe/layers.py:262-286: their score-weighted sum
                # is (sum of the token's scores) x that row
                total = score.sum(dim=-1, keepdim=True)

                def fill(t):
                    for k, v in self.mask_dict.items():
                        row = (total * v.to(total.dtype).view(1, -1)).to(t.dtype)
                        t = torch.where((mask == k).view(-1, 1), row, t)
                    return t
                out = tree.map_structure(fill, out)
            return out

        if masked:
            mask = self.mask.view(-1)
            keep = mask == 0
            moe_inp = tree.map_structure(lambda t: t[keep, :], moe_inp)
            gate_top_k_idx = gate_top_k_idx[keep, :]

        fwd = _fmoe_general_global_forward(
            moe_inp, gate_top_k_idx, self.expert_fn, self.num_expert,
            self.world_size, experts=self.experts)

        if masked:
            def recover(t):
                dim = t.shape[-1]
                t = t.view(-1, self.top_k, dim)
                full = torch.zeros(mask.shape[0], self.top_k, dim,
                                   device=t.device, dtype=t.dtype)
                full[keep] = t
                for k, v in self.mask_dict.items():
                    full[mask == k] = v
                return full
            moe_outp = tree.map_structure(recover, fwd)
        else:
            moe_outp = tree.map_structure(
                lambda t: t.view(-1, self.top_k, t.shape[-1]), fwd)

        gate_score = gate_score.view(-1, 1, self.top_k)
        moe_outp = tree.map_structure(
            lambda t: torch.bmm(gate_score.to(t.dtype), t).reshape(-1, t.shape[-1]),
            moe_outp)
        sizes = tree.flatten(tree.map_structure(lambda t: t.shape[0], moe_outp))
        assert all(s == sizes[0] for s in sizes), \
            "MoE outputs must have the same batch size"
        return moe_outp
