r"""The MoE feed-forward block of a Transformer, mirroring fmoe/transformer.py."""
from __future__ import annotations

import torch
import torch.nn as nn

from .functions import SegmentTable, apply_activation
from .layers import FMoE
from .linear import FMoELinear


class _Expert(nn.Module):
    r"""`num_expert` two-layer MLPs held as two FMoELinear modules
    (fmoe/transformer.py:11-31).  Accepts host counts or a device-side
    SegmentTable as `fwd_expert_count`."""

    accepts_segment_table = True

    def __init__(self, num_expert, d_model, d_hidden, activation, rank=0):
        super().__init__()
        self.htoh4 = FMoELinear(num_expert, d_model, d_hidden, bias=True, rank=rank)
        self.h4toh = FMoELinear(num_expert, d_hidden, d_model, bias=True, rank=rank)
        self.activation = activation

    def forward(self, inp, fwd_expert_count):
        x = self.htoh4(inp, fwd_expert_count)
        # with a device-side segment table, the activation skips the dead rows
        live = fwd_expert_count.seg_off[-1:] if isinstance(fwd_expert_count, SegmentTable) else None
        x = apply_activation(self.activation, x, live)
        return self.h4toh(x, fwd_expert_count)


class FMoETransformerMLP(FMoE):
    r"""A complete MoE MLP block (fmoe/transformer.py:34-66).

    * `activation`: the non-linearity between the two expert layers.
    * `d_hidden`: width of the hidden layer.
    * `fused` (this build): True keeps all experts in one `_Expert` whose
      weights are `[E, out, in]` tensors and runs the device-side dispatch;
      False builds `num_expert` single-expert modules as the reference does
      (state-dict keys `experts.<i>.htoh4.weight`), which costs a host copy of
      the counts and a Python loop per forward.  Checkpoints in either layout
      load into either.
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
