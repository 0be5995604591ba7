r"""Capacity helper shared by the balanced gates (fmoe/gates/utils.py:9-26)."""
import torch

from .. import fmoe_cuda as fmoe_native
from ..functions import count_by_gate


def limit_by_capacity(topk_idx, num_expert, world_size, capacity):
    r"""Clips every expert to `capacity` slots; earlier slots win.  Returns
    `(new_local_count, new_global_count, topk_idx with -1 where dropped)`."""
    with torch.no_grad():
        cap = torch.full((num_expert,), int(capacity), dtype=torch.int32,
                         device=topk_idx.device)
        _pos, _lec, gec = count_by_gate(topk_idx, num_expert, world_size,
                                        require_pos=False)
        new_gec = fmoe_native.limit_by_capacity(gec, cap, num_expert, world_size)
        new_lec = new_gec  # one worker: nothing to exchange
        topk_idx = fmoe_native.prune_gate_by_capacity(
            topk_idx.contiguous(), new_lec.to(torch.int32), num_expert, world_size)
    return new_lec, new_gec, topk_idx
