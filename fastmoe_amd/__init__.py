r"""fastmoe_amd: the single-GPU MoE-layer hot path of FastMoE, native to MI355X.

`FMoE`, `FMoELinear`, `FMoETransformerMLP` and the gates keep the reference's
interface; `fmoe_cuda` is the operator module that stands in for the
reference's compiled extension of the same name.
"""
from . import fmoe_cuda
from .gates import BaseGate, GShardGate, NaiveGate, SwitchGate
from .layers import FMoE
from .linear import FMoELinear
from .transformer import FMoETransformerMLP


def install_as_fmoe_cuda(compiled: bool = True) -> None:
    """Registers an operator module as `fmoe_cuda`, so that the reference's
    own Python package (`import fmoe_cuda` in fmoe/functions.py:9) binds to the
    MI355X kernels: the pybind11 extension of that name (cuda/fmoe_cuda.cpp:104-125
    rebuilt on the C ABI), or with `compiled=False` the ctypes module."""
    import sys

    if compiled:
        from . import _ext

        sys.modules["fmoe_cuda"] = _ext.load()
    else:
        sys.modules["fmoe_cuda"] = fmoe_cuda.ctypes_ops


def graphed(layer, sample_input, num_warmup_iters: int = 3):
    """The layer with its forward and its backward captured in one HIP graph each
    (`torch.cuda.make_graphed_callables`): for workloads so small that a step is the
    host's time to enqueue it (512 tokens, 128 -> 256, 4 experts: 0.30 ms eager, 0.17 ms
    replayed).  The device-side dispatch reads nothing back to the host, so the capture
    is legal and a replay routes new data anew; results are the eager layer's bits.
    `sample_input` fixes shape, dtype and device of every later call and has to require
    a gradient if the inputs will.  The library's one-time set-up is made before the
    capture."""
    import torch

    fmoe_cuda.init(sample_input.device)
    return torch.cuda.make_graphed_callables(layer, (sample_input,),
                                             num_warmup_iters=num_warmup_iters)


__all__ = ["FMoE", "FMoELinear", "FMoETransformerMLP", "BaseGate", "NaiveGate",
           "GShardGate", "SwitchGate", "fmoe_cuda", "install_as_fmoe_cuda", "graphed"]
