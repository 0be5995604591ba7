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


__all__ = ["FMoE", "FMoELinear", "FMoETransformerMLP", "BaseGate", "NaiveGate",
           "GShardGate", "SwitchGate", "fmoe_cuda", "install_as_fmoe_cuda"]
