"""Drop-in for the reference's compiled ``fmoe_cuda`` extension on MI355X.

Same function names, argument order, side effects and error type
(``RuntimeError``) as the pybind11 module in cuda/fmoe_cuda.cpp:104-125 of the
reference.  Beyond that surface it exposes the native dispatch ops
(``local_scatter``, ``local_gather``) and the synchronisation-free fused ops used
by this package's own layer (``route``, ``grouped_linear_*``, ``gather_combine_*``,
``scatter_reduce``), all on torch's current HIP stream.

Two bindings of the same C ABI (include/fmoe_hip.h, libfmoe_hip.so) exist:

* the compiled pybind11 extension built from csrc/fmoe_cuda_ext.cpp, the form of the
  reference's own module (cuda/fmoe_cuda.cpp:104-125, setup.py:52-69): one C++ call
  per operator.  It is the default;
* ctypes calls from ``_ctypes_ops.py``, which need nothing but the shared library:
  ``FMOE_BINDING=ctypes`` in the environment selects them, and they take over (with a
  warning) when the extension can neither be loaded nor built.

Whichever is bound, ``ctypes_ops`` is the ctypes module, ``BINDING`` names the choice,
and both feed the per-op event hook below.  Every function needs the HIP library and
HIP tensors; nothing here computes on the CPU.
"""
from __future__ import annotations

import os
import warnings

import torch

from . import _ctypes_ops as ctypes_ops

# Optional per-op timing: when `profile_hook` is set to a callable it receives
# (op name, start event, end event) for every launch group, with both events
# recorded on the stream the kernels run on.  Off (None) by default.  An event
# costs a few microseconds of idle GPU, so `profile_only` (a set of op names)
# can restrict the pairs to the ops of interest.
profile_hook = None
profile_only = None

MAX_GATE_TOP_K = ctypes_ops.MAX_GATE_TOP_K   # FMOE_MAX_GATE_TOP_K of the C ABI
init = ctypes_ops.init                       # one-time GPU set-up (fmoe_init), either binding

OPERATORS = ("expert_count", "assign_pos", "linear_forward", "linear_backward",
             "limit_by_capacity", "prune_gate_by_capacity", "local_scatter", "scatter_tokens",
             "local_gather", "route", "route_static", "grouped_linear_fwd",
             "grouped_linear_bwd", "pointer_table", "grouped_linear_fwd_ptrs",
             "grouped_linear_bwd_ptrs", "gather_combine_fwd", "gather_combine_bwd",
             "scatter_reduce", "topk_softmax_fwd", "topk_softmax_bwd", "gelu_fwd", "gelu_bwd",
             "set_gemm_path", "_seg_off_from_counts")


def _hooked(op_name, fn):
    """A compiled operator that reports to `profile_hook` the way the ctypes ones do."""

    def op(*args, **kwargs):
        if profile_hook is None:
            return fn(*args, **kwargs)
        name = op_name
        if name == "grouped_linear_fwd_ptrs":
            name = ("grouped_linear_fwd_act" if kwargs.get("with_gelu") or
                    (len(args) > 5 and args[5]) else "grouped_linear_fwd")
        elif name == "grouped_linear_fwd" and (kwargs.get("with_gelu") or
                                               (len(args) > 4 and args[4])):
            name = "grouped_linear_fwd_act"
        elif name in ("grouped_linear_bwd", "grouped_linear_bwd_ptrs"):
            # need_bias, need_dx, need_dw are arguments 4..6
            dx = kwargs.get("need_dx", args[5] if len(args) > 5 else True)
            dw = kwargs.get("need_dw", args[6] if len(args) > 6 else True)
            name = ("grouped_linear_bwd" if dx and dw else "grouped_linear_dgrad" if dx else
                    "grouped_linear_wgrad" if dw else "grouped_linear_bias_grad")
        if profile_only is not None and name not in profile_only:
            return fn(*args, **kwargs)
        first = next((a for a in args if isinstance(a, torch.Tensor) and a.is_cuda), None)
        if first is None:
            return fn(*args, **kwargs)
        stream = torch.cuda.current_stream(first.device)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        out = fn(*args, **kwargs)
        end.record(stream)
        profile_hook(name, start, end)
        return out

    op.__name__ = op_name
    op.__doc__ = getattr(ctypes_ops, op_name).__doc__
    return op


def _bind(binding: str) -> None:
    g = globals()
    if binding == "compiled":
        from . import _ext

        compiled = _ext.load()
        for name in OPERATORS:
            g[name] = _hooked(name, getattr(compiled, name))
    else:
        for name in OPERATORS:
            g[name] = getattr(ctypes_ops, name)
    g["BINDING"] = binding


_want = os.environ.get("FMOE_BINDING", "").strip().lower()
if _want in ("", "compiled", "ext", "pybind"):
    try:
        _bind("compiled")
    except Exception as exc:   # no compiler / headers for the extension on this machine
        if _want:
            raise
        warnings.warn(f"fastmoe_amd: the compiled fmoe_cuda extension is unavailable ({exc}); "
                      "using the ctypes binding of the same library")
        _bind("ctypes")
elif _want == "ctypes":
    _bind("ctypes")
else:
    raise ImportError(f"FMOE_BINDING={_want!r}: expected 'compiled' or 'ctypes'")
