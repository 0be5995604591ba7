"""Loads libfmoe_hip.so (the C ABI declared in include/fmoe_hip.h) with ctypes.

There is no CPU fallback: if the library is neither prebuilt nor buildable the
import of the operator module fails with an explicit error.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_int32, c_int64, c_void_p

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libfmoe_hip.so")

_lib = None

# name -> (restype, argtypes); one entry per declaration in include/fmoe_hip.h
SIGNATURES = {
    "fmoe_version": (c_char_p, []),
    "fmoe_last_error": (c_char_p, []),
    "fmoe_init": (c_int, [c_void_p]),
    "fmoe_expert_count": (c_int, [c_void_p, c_int64, c_void_p, c_int32, c_void_p]),
    "fmoe_route_workspace_bytes": (c_int64, [c_int64, c_int32]),
    "fmoe_assign_pos": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int32,
                                c_void_p, c_int64, c_void_p]),
    "fmoe_route": (c_int, [c_void_p, c_int64, c_int32, c_void_p, c_void_p,
                           c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "fmoe_route_static": (c_int, [c_void_p, c_int64, c_int32, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_void_p]),
    "fmoe_limit_by_capacity": (c_int, [c_void_p, c_void_p, c_void_p, c_int64,
                                       c_int64, c_void_p]),
    "fmoe_prune_gate_by_capacity": (c_int, [c_void_p, c_void_p, c_void_p, c_int64,
                                            c_int64, c_int64, c_void_p, c_int64,
                                            c_void_p]),
    "fmoe_local_scatter": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                   c_int64, c_void_p, c_int, c_void_p]),
    "fmoe_local_gather": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                  c_int64, c_void_p, c_int, c_int, c_void_p]),
    "fmoe_gather_combine_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int64, c_int64, c_int64, c_int, c_void_p]),
    "fmoe_gather_combine_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_int64, c_int64,
                                        c_int64, c_int, c_void_p]),
    "fmoe_scatter_reduce": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                    c_int64, c_int, c_void_p]),
    "fmoe_grouped_linear_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_int64, c_int64, c_int64,
                                        c_int64, c_int, c_void_p]),
    "fmoe_grouped_linear_fwd_act": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                            c_int64, c_int, c_void_p]),
    "fmoe_grouped_linear_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_void_p, c_int64,
                                        c_int64, c_int64, c_int64, c_int, c_void_p]),
    "fmoe_grouped_linear_bwd_act": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_void_p, c_int64,
                                            c_int64, c_int64, c_int64, c_int, c_void_p]),
    "fmoe_grouped_linear_fwd_ptrs": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                             c_void_p, c_int64, c_int64, c_int64, c_int64,
                                             c_int, c_void_p]),
    "fmoe_grouped_linear_bwd_ptrs": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                             c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                             c_int64, c_int64, c_int, c_void_p]),
    "fmoe_pointer_table": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "fmoe_seg_off_from_host_counts": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "fmoe_topk_softmax_fwd": (c_int, [c_void_p, c_int64, c_int32, c_int32, c_void_p, c_void_p,
                                      c_int, c_void_p]),
    "fmoe_topk_softmax_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32,
                                      c_int32, c_int, c_void_p]),
    "fmoe_scatter_tokens": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                    c_int, c_void_p]),
    "fmoe_gelu_fwd": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int, c_void_p]),
    "fmoe_gelu_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int,
                              c_void_p]),
    "fmoe_set_gemm_path": (c_int, [c_int]),
}


def _preload_torch_hip_runtime() -> None:
    """Make the process use ONE HIP runtime: the one torch already mapped.

    libfmoe_hip.so asks for libamdhip64.so.7 by soname; once torch's copy is
    mapped the dynamic loader reuses it, so streams and pointers are shared.
    """
    try:
        import torch  # noqa: F401  (maps torch/lib/libamdhip64.so)
    except Exception:  # pragma: no cover - torch is optional for the C ABI
        pass


def load(build_if_missing: bool = True) -> ctypes.CDLL:
    """Returns the loaded library, building it first if no binary exists."""
    global _lib
    if _lib is not None:
        return _lib
    from . import build as _build

    if not os.path.exists(LIB_PATH):
        if not build_if_missing:
            raise ImportError(f"{LIB_PATH} is missing; run `python fastmoe_amd/build.py`")
        _build.build(verbose=False)
    elif os.path.isdir(_build.CSRC):
        # a binary left behind by an earlier state of csrc/ must not be loaded
        # silently: the kernels and the signature table below would disagree
        want, have = _build.source_hash(), _build.built_hash(LIB_PATH)
        if want != have:
            if not (build_if_missing and os.path.exists(_build.HIPCC)):
                raise ImportError(
                    f"{LIB_PATH} was built from other sources (digest {have}, csrc/ has "
                    f"{want}); run `python fastmoe_amd/build.py`")
            _build.build(verbose=False)
    _preload_torch_hip_runtime()
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class FMoEError(RuntimeError):
    """A C-ABI call returned a negative status."""


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().fmoe_last_error().decode("utf-8", "replace")
        raise FMoEError(f"{what} failed (status {status}): {msg}")
