"""Loads the compiled PyTorch binding: the pybind11 module `fmoe_cuda` built from
csrc/fmoe_cuda_ext.cpp (same functions as the ctypes module fmoe_cuda.py, one
C++ call per operator instead of a Python wrapper around ctypes)."""
from __future__ import annotations

import importlib.util
import os
import sys

from . import _lib

_mod = None


def load(build_if_missing: bool = True):
    """Returns the compiled module, building it first if no binary exists."""
    global _mod
    if _mod is not None:
        return _mod
    from . import build as _build

    _lib.load()                      # libfmoe_hip.so first: the extension links to it
    path = _build.ext_path()
    # a binary compiled from another state of its source or of the C ABI header
    stale = (os.path.exists(path) and os.path.exists(_build.EXT_SRC)
             and _build.ext_built_hash(path) != _build.ext_source_hash())
    if not os.path.exists(path) or stale:
        if not build_if_missing:
            raise ImportError(f"{path} is missing or was built from other sources; run "
                              "`python fastmoe_amd/build.py`")
        _build.build_extension(verbose=False)
    import torch  # noqa: F401  (the module links to libtorch)

    spec = importlib.util.spec_from_file_location("fmoe_cuda", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    _mod = mod
    return mod


def install() -> None:
    """Registers the compiled module as top-level `fmoe_cuda`."""
    sys.modules["fmoe_cuda"] = load()
