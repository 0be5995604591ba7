"""Builds libfmoe_hip.so (HIP kernels + C ABI) for gfx950 with plain hipcc.

Run as ``python fastmoe_amd/build.py`` (as a script, so that a stale library
from an earlier build is not loaded by the package import first).  The library is torch-free; it is
written next to the package (fastmoe_amd/lib/) so a prebuilt copy travels with
the source tree.  Building needs no GPU (hipcc cross-compiles).
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libfmoe_hip.so")

# the two heavy translation units first, so that they compile side by side
SOURCES = ["gemm_mfma_bf16.hip", "gemm_mfma_f16.hip", "api.hip", "route.hip", "dispatch.hip",
           "gate.hip", "act.hip", "gemm_simt.hip", "gemm_mfma.hip", "gemm_mfma_wide.hip"]
HEADERS = ["common.h", "gemm.h", "dma_desc.h", "gemm_mfma_impl.h",
           os.path.join("..", "..", "include", "fmoe_hip.h")]
# the library carries a digest of the files it was built from behind this marker
HASH_MARKER = "fmoe-src:"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-inline-asm",   # m0 is written by the LDS-copy instruction sequence
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# Extra compiler flags for experiments with the kernels' named constants, e.g.
# FMOE_EXTRA_HIPCC_FLAGS="-DFMOE_PATCH_ROWS=8 -DFMOE_PATCH_COLS=4" (the order in which
# a launch walks its tiles); they enter the digest, so a library built with them is
# never mistaken for the plain one.
EXTRA_FLAGS = os.environ.get("FMOE_EXTRA_HIPCC_FLAGS", "").split()


def source_hash() -> str:
    """Digest (12 hex digits) of every source and header the library is built from."""
    import hashlib

    h = hashlib.sha256()
    for name in SOURCES + HEADERS:
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read() + b"\0")
    if EXTRA_FLAGS:
        h.update(" ".join(EXTRA_FLAGS).encode())
    return h.hexdigest()[:12]


def built_hash(lib_path: str = LIB_PATH):
    """The digest a built library carries, read from the file without loading it
    (None if the file has none)."""
    with open(lib_path, "rb") as f:
        blob = f.read()
    at = blob.find(HASH_MARKER.encode())
    if at < 0:
        return None
    return blob[at + len(HASH_MARKER):at + len(HASH_MARKER) + 12].decode("ascii", "replace")


def _compile(src: str, verbose: bool) -> str:
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *EXTRA_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    if src == "api.hip":
        cmd.insert(-4, f'-DFMOE_SOURCE_HASH="{source_hash()}"')
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = True, jobs: int = 6) -> str:
    """Compiles every source and links the shared library; returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, verbose), SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


EXT_DIR = os.path.join(PKG_DIR, "ext")
EXT_SRC = os.path.join(CSRC, "fmoe_cuda_ext.cpp")


EXT_HASH_MARKER = "fmoe-ext:"


def ext_source_hash() -> str:
    """Digest of what the extension is compiled from: its source and the C ABI header."""
    import hashlib

    h = hashlib.sha256()
    for path in (EXT_SRC, os.path.join(PKG_DIR, "..", "include", "fmoe_hip.h")):
        with open(path, "rb") as f:
            h.update(f.read() + b"\0")
    return h.hexdigest()[:12]


def ext_built_hash(path: str):
    """The digest a built extension carries (None if it has none)."""
    with open(path, "rb") as f:
        blob = f.read()
    at = blob.find(EXT_HASH_MARKER.encode())
    if at < 0:
        return None
    at += len(EXT_HASH_MARKER)
    return blob[at:at + 12].decode("ascii", "replace")


def ext_path() -> str:
    import sysconfig

    return os.path.join(EXT_DIR, "fmoe_cuda" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_extension(verbose: bool = True) -> str:
    """Compiles the pybind11 module `fmoe_cuda` (csrc/fmoe_cuda_ext.cpp: no
    kernels, plain C++ against the torch headers) and links it to
    libfmoe_hip.so, which must have been built.  Returns its path."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(EXT_DIR, exist_ok=True)
    out = ext_path()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=fmoe_cuda",
           f'-DFMOE_EXT_SOURCE_HASH="{ext_source_hash()}"',
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-Wno-deprecated-declarations"]
    cmd += ["-I" + p for p in ce.include_paths("cuda")]
    cmd += ["-I" + sysconfig.get_paths()["include"]]
    cmd += [EXT_SRC, "-o", out + ".tmp", "-L" + torch_lib, "-L" + LIB_DIR,
            "-lfmoe_hip", "-ltorch_python", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10",
            "-lc10_hip", "-Wl,-rpath,$ORIGIN/../lib", "-Wl,-rpath," + torch_lib]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"building the fmoe_cuda extension failed:\n{res.stderr[-4000:]}")
    os.replace(out + ".tmp", out)
    return out


if __name__ == "__main__":
    print(build())
    print(build_extension())
