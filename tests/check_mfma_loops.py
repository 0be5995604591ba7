"""Checks what the compiler made of the K loops of fastmoe_amd/csrc/gemm_mfma_impl.h.

    python tests/check_mfma_loops.py [--all-dtypes] [--keep FILE.s]

The kernels copy their operands into LDS with `buffer_load ... lds` written as inline
assembly, and wait for them with their own `s_waitcnt vmcnt(n)`: the compiler does not
know that those copies are in flight.  Three things it may do to an MFMA loop
therefore cost far more than they look (each was seen, each time after a change to an
EPILOGUE, never to the loop itself):

* an `s_waitcnt vmcnt(n)` of its own inside the loop (it counts only the loads it
  knows about, so the wait drains the whole queue of copies: two of them made the
  forward kernel 6 % slower);
* accumulator moves (`v_accvgpr_*`) inside the loop, when two variants of the code
  that reads the accumulators want them in different registers (40 moves per slice,
  4 %);
* scratch accesses inside the loop (spills).

The script compiles the file to assembly for gfx950 (bf16 kernels only unless
--all-dtypes: about 1.5 instead of 3.5 minutes), finds every loop with at least 16
MFMAs and fewer than 700 lines, and reports the three counts; exit status 1 if any is
not zero.  A `flat_load` anywhere in a kernel of the file is reported as well.
"""
from __future__ import annotations

import argparse
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(os.path.dirname(HERE), "fastmoe_amd")
CSRC = os.path.join(PKG, "csrc")


def _library_build():
    """fastmoe_amd/build.py (the library's own compiler and flags), loaded by path: the
    package itself is not imported, so no library has to exist yet."""
    import importlib.util

    spec = importlib.util.spec_from_file_location(
        "fmoe_library_build", os.path.join(PKG, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def compile_to_assembly(out_path: str, all_dtypes: bool) -> None:
    _build = _library_build()

    # one translation unit per element type; their assembly is concatenated
    units = ["gemm_mfma_bf16.hip"] + (["gemm_mfma_f16.hip"] if all_dtypes else [])
    with open(out_path, "w") as out:
        for unit in units:
            part = out_path + "." + unit + ".s"
            cmd = [_build.HIPCC, *_build.FLAGS, "--cuda-device-only", "-S",
                   os.path.join(CSRC, unit), "-o", part]
            res = subprocess.run(cmd, capture_output=True, text=True)
            if res.returncode != 0:
                raise RuntimeError("hipcc failed:\n" + res.stderr[-4000:])
            with open(part) as f:
                out.write(f.read())
            os.remove(part)


def scan(asm_text: str):
    """([(kernel, [(mfmas, lines, compiler_vmcnt_waits, accvgpr_moves, scratch_ops)])],
    {kernel: flat loads anywhere in its body})"""
    lines = asm_text.split("\n")
    out = []
    flat = {}
    for start in (i for i, l in enumerate(lines) if re.match(r"^_ZN4fmoe\S+:", l)):
        name = lines[start].split(":")[0]
        end = next((i for i in range(start, len(lines)) if lines[i].startswith(".Lfunc_end")),
                   None)
        if end is None:
            continue
        body = lines[start:end]
        n_flat = sum(1 for x in body if re.match(r"^\s+flat_load", x))
        if n_flat:
            flat[name] = n_flat
        labels = {}
        for i, l in enumerate(body):
            m = re.match(r"^(\.LBB\d+_\d+):", l)
            if m:
                labels[m.group(1)] = i
        loops = []
        for i, l in enumerate(body):
            m = re.search(r"s_cbranch\w*\s+(\.LBB\d+_\d+)", l)
            if not (m and m.group(1) in labels and labels[m.group(1)] < i):
                continue
            block = body[labels[m.group(1)]:i + 1]
            mfmas = sum(1 for x in block if "v_mfma" in x)
            if mfmas < 16 or len(block) >= 700:
                continue
            in_asm = False
            waits = moves = scratch = 0
            for x in block:
                if "ASMSTART" in x:
                    in_asm = True
                elif "ASMEND" in x:
                    in_asm = False
                elif not in_asm and "s_waitcnt" in x and "vmcnt" in x:
                    waits += 1
                moves += "v_accvgpr" in x
                scratch += "scratch_" in x
            loops.append((mfmas, len(block), waits, moves, scratch))
        if loops:
            out.append((name, loops))
    return out, flat


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--all-dtypes", action="store_true", help="also the f16 kernels")
    ap.add_argument("--keep", metavar="FILE", help="keep the assembly in FILE")
    ap.add_argument("--assembly", metavar="FILE", help="scan FILE instead of compiling")
    args = ap.parse_args()
    if args.assembly:
        text = open(args.assembly).read()
    else:
        build_dir = os.path.join(CSRC, "build")      # the library's object directory
        os.makedirs(build_dir, exist_ok=True)
        path = args.keep or os.path.join(build_dir, "gemm_mfma_loops.%d.s" % os.getpid())
        try:
            compile_to_assembly(path, args.all_dtypes)
            text = open(path).read()
        finally:
            if not args.keep and os.path.exists(path):
                os.remove(path)
    found, flat = scan(text)
    bad = 0
    # The activation epilogues index an LDS table with an offset that may lie outside
    # the table (the result is then recomputed): harmless as an LDS read, a wild global
    # read if the compiler ever lost the pointer's address space and emitted a flat load.
    for name, n in flat.items():
        print("%s: %d flat_load instructions (LDS / global pointers must keep their "
              "address spaces)" % (name[:80], n))
        bad += n
    for name, loops in found:
        short = re.sub(r"_ZN4fmoe\d+", "", name).replace("14__hip_bfloat16", "bf16")
        short = short.replace("6__half", "f16")[:64]
        flagged = [l for l in loops if l[2] or l[3] or l[4]]
        bad += len(flagged)
        print("%-66s %2d loops%s" % (short, len(loops), "" if not flagged else
              "  BAD (mfmas, lines, vmcnt waits, acc moves, scratch): " + str(flagged)))
    print("%d kernels, %d loops, %d flagged" % (len(found), sum(len(l) for _, l in found), bad))
    if not found:
        print("no MFMA loops found: the scan does not fit the compiler's output any more")
        return 1
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
