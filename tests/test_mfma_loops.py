"""The K loops of the matrix-core GEMM as the compiler emits them: no wait of the
compiler's own on the memory counter, no accumulator moves, no scratch access (see
tests/check_mfma_loops.py for why each of them is expensive here).  Needs
hipcc but no GPU; about a minute and a half."""
import os
import subprocess
import sys

import pytest

from conftest import ROOT


def test_compiler_leaves_the_mfma_loops_alone():
    from fastmoe_amd import build as lib_build

    if not os.path.exists(lib_build.HIPCC):
        pytest.skip("no hipcc on this machine")
    res = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "check_mfma_loops.py")],
                         capture_output=True, text=True, timeout=900)
    assert res.returncode == 0, (res.stdout + res.stderr)[-3000:]
    assert " 0 flagged" in res.stdout
