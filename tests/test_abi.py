"""The C-ABI library loads and exports exactly what include/fmoe_hip.h declares
(no compute calls: this runs without a GPU)."""
import os
import re

from conftest import ROOT


def _declared():
    text = open(os.path.join(ROOT, "include", "fmoe_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fmoe_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_reference_surface():
    names = _declared()
    for need in ["fmoe_expert_count", "fmoe_assign_pos", "fmoe_local_scatter",
                 "fmoe_local_gather", "fmoe_grouped_linear_fwd",
                 "fmoe_grouped_linear_bwd", "fmoe_limit_by_capacity",
                 "fmoe_prune_gate_by_capacity"]:
        assert need in names


def test_library_exports_every_declared_symbol():
    from fastmoe_amd import _lib

    lib = _lib.load()
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in fmoe_hip.h but not exported"
    assert set(_lib.SIGNATURES) == set(_declared())
    assert b"gfx950" in lib.fmoe_version()


def test_argument_errors_are_reported_not_fatal():
    from fastmoe_amd import _lib

    lib = _lib.load()
    # bad sizes are rejected before any launch, so this is safe without a GPU
    assert lib.fmoe_route_workspace_bytes(-1, 4) < 0
    assert lib.fmoe_route_workspace_bytes(4096, 8) >= 4 * 2 * 8
    rc = lib.fmoe_expert_count(None, -5, None, 4, None)
    assert rc == -1 and b"bad sizes" in lib.fmoe_last_error()
    rc = lib.fmoe_route(None, 10, 5000, None, None, None, None, None, 0, None)
    assert rc == -2 and b"FMOE_MAX_EXPERTS" in lib.fmoe_last_error()
    rc = lib.fmoe_gather_combine_fwd(None, None, None, None, 4, 65, 8, 3, None)
    assert rc == -2
    assert lib.fmoe_set_gemm_path(7) == -1 and lib.fmoe_set_gemm_path(6) == 0
    assert lib.fmoe_set_gemm_path(0) == 0


def test_product_does_not_touch_the_oracle():
    """No file of the package may import or open anything under oracle/."""
    pkg = os.path.join(ROOT, "fastmoe_amd")
    for dirpath, _dirs, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"
