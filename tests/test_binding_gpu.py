"""The compiled PyTorch binding (pybind11 module `fmoe_cuda`, the form of the
reference's cuda/fmoe_cuda.cpp:104-125) against the ctypes module: the same C
ABI underneath, so every operator must return bit-identical tensors; then the
routing / dispatch / linear / layer suites once more in a child process with
FMOE_BINDING=ctypes: the whole Python layer runs on the extension by default, and
there on the ctypes calls."""
import os
import subprocess
import sys

import pytest
import torch

from conftest import ROOT
from helpers import make_gate, randn


def _same(a, b):
    if a is None or b is None:
        return a is None and b is None
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a, b)


@pytest.mark.gpu
def test_compiled_module_matches_the_ctypes_module_bit_for_bit():
    from fastmoe_amd import _ext, fmoe_cuda

    py = fmoe_cuda.ctypes_ops
    cx = _ext.load()
    assert fmoe_cuda.BINDING == "compiled"      # the default
    e, k, t, d, h = 6, 2, 300, 64, 96
    gate = torch.from_numpy(make_gate(t, k, e, drop=0.1, seed=3, empty=(4,))).cuda()
    # routing
    ra, rb = py.route(gate, e), cx.route(gate, e)
    n_valid = int(ra[2][-1])
    assert _same(ra[0][:n_valid], rb[0][:n_valid]) and all(_same(a, b) for a, b in
                                                            zip(ra[1:], rb[1:]))
    pos, count, seg, inv = ra
    ha, hb = torch.zeros(e, dtype=torch.int32).cuda(), torch.zeros(e, dtype=torch.int32).cuda()
    py.expert_count(gate, ha)
    cx.expert_count(gate, hb)
    assert _same(ha, hb)
    cum = torch.cumsum(ha, 0).int()
    pa, pb = torch.zeros(n_valid, dtype=torch.int64).cuda(), torch.zeros(n_valid, dtype=torch.int64).cuda()
    ca, cb = cum.clone(), cum.clone()
    py.assign_pos(ca, gate, pa)
    cx.assign_pos(cb, gate, pb)
    assert _same(pa, pb) and _same(ca, cb)
    cap_a = torch.full((e,), 70, dtype=torch.int32).cuda()
    cap_b = cap_a.clone()
    assert _same(py.limit_by_capacity(count, cap_a, e, 1), cx.limit_by_capacity(count, cap_b, e, 1))
    assert _same(cap_a, cap_b)
    ea, eb = torch.full((e,), 70, dtype=torch.int32).cuda(), torch.full((e,), 70, dtype=torch.int32).cuda()
    assert _same(py.prune_gate_by_capacity(gate.clamp(min=0), ea, e, 1),
                 cx.prune_gate_by_capacity(gate.clamp(min=0), eb, e, 1)) and _same(ea, eb)
    for dtype in (torch.float32, torch.bfloat16):
        x = randn((t, d), dtype, 1).cuda()
        w = randn((e, h, d), dtype, 2, 0.1).cuda()
        b = randn((e, h), dtype, 3).cuda()
        score = randn((t, k), dtype, 4).cuda()
        # dispatch
        buf = py.local_scatter(x, pos[:n_valid], k)
        assert _same(buf, cx.local_scatter(x, pos[:n_valid], k))
        assert _same(py.scatter_tokens(x, inv, k)[:n_valid], cx.scatter_tokens(x, inv, k)[:n_valid])
        assert _same(py.local_gather(buf, pos[:n_valid], t * k, False),
                     cx.local_gather(buf, pos[:n_valid], t * k, False))
        # expert GEMMs, device-side segments and the reference's host counts
        ya, yb = py.grouped_linear_fwd(buf, seg, w, b), cx.grouped_linear_fwd(buf, seg, w, b)
        assert _same(ya, yb)
        assert _same(py.linear_forward(buf, count.cpu(), w, b), cx.linear_forward(buf, count.cpu(), w, b))
        assert _same(ya, cx.linear_forward(buf, count.cpu(), w, b))
        dy = randn(tuple(ya.shape), dtype, 5).cuda()
        ga, gb = py.grouped_linear_bwd(dy, buf, seg, w), cx.grouped_linear_bwd(dy, buf, seg, w)
        assert all(_same(a, c) for a, c in zip(ga, gb))
        la, lb = py.linear_backward(dy, buf, count.cpu(), w, b), cx.linear_backward(dy, buf, count.cpu(), w, b)
        assert all(_same(a, c) for a, c in zip(la, lb))
        ga, gb = (py.grouped_linear_bwd(dy, buf, seg, w, need_bias=False, need_dw=False),
                  cx.grouped_linear_bwd(dy, buf, seg, w, need_bias=False, need_dw=False))
        assert _same(ga[0], gb[0]) and gb[1] is None and gb[2] is None
        # combine both ways, scatter backward
        full = torch.zeros(t * k, d, dtype=dtype).cuda()
        full[:n_valid] = buf
        assert _same(py.gather_combine_fwd(full, inv, score, t, k),
                     cx.gather_combine_fwd(full, inv, score, t, k))
        ba, bb = (py.gather_combine_bwd(x, full, inv, score, t, k),
                  cx.gather_combine_bwd(x, full, inv, score, t, k))
        assert _same(ba[0][:n_valid], bb[0][:n_valid]) and _same(ba[1], bb[1])
        assert _same(py.scatter_reduce(full, inv, t, k), cx.scatter_reduce(full, inv, t, k))
        # gate and activation
        logits = randn((t, e), dtype, 6).cuda()
        ta, tb = py.topk_softmax_fwd(logits, k), cx.topk_softmax_fwd(logits, k)
        assert _same(ta[0], tb[0]) and _same(ta[1], tb[1])
        assert _same(py.topk_softmax_bwd(score, ta[1], ta[0], e), cx.topk_softmax_bwd(score, tb[1], tb[0], e))
        assert _same(py.gelu_fwd(ya), cx.gelu_fwd(ya))
        assert _same(py.gelu_bwd(dy, ya), cx.gelu_bwd(dy, ya))
    # errors are RuntimeErrors, as the reference's AT_ASSERTM failures are
    with pytest.raises(RuntimeError):
        cx.expert_count(gate.cpu(), ha)
    with pytest.raises(RuntimeError):
        cx.grouped_linear_fwd(x, seg, w.float(), None)
    with pytest.raises(RuntimeError):
        cx.topk_softmax_fwd(torch.zeros(4, 3).cuda(), 4)


@pytest.mark.gpu
@pytest.mark.timeout(900)
@pytest.mark.parametrize("suites", [
    ("tests/test_routing_gpu.py", "tests/test_dispatch_gpu.py", "tests/test_act_gpu.py"),
    ("tests/test_linear_gpu.py",),
    ("tests/test_layer_gpu.py", "tests/test_fused_act_gpu.py"),
], ids=["routing-dispatch-act", "linear", "layer-fused_act"])
def test_suites_pass_on_the_ctypes_binding(suites):
    """Routing, dispatch, linear, activation and layer suites with the package bound
    to the ctypes calls instead of the compiled extension (one child process per group of
    suites, so that none runs for minutes without a sign of life; the big benchmark-size
    cases stay with the default binding).  The activation suites also watch the per-op
    event hook, which both bindings must feed alike."""
    env = dict(os.environ, FMOE_BINDING="ctypes")
    cmd = [sys.executable, "-m", "pytest", "-x", "-q", "-m", "gpu", "-p", "no:cacheprovider",
           *suites, "-k", "not full_size and not config2"]
    res = subprocess.run(cmd, cwd=ROOT, env=env, capture_output=True, text=True, timeout=850)
    tail = (res.stdout + res.stderr)[-3000:]
    assert res.returncode == 0, tail
    assert " passed" in res.stdout, tail


def test_compiled_module_loads_and_has_the_reference_surface():
    """No GPU needed: the extension imports, carries the six functions of
    cuda/fmoe_cuda.cpp:117-124 and turns a host tensor into a RuntimeError."""
    from fastmoe_amd import _ext

    m = _ext.load()
    for name in ("expert_count", "assign_pos", "linear_forward", "linear_backward",
                 "limit_by_capacity", "prune_gate_by_capacity"):
        assert callable(getattr(m, name))
    assert m.__name__ == "fmoe_cuda" and m.binding == "compiled"
    with pytest.raises(RuntimeError):
        m.expert_count(torch.zeros(4, dtype=torch.int64), torch.zeros(2, dtype=torch.int32))
    with pytest.raises(RuntimeError):
        m.linear_forward(torch.zeros(4, 8), torch.zeros(2, dtype=torch.int64), torch.zeros(2, 8, 8))
