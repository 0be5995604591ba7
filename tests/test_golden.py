"""Committed fixtures (tests/golden/, written by make_golden.py from the pinned
CPU checker): the checker must keep reproducing them on the CPU, and the HIP
kernels must reproduce them on the GPU."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _routing():
    with open(os.path.join(GOLD, "routing_cases.json")) as f:
        return json.load(f)


def _layer():
    return dict(np.load(os.path.join(GOLD, "layer_case.npz")))


def test_checker_reproduces_routing_fixtures():
    for c in _routing():
        g, e = np.array(c["gate"], np.int64), c["n_expert"]
        pos, count, seg_off, inv = O.route(g, e)
        assert pos.tolist() == c["pos"] and count.tolist() == c["count"]
        assert seg_off.tolist() == c["seg_off"] and inv.tolist() == c["inv"]
        cap = np.array(c["capacity"], np.int32)
        assert O.prune_gate_by_capacity(g, cap, e).tolist() == c["pruned"]
        assert cap.tolist() == c["capacity_after_prune"]
        cap = np.array(c["capacity"], np.int32)
        assert O.limit_by_capacity(np.array(c["count"]), cap, e, 1).tolist() == c["limited"]
        assert cap.tolist() == c["capacity_after_limit"]


def test_checker_reproduces_layer_fixture():
    L = _layer()
    t = {k: torch.from_numpy(v) for k, v in L.items()}
    leaves = {k: t[k].clone().requires_grad_(True) for k in ("x", "w1", "b1", "w2", "b2", "score")}
    out = O.brute_force_moe_mlp(leaves["x"], t["idx"], leaves["score"], leaves["w1"],
                                leaves["b1"], leaves["w2"], leaves["b2"])
    (out * t["probe"]).sum().backward()
    assert np.allclose(out.detach().numpy(), L["out"], rtol=0, atol=1e-12)
    for name, key in (("x", "dx"), ("w1", "dw1"), ("b1", "db1"), ("w2", "dw2"),
                      ("b2", "db2"), ("score", "dscore")):
        assert np.allclose(leaves[name].grad.numpy(), L[key], rtol=0, atol=1e-11), key
    # dropped slots get no score gradient
    assert L["dscore"][3, 1] == 0 and L["dscore"][17, 0] == 0


@pytest.mark.gpu
def test_kernels_reproduce_routing_fixtures():
    from fastmoe_amd import fmoe_cuda

    for c in _routing():
        e = c["n_expert"]
        g = torch.tensor(c["gate"], dtype=torch.int64, device="cuda")
        pos, count, seg, inv = fmoe_cuda.route(g, e)
        nv = c["seg_off"][-1]
        assert pos.cpu().tolist()[:nv] == c["pos"] and count.cpu().tolist() == c["count"]
        assert seg.cpu().tolist() == c["seg_off"] and inv.cpu().tolist() == c["inv"]
        cap = torch.tensor(c["capacity"], dtype=torch.int32, device="cuda")
        assert fmoe_cuda.prune_gate_by_capacity(g, cap, e, 1).cpu().tolist() == c["pruned"]
        assert cap.cpu().tolist() == c["capacity_after_prune"]
        cap = torch.tensor(c["capacity"], dtype=torch.int32, device="cuda")
        lim = fmoe_cuda.limit_by_capacity(torch.tensor(c["count"], device="cuda"), cap, e, 1)
        assert lim.cpu().tolist() == c["limited"] and cap.cpu().tolist() == c["capacity_after_limit"]


@pytest.mark.gpu
@pytest.mark.parametrize("dt,tol", [(torch.float64, 1e-10), (torch.float32, 2e-5),
                                    (torch.bfloat16, 2e-2)])
def test_kernels_reproduce_layer_fixture(dt, tol):
    """The fused dispatch + grouped GEMMs + combine on the fixture's routing."""
    from fastmoe_amd.functions import FusedGatherCombine, FusedScatter, RoutePlan
    from fastmoe_amd.linear import MOELinear

    L = {k: torch.from_numpy(v) for k, v in _layer().items()}
    leaves = {k: L[k].to(dt).cuda().requires_grad_(True)
              for k in ("x", "w1", "b1", "w2", "b2", "score")}
    plan = RoutePlan(L["idx"].cuda(), 4)
    rows = FusedScatter.apply(leaves["x"], plan)
    hid = MOELinear.apply(rows, plan.segments, leaves["w1"], leaves["b1"])
    hid = torch.nn.functional.gelu(hid)
    rows_out = MOELinear.apply(hid, plan.segments, leaves["w2"], leaves["b2"])
    out = FusedGatherCombine.apply(rows_out, leaves["score"], plan)
    (out.double() * L["probe"].cuda()).sum().backward()

    def rel(a, b):
        b = b.double()
        return ((a.double().cpu() - b).abs().max() / b.abs().max()).item()

    # rounded inputs differ from the float64 fixture by the dtype's epsilon,
    # which the tolerance (max |err| / max |ref|) covers
    assert rel(out, L["out"]) <= tol
    for name, key in (("x", "dx"), ("w1", "dw1"), ("b1", "db1"), ("w2", "dw2"),
                      ("b2", "db2"), ("score", "dscore")):
        assert rel(leaves[name].grad, L[key]) <= tol, key
