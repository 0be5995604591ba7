"""Routing and capacity kernels against the CPU checker: bit-exact."""
import numpy as np
import pytest
import torch

from helpers import make_gate, zipf_gate
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _cuda(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


CASES = [  # n_tokens, top_k, n_expert, drop
    (1, 1, 1, 0.0),
    (12, 2, 8, 0.3),
    (4, 3, 4, 0.0),
    (63, 1, 5, 0.5),
    (64, 2, 64, 0.0),
    (1000, 2, 16, 0.1),
    (2048, 1, 3, 0.0),       # exactly one block
    (2049, 1, 3, 0.0),       # one slot into the second block
    (8192, 2, 16, 0.0),      # config 2
    (16384, 2, 8, 0.0),      # config 4
    (8192, 8, 128, 0.0),     # config 5 shape
    (5000, 2, 1000, 0.2),    # many experts
    (3000, 2, 4096, 0.0),    # the LDS limit
    (4096, 1, 512, 0.05),    # the largest problem routed by a single workgroup
    (4097, 1, 512, 0.05),    # one slot more: three kernels
    (1363, 3, 7, 0.05),      # 4089 slots: ragged last row
    (40000, 2, 64, 0.1),     # 80000 slots: three kernels
    (1500, 2, 513, 0.0),     # one expert too many for the single workgroup
]


@pytest.mark.parametrize("n,k,e,drop", CASES)
def test_expert_count(n, k, e, drop):
    from fastmoe_amd import fmoe_cuda

    g = make_gate(n, k, e, drop, seed=n + e)
    want = O.expert_count(g, e)
    out = torch.zeros(e, dtype=torch.int32, device="cuda")
    fmoe_cuda.expert_count(_cuda(g), out)
    assert np.array_equal(out.cpu().numpy(), want)
    fmoe_cuda.expert_count(_cuda(g), out)  # accumulates
    assert np.array_equal(out.cpu().numpy(), 2 * want)


def test_expert_count_skips_out_of_range_and_handles_large_expert_sets():
    from fastmoe_amd import fmoe_cuda

    g = np.array([0, 3, -1, 7, 4, 2, 2, -5, 100], np.int64)
    out = torch.zeros(4, dtype=torch.int32, device="cuda")
    fmoe_cuda.expert_count(_cuda(g), out)
    assert out.cpu().tolist() == O.expert_count(g, 4).tolist() == [1, 0, 2, 1]
    e = 5000  # beyond the LDS-resident path
    g = make_gate(3000, 2, e, 0.1, seed=5)
    out = torch.zeros(e, dtype=torch.int32, device="cuda")
    fmoe_cuda.expert_count(_cuda(g), out)
    assert np.array_equal(out.cpu().numpy(), O.expert_count(g, e))
    empty = torch.zeros(4, dtype=torch.int32, device="cuda")
    fmoe_cuda.expert_count(torch.empty(0, dtype=torch.int64, device="cuda"), empty)
    assert empty.sum().item() == 0


@pytest.mark.parametrize("n,k,e,drop", CASES)
def test_assign_pos_and_route(n, k, e, drop):
    from fastmoe_amd import fmoe_cuda

    g = make_gate(n, k, e, drop, seed=7 * n + e)
    pos_w, count_w, seg_w, inv_w = O.route(g, e)
    # legacy pair: histogram + cumsum on the host side, then assign_pos
    cum = _cuda(np.cumsum(count_w).astype(np.int32))
    pos = torch.full((int(count_w.sum()),), -9, dtype=torch.int64, device="cuda")
    fmoe_cuda.assign_pos(cum, _cuda(g), pos)
    assert np.array_equal(pos.cpu().numpy(), pos_w)
    assert np.array_equal(cum.cpu().numpy(), seg_w[:-1])  # left as exclusive prefix
    # fused call
    pos2, count2, seg2, inv2 = fmoe_cuda.route(_cuda(g), e)
    nv = int(seg_w[-1])
    assert np.array_equal(count2.cpu().numpy(), count_w)
    assert np.array_equal(seg2.cpu().numpy(), seg_w)
    assert np.array_equal(pos2.cpu().numpy()[:nv], pos_w)
    assert np.array_equal(inv2.cpu().numpy(), inv_w)


def test_route_all_dropped_and_empty():
    from fastmoe_amd import fmoe_cuda

    g = np.full((10, 2), -1, np.int64)
    pos, count, seg, inv = fmoe_cuda.route(_cuda(g), 4)
    assert count.cpu().tolist() == [0, 0, 0, 0] and seg.cpu().tolist() == [0] * 5
    assert inv.cpu().tolist() == [-1] * 20
    pos, count, seg, inv = fmoe_cuda.route(torch.empty((0, 2), dtype=torch.int64, device="cuda"), 3)
    assert count.cpu().tolist() == [0, 0, 0] and seg.cpu().tolist() == [0, 0, 0, 0]


def test_count_by_gate_matches_reference_shapes():
    from fastmoe_amd.functions import count_by_gate, prepare_forward

    g = make_gate(12, 2, 4, 0.3, seed=1)
    pos_w, count_w, _seg, _inv = O.route(g, 4)
    pos, lec, gec = count_by_gate(_cuda(g), 4, 1)
    assert pos.dtype == torch.int64 and lec.dtype == torch.int64 and lec is gec
    assert np.array_equal(pos.cpu().numpy(), pos_w)
    assert np.array_equal(lec.cpu().numpy(), count_w)
    none, lec2, _ = count_by_gate(_cuda(g), 4, 1, require_pos=False)
    assert none is None and np.array_equal(lec2.cpu().numpy(), count_w)
    pos, lec, gec, fec, fbs = prepare_forward(_cuda(g), 4, 1)
    assert not lec.is_cuda and not fec.is_cuda and fbs == int(count_w.sum())


@pytest.mark.parametrize("e,w", [(1, 1), (16, 1), (64, 1), (5, 7), (300, 3)])
def test_limit_by_capacity(e, w):
    from fastmoe_amd import fmoe_cuda

    rng = np.random.default_rng(e * 31 + w)
    ec = rng.integers(0, 60, size=e * w).astype(np.int64)
    cap0 = rng.integers(0, 100, size=e).astype(np.int32)
    cap_w = cap0.copy()
    want = O.limit_by_capacity(ec, cap_w, e, w)
    cap = _cuda(cap0)
    got = fmoe_cuda.limit_by_capacity(_cuda(ec), cap, e, w)
    assert got.dtype == torch.int64
    assert np.array_equal(got.cpu().numpy(), want)
    assert np.array_equal(cap.cpu().numpy(), cap_w)


@pytest.mark.parametrize("n,k,e,drop", CASES)
def test_prune_gate_by_capacity(n, k, e, drop):
    from fastmoe_amd import fmoe_cuda

    g = make_gate(n, k, e, drop, seed=3 * n + e)
    rng = np.random.default_rng(n)
    cap0 = rng.integers(0, max(2, 2 * n * k // e), size=e).astype(np.int32)
    cap_w = cap0.copy()
    want = O.prune_gate_by_capacity(g, cap_w, e)
    cap = _cuda(cap0)
    got = fmoe_cuda.prune_gate_by_capacity(_cuda(g), cap, e, 1)
    assert got.shape == g.shape
    assert np.array_equal(got.cpu().numpy(), want)
    assert np.array_equal(cap.cpu().numpy(), cap_w)


def test_config3_capacity_chain_is_bit_exact():
    """Zipf(1.2) routing, 16384 tokens, 64 experts, capacity 640 per expert."""
    from fastmoe_amd.gates import limit_by_capacity

    g = zipf_gate(16384, 64, 1.2, seed=0)
    cap = 640
    count = O.expert_count(g, 64).astype(np.int64)
    capv = np.full(64, cap, np.int32)
    new_w = O.limit_by_capacity(count, capv, 64, 1)
    pruned_w = O.prune_gate_by_capacity(g, new_w.astype(np.int32), 64)
    new_lec, new_gec, pruned = limit_by_capacity(_cuda(g), 64, 1, cap)
    assert np.array_equal(new_lec.cpu().numpy(), new_w)
    assert np.array_equal(pruned.cpu().numpy(), pruned_w)
    kept = (pruned_w >= 0).sum()
    assert kept == np.minimum(count, cap).sum() and kept < g.size
    # size-independent properties of the drop mask
    p = pruned.cpu().numpy()
    assert np.all((p == g) | (p == -1))
    assert np.bincount(p[p >= 0], minlength=64).max() <= cap
