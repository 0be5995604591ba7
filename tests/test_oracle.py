"""Pins the CPU checker (oracle/) before anything is compared against it.

Each check uses a formulation independent of the oracle's own loop: a library
routine, a closed form, an invariant, or brute force on tiny inputs.  The
reference ships no golden vectors for this path (its tests are differential,
tests/test_numerical.py, tests/test_local_exchange.py), so these are the pins.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O

RNG = np.random.default_rng(20240607)


def _gate(n, k, n_expert, drop=0.0):
    g = RNG.integers(0, n_expert, size=(n, k))
    if drop:
        g[RNG.random((n, k)) < drop] = -1
    return g.astype(np.int64)


@pytest.mark.parametrize("n,k,e,drop", [(0, 2, 4, 0), (1, 1, 1, 0), (12, 2, 8, 0.3),
                                       (1000, 3, 16, 0.1), (4097, 2, 130, 0.0)])
def test_expert_count_is_bincount(n, k, e, drop):
    g = _gate(n, k, e, drop)
    flat = g.reshape(-1)
    want = np.bincount(flat[flat >= 0], minlength=e)
    got = O.expert_count(g, e)
    assert got.dtype == np.int32 and np.array_equal(got, want)
    # accumulates into the caller's buffer
    again = O.expert_count(g, e, into=got.copy())
    assert np.array_equal(again, 2 * want)
    # out-of-range values are ignored, like -1
    g2 = np.concatenate([flat, [e, e + 5, -3]])
    assert np.array_equal(O.expert_count(g2, e), want)


@pytest.mark.parametrize("n,k,e,drop", [(1, 1, 1, 0), (12, 2, 8, 0.3), (333, 2, 7, 0.5),
                                       (5000, 2, 64, 0.05)])
def test_assign_pos_is_stable_argsort(n, k, e, drop):
    g = _gate(n, k, e, drop)
    flat = g.reshape(-1)
    order = np.argsort(flat, kind="stable")
    want = order[flat[order] >= 0]
    pos, count, seg_off, inv = O.route(g, e)
    assert np.array_equal(pos, want)
    # invariants that hold for ANY legal arrival order of the reference kernel
    assert sorted(pos.tolist()) == np.flatnonzero(flat >= 0).tolist()
    for x in range(e):
        seg = pos[seg_off[x]:seg_off[x + 1]]
        assert np.all(flat[seg] == x) and seg.size == count[x]
    assert np.array_equal(inv[pos], np.arange(pos.size))
    assert np.all(inv[flat < 0] == -1)
    # side effect: the inclusive prefix becomes the exclusive one
    cum = np.cumsum(count).astype(np.int32)
    O.assign_pos(cum, g)
    assert np.array_equal(cum, seg_off[:-1])


def test_limit_by_capacity_one_worker_is_min():
    ec = RNG.integers(0, 50, size=16)
    cap0 = RNG.integers(0, 40, size=16).astype(np.int32)
    cap = cap0.copy()
    eca = O.limit_by_capacity(ec, cap, 16, 1)
    assert np.array_equal(eca, np.minimum(ec, cap0))
    assert np.array_equal(cap, cap0 - ec)  # the full proposal is subtracted


def test_limit_by_capacity_many_workers_invariants():
    e, w = 5, 7
    ec = RNG.integers(0, 30, size=(w, e))
    cap0 = RNG.integers(0, 90, size=e).astype(np.int32)
    cap = cap0.copy()
    eca = O.limit_by_capacity(ec, cap, e, w).reshape(w, e)
    assert np.all(eca >= 0) and np.all(eca <= ec)
    assert np.all(eca.sum(0) <= cap0)
    # workers are served in ascending order: worker w sees cap - sum of earlier proposals
    seen = cap0[None, :] - np.concatenate([np.zeros((1, e), int), np.cumsum(ec, 0)[:-1]])
    assert np.array_equal(eca, np.clip(np.minimum(ec, seen), 0, None))
    assert np.array_equal(cap, cap0 - ec.sum(0))


@pytest.mark.parametrize("n,k,e", [(16, 2, 4), (257, 1, 3), (4000, 2, 64)])
def test_prune_gate_keeps_the_first_cap_slots(n, k, e):
    g = _gate(n, k, e)
    flat = g.reshape(-1)
    cap0 = RNG.integers(0, max(2, 2 * n * k // e), size=e).astype(np.int32)
    cap = cap0.copy()
    out = O.prune_gate_by_capacity(g, cap, e)
    assert out.shape == g.shape
    # rank of every slot among the slots of its expert, from a stable sort
    order = np.argsort(flat, kind="stable")
    start = np.concatenate([[0], np.cumsum(np.bincount(flat, minlength=e))])
    rank = np.empty_like(flat)
    rank[order] = np.arange(flat.size) - start[flat[order]]
    want = np.where(rank < cap0[flat], flat, -1)
    assert np.array_equal(out.reshape(-1), want)
    kept = np.bincount(want[want >= 0], minlength=e)
    assert np.array_equal(kept, np.minimum(np.bincount(flat, minlength=e), cap0))
    assert np.array_equal(cap, cap0 - np.bincount(flat, minlength=e))


def test_prune_gate_passes_dropped_slots_through():
    g = np.array([0, -1, 0, 1, -1, 0], np.int64)
    cap = np.array([2, 5], np.int32)
    out = O.prune_gate_by_capacity(g, cap, 2)
    assert out.tolist() == [0, -1, 0, 1, -1, -1]
    assert cap.tolist() == [-1, 4]


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16])
def test_scatter_gather_are_fancy_indexing(dtype):
    x = RNG.standard_normal((12, 6)).astype(dtype)
    g = _gate(12, 2, 4, 0.25)
    pos, _c, _s, _i = O.route(g, 4)
    buf = O.local_scatter(x, pos, 2)
    assert np.array_equal(buf, x[pos // 2])
    back = O.local_gather(buf, pos, 24)
    want = np.zeros((24, 6), dtype)
    want[pos] = buf
    assert np.array_equal(back, want)
    summed = O.local_gather_add(buf.astype(np.float64), pos // 2, 12)
    want2 = np.zeros((12, 6))
    np.add.at(want2, pos // 2, buf.astype(np.float64))
    assert np.allclose(summed, want2, rtol=0, atol=1e-12)


def test_combine_is_einsum():
    s = RNG.standard_normal((9, 3))
    o = RNG.standard_normal((27, 5))
    assert np.allclose(O.combine(s, o), np.einsum("tk,tkd->td", s, o.reshape(9, 3, 5)),
                       rtol=0, atol=1e-12)


def _segments(cnt):
    off = np.concatenate([[0], np.cumsum(cnt)])
    return [(int(off[i]), int(off[i + 1])) for i in range(len(cnt))]


@pytest.mark.parametrize("cnt", [[5], [3, 0, 4, 1], [0, 0, 6], [2, 2, 2, 2, 0]])
def test_linear_forward_backward_match_torch_autograd(cnt):
    e, in_f, out_f = len(cnt), 7, 5
    n = sum(cnt)
    x = torch.tensor(RNG.standard_normal((n, in_f)), requires_grad=True)
    w = torch.tensor(RNG.standard_normal((e, out_f, in_f)), requires_grad=True)
    b = torch.tensor(RNG.standard_normal((e, out_f)), requires_grad=True)
    dy = torch.tensor(RNG.standard_normal((n, out_f)))
    ys = [F.linear(x[a:z], w[i], b[i]) for i, (a, z) in enumerate(_segments(cnt))]
    y = torch.cat(ys, 0)
    y.backward(dy)
    got_y = O.linear_forward(x.detach().numpy(), w.detach().numpy(), b.detach().numpy(), cnt)
    assert np.allclose(got_y, y.detach().numpy(), rtol=0, atol=1e-12)
    no_bias = O.linear_forward(x.detach().numpy(), w.detach().numpy(), None, cnt)
    want_nb = torch.cat([F.linear(x[a:z], w[i]) for i, (a, z) in enumerate(_segments(cnt))], 0)
    assert np.allclose(no_bias, want_nb.detach().numpy(), rtol=0, atol=1e-12)
    dx, dw, db = O.linear_backward(dy.numpy(), x.detach().numpy(), w.detach().numpy(), cnt)
    assert np.allclose(dx, x.grad.numpy(), rtol=0, atol=1e-12)
    assert np.allclose(dw, w.grad.numpy(), rtol=0, atol=1e-12)
    assert np.allclose(db, b.grad.numpy(), rtol=0, atol=1e-12)
    for i, c in enumerate(cnt):  # empty experts get exact zeros
        if c == 0:
            assert not dw[i].any() and not db[i].any()


def test_one_expert_reduces_to_nn_linear():
    lin = torch.nn.Linear(6, 4).double()
    x = torch.tensor(RNG.standard_normal((10, 6)))
    got = O.linear_forward(x.numpy(), lin.weight.detach().numpy()[None],
                           lin.bias.detach().numpy()[None], [10])
    assert np.allclose(got, lin(x).detach().numpy(), rtol=0, atol=1e-12)


def _per_token_brute_force(x, idx, score, w1, b1, w2, b2):
    """Row-by-row evaluation, the semantics of tests/moe.py:64-75."""
    out = torch.zeros(x.shape[0], w2.shape[1], dtype=x.dtype)
    for t in range(x.shape[0]):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            if e < 0:
                continue
            h = F.gelu(w1[e] @ x[t] + b1[e])
            out[t] += score[t, j] * (w2[e] @ h + b2[e])
    return out


def test_brute_force_layer_matches_per_token_loop_and_k1_mlp():
    torch.manual_seed(3)
    t, d, h, e, k = 9, 6, 10, 4, 2
    x = torch.randn(t, d, dtype=torch.float64)
    w1, b1 = torch.randn(e, h, d, dtype=torch.float64), torch.randn(e, h, dtype=torch.float64)
    w2, b2 = torch.randn(e, d, h, dtype=torch.float64), torch.randn(e, d, dtype=torch.float64)
    idx = torch.tensor(_gate(t, k, e, 0.2))
    score = torch.rand(t, k, dtype=torch.float64)
    got = O.brute_force_moe_mlp(x, idx, score, w1, b1, w2, b2)
    want = _per_token_brute_force(x, idx, score, w1, b1, w2, b2)
    assert torch.allclose(got, want, rtol=0, atol=1e-12)
    # k = 1 with weight 1 is a plain per-expert MLP
    idx1 = torch.tensor(_gate(t, 1, e))
    got1 = O.brute_force_moe_mlp(x, idx1, torch.ones(t, 1, dtype=torch.float64),
                                 w1, b1, w2, b2)
    for r in range(t):
        ee = int(idx1[r, 0])
        ref = w2[ee] @ F.gelu(w1[ee] @ x[r] + b1[ee]) + b2[ee]
        assert torch.allclose(got1[r], ref, rtol=0, atol=1e-12)
    # and it is differentiable
    x.requires_grad_(True)
    O.brute_force_moe_mlp(x, idx, score, w1, b1, w2, b2).sum().backward()
    assert x.grad is not None and torch.isfinite(x.grad).all()


def test_topk_softmax_against_torch_and_ties():
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(5)
    logits = rng.standard_normal((37, 11))
    idx, score = O.topk_softmax(logits, 3)
    val, tidx = torch.topk(torch.from_numpy(logits), 3, dim=-1, largest=True, sorted=True)
    assert (idx == tidx.numpy()).all()                    # no ties in random data
    np.testing.assert_allclose(score, F.softmax(val, dim=-1).numpy(), rtol=1e-12)
    # ties go to the lower index, -inf entries are never preferred to finite ones
    tied = np.array([[1.0, 3.0, 3.0, -np.inf, 3.0], [0.0, 0.0, 0.0, 0.0, 0.0]])
    idx, score = O.topk_softmax(tied, 2)
    assert idx.tolist() == [[1, 2], [0, 1]]
    np.testing.assert_allclose(score, [[0.5, 0.5], [0.5, 0.5]])
    # backward against autograd of the torch formulation
    lt = torch.from_numpy(logits).requires_grad_(True)
    v, i = torch.topk(lt, 3, dim=-1)
    sc = F.softmax(v, dim=-1)
    g = torch.from_numpy(rng.standard_normal((37, 3)))
    sc.backward(g)
    got = O.topk_softmax_backward(g.numpy(), sc.detach().numpy(), i.numpy(), 11)
    np.testing.assert_allclose(got, lt.grad.numpy(), rtol=1e-10, atol=1e-14)


def test_gelu_against_torch_and_identities():
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(11)
    x = np.concatenate([rng.standard_normal(500) * 3, [0.0, -0.0, 1e-30, -40.0, 40.0, -8.5]])
    want = F.gelu(torch.from_numpy(x)).numpy()                 # library routine, float64
    # (torch evaluates 1 + erf, which cancels in the negative tail: absolute there)
    np.testing.assert_allclose(O.gelu(x), want, rtol=1e-12, atol=2e-15)
    # x Phi(x) - (-x) Phi(-x) = x (Phi(x) + Phi(-x)) = x
    np.testing.assert_allclose(O.gelu(x) - O.gelu(-x), x, rtol=1e-12, atol=1e-15)
    # the negative tail keeps its digits: x Phi(x) with Phi(-8.5) = 9.48e-18 from libm
    import math
    phi = 0.5 * math.erfc(8.5 / math.sqrt(2.0))
    assert 9.47e-18 < phi < 9.49e-18
    assert abs(O.gelu(np.array([-8.5]))[0] / (-8.5 * phi) - 1) < 1e-12
    # backward: autograd of the library routine, and gelu'(x) + gelu'(-x) = 1
    xt = torch.from_numpy(x).requires_grad_(True)
    g = rng.standard_normal(x.size)
    F.gelu(xt).backward(torch.from_numpy(g))
    np.testing.assert_allclose(O.gelu_backward(g, x), xt.grad.numpy(), rtol=1e-11, atol=1e-14)
    one = np.ones_like(x)
    np.testing.assert_allclose(O.gelu_backward(one, x) + O.gelu_backward(one, -x), one,
                               rtol=1e-12)
    assert O.gelu_backward(np.array([1.0]), np.array([0.0]))[0] == 0.5
