"""Row-moving kernels against the CPU checker: copies bit-exact, weighted sums
within the dtype's tolerance."""
import numpy as np
import pytest
import torch

from helpers import DTYPES, TOL, make_gate, max_rel_err, randn
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

SHAPES = [  # n_tokens, top_k, n_expert, d, drop
    (12, 2, 4, 6, 0.3),       # the reference's own scatter test shape (d = 6)
    (12, 1, 1, 6, 0.0),
    (5, 3, 4, 16, 0.0),
    (100, 2, 8, 64, 0.2),
    (257, 2, 8, 1000, 0.1),   # rows of 2000 B: 16-byte packs with a tail loop
    (64, 8, 16, 2048, 0.0),
    (33, 2, 4, 4096 + 8, 0.5),
]


def _np_dtype(dt):
    return {torch.float32: np.float32, torch.float64: np.float64,
            torch.float16: np.float16}.get(dt)


def _bits(t):
    """Raw bits as integers, so bf16 can be compared exactly through numpy."""
    view = {2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()]
    return t.contiguous().view(view).cpu().numpy()


@pytest.mark.parametrize("dt", ["f32", "f64", "f16", "bf16"])
@pytest.mark.parametrize("n,k,e,d,drop", SHAPES)
def test_scatter_and_gather_are_exact_copies(dt, n, k, e, d, drop):
    from fastmoe_amd import fmoe_cuda

    dtype = DTYPES[dt]
    g = make_gate(n, k, e, drop, seed=n + d)
    pos, _count, seg_off, inv = O.route(g, e)
    x = randn((n, d), dtype, seed=1)
    xb = _bits(x)
    pos_c = torch.from_numpy(pos).cuda()
    buf = fmoe_cuda.local_scatter(x.cuda(), pos_c, k)
    want = O.local_scatter(xb, pos, k)
    assert np.array_equal(_bits(buf), want)
    # the reference passes pos // k itself (fmoe/layers.py:49-53)
    buf2 = fmoe_cuda.local_scatter(x.cuda(), pos_c // k)
    assert np.array_equal(_bits(buf2), want)
    # rows beyond the device-side live count are left alone
    live = torch.tensor([max(pos.size - 3, 0)], dtype=torch.int32, device="cuda")
    full = torch.full((pos.size, d), 7, dtype=dtype, device="cuda")
    part = fmoe_cuda.local_scatter(x.cuda(), pos_c, k, n_rows_dev=live)
    assert np.array_equal(_bits(part)[: int(live.item())], want[: int(live.item())])
    del full
    back = fmoe_cuda.local_gather(buf, pos_c, n * k, maybe_overlap=False)
    assert np.array_equal(_bits(back), O.local_gather(want, pos, n * k))
    # the same rows written in token order from the inverse map
    buf3 = fmoe_cuda.scatter_tokens(x.cuda(), torch.from_numpy(inv.astype(np.int32)).cuda(), k)
    assert np.array_equal(_bits(buf3)[: pos.size], want)


@pytest.mark.parametrize("dt", ["f32", "f64", "bf16"])
def test_gather_with_overlap_sums_rows(dt):
    from fastmoe_amd import fmoe_cuda

    dtype = DTYPES[dt]
    n, k, e, d = 50, 3, 4, 24
    g = make_gate(n, k, e, 0.2, seed=9)
    pos, *_ = O.route(g, e)
    rows = randn((pos.size, d), dtype, seed=2)
    got = fmoe_cuda.local_gather(rows.cuda(), torch.from_numpy(pos // k).cuda(), n, True)
    want = torch.from_numpy(O.local_gather_add(rows.double().numpy(), pos // k, n))
    assert max_rel_err(got, want) <= TOL[dtype]


@pytest.mark.parametrize("dt", ["f32", "f64", "f16", "bf16"])
@pytest.mark.parametrize("n,k,e,d,drop", SHAPES)
def test_gather_combine_forward_backward(dt, n, k, e, d, drop):
    from fastmoe_amd import fmoe_cuda

    dtype = DTYPES[dt]
    g = make_gate(n, k, e, drop, seed=n * 3 + d)
    pos, _count, seg_off, inv = O.route(g, e)
    nv = pos.size
    buf = randn((n * k, d), dtype, seed=3)       # rows beyond nv are dead
    score = randn((n, k), dtype, seed=4).abs()
    dy = randn((n, d), dtype, seed=5)
    inv_c = torch.from_numpy(inv).cuda()

    # forward: gather into slot order (zeros where dropped), then weight and sum
    slots = O.local_gather(buf.double().numpy()[:nv], pos, n * k)
    want_y = torch.from_numpy(O.combine(score.double().numpy(), slots))
    y = fmoe_cuda.gather_combine_fwd(buf.cuda(), inv_c, score.cuda(), n, k)
    assert y.dtype == dtype and max_rel_err(y, want_y) <= TOL[dtype]

    # backward of the same composition by autograd on the CPU, in float64
    b64 = buf.double().clone().requires_grad_(True)
    s64 = score.double().clone().requires_grad_(True)
    idx = torch.from_numpy(inv.astype(np.int64))
    live = (idx >= 0).unsqueeze(1)
    rows = b64[idx.clamp(min=0)] * live
    yy = torch.bmm(s64.view(n, 1, k), rows.view(n, k, d)).view(n, d)
    yy.backward(dy.double())
    dbuf, dscore = fmoe_cuda.gather_combine_bwd(dy.cuda(), buf.cuda(), inv_c,
                                                score.cuda(), n, k)
    assert max_rel_err(dbuf[:nv], b64.grad[:nv]) <= TOL[dtype]
    assert max_rel_err(dscore, s64.grad) <= TOL[dtype]
    dropped = torch.from_numpy(inv < 0).view(n, k)
    assert (dscore.cpu()[dropped] == 0).all()

    # scatter backward: a token's k rows summed in slot order
    dbuf_in = randn((n * k, d), dtype, seed=6)
    want_dx = (dbuf_in.double()[idx.clamp(min=0)] * live).view(n, k, d).sum(1)
    dx = fmoe_cuda.scatter_reduce(dbuf_in.cuda(), inv_c, n, k)
    assert max_rel_err(dx, want_dx) <= TOL[dtype]


def test_full_size_round_trip_and_linearity():
    """Config-5-sized dispatch (8192 tokens, top-8, d = 2048, bf16) through
    size-independent properties: scatter then gather restores every live slot,
    the combine is linear in the scores, and all-ones scores give the row sum."""
    from fastmoe_amd import fmoe_cuda

    n, k, e, d = 8192, 8, 128, 2048
    g = torch.from_numpy(make_gate(n, k, e, 0.05, seed=11, empty=range(0, 128, 10))).cuda()
    pos, count, seg, inv = fmoe_cuda.route(g, e)
    nv = int(seg[-1].item())
    assert nv == int((g >= 0).sum().item())
    p = pos[:nv]
    assert torch.equal(torch.sort(p).values, torch.nonzero(g.view(-1) >= 0).view(-1))
    assert bool((g.view(-1)[p][1:] >= g.view(-1)[p][:-1]).all())      # grouped by expert
    x = torch.randn(n, d, device="cuda", dtype=torch.bfloat16)
    buf = fmoe_cuda.local_scatter(x, pos, k, seg[-1:])
    assert torch.equal(buf[:nv], x[p // k])
    back = fmoe_cuda.local_gather(buf[:nv].contiguous(), p, n * k, False)
    want = x.repeat_interleave(k, 0) * (g.view(-1, 1) >= 0)
    assert torch.equal(back, want)
    ones = torch.ones(n, k, device="cuda", dtype=torch.bfloat16)
    y1 = fmoe_cuda.gather_combine_fwd(buf, inv, ones, n, k).float()
    ref = (x.float() * (g >= 0).sum(1, keepdim=True))
    assert (y1 - ref).abs().max().item() <= 2e-2 * ref.abs().max().item()
    y2 = fmoe_cuda.gather_combine_fwd(buf, inv, 2 * ones, n, k).float()
    assert (y2 - 2 * y1).abs().max().item() <= 2e-2 * ref.abs().max().item()
