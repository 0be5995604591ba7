"""Grouped expert GEMMs (forward, input/weight/bias gradients) against the CPU
checker, for every dtype and both kernel families."""
import numpy as np
import pytest
import torch

from helpers import DTYPES, TOL, max_rel_err, randn
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

# counts per expert, in_feat, out_feat
SHAPES = [
    ([4], 16, 32),
    ([3, 0, 4, 1], 16, 32),                 # reference test shape, one empty expert
    ([0, 0, 6], 7, 5),                      # odd sizes: scalar kernel only
    ([5, 9, 2, 0, 0, 17, 1, 3], 24, 40),
    ([130, 0, 1, 255, 64], 64, 72),         # partial tiles in M, N and K
    ([100, 300, 7], 136, 264),              # K and N beyond one tile
    ([0, 513, 0, 11], 256, 128),
]


def _run(counts, in_f, out_f, dtype, with_bias, path, extra_rows=0):
    from fastmoe_amd import fmoe_cuda

    e, n = len(counts), sum(counts)
    x = randn((n + extra_rows, in_f), dtype, 1)
    w = randn((e, out_f, in_f), dtype, 2, 0.3)
    b = randn((e, out_f), dtype, 3) if with_bias else None
    dy = randn((n + extra_rows, out_f), dtype, 4)
    cnt = torch.tensor(counts, dtype=torch.int64)
    fmoe_cuda.set_gemm_path(path)
    try:
        y = fmoe_cuda.linear_forward(x.cuda(), cnt, w.cuda(), None if b is None else b.cuda())
        dx, dw, db = fmoe_cuda.linear_backward(dy.cuda(), x.cuda(), cnt, w.cuda(),
                                               None if b is None else b.cuda())
        torch.cuda.synchronize()
    finally:
        fmoe_cuda.set_gemm_path(0)
    xn, wn, dyn = x.double().numpy(), w.double().numpy(), dy.double().numpy()
    bn = None if b is None else b.double().numpy()
    want_y = O.linear_forward(xn[:n], wn, bn, counts)
    want_dx, want_dw, want_db = O.linear_backward(dyn[:n], xn[:n], wn, counts)
    tol = TOL[dtype]
    assert y.shape == (n + extra_rows, out_f) and y.dtype == dtype
    assert max_rel_err(y[:n], torch.from_numpy(want_y)) <= tol
    assert max_rel_err(dx[:n], torch.from_numpy(want_dx)) <= tol
    assert dw.shape == (e, out_f, in_f)
    assert max_rel_err(dw, torch.from_numpy(want_dw)) <= tol
    assert max_rel_err(db, torch.from_numpy(want_db)) <= tol
    for i, c in enumerate(counts):   # exact zeros for experts without rows
        if c == 0:
            assert not dw[i].any().item() and not db[i].any().item()


@pytest.mark.parametrize("dt", ["f32", "f64", "f16", "bf16"])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("counts,in_f,out_f", SHAPES)
def test_scalar_kernel(dt, with_bias, counts, in_f, out_f):
    _run(counts, in_f, out_f, DTYPES[dt], with_bias, path=1)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("counts,in_f,out_f", SHAPES)
def test_matrix_core_kernel(dt, with_bias, counts, in_f, out_f):
    _run(counts, in_f, out_f, DTYPES[dt], with_bias, path=0)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
def test_matrix_core_large_tiles_and_dead_rows(dt):
    # a mid-size problem with the tile shape left to the library; 37 rows past
    # seg_off[E] are dead and must not be read as part of any expert
    _run([1000, 0, 1531, 800], 512, 1024, DTYPES[dt], True, path=0, extra_rows=37)


# every tile configuration of the matrix-core kernel, forced, on shapes with
# partial tiles in M, N and K, remainders of every length class (none, up to 64,
# up to 128, above half a tile), empty experts and dead rows at the end
FORCED = [
    ([300, 0, 257, 64, 1, 200, 513], 136, 264),
    ([1024 + 17, 1024 - 9, 0, 130], 72, 520),
    ([255, 129, 128, 65, 63], 264, 256),
    ([520, 260, 0, 256], 352, 384),         # last column tile exactly / under half a tile
]


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("tile", [1, 2, 3, 4])
@pytest.mark.parametrize("counts,in_f,out_f", FORCED)
def test_matrix_core_forced_tile(dt, tile, counts, in_f, out_f):
    _run(counts, in_f, out_f, DTYPES[dt], True, path=1 + tile, extra_rows=5)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
def test_matrix_core_narrow_remainder_tiles(dt):
    """With K >= 2048 and few remainder tiles in the launch, the remainders (1, 44, 64
    and 100 rows here, behind 0 to 2 full tiles) run as 64-column (forward) and
    128-column (dX) tiles; feature sizes that end inside such a tile, K with a tail."""
    _run([300, 0, 257, 64, 1, 200, 513, 356], 2056, 2112, DTYPES[dt], True, path=0, extra_rows=3)


@pytest.mark.parametrize("dt", ["f32", "f64"])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("counts,in_f,out_f", SHAPES + FORCED)
def test_matrix_core_full_precision(dt, with_bias, counts, in_f, out_f):
    # f32 / f64 on their matrix-core kernel (shapes that are not multiples of 4
    # still take the scalar kernel)
    _run(counts, in_f, out_f, DTYPES[dt], with_bias, path=0, extra_rows=3)


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_matrix_core_full_precision_many_tiles(dt):
    _run([2100, 0, 1500, 4000, 37, 900], 256, 512, DTYPES[dt], True, path=0, extra_rows=9)


@pytest.mark.parametrize("n_expert", [257, 600, 4096])
def test_matrix_core_many_experts(n_expert):
    # more experts than threads in a block: every thread of the tile search owns
    # a run of experts; two thirds of them are empty
    rng = np.random.default_rng(n_expert)
    counts = (rng.integers(0, 30, n_expert) * (rng.random(n_expert) < 0.34)).tolist()
    counts[-1] = 5
    _run(counts, 32, 48, torch.bfloat16, True, path=0, extra_rows=3)


def test_device_side_counts_and_seg_off_upload():
    from fastmoe_amd import fmoe_cuda

    counts = [3, 0, 4, 1]
    cnt = torch.tensor(counts, dtype=torch.int64)
    seg_h = fmoe_cuda._seg_off_from_counts(cnt, torch.device("cuda"))
    seg_d = fmoe_cuda._seg_off_from_counts(cnt.cuda(), torch.device("cuda"))
    assert seg_h.cpu().tolist() == seg_d.cpu().tolist() == [0, 3, 3, 7, 8]
    big = torch.arange(1300, dtype=torch.int64) % 5          # more than one upload chunk
    seg = fmoe_cuda._seg_off_from_counts(big, torch.device("cuda"))
    assert seg.cpu().tolist() == [0] + torch.cumsum(big, 0).tolist()


def test_errors_are_runtime_errors():
    from fastmoe_amd import fmoe_cuda

    x = torch.zeros(4, 8, device="cuda")
    w = torch.zeros(2, 8, 8, device="cuda")
    with pytest.raises(RuntimeError):
        fmoe_cuda.linear_forward(x, torch.tensor([2, 2]), w.half(), None)   # dtype clash
    with pytest.raises(RuntimeError):
        fmoe_cuda.linear_forward(x.cpu(), torch.tensor([2, 2]), w, None)    # host tensor
    with pytest.raises(RuntimeError):
        fmoe_cuda.expert_count(torch.zeros(4, device="cuda"),               # wrong dtype
                               torch.zeros(2, dtype=torch.int32, device="cuda"))


@pytest.mark.parametrize("cfg", ["cfg2", "cfg4", "cfg5"])
def test_full_size_gemm_properties(cfg):
    """Full-size grouped GEMMs (the balanced, the largest and the fine-grained workload)
    checked through properties that do not need a CPU evaluation: agreement with fp32 matmul of sampled rows, exact zeros
    for empty experts, and linearity in the input."""
    from fastmoe_amd import fmoe_cuda

    if cfg == "cfg2":
        e, d, h, n = 16, 1024, 4096, 16384
        counts = torch.full((e,), n // e, dtype=torch.int64)
    elif cfg == "cfg4":
        e, d, h, n = 8, 4096, 14336, 32768
        g = torch.Generator().manual_seed(4)
        counts = torch.bincount(torch.randint(0, e, (n,), generator=g), minlength=e)
    else:
        e, d, h, n = 128, 2048, 1408, 65536
        g = torch.Generator().manual_seed(0)
        raw = torch.rand(e, generator=g)
        raw[::10] = 0                                     # 13 empty experts
        counts = torch.floor(raw / raw.sum() * n).long()
        counts[1] += n - counts.sum()
    dt = torch.bfloat16
    x = torch.randn(n, d, device="cuda", dtype=dt)
    w = (torch.randn(e, h, d, device="cuda") * 0.02).to(dt)
    b = (torch.randn(e, h, device="cuda") * 0.02).to(dt)
    y = fmoe_cuda.linear_forward(x, counts, w, b)
    off = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(counts, 0)])
    rng = np.random.default_rng(0)
    for ex in rng.choice(np.flatnonzero(counts.numpy() > 0), 6, replace=False):
        a, z = int(off[ex]), int(off[ex + 1])
        rows = torch.from_numpy(rng.integers(a, z, size=min(64, z - a))).cuda()
        ref = x[rows].float() @ w[ex].float().t() + b[ex].float()
        assert max_rel_err(y[rows], ref) <= 2e-2
    y2 = fmoe_cuda.linear_forward(x * 2, counts, w, None)
    y1 = fmoe_cuda.linear_forward(x, counts, w, None)
    assert max_rel_err(y2, 2 * y1.float()) <= 2e-2
    dy = torch.randn(n, h, device="cuda", dtype=dt)
    dx, dw, db = fmoe_cuda.linear_backward(dy, x, counts, w, b)
    for ex in rng.choice(np.flatnonzero(counts.numpy() > 0), 3, replace=False):
        a, z = int(off[ex]), int(off[ex + 1])
        ref_dw = dy[a:z].float().t() @ x[a:z].float()
        assert max_rel_err(dw[ex], ref_dw) <= 2e-2
        assert max_rel_err(db[ex], dy[a:z].float().sum(0)) <= 2e-2
        rows = torch.from_numpy(rng.integers(a, z, size=min(64, z - a))).cuda()
        assert max_rel_err(dx[rows], dy[rows].float() @ w[ex].float()) <= 2e-2
    for ex in np.flatnonzero(counts.numpy() == 0):
        assert not dw[ex].any().item() and not db[ex].any().item()


@pytest.mark.parametrize("seed", range(24))
def test_random_ragged_shapes_against_torch(seed):
    """Random expert counts, row counts (empty experts included) and feature
    sizes through the automatic kernel choice, against per-expert float32
    matmuls of the same rounded operands on the GPU."""
    from fastmoe_amd import fmoe_cuda

    rng = np.random.default_rng(1000 + seed)
    dt = [torch.bfloat16, torch.float16, torch.float32][seed % 3]
    step = 4 if dt == torch.float32 else 8
    e = int(rng.integers(1, 40))
    in_f = int(rng.integers(1, 90)) * step
    out_f = int(rng.integers(1, 90)) * step
    if seed % 4 == 0:                      # a last column tile at most half full
        out_f = 256 * int(rng.integers(1, 4)) + step * int(rng.integers(1, 16))
    counts = rng.integers(0, 700, e) * (rng.random(e) < 0.8)
    if seed % 5 == 0:
        counts[rng.integers(0, e)] += 2048     # one expert with many full tiles
    counts = torch.from_numpy(counts.astype(np.int64))
    n = int(counts.sum())
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n + 2, in_f, generator=g).to(dt).cuda()
    w = (torch.randn(e, out_f, in_f, generator=g) * 0.2).to(dt).cuda()
    b = torch.randn(e, out_f, generator=g).to(dt).cuda()
    dy = torch.randn(n + 2, out_f, generator=g).to(dt).cuda()
    y = fmoe_cuda.linear_forward(x, counts, w, b)
    dx, dw, db = fmoe_cuda.linear_backward(dy, x, counts, w, b)
    tol = 2e-2 if dt == torch.bfloat16 else (4e-3 if dt == torch.float16 else 1e-4)
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        off = 0
        for ex in range(e):
            c = int(counts[ex])
            xs, ds, wf = x[off:off + c].float(), dy[off:off + c].float(), w[ex].float()
            if c:
                assert max_rel_err(y[off:off + c], xs @ wf.t() + b[ex].float()) <= tol
                assert max_rel_err(dx[off:off + c], ds @ wf) <= tol
            assert max_rel_err(dw[ex], ds.t() @ xs) <= tol
            assert max_rel_err(db[ex], ds.sum(0)) <= tol
            off += c
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
