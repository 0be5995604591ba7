"""GELU kernels (the activation between the two expert layers) against the CPU
checker: every 16-bit pattern for bf16/f16, random data for f32/f64."""
import numpy as np
import pytest
import torch

from helpers import DTYPES
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _all_patterns(dtype):
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    return bits.view(dtype)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_forward_every_16_bit_pattern(dt):
    """gelu of every representable argument is the float64 value correctly
    rounded to the type, and agrees with torch's
    own kernel to the accuracy of that kernel's float32 evaluation."""
    from fastmoe_amd import fmoe_cuda

    dtype = DTYPES[dt]
    x = _all_patterns(dtype)
    y = fmoe_cuda.gelu_fwd(x.cuda()).cpu()
    finite = torch.isfinite(x)
    exact = O.gelu(x[finite].double().numpy())
    got = y[finite]
    # correctly rounded: within half a unit in the last place of the exact value
    # (a tie may go either way: the table rounds through float32)
    mant, min_exp = (7, -126) if dt == "bf16" else (10, -14)
    expo = np.floor(np.log2(np.maximum(np.abs(exact), 2.0 ** min_exp)))
    half_ulp = 2.0 ** (expo - mant - 1)
    assert (np.abs(got.double().numpy() - exact) <= half_ulp * (1 + 1e-9)).all()
    want = torch.from_numpy(exact).float().to(dtype)
    assert (got.view(torch.int16) != want.view(torch.int16)).sum().item() <= 4
    assert torch.isnan(y[torch.isnan(x)]).all()
    # torch evaluates 0.5 x (1 + erf) in float32: one unit in the last place of the
    # type, plus the cancellation of 1 + erf (6e-8) times |x| in the negative tail
    theirs = torch.nn.functional.gelu(x.cuda()).cpu()[finite].double()
    ulp = 2.0 ** -7 if dt == "bf16" else 2.0 ** -10
    slack = ulp * theirs.abs() + 1e-7 * x[finite].double().abs() + 1e-7
    assert ((got.double() - theirs).abs() <= slack).all()


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_backward_every_16_bit_pattern(dt):
    from fastmoe_amd import fmoe_cuda

    dtype = DTYPES[dt]
    x = _all_patterns(dtype)
    x = x[torch.isfinite(x)]
    g = torch.Generator().manual_seed(1)
    dy = torch.randn(x.numel(), generator=g).to(dtype)
    dx = fmoe_cuda.gelu_bwd(dy.cuda(), x.cuda()).cpu()
    want = O.gelu_backward(dy.double().numpy(), x.double().numpy())
    # one rounding of the product of dy and the float32 derivative
    eps = 2.0 ** -8 if dt == "bf16" else 2.0 ** -11
    err = np.abs(dx.double().numpy() - want)
    assert (err <= eps * np.abs(want) * 1.01 + 1e-7).all()


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_full_precision(dt):
    from fastmoe_amd import fmoe_cuda

    dtype = DTYPES[dt]
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(100003, generator=g, dtype=torch.float64) * 3).to(dtype)
    dy = torch.randn(100003, generator=g, dtype=torch.float64).to(dtype)
    tol = 1e-13 if dt == "f64" else 3e-7
    y = fmoe_cuda.gelu_fwd(x.cuda()).cpu()
    assert np.abs(y.double().numpy() - O.gelu(x.double().numpy())).max() <= tol * 12
    dx = fmoe_cuda.gelu_bwd(dy.cuda(), x.cuda()).cpu()
    want = O.gelu_backward(dy.double().numpy(), x.double().numpy())
    assert np.abs(dx.double().numpy() - want).max() <= tol * 12


@pytest.mark.parametrize("n", [0, 1, 7, 8, 9, 4099, 8 * 1024 * 4 * 3 + 5])
def test_sizes_tails_and_unaligned_views(n):
    """The table kernels move 16-byte packs; tails and views that start off a
    16-byte boundary take the element-wise kernels and must agree exactly."""
    from fastmoe_amd import fmoe_cuda

    g = torch.Generator().manual_seed(n)
    base = (torch.randn(n + 3, generator=g) * 2).to(torch.bfloat16).cuda()
    dyb = torch.randn(n + 3, generator=g).to(torch.bfloat16).cuda()
    ref_y = fmoe_cuda.gelu_fwd(base.clone())
    ref_dx = fmoe_cuda.gelu_bwd(dyb.clone(), base.clone())
    for off in (0, 1, 3):
        x = base[off:off + n]
        y = fmoe_cuda.gelu_fwd(x)
        assert torch.equal(y, ref_y[off:off + n])
        dx = fmoe_cuda.gelu_bwd(dyb[off:off + n], x)
        assert torch.equal(dx, ref_dx[off:off + n])


def test_expert_module_uses_the_kernel_only_for_exact_gelu():
    from fastmoe_amd import fmoe_cuda
    from fastmoe_amd.functions import apply_activation

    x = torch.randn(64, 32, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    seen = []
    fmoe_cuda.profile_hook = lambda name, a, b: seen.append(name)
    try:
        y = apply_activation(torch.nn.GELU(), x)
        y.sum().backward()
        apply_activation(torch.nn.GELU(approximate="tanh"), x)
        apply_activation(torch.nn.ReLU(), x)
    finally:
        fmoe_cuda.profile_hook = None
    assert seen == ["gelu_fwd", "gelu_bwd"]
    want = O.gelu_backward(np.ones(x.numel()), x.detach().double().cpu().numpy().ravel())
    assert np.abs(x.grad.double().cpu().numpy().ravel() - want).max() <= 2.0 ** -8 * 1.2


@pytest.mark.parametrize("dt", ["bf16", "f32"])
def test_live_row_hint_skips_dead_rows(dt):
    """With a device-side count of live rows only those rows are computed; the
    rest of the output is left as it was."""
    from fastmoe_amd import fmoe_cuda
    from fastmoe_amd._ctypes_ops import _L, _dt, _lib, _stream

    dtype = DTYPES[dt]
    g = torch.Generator().manual_seed(5)
    x = torch.randn(37, 64, generator=g).to(dtype).cuda()
    dy = torch.randn(37, 64, generator=g).to(dtype).cuda()
    full_y = fmoe_cuda.gelu_fwd(x)
    full_dx = fmoe_cuda.gelu_bwd(dy, x)
    for live in (0, 1, 20, 37, 50):
        n_rows = torch.tensor([live], dtype=torch.int32, device="cuda")
        y = torch.full_like(x, 7.0)
        dx = torch.full_like(x, 7.0)
        _lib.check(_L.fmoe_gelu_fwd(x.data_ptr(), y.data_ptr(), x.numel(), n_rows.data_ptr(), 64,
                                    _dt(x, "x"), _stream(x)), "gelu_fwd")
        _lib.check(_L.fmoe_gelu_bwd(dy.data_ptr(), x.data_ptr(), dx.data_ptr(), x.numel(),
                                    n_rows.data_ptr(), 64, _dt(x, "x"), _stream(x)), "gelu_bwd")
        k = min(live, 37)
        assert torch.equal(y[:k], full_y[:k]) and torch.equal(dx[:k], full_dx[:k])
        assert (y[k:] == 7.0).all() and (dx[k:] == 7.0).all()
    # through the binding the hint rides on the autograd function
    from fastmoe_amd.functions import apply_activation
    xr = x.clone().requires_grad_(True)
    n_rows = torch.tensor([20], dtype=torch.int32, device="cuda")
    out = apply_activation(torch.nn.GELU(), xr, n_rows)
    out[:20].float().sum().backward()
    assert torch.equal(out[:20], full_y[:20])
    ones = torch.ones_like(x)
    assert torch.equal(xr.grad[:20], fmoe_cuda.gelu_bwd(ones, x)[:20])
