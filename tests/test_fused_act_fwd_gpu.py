"""The forward of `gelu(linear(x))` with the activation applied by the grouped GEMM's
own output tiles (fmoe_grouped_linear_fwd_act) against the two separate steps it
replaces: the same bits in both results, on every kernel path, for every 16-bit
value of the linear layer's output."""
import numpy as np
import pytest
import torch

from helpers import DTYPES, randn
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _seg(counts):
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    return torch.from_numpy(off).cuda()


def _bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else
                               (torch.int32 if t.element_size() == 4 else torch.int64))


SHAPES = [  # rows per expert, in_feat, out_feat
    ([300, 0, 129, 64, 1, 0, 513], 256, 128),     # ragged, empty experts, all tile heights
    ([1024, 1024], 512, 256),                     # full 256-row tiles only
    ([7, 250], 136, 72),                          # widths that are no multiple of a tile
    ([0, 0, 0], 64, 64),                          # no rows at all
    ([700], 1024, 64),
    ([300, 0, 129, 64, 1, 0, 513, 356], 2048, 264),   # K = 2048: narrow remainder tiles
    ([900, 800, 1000], 64, 136),                  # enough rows per expert for the automatic choice
]


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("with_bias", [True, False])
@pytest.mark.parametrize("counts,in_f,out_f", SHAPES)
def test_same_bits_as_linear_forward_then_gelu(dt, with_bias, counts, in_f, out_f):
    from fastmoe_amd import fmoe_cuda

    dtype = DTYPES[dt]
    n, e = int(sum(counts)), len(counts)
    seg = _seg(counts)
    x = randn((n + 3, in_f), dtype, 1, 1.0).cuda()          # 3 rows behind the last segment
    w = randn((e, out_f, in_f), dtype, 2, 0.08).cuda()
    b = randn((e, out_f), dtype, 3, 1.0).cuda() if with_bias else None
    for path in (0, 2, 3, 4, 5, 1):                          # automatic, the four tile shapes, scalar
        fmoe_cuda.set_gemm_path(path)
        try:
            y0 = fmoe_cuda.grouped_linear_fwd(x, seg, w, b)
            y1, a1 = fmoe_cuda.grouped_linear_fwd(x, seg, w, b, with_gelu=True)
        finally:
            fmoe_cuda.set_gemm_path(0)
        assert y1.shape == a1.shape == (n + 3, out_f) and a1.dtype == dtype
        if n == 0:
            continue
        a0 = fmoe_cuda.gelu_fwd(y0[:n].contiguous())
        assert torch.equal(_bits(y0[:n]), _bits(y1[:n])), path
        assert torch.equal(_bits(a0), _bits(a1[:n])), path
    if n:
        # and against the float64 checker: gelu of the rounded linear output
        ref = O.gelu(y1[:n].double().cpu().numpy())
        err = np.abs(a1[:n].double().cpu().numpy() - ref).max()
        tol = {"bf16": 2.0 ** -8, "f16": 2.0 ** -11, "f32": 2e-6}[dt]
        assert err <= tol * max(np.abs(ref).max(), 1.0)


def test_every_bf16_value_through_the_output_tiles():
    """All 65536 bf16 patterns as outputs of the linear layer (an identity weight):
    zeros, denormals, the range the in-kernel table covers, the ranges either side of
    it, infinities, NaNs; on every tile shape."""
    from fastmoe_amd import fmoe_cuda

    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16).reshape(256, 256).cuda()
    w = torch.eye(256, dtype=torch.bfloat16).reshape(1, 256, 256).cuda()
    seg = _seg([256])
    for path in (2, 3, 4, 5):
        fmoe_cuda.set_gemm_path(path)
        try:
            y, a = fmoe_cuda.grouped_linear_fwd(x, seg, w, None, with_gelu=True)
        finally:
            fmoe_cuda.set_gemm_path(0)
        # y = x * 1 + zeros: the patterns come through, but for -0 (+0 after the sum),
        # denormals (flushed by the matrix cores) and the rows an inf or NaN spoils
        clean = torch.isfinite(x).all(dim=1)
        assert (_bits(y)[clean] == _bits(x)[clean]).float().mean().item() > 0.98
        assert torch.equal(_bits(a), _bits(fmoe_cuda.gelu_fwd(y)))
    # only values the in-kernel table covers (2^-28 <= |x| < 16, both signs, its two
    # ends included): no lane leaves the table in LDS
    inside = torch.cat([torch.arange(0x3180, 0x4180), torch.arange(0xB180, 0xC180)])
    xin = inside.repeat(8).to(torch.int32).to(torch.int16).view(torch.bfloat16)
    xin = xin[torch.randperm(65536, generator=torch.Generator().manual_seed(5))]
    xin = xin.reshape(256, 256).cuda()
    fmoe_cuda.set_gemm_path(5)
    try:
        y, a = fmoe_cuda.grouped_linear_fwd(xin, seg, w, None, with_gelu=True)
    finally:
        fmoe_cuda.set_gemm_path(0)
    assert torch.equal(_bits(y), _bits(xin))
    assert torch.equal(_bits(a), _bits(fmoe_cuda.gelu_fwd(xin)))


@pytest.mark.parametrize("dt", ["bf16", "f32"])
def test_expert_module_runs_no_activation_kernel_of_its_own(dt):
    """_Expert with torch.nn.GELU(): forward and backward make no gelu_fwd / gelu_bwd
    call through the operator module (one entry point per direction covers the
    activation), and outputs and gradients are those of the two linear nodes with the
    activation node between them."""
    from fastmoe_amd import fmoe_cuda
    from fastmoe_amd.functions import apply_activation
    from fastmoe_amd.linear import MOELinear
    from fastmoe_amd.transformer import _Expert

    dtype = DTYPES[dt]
    torch.manual_seed(7)
    ex = _Expert(3, 64, 128, torch.nn.GELU()).cuda().to(dtype)
    ex.htoh4.bias.data.normal_()
    ex.h4toh.bias.data.normal_()
    counts = torch.tensor([70, 0, 130])
    x = randn((200, 64), dtype, 9).cuda()
    dy = randn((200, 64), dtype, 10).cuda()

    def run(fn):
        xi = x.clone().requires_grad_(True)
        for p in ex.parameters():
            p.grad = None
        y = fn(xi)
        y.backward(dy)
        return [y.detach(), xi.grad] + [p.grad.clone() for p in ex.parameters()]

    from fastmoe_amd.linear import MOELinearGelu

    seen, act_grads = [], []
    inner = MOELinearGelu.backward

    def spy(ctx, grad_pre, grad_act):
        act_grads.append(grad_act)
        return inner(ctx, grad_pre, grad_act)

    fmoe_cuda.profile_hook = lambda name, a, b: seen.append(name)
    MOELinearGelu.backward = staticmethod(spy)
    try:
        got = run(lambda xi: ex(xi, counts))
    finally:
        fmoe_cuda.profile_hook = None
        MOELinearGelu.backward = staticmethod(inner)
    assert "gelu_fwd" not in seen and "gelu_bwd" not in seen
    # no zero tensor of the activation's size is made for the output that carries no gradient
    assert act_grads == [None]
    assert seen.count("grouped_linear_fwd_act") == 1 and seen.count("grouped_linear_fwd") == 1
    assert seen.count("grouped_linear_bwd") == 2

    def separate(xi):
        h = MOELinear.apply(xi, counts, ex.htoh4.weight, ex.htoh4.bias)
        h = apply_activation(ex.activation, h)
        return MOELinear.apply(h, counts, ex.h4toh.weight, ex.h4toh.bias)

    want = run(separate)
    for g, w in zip(got, want):
        assert torch.equal(g, w)


def test_forward_hooks_on_the_linear_modules_still_fire():
    from fastmoe_amd.transformer import _Expert

    ex = _Expert(2, 32, 64, torch.nn.GELU()).cuda().to(torch.bfloat16)
    x = randn((50, 32), torch.bfloat16, 3).cuda()
    counts = torch.tensor([20, 30])
    plain = ex(x, counts)
    calls = []
    h1 = ex.htoh4.register_forward_hook(lambda m, i, o: calls.append("htoh4"))
    h2 = ex.h4toh.register_forward_hook(lambda m, i, o: calls.append("h4toh"))
    try:
        hooked = ex(x, counts)
    finally:
        h1.remove()
        h2.remove()
    assert calls == ["htoh4", "h4toh"] and torch.equal(plain, hooked)


def test_switch_keeps_the_activation_a_kernel_of_its_own():
    """set_gemm_path(6): the same entry point runs the GEMM followed by the activation
    kernel; the same bits as from the fused tiles."""
    from fastmoe_amd import fmoe_cuda

    counts = [1100, 0, 900, 1024, 1, 0, 813]
    seg = torch.from_numpy(np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)).cuda()
    n = sum(counts)
    x = randn((n, 256), torch.bfloat16, 1, 1.0).cuda()
    w = randn((len(counts), 128, 256), torch.bfloat16, 2, 0.08).cuda()
    b = randn((len(counts), 128), torch.bfloat16, 3, 1.0).cuda()
    y, a = fmoe_cuda.grouped_linear_fwd(x, seg, w, b, with_gelu=True)    # fused (>= 768 rows/expert)
    fmoe_cuda.set_gemm_path(6)
    try:
        y2, a2 = fmoe_cuda.grouped_linear_fwd(x, seg, w, b, with_gelu=True)
    finally:
        fmoe_cuda.set_gemm_path(0)
    assert torch.equal(y.view(torch.int16)[:n], y2.view(torch.int16)[:n])
    assert torch.equal(a.view(torch.int16)[:n], a2.view(torch.int16)[:n])
