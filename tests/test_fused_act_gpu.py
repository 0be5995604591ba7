"""The backward of `linear(gelu(pre))` with gelu' applied inside the grouped
GEMM's epilogue (fmoe_grouped_linear_bwd_act) against the two separate steps it
replaces: the same bits out, on every kernel path, for every 16-bit argument."""
import numpy as np
import pytest
import torch

from helpers import DTYPES, randn
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _seg(counts):
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    return torch.from_numpy(off).cuda()


def _same_bits(a, b):
    """Equal element by element, NaN matching NaN."""
    a, b = a.float(), b.float()
    return bool(((a == b) | (torch.isnan(a) & torch.isnan(b))).all())


def _two_steps(fmoe_cuda, dy, act, seg, w, pre, **kw):
    dx, dw, db = fmoe_cuda.grouped_linear_bwd(dy, act, seg, w, **kw)
    if dx is not None:
        dx = fmoe_cuda.gelu_bwd(dx, pre, seg[-1:])
    return dx, dw, db


SHAPES = [  # rows per expert, in_feat, out_feat
    ([300, 0, 129, 64, 1, 0, 513], 256, 128),     # ragged, empty experts, all tile heights
    ([1024, 1024], 512, 256),                     # full 256-row tiles only
    ([7, 250], 136, 72),                          # widths that are no multiple of a tile
    ([0, 0, 0], 64, 64),                          # no rows at all
    ([700], 1024, 64),
    ([300, 0, 129, 64, 1, 0, 513, 356], 264, 2048),   # K = 2048: narrow remainder tiles of dX
]


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("counts,in_f,out_f", SHAPES)
def test_same_bits_as_linear_backward_then_gelu_backward(dt, counts, in_f, out_f):
    from fastmoe_amd import fmoe_cuda

    dtype = DTYPES[dt]
    n, e = int(sum(counts)), len(counts)
    slack = 5                                   # rows behind the last segment stay untouched
    seg = _seg(counts)
    pre = randn((n + slack, in_f), dtype, 1, 1.5).cuda()
    act = fmoe_cuda.gelu_fwd(pre)
    dy = randn((n + slack, out_f), dtype, 2).cuda()
    w = randn((e, out_f, in_f), dtype, 3, 0.05).cuda()
    want = _two_steps(fmoe_cuda, dy, act, seg, w, pre)
    got = fmoe_cuda.grouped_linear_bwd(dy, act, seg, w, act_pre=pre)
    assert _same_bits(got[0][:n], want[0][:n])
    assert torch.equal(got[1], want[1]) and torch.equal(got[2], want[2])
    # dX alone (the launch without the dW tiles)
    got = fmoe_cuda.grouped_linear_bwd(dy, act, seg, w, need_bias=False, need_dw=False,
                                       act_pre=pre)
    assert _same_bits(got[0][:n], want[0][:n]) and got[1] is None and got[2] is None
    # and against the float64 checker: (dy W) .* gelu'(pre), one rounding of dy W to the
    # storage type before the factor
    if n:
        e_of_row = np.repeat(np.arange(e), counts)
        dh = torch.einsum("no,noi->ni", dy[:n].double().cpu(), w.double().cpu()[e_of_row])
        ref = O.gelu_backward(dh.numpy().ravel(), pre[:n].double().cpu().numpy().ravel())
        err = np.abs(got[0][:n].double().cpu().numpy().ravel() - ref).max()
        tol = {"bf16": 2e-2, "f16": 4e-3, "f32": 2e-5}[dt]
        assert err <= tol * max(np.abs(ref).max(), 1e-30)


@pytest.mark.parametrize("path", [1, 2, 3, 4, 5])
def test_every_forced_kernel_path_agrees(path):
    """Tile configurations 1-4 of the matrix-core kernel (paths 2-5) apply the
    factor in their epilogues; path 1 (no matrix cores) runs the activation kernel."""
    from fastmoe_amd import fmoe_cuda

    counts, in_f, out_f = [300, 0, 129, 64, 1, 0, 513], 384, 128
    n, e = sum(counts), len(counts)
    seg = _seg(counts)
    pre = randn((n, in_f), torch.bfloat16, 4, 2.0).cuda()
    act = fmoe_cuda.gelu_fwd(pre)
    dy = randn((n, out_f), torch.bfloat16, 5).cuda()
    w = randn((e, out_f, in_f), torch.bfloat16, 6, 0.05).cuda()
    fmoe_cuda.set_gemm_path(path)
    try:
        want = _two_steps(fmoe_cuda, dy, act, seg, w, pre)
        got = fmoe_cuda.grouped_linear_bwd(dy, act, seg, w, act_pre=pre)
        alone = fmoe_cuda.grouped_linear_bwd(dy, act, seg, w, need_bias=False, need_dw=False,
                                             act_pre=pre)
    finally:
        fmoe_cuda.set_gemm_path(0)
    assert _same_bits(got[0], want[0]) and _same_bits(alone[0], want[0])
    assert torch.equal(got[1], want[1]) and torch.equal(got[2], want[2])


def test_every_bf16_argument_through_the_epilogue():
    """All 65536 bf16 patterns as pre-activations (zeros, denormals, the range the
    in-kernel table covers, the ranges either side of it, infinities, NaNs), with an
    identity weight so that dY W = dY exactly: the epilogue's factor must be the
    activation kernel's, bit for bit."""
    from fastmoe_amd import fmoe_cuda

    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    pre = bits.view(torch.bfloat16).reshape(256, 256).cuda()
    w = torch.eye(256, dtype=torch.bfloat16).reshape(1, 256, 256).cuda()
    seg = _seg([256])
    act = torch.zeros_like(pre)                   # only feeds dW, which is not asked for
    for seed, scale in ((7, 1.0), (8, 37.0)):
        dy = randn((256, 256), torch.bfloat16, seed, scale).cuda()
        want = fmoe_cuda.gelu_bwd(dy, pre)
        got = fmoe_cuda.grouped_linear_bwd(dy, act, seg, w, need_bias=False, need_dw=False,
                                           act_pre=pre)[0]
        assert _same_bits(got, want)
        got = fmoe_cuda.grouped_linear_bwd(dy, act, seg, w, act_pre=pre)[0]
        assert _same_bits(got, want)
    # only the arguments the in-kernel table covers (2^-28 <= |x| < 16, both signs,
    # each 8 times): every lane stays on the table in LDS, its two ends included
    inside = torch.cat([torch.arange(0x3180, 0x4180), torch.arange(0xB180, 0xC180)])
    pre_in = inside.repeat(8).to(torch.int32).to(torch.int16).view(torch.bfloat16)
    pre_in = pre_in[torch.randperm(65536, generator=torch.Generator().manual_seed(3))]
    pre_in = pre_in.reshape(256, 256).cuda()
    dy = randn((256, 256), torch.bfloat16, 11, 3.0).cuda()
    want = fmoe_cuda.gelu_bwd(dy, pre_in)
    got = fmoe_cuda.grouped_linear_bwd(dy, act, seg, w, need_bias=False, need_dw=False,
                                       act_pre=pre_in)[0]
    assert torch.equal(got, want)
    # dy = 1: the factor itself, against the float64 derivative
    ones = torch.ones(256, 256, dtype=torch.bfloat16).cuda()
    got = fmoe_cuda.grouped_linear_bwd(ones, act, seg, w, need_bias=False, need_dw=False,
                                       act_pre=pre)[0].cpu()
    finite = torch.isfinite(pre.cpu())
    ref = O.gelu_backward(np.ones(int(finite.sum())), pre.cpu()[finite].double().numpy())
    assert np.abs(got[finite].double().numpy() - ref).max() <= 2.0 ** -8 * 1.2
    assert torch.isnan(got[torch.isnan(pre.cpu())]).all()


@pytest.mark.parametrize("dt", ["bf16", "f32"])
def test_expert_module_backward_runs_without_the_activation_kernel(dt):
    """_Expert with torch.nn.GELU(): the layer's backward makes no gelu_bwd call for
    any dtype (one entry point covers the activation), and its gradients are the ones
    of the two linear nodes with the activation node between them."""
    from fastmoe_amd import fmoe_cuda
    from fastmoe_amd.functions import apply_activation
    from fastmoe_amd.linear import MOELinear
    from fastmoe_amd.transformer import _Expert

    dtype = DTYPES[dt]
    torch.manual_seed(5)
    ex = _Expert(3, 64, 128, torch.nn.GELU()).cuda().to(dtype)
    ex.htoh4.bias.data.normal_()
    ex.h4toh.bias.data.normal_()
    counts = torch.tensor([70, 0, 130])
    x = randn((200, 64), dtype, 9).cuda()
    dy = randn((200, 64), dtype, 10).cuda()

    def grads(fn):
        xi = x.clone().requires_grad_(True)
        for p in ex.parameters():
            p.grad = None
        fn(xi).backward(dy)
        return [xi.grad] + [p.grad.clone() for p in ex.parameters()]

    seen = []
    fmoe_cuda.profile_hook = lambda name, a, b: seen.append(name)
    try:
        got = grads(lambda xi: ex(xi, counts))
    finally:
        fmoe_cuda.profile_hook = None
    assert "gelu_bwd" not in seen and seen.count("grouped_linear_bwd") == 2

    def separate(xi):
        h = MOELinear.apply(xi, counts, ex.htoh4.weight, ex.htoh4.bias)
        h = apply_activation(ex.activation, h)
        return MOELinear.apply(h, counts, ex.h4toh.weight, ex.h4toh.bias)

    want = grads(separate)
    for g, w in zip(got, want):
        assert torch.equal(g, w)


def test_other_activations_keep_their_own_backward():
    from fastmoe_amd import fmoe_cuda
    from fastmoe_amd.transformer import _Expert

    ex = _Expert(2, 32, 64, torch.nn.ReLU()).cuda()
    x = torch.randn(50, 32, device="cuda", requires_grad=True)
    seen = []
    fmoe_cuda.profile_hook = lambda name, a, b: seen.append(name)
    try:
        ex(x, torch.tensor([20, 30])).sum().backward()
    finally:
        fmoe_cuda.profile_hook = None
    assert "gelu_fwd" not in seen and seen.count("grouped_linear_bwd") == 2
    ref = _Expert(2, 32, 64, torch.nn.ReLU()).cuda()
    ref.load_state_dict(ex.state_dict())
    xr = x.detach().clone().requires_grad_(True)
    h = torch.relu(torch.einsum("ni,noi->no", xr[:20], ref.htoh4.weight[:1].expand(20, -1, -1))
                   + ref.htoh4.bias[0])
    y0 = h @ ref.h4toh.weight[0].t() + ref.h4toh.bias[0]
    y0.sum().backward()
    assert (x.grad[:20] - xr.grad[:20]).abs().max().item() <= 1e-4
