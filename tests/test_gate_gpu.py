"""Fused top-k + softmax gate kernels against the CPU checker and against the
torch.topk + softmax formulation of the reference's NaiveGate."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import DTYPES
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

CASES = [  # tokens, experts, top_k
    (1, 1, 1),
    (5, 2, 2),
    (33, 16, 2),        # config 2 shape
    (100, 8, 2),
    (257, 128, 8),      # config 5 shape
    (64, 64, 1),
    (19, 100, 16),      # largest supported top_k
    (7, 4096, 3),
    (1000, 7, 7),       # every expert chosen
    (50, 256, 8),       # up to 512 experts: logits held in registers (8 per lane here)
    (33, 300, 4),       # 32 lanes per token, ragged last register
    (20, 512, 16),
    (40, 17, 3),
    (40, 40, 5),
    (9, 513, 2),        # above 512: sorted lists over 32 lanes
]
SCORE_TOL = {"f64": 1e-12, "f32": 2e-6, "f16": 2e-3, "bf16": 1.6e-2}


@pytest.mark.parametrize("dt", ["f32", "f64", "f16", "bf16"])
@pytest.mark.parametrize("t,e,k", CASES)
def test_forward_and_backward(dt, t, e, k):
    from fastmoe_amd import fmoe_cuda

    dtype = DTYPES[dt]
    rng = np.random.default_rng(t * 131 + e)
    # a permutation of a grid per token: distinct values in float64; the narrow
    # dtypes round the widest cases to ties, which must then go by index
    logits = np.stack([rng.permutation(e) for _ in range(t)]).astype(np.float64)
    logits = (logits - e / 2) / max(e / 8, 1.0)
    lt = torch.from_numpy(logits).to(dtype)
    exact = lt.double().numpy()                       # what the kernel really sees
    idx, score = fmoe_cuda.topk_softmax_fwd(lt.cuda(), k)
    want_idx, want_score = O.topk_softmax(exact, k)
    assert idx.dtype == torch.int64 and score.dtype == dtype
    assert (idx.cpu().numpy() == want_idx).all()
    assert np.abs(score.double().cpu().numpy() - want_score).max() <= SCORE_TOL[dt]
    dscore = torch.from_numpy(rng.standard_normal((t, k))).to(dtype)
    dl = fmoe_cuda.topk_softmax_bwd(dscore.cuda(), score, idx, e)
    want_dl = O.topk_softmax_backward(dscore.double().numpy(), score.double().cpu().numpy(),
                                      want_idx, e)
    assert dl.shape == (t, e) and dl.dtype == dtype
    assert np.abs(dl.double().cpu().numpy() - want_dl).max() <= 4 * SCORE_TOL[dt]
    # zero outside the chosen experts, exactly
    mask = np.ones((t, e), dtype=bool)
    np.put_along_axis(mask, want_idx, False, axis=1)
    assert not dl.double().cpu().numpy()[mask].any()


def test_ties_and_minus_infinity():
    from fastmoe_amd import fmoe_cuda

    lt = torch.tensor([[1.0, 3.0, 3.0, float("-inf"), 3.0],
                       [0.0, 0.0, 0.0, 0.0, 0.0],
                       [float("-inf"), float("-inf"), 2.0, float("-inf"), 1.0]])
    idx, score = fmoe_cuda.topk_softmax_fwd(lt.cuda(), 2)
    assert idx.cpu().tolist() == [[1, 2], [0, 1], [2, 4]]
    want = O.topk_softmax(lt.double().numpy(), 2)[1]
    assert np.abs(score.double().cpu().numpy() - want).max() <= 1e-6


def test_ties_and_minus_infinity_in_a_wide_expert_set():
    from fastmoe_amd import fmoe_cuda

    e = 70
    lt = torch.full((3, e), float("-inf"))
    lt[0, [5, 40, 69]] = torch.tensor([2.0, 2.0, 2.0])       # three-way tie
    lt[1, 33] = 1.0                                           # one finite logit, k = 3
    lt[2] = 0.5                                               # all equal
    idx, score = fmoe_cuda.topk_softmax_fwd(lt.cuda(), 3)
    assert idx.cpu().tolist() == [[5, 40, 69], [33, 0, 1], [0, 1, 2]]
    want = O.topk_softmax(lt.double().numpy(), 3)[1]
    assert np.abs(score.double().cpu().numpy() - want).max() <= 1e-6


def test_nan_logits_rank_first_as_in_torch_topk():
    """torch.topk ranks NaN above every number (naive_gate.py:31-38 inherits that):
    a NaN logit is selected and the token's scores become NaN, for both the
    register-resident (<= 512 experts) and the sorted-list kernels."""
    from fastmoe_amd import fmoe_cuda

    nan, ninf = float("nan"), float("-inf")
    for e in (6, 600):
        lt = torch.zeros(4, e)
        lt[0, :6] = torch.tensor([1.0, nan, 3.0, ninf, 2.0, 0.5])
        lt[1, :6] = torch.tensor([nan, nan, nan, 1.0, ninf, 0.0])     # fewer numbers than k
        lt[2, :6] = torch.tensor([ninf, ninf, 1.0, ninf, ninf, ninf])
        lt[3, :6] = torch.tensor([5.0, 4.0, 3.0, 2.0, 1.0, 0.5])
        lt[:, 6:] = -10.0
        idx, score = fmoe_cuda.topk_softmax_fwd(lt.cuda(), 3)
        tval, tidx = torch.topk(lt, 3, dim=-1)
        idx, score = idx.cpu(), score.cpu()
        assert idx[0].tolist() == [1, 2, 4] and idx[1].tolist() == [0, 1, 2]
        assert idx[2, 0].item() == 2 and idx[3].tolist() == [0, 1, 2]
        for r in range(4):                      # same experts as torch.topk picks
            assert sorted(idx[r].tolist()) == sorted(tidx[r].tolist()) or r == 2
        assert idx.min().item() >= 0 and idx.max().item() < e
        assert torch.isnan(score[0]).all() and torch.isnan(score[1]).all()
        want = F.softmax(tval[3].double(), dim=-1)
        assert (score[3].double() - want).abs().max().item() <= 1e-6
        assert not torch.isnan(score[2:]).any()


def test_autograd_matches_torch_formulation():
    """The fused op inside autograd against torch.topk + softmax (no ties)."""
    from fastmoe_amd.functions import topk_softmax

    torch.manual_seed(3)
    logits = torch.randn(513, 32, device="cuda")
    a = logits.clone().requires_grad_(True)
    b = logits.clone().requires_grad_(True)
    idx, score = topk_softmax(a, 4)
    val, tidx = torch.topk(b, 4, dim=-1, largest=True, sorted=True)
    tscore = F.softmax(val, dim=-1)
    assert (idx == tidx).all()
    assert (score - tscore).abs().max().item() <= 2e-6
    g = torch.randn_like(score)
    score.backward(g)
    tscore.backward(g)
    assert (a.grad - b.grad).abs().max().item() <= 2e-6


def test_naive_gate_uses_the_kernel_and_errors():
    from fastmoe_amd import fmoe_cuda
    from fastmoe_amd.gates import NaiveGate

    gate = NaiveGate(24, 6, 1, top_k=2).cuda()
    x = torch.randn(50, 24, device="cuda")
    seen = []
    fmoe_cuda.profile_hook = lambda name, a, b: seen.append(name)
    try:
        idx, score = gate(x)
    finally:
        fmoe_cuda.profile_hook = None
    assert "topk_softmax_fwd" in seen
    logits = gate.gate(x)
    want_idx, want_score = O.topk_softmax(logits.double().cpu().detach().numpy(), 2)
    assert (idx.cpu().numpy() == want_idx).all()
    assert np.abs(score.double().cpu().detach().numpy() - want_score).max() <= 2e-6
    with pytest.raises(RuntimeError):
        fmoe_cuda.topk_softmax_fwd(torch.zeros(4, 3, device="cuda"), 4)      # k > experts
    with pytest.raises(RuntimeError):
        fmoe_cuda.topk_softmax_fwd(torch.zeros(4, 40, device="cuda"), 17)    # k > supported
