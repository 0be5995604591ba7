"""Seeded input generators and comparison helpers shared by the tests."""
import numpy as np
import torch

DTYPES = {"f32": torch.float32, "f64": torch.float64, "f16": torch.float16,
          "bf16": torch.bfloat16}


def make_gate(n_tokens, top_k, n_expert, drop=0.0, seed=0, empty=()):
    """int64 [n_tokens, top_k] expert choices; `drop` fraction set to -1;
    experts listed in `empty` never chosen."""
    rng = np.random.default_rng(seed)
    allowed = np.array([e for e in range(n_expert) if e not in set(empty)])
    g = allowed[rng.integers(0, allowed.size, size=(n_tokens, top_k))]
    if drop:
        g[rng.random((n_tokens, top_k)) < drop] = -1
    return g.astype(np.int64)


def zipf_gate(n_tokens, n_expert, s=1.2, seed=0):
    """Two distinct experts per token drawn from p_e ~ e^-s."""
    g = torch.Generator().manual_seed(seed)
    p = torch.arange(1, n_expert + 1, dtype=torch.float64) ** (-s)
    idx = torch.multinomial((p / p.sum()).expand(n_tokens, -1), 2, replacement=False,
                            generator=g)
    return idx.numpy().astype(np.int64)


def randn(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g, dtype=torch.float64) * scale).to(dtype)


def max_rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """max |got - want| / max |want| in float64 (0 if both are all zero)."""
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    denom = want.abs().max().item()
    err = (got - want).abs().max().item()
    return err / denom if denom > 0 else err


def max_row_rel_err(got: torch.Tensor, want: torch.Tensor, floor: float = 1e-3) -> float:
    """max over rows of (max |got - want| in the row) / (max |want| in the row):
    the norm-wise bound of max_rel_err applied row by row (rows = the leading
    dimension: tokens, or the experts of a weight gradient), so that a tile of
    wrong values in a row of small magnitude cannot hide behind a large row
    elsewhere.  Rows whose own maximum is below `floor` x the global maximum
    are measured against that floor (a row of zeros has no scale of its own)."""
    got = got.detach().double().cpu().reshape(got.shape[0], -1)
    want = want.detach().double().cpu().reshape(want.shape[0], -1)
    scale = want.abs().amax(dim=1)
    scale = torch.clamp(scale, min=floor * max(scale.max().item(), 1e-300))
    return ((got - want).abs().amax(dim=1) / scale).max().item()


# tolerances: max |err| / max |ref| against a float64 evaluation of the same
# rounded inputs.  bf16/f16: the 2e-2 bound stated for the GEMM and combine
# outputs; f32: 1e-3 absolute in the reference's own tests
# (tests/test_numerical.py:51-68), far tighter here.
TOL = {torch.float64: 1e-12, torch.float32: 2e-5, torch.float16: 4e-3,
       torch.bfloat16: 2e-2}
