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


# tolerances: max |err| / max |ref| against a float64 evaluation of the same
# rounded inputs.  bf16/f16: the 2e-2 bound stated for the GEMM and combine
# outputs; f32: 1e-3 absolute in the reference's own tests
# (tests/test_numerical.py:51-68), far tighter here.
TOL = {torch.float64: 1e-12, torch.float32: 2e-5, torch.float16: 4e-3,
       torch.bfloat16: 2e-2}
