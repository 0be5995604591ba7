"""Writes tests/golden/routing_cases.json and tests/golden/layer_case.npz.

The reference ships no golden vectors for this path, so these fixtures are
produced by the CPU checker (oracle/) once it is pinned by tests/test_oracle.py,
from seeded inputs.  They freeze today's expected outputs so that neither the
checker nor the HIP kernels can drift silently: tests/test_golden.py compares
the checker against them on the CPU and the kernels against them on the GPU.

    python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import moe_oracle as O  # noqa: E402


def routing_cases():
    rng = np.random.default_rng(7)
    cases = []
    for n, k, e, drop in [(6, 2, 4, 0.0), (12, 2, 8, 0.3), (9, 3, 5, 0.2), (40, 1, 3, 0.5),
                          (70, 2, 16, 0.1)]:
        g = rng.integers(0, e, size=(n, k))
        g[rng.random((n, k)) < drop] = -1
        pos, count, seg_off, inv = O.route(g, e)
        cap0 = rng.integers(0, max(2, 2 * n * k // e), size=e).astype(np.int32)
        cap = cap0.copy()
        pruned = O.prune_gate_by_capacity(g, cap, e)
        lim_cap = cap0.copy()
        limited = O.limit_by_capacity(count, lim_cap, e, 1)
        cases.append(dict(n_expert=e, gate=g.tolist(), count=count.tolist(),
                          seg_off=seg_off.tolist(), pos=pos.tolist(), inv=inv.tolist(),
                          capacity=cap0.tolist(), pruned=pruned.tolist(),
                          capacity_after_prune=cap.tolist(), limited=limited.tolist(),
                          capacity_after_limit=lim_cap.tolist()))
    return cases


def layer_case():
    """A 24-token, 4-expert, top-2 GELU MoE MLP in float64: inputs, weights,
    routing, output and all gradients of loss = sum(out * probe)."""
    g = torch.Generator().manual_seed(11)
    t, d, h, e, k = 24, 16, 24, 4, 2
    x = torch.randn(t, d, generator=g, dtype=torch.float64, requires_grad=True)
    w1 = (torch.randn(e, h, d, generator=g, dtype=torch.float64) * 0.3).requires_grad_(True)
    b1 = (torch.randn(e, h, generator=g, dtype=torch.float64) * 0.1).requires_grad_(True)
    w2 = (torch.randn(e, d, h, generator=g, dtype=torch.float64) * 0.3).requires_grad_(True)
    b2 = (torch.randn(e, d, generator=g, dtype=torch.float64) * 0.1).requires_grad_(True)
    idx = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(t)])
    idx[3, 1] = -1
    idx[17, 0] = -1
    score = torch.rand(t, k, generator=g, dtype=torch.float64).requires_grad_(True)
    probe = torch.randn(t, d, generator=g, dtype=torch.float64)
    out = O.brute_force_moe_mlp(x, idx, score, w1, b1, w2, b2)
    (out * probe).sum().backward()
    return dict(x=x.detach().numpy(), w1=w1.detach().numpy(), b1=b1.detach().numpy(),
                w2=w2.detach().numpy(), b2=b2.detach().numpy(), idx=idx.numpy(),
                score=score.detach().numpy(), probe=probe.numpy(),
                out=out.detach().numpy(), dx=x.grad.numpy(), dw1=w1.grad.numpy(),
                db1=b1.grad.numpy(), dw2=w2.grad.numpy(), db2=b2.grad.numpy(),
                dscore=score.grad.numpy())


if __name__ == "__main__":
    with open(os.path.join(HERE, "routing_cases.json"), "w") as f:
        json.dump(routing_cases(), f)
    np.savez_compressed(os.path.join(HERE, "layer_case.npz"), **layer_case())
    print("wrote", os.listdir(HERE))
