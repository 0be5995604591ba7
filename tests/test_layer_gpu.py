"""The whole MoE layer against the brute-force restatement of the reference's
test oracle (tests/moe.py:30-49), mirroring tests/test_numerical.py,
tests/test_zero.py and the invariants of tests/test_gates.py."""
import math

import pytest
import torch
import torch.nn.functional as F

from helpers import DTYPES, TOL, max_rel_err, max_row_rel_err
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _layer_vs_brute_force(moe, x, dtype, activation=F.gelu):
    """Runs the HIP layer and the CPU brute force on the same weights, gate
    decisions and inputs; returns (name, got, want) triples."""
    ex = moe.experts
    x_dev = x.clone().cuda().requires_grad_(True)
    out = moe(x_dev)
    out.float().mean().backward()
    with torch.no_grad():
        idx, score = moe.gate(x.cuda())
    w1, b1 = ex.htoh4.weight, ex.htoh4.bias
    w2, b2 = ex.h4toh.weight, ex.h4toh.bias
    cpu = [t.detach().double().cpu().requires_grad_(True) for t in (w1, b1, w2, b2)]
    x_cpu = x.double().requires_grad_(True)
    # the gate's scores depend on x; keep that path out of the comparison of
    # the expert gradients by differentiating the scores separately
    s_cpu = score.double().cpu().requires_grad_(True)
    want = O.brute_force_moe_mlp(x_cpu, idx.cpu(), s_cpu, *cpu, activation=activation)
    want.mean().backward()
    triples = [("out", out, want),
               ("dW1", w1.grad, cpu[0].grad), ("db1", b1.grad, cpu[1].grad),
               ("dW2", w2.grad, cpu[2].grad), ("db2", b2.grad, cpu[3].grad)]
    return triples, x_dev.grad, x_cpu.grad, s_cpu.grad


class _FusedMoE(torch.nn.Module):
    pass


def _make(num_expert, d_model, d_hidden, top_k, dtype, seed=0, scale=1.0):
    from fastmoe_amd import FMoETransformerMLP

    torch.manual_seed(seed)
    moe = FMoETransformerMLP(num_expert, d_model, d_hidden, top_k=top_k)
    g = torch.Generator().manual_seed(seed + 1)
    with torch.no_grad():
        for p in moe.experts.parameters():
            p.copy_(torch.randn(p.shape, generator=g) * scale)
    return moe.to(dtype).cuda()


@pytest.mark.parametrize("num_expert", [4, 8])
@pytest.mark.parametrize("top_k", [2, 3])
@pytest.mark.parametrize("dt", ["f32", "f16", "bf16"])
def test_fmoe_linear_shapes_of_the_reference_suite(num_expert, top_k, dt):
    """tests/test_numerical.py::test_fmoe_linear: batch 4, d_model 16, d_hidden 32."""
    dtype = DTYPES[dt]
    moe = _make(num_expert, 16, 32, top_k, dtype, seed=42, scale=0.5)
    torch.manual_seed(42)
    x = torch.rand(4, 16).to(dtype)
    triples, dx, _dx_cpu, _ds = _layer_vs_brute_force(moe, x, dtype)
    for name, got, want in triples:
        assert max_rel_err(got, want) <= TOL[dtype], name
    assert dx is not None and torch.isfinite(dx.float()).all()


def test_config1_fp32_layer_and_all_gradients():
    """512 tokens, d_model 128, d_hidden 256, 4 experts, top-2 NaiveGate, GELU,
    inputs and weights N(0, 0.02), seed 0; forward and every gradient."""
    from fastmoe_amd import FMoETransformerMLP

    torch.manual_seed(0)
    moe = FMoETransformerMLP(4, 128, 256, top_k=2)
    g = torch.Generator().manual_seed(0)
    with torch.no_grad():
        for p in moe.parameters():
            p.copy_(torch.randn(p.shape, generator=g) * 0.02)
    moe = moe.cuda()
    x = torch.randn(512, 128, generator=g) * 0.02

    x_dev = x.clone().cuda().requires_grad_(True)
    out = moe(x_dev)
    out.sum().backward()

    # CPU: the same gate (torch ops) feeding the brute-force experts, in float64
    from fastmoe_amd.gates import NaiveGate
    gate = NaiveGate(128, 4, 1, top_k=2)
    gate.load_state_dict(moe.gate.state_dict())
    gate = gate.double()
    ex = moe.experts
    cpu = [t.detach().double().cpu().requires_grad_(True)
           for t in (ex.htoh4.weight, ex.htoh4.bias, ex.h4toh.weight, ex.h4toh.bias)]
    x_cpu = x.double().requires_grad_(True)
    idx, score = gate(x_cpu)
    with torch.no_grad():
        idx_dev, _ = moe.gate(x.cuda())
    assert torch.equal(torch.sort(idx, 1).values, torch.sort(idx_dev.cpu(), 1).values)
    want = O.brute_force_moe_mlp(x_cpu, idx, score, *cpu)
    want.sum().backward()
    tol = 1e-4
    assert max_rel_err(out, want) <= tol
    assert max_rel_err(x_dev.grad, x_cpu.grad) <= tol
    assert max_rel_err(ex.htoh4.weight.grad, cpu[0].grad) <= tol
    assert max_rel_err(ex.htoh4.bias.grad, cpu[1].grad) <= tol
    assert max_rel_err(ex.h4toh.weight.grad, cpu[2].grad) <= tol
    assert max_rel_err(ex.h4toh.bias.grad, cpu[3].grad) <= tol
    assert max_rel_err(moe.gate.gate.weight.grad, gate.gate.weight.grad) <= tol


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_medium_layer_on_the_matrix_cores(dt):
    """Shapes that take the MFMA kernels (features multiples of 8), ragged and
    empty experts, bf16/f16 tolerance 2e-2 / 4e-3 on out and every gradient."""
    dtype = DTYPES[dt]
    moe = _make(8, 256, 512, 2, dtype, seed=3, scale=0.05)
    with torch.no_grad():                       # starve experts 2 and 5
        moe.gate.gate.bias[2] = -1e4
        moe.gate.gate.bias[5] = -1e4
    x = torch.randn(700, 256, generator=torch.Generator().manual_seed(8)).to(dtype)
    triples, dx, dx_cpu, _ = _layer_vs_brute_force(moe, x, dtype)
    # with a mean() loss the f16 weight gradients sit in the subnormal range
    # (|dW| ~ 1e-5), where f16 keeps fewer than 11 bits: 1e-2 there
    tol = max(TOL[dtype], 1e-2)
    for name, got, want in triples:
        assert max_rel_err(got, want) <= tol, name
    ex = moe.experts
    assert not ex.htoh4.weight.grad[2].any().item()
    assert not ex.h4toh.bias.grad[5].any().item()


def test_fused_and_reference_layouts_agree_and_exchange_checkpoints():
    from fastmoe_amd import FMoETransformerMLP

    torch.manual_seed(1)
    fused = FMoETransformerMLP(4, 32, 64, top_k=2).cuda()
    plain = FMoETransformerMLP(4, 32, 64, top_k=2, fused=False).cuda()
    plain.load_state_dict(fused.state_dict())          # fused keys -> per-expert keys
    assert "experts.0.htoh4.weight" in plain.state_dict()
    x = torch.randn(50, 32, device="cuda")
    a, b = fused(x), plain(x)
    assert max_rel_err(a, b) <= 1e-5
    again = FMoETransformerMLP(4, 32, 64, top_k=2).cuda()
    again.load_state_dict(plain.state_dict())          # and back
    assert torch.equal(again.experts.htoh4.weight, fused.experts.htoh4.weight)
    # 3-d input keeps its shape (fmoe/transformer.py:58-66)
    assert fused(x.view(5, 10, 32)).shape == (5, 10, 32)


class _Doubler(torch.nn.Module):
    def __init__(self, d_model):
        super().__init__()
        self.lin = torch.nn.Linear(d_model, d_model)

    def forward(self, x, fec=None):
        return self.lin(x)


def test_arbitrary_expert_modules_follow_the_reference_route():
    """tests/test_numerical.py::test_fmoe: a list of ordinary modules as experts."""
    from fastmoe_amd import FMoE

    torch.manual_seed(5)
    moe = FMoE(num_expert=3, d_model=8, top_k=2, expert=_Doubler).cuda()
    x = torch.randn(20, 8, device="cuda", requires_grad=True)
    out = moe(x)
    out.sum().backward()
    with torch.no_grad():
        idx, score = moe.gate(x)
        want = torch.zeros_like(out)
        for t in range(20):
            for j in range(2):
                want[t] += score[t, j] * moe.experts[int(idx[t, j])](x[t])
    assert max_rel_err(out, want) <= 1e-5
    assert x.grad is not None and moe.experts[0].lin.weight.grad is not None


class _ConstantGate(torch.nn.Module):
    def __init__(self, d_model, num_expert, world_size, top_k=1):
        super().__init__()
        self.top_k = top_k

    def forward(self, inp):
        idx = torch.zeros((inp.shape[0], self.top_k), dtype=torch.int64, device=inp.device)
        score = torch.ones((inp.shape[0], 1, self.top_k), device=inp.device) / 2
        return idx, score


def test_zero_token_experts_and_mask():
    """tests/test_zero.py: every token to expert 0, expert 1 idle; masked rows
    replaced from mask_dict."""
    from fastmoe_amd import FMoETransformerMLP
    from fastmoe_amd.layers import _fmoe_general_global_forward

    inp = torch.rand(4, 8).cuda()
    gate = torch.zeros(4, dtype=torch.int64).cuda()
    out = _fmoe_general_global_forward(inp, gate, lambda x, y: x, 2, 1)
    assert torch.equal(out, inp)
    mask = torch.zeros(4, dtype=torch.long)
    mask[1] = 1
    model = FMoETransformerMLP(2, 8, 32, gate=_ConstantGate, mask=mask.cuda(),
                               mask_dict={1: torch.zeros(8).cuda()}, top_k=1).cuda()
    out = model(inp)
    assert out.shape == (4, 8) and not out[1].any().item() and out[0].any().item()
    model2 = FMoETransformerMLP(2, 8, 32, gate=_ConstantGate, top_k=1).cuda()
    out2 = model2(inp)
    out2.sum().backward()
    assert not model2.experts.htoh4.weight.grad[1].any().item()


@pytest.mark.parametrize("n_expert,cap", [(4, 0.1), (4, 1.1)])
def test_gshard_gate_invariants(n_expert, cap):
    """tests/test_gates.py:31-56: per-expert load <= ceil(cap * batch), kept
    scores equal the plain top-2 softmax."""
    from fastmoe_amd.gates import GShardGate, NaiveGate

    torch.manual_seed(0)
    gate = GShardGate(1024, n_expert, 1, capacity=(cap, cap)).cuda()
    x = torch.rand(16, 1024).cuda()
    idx, val = gate(x)
    loss = gate.get_loss()
    counts = torch.bincount(idx[idx >= 0].view(-1), minlength=n_expert)
    assert counts.max().item() <= math.ceil(cap * 16)
    logits = gate.gate(x)
    tv, _ti = torch.topk(logits, k=2, dim=-1, largest=True, sorted=False)
    ref = F.softmax(tv, dim=-1)
    keep = idx != -1
    assert torch.equal(val[keep], ref[keep])
    # the balance loss (fmoe/gates/gshard_gate.py:26-33) from torch.bincount
    _i, _v, lg = NaiveGate.forward(gate, x, return_all_scores=True)
    frac = torch.bincount(_i[:, 0], minlength=n_expert).float() / 16
    want = torch.mean(frac * F.softmax(lg, dim=1).mean(dim=0)) * n_expert ** 2
    assert abs(loss.item() - want.item()) <= 1e-6 * max(1.0, abs(want.item()))


@pytest.mark.parametrize("n_expert,cap", [(1, 0.1), (16, 0.8)])
def test_switch_gate_invariants(n_expert, cap):
    """tests/test_gates.py:74-113."""
    from fastmoe_amd.gates import SwitchGate

    torch.manual_seed(0)
    gate = SwitchGate(1024, n_expert, 1, capacity=(cap, cap)).cuda().eval()
    x = torch.rand(4096, 1024).cuda()
    idx, val = gate(x)
    counts = torch.bincount(idx[idx >= 0].view(-1), minlength=n_expert)
    assert counts.max().item() <= math.ceil(cap * 4096)
    score = F.softmax(gate.gate(x).float(), dim=-1)
    keep = (idx != -1).view(-1)
    rows = torch.nonzero(keep).view(-1)
    assert torch.equal(val.view(-1)[rows], score[rows, idx.view(-1)[rows]])
    # the balance loss (fmoe/gates/switch_gate.py:49-57) from torch.bincount
    kept = idx[idx > -1]
    frac = torch.bincount(kept, minlength=n_expert).float() / kept.numel()
    want = (frac * (score.sum(dim=0) / kept.numel())).sum() * n_expert
    assert abs(gate.get_loss().item() - want.item()) <= 1e-5 * max(1.0, abs(want.item()))


def test_dropped_slots_flow_through_the_layer():
    """A gate that drops slots (-1): the layer output equals the brute force
    with those slots contributing zero, and their scores get zero gradient."""
    from fastmoe_amd import FMoETransformerMLP
    from fastmoe_amd.gates import GShardGate

    torch.manual_seed(2)
    moe = FMoETransformerMLP(4, 64, 128, top_k=2, gate=GShardGate).cuda()
    moe.gate.capacity = (0.3, 0.3)
    moe.gate.random_routing = False
    x = torch.randn(200, 64)
    x_dev = x.cuda().requires_grad_(True)
    out = moe(x_dev)
    out.sum().backward()
    with torch.no_grad():
        idx, score = moe.gate(x.cuda())
    assert (idx == -1).any().item()
    ex = moe.experts
    want = O.brute_force_moe_mlp(x.double(), idx.cpu(), score.double().cpu(),
                                 ex.htoh4.weight.detach().double().cpu(),
                                 ex.htoh4.bias.detach().double().cpu(),
                                 ex.h4toh.weight.detach().double().cpu(),
                                 ex.h4toh.bias.detach().double().cpu())
    assert max_rel_err(out, want) <= 1e-4


@pytest.mark.parametrize("n_expert,top_k", [(24, 20), (80, 70)])
def test_top_k_beyond_the_gate_and_combine_kernels(n_expert, top_k):
    """top_k above 16 leaves the fused gate kernel for torch.topk + softmax (the
    reference's own formulation, naive_gate.py:31-38); above 64 the layer also
    leaves the fused combine kernels for the reference-shaped route (MOEScatter ->
    experts -> MOEGather + bmm).  Both against the brute force, with gradients."""
    from fastmoe_amd import FMoETransformerMLP

    torch.manual_seed(21)
    moe = FMoETransformerMLP(n_expert, 32, 48, top_k=top_k).cuda()
    x = torch.randn(150, 32)
    dy = torch.randn(150, 32)
    x_dev = x.cuda().requires_grad_(True)
    out = moe(x_dev)
    out.backward(dy.cuda())
    with torch.no_grad():
        idx, score = moe.gate(x.cuda())
    assert tuple(idx.shape) == (150, top_k)
    assert all(len(set(r)) == top_k for r in idx.cpu().tolist())     # k distinct experts
    ex = moe.experts
    ps = [p.detach().double().cpu().requires_grad_(True)
          for p in (ex.htoh4.weight, ex.htoh4.bias, ex.h4toh.weight, ex.h4toh.bias)]
    xr = x.double().requires_grad_(True)
    # the gate itself, recomputed on the host: logits -> top-k -> softmax over the k values
    logits = xr @ moe.gate.gate.weight.detach().double().cpu().t() \
        + moe.gate.gate.bias.detach().double().cpu()
    ref_score = torch.softmax(torch.gather(logits, 1, idx.cpu()), dim=-1)
    assert (ref_score - score.double().cpu()).abs().max().item() <= 1e-5
    want = O.brute_force_moe_mlp(xr, idx.cpu(), ref_score, *ps)
    want.backward(dy.double())
    assert max_rel_err(out, want) <= 1e-4
    assert max_rel_err(x_dev.grad, xr.grad) <= 1e-4
    for dev, ref in zip((ex.htoh4.weight, ex.htoh4.bias, ex.h4toh.weight, ex.h4toh.bias), ps):
        assert max_rel_err(dev.grad, ref.grad) <= 1e-4


def test_config2_full_size_layer_against_brute_force():
    """The benchmark workload itself (8192 tokens, d_model 1024, d_hidden 4096,
    16 experts, top-2, bf16): output, input gradient and all four expert
    gradients against the float32 brute force on the host, 2e-2."""
    dtype = torch.bfloat16
    moe = _make(16, 1024, 4096, 2, dtype, seed=11, scale=0.02)
    g = torch.Generator().manual_seed(12)
    x = torch.randn(8192, 1024, generator=g).to(dtype)
    dy = torch.randn(8192, 1024, generator=g).to(dtype)
    ex = moe.experts
    x_dev = x.clone().cuda().requires_grad_(True)
    out = moe(x_dev)
    out.backward(dy.cuda())
    with torch.no_grad():
        idx, score = moe.gate(x.cuda())
    cpu = [t.detach().float().cpu().requires_grad_(True)
           for t in (ex.htoh4.weight, ex.htoh4.bias, ex.h4toh.weight, ex.h4toh.bias)]
    x_cpu = x.float().requires_grad_(True)
    s_cpu = score.float().cpu()          # the gate's own path is not under test here
    want = O.brute_force_moe_mlp(x_cpu, idx.cpu(), s_cpu, *cpu)
    want.backward(dy.float())
    tol = TOL[dtype]
    assert max_rel_err(out, want) <= tol
    assert max_row_rel_err(out, want) <= 3e-2          # and token by token
    grads = [ex.htoh4.weight.grad, ex.htoh4.bias.grad, ex.h4toh.weight.grad, ex.h4toh.bias.grad]
    for name, got, ref in zip(("dW1", "db1", "dW2", "db2"), grads, cpu):
        assert max_rel_err(got, ref.grad) <= tol, name
        assert max_row_rel_err(got, ref.grad) <= 3e-2, name    # expert by expert
    # dx on the device also carries the gate's share (d score / d x); compare the
    # experts' share by removing it: run the layer again with the scores detached
    x2 = x.clone().cuda().requires_grad_(True)
    hook = moe.gate.register_forward_hook(lambda m, a, o: (o[0], o[1].detach()))
    try:
        moe(x2).backward(dy.cuda())
    finally:
        hook.remove()
    assert max_rel_err(x2.grad, x_cpu.grad) <= tol
    assert max_row_rel_err(x2.grad, x_cpu.grad) <= 3e-2


@pytest.mark.parametrize("dt,top_k", [("bf16", 2), ("f32", 3), ("bf16", 8)])
def test_whole_layer_node_matches_the_chain_of_nodes(dt, top_k):
    """FusedExpertLayer (dispatch, experts and combine as one autograd node) runs the
    same kernels in the same order as the chain FusedScatter -> MOELinearGelu ->
    MOEGeluLinear -> FusedGatherCombine: identical bits in the output and in every
    gradient.  A hook on the activation module switches the single node off."""
    from fastmoe_amd import FMoETransformerMLP

    dtype = DTYPES[dt]
    torch.manual_seed(9)
    moe = FMoETransformerMLP(12, 64, 96, top_k=top_k).to(dtype).cuda()
    x = torch.randn(200, 64, device="cuda").to(dtype)
    dy = torch.randn(200, 64, device="cuda").to(dtype)

    def run():
        for p in moe.parameters():
            p.grad = None
        a = x.clone().requires_grad_(True)
        out = moe(a)
        out.backward(dy)
        return [out, a.grad] + [p.grad for p in moe.parameters()]

    assert moe.experts.can_run_layer(x, top_k)
    whole = run()
    hook = moe.experts.activation.register_forward_hook(lambda m, i, o: None)
    assert not moe.experts.can_run_layer(x, top_k)
    hook.remove()
    moe.experts.can_run_layer = lambda inp, k: False      # the chain of nodes
    try:
        chain = run()
    finally:
        del moe.experts.can_run_layer
    for got, want in zip(whole, chain):
        assert (got is None) == (want is None)
        if got is not None:
            assert torch.equal(got, want)
