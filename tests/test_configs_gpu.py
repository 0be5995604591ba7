"""The benchmark workloads themselves (bench.py's seeded cfg3, cfg4, cfg5) run as
a whole layer, forward and backward, against the brute-force restatement of the
reference's test oracle (tests/moe.py:30-49) on the host: all of it where the
host can afford the arithmetic (cfg3, cfg5), a fixed sample of tokens and one
whole expert for the Mixtral-sized cfg4.  Tolerance: the bf16 bound 2e-2, both
norm-wise and row by row.  Also the reference-shaped dispatch (MOEScatter /
MOEGather, module-list experts) through autograd, and nested (dict / list)
inputs as in tests/test_mimo.py."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import DTYPES, TOL, max_rel_err, max_row_rel_err
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu

ROW_TOL = 2e-2      # row-wise bound for bf16 results, the same as the norm-wise one


def _bench_layer(name):
    import bench

    cfg = dict(bench.CONFIGS[name], name=name)
    layer, x, dy = bench.build_layer(cfg)
    return cfg, layer, x, dy


def _run_device(layer, x, dy, detach_score=False):
    """Forward + backward on the GPU.  With detach_score the gate's scores carry
    no gradient, so x.grad is the experts' share alone (what the oracle computes
    when it is handed the scores as constants)."""
    for p in layer.parameters():
        p.grad = None
    xd = x.detach().clone().requires_grad_(True)
    hook = None
    if detach_score:
        hook = layer.gate.register_forward_hook(lambda m, a, o: (o[0], o[1].detach()))
    try:
        out = layer(xd)
        out.backward(dy)
    finally:
        if hook is not None:
            hook.remove()
    torch.cuda.synchronize()
    return out.detach(), xd.grad.detach()


def _expert_params_cpu(layer, experts=None):
    ex = layer.experts
    sel = slice(None) if experts is None else experts
    return [t.detach()[sel].float().cpu().requires_grad_(True)
            for t in (ex.htoh4.weight, ex.htoh4.bias, ex.h4toh.weight, ex.h4toh.bias)]


def _check(name, got, want, tol=TOL[torch.bfloat16], row_tol=ROW_TOL):
    assert max_rel_err(got, want) <= tol, f"{name}: norm-wise"
    assert max_row_rel_err(got, want) <= row_tol, f"{name}: row-wise"


def _full_layer_check(name, expect_drops=False, expect_empty=0):
    cfg, layer, x, dy = _bench_layer(name)
    out, dx = _run_device(layer, x, dy, detach_score=True)
    with torch.no_grad():
        idx, score = layer.gate(x)
    ex = layer.experts
    counts = torch.bincount(idx[idx >= 0].view(-1), minlength=cfg["E"])
    if expect_drops:
        assert (idx == -1).any().item() and counts.max().item() <= layer.gate.capacity
    assert int((counts == 0).sum()) >= expect_empty
    cpu = _expert_params_cpu(layer)
    x_cpu = x.float().cpu().requires_grad_(True)
    want = O.brute_force_moe_mlp(x_cpu, idx.cpu(), score.float().cpu(), *cpu)
    want.backward(dy.float().cpu())
    _check("out", out, want)
    _check("dx", dx, x_cpu.grad)
    grads = (ex.htoh4.weight.grad, ex.htoh4.bias.grad, ex.h4toh.weight.grad, ex.h4toh.bias.grad)
    for gname, got, ref in zip(("dW1", "db1", "dW2", "db2"), grads, cpu):
        _check(gname, got, ref.grad)
    # experts without rows: exactly zero gradients
    for e in torch.nonzero(counts == 0).view(-1).tolist():
        for got in grads:
            assert not got[e].any().item()


@pytest.mark.timeout(900)
def test_config3_zipf_routing_with_capacity_full_layer():
    """16384 tokens, d_model 2048, d_hidden 8192, 64 experts, top-2, Zipf(1.2)
    choices clipped to 640 rows per expert: half of the expert-ordered buffers is
    dead rows, the experts have 2.5 tiles of rows each."""
    _full_layer_check("cfg3", expect_drops=True)


@pytest.mark.timeout(900)
def test_config5_fine_grained_experts_full_layer():
    """8192 tokens, d_model 2048, d_hidden 1408, 128 experts of which 13 get no
    token, top-8 (token-ordered scatter, tiny and empty grouped GEMMs)."""
    _full_layer_check("cfg5", expect_empty=13)


@pytest.mark.timeout(900)
def test_config4_mixtral_sized_layer_on_a_sample():
    """16384 tokens, d_model 4096, d_hidden 14336, 8 experts, top-2: 23 TFLOP per
    step, too much for the host in full.  The oracle is evaluated on a fixed
    sample of 384 tokens (their outputs and input gradients need nothing else)
    and, expert by expert, on ALL rows of each of the eight experts (an expert's
    four parameter gradients need nothing but its own rows)."""
    cfg, layer, x, dy = _bench_layer("cfg4")
    out, dx = _run_device(layer, x, dy, detach_score=True)
    with torch.no_grad():
        idx, score = layer.gate(x)
    idx_c, score_c = idx.cpu(), score.float().cpu()
    ex = layer.experts
    grads = (ex.htoh4.weight.grad, ex.htoh4.bias.grad, ex.h4toh.weight.grad, ex.h4toh.bias.grad)

    # (a) a sample of tokens, all experts
    g = torch.Generator().manual_seed(4)
    sample = torch.randperm(cfg["T"], generator=g)[:384].sort().values
    cpu = [t.detach().float().cpu() for t in (ex.htoh4.weight, ex.htoh4.bias,
                                              ex.h4toh.weight, ex.h4toh.bias)]
    xs = x[sample.cuda()].float().cpu().requires_grad_(True)
    want = O.brute_force_moe_mlp(xs, idx_c[sample], score_c[sample], *cpu)
    want.backward(dy[sample.cuda()].float().cpu())
    _check("out[sample]", out[sample.cuda()], want)
    _check("dx[sample]", dx[sample.cuda()], xs.grad)
    del cpu

    # (b) every row of one expert at a time: its slots keep their index (renamed 0),
    # all other slots are dropped, and the weights handed over are that expert's alone
    for e in range(cfg["E"]):
        rows = torch.nonzero((idx_c == e).any(dim=1)).view(-1)
        sub_idx = torch.where(idx_c[rows] == e, 0, -1)
        one = _expert_params_cpu(layer, experts=slice(e, e + 1))
        xe = x[rows.cuda()].float().cpu()
        got = O.brute_force_moe_mlp(xe, sub_idx, score_c[rows], *one)
        got.backward(dy[rows.cuda()].float().cpu())
        for gname, dev, ref in zip(("dW1", "db1", "dW2", "db2"), grads, one):
            _check(f"{gname}[{e}]", dev[e:e + 1], ref.grad)


class _PlainExpert(torch.nn.Module):
    """A single-expert MLP like the reference's _Expert(1, ...) (fmoe/transformer.py:11-31),
    as an ordinary module: FMoE has to slice rows for it on the host."""

    def __init__(self, d_model, d_hidden=64):
        super().__init__()
        from fastmoe_amd import FMoELinear

        self.htoh4 = FMoELinear(1, d_model, d_hidden, bias=True)
        self.h4toh = FMoELinear(1, d_hidden, d_model, bias=True)

    def forward(self, inp, fwd_expert_count):
        return self.h4toh(F.gelu(self.htoh4(inp, fwd_expert_count)), fwd_expert_count)


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_reference_shaped_route_through_autograd(dt):
    """Ordinary modules as experts take _fmoe_general_global_forward: MOEScatter ->
    per-expert modules -> MOEGather -> bmm.  Output, input gradient and every
    expert's parameter gradients against the brute force, through autograd
    (MOEScatter.backward / MOEGather.backward included), with dropped slots."""
    from fastmoe_amd import FMoE
    from fastmoe_amd.gates import GShardGate

    dtype = DTYPES[dt]
    torch.manual_seed(7)
    plain = FMoE(num_expert=4, d_model=32, top_k=2, gate=GShardGate, expert=_PlainExpert)
    assert not plain._device_side_dispatch()
    g = torch.Generator().manual_seed(8)
    with torch.no_grad():
        for p in plain.parameters():
            p.copy_(torch.randn(p.shape, generator=g) * 0.3)
    plain = plain.to(dtype).cuda()
    plain.gate.capacity = (0.4, 0.4)            # forces drops
    plain.gate.random_routing = False
    x = torch.randn(150, 32, generator=g).to(dtype)
    dy = torch.randn(150, 32, generator=g).to(dtype)
    xd = x.cuda().requires_grad_(True)
    hook = plain.gate.register_forward_hook(lambda m, a, o: (o[0], o[1].detach()))
    try:
        out = plain(xd)
        out.backward(dy.cuda())
    finally:
        hook.remove()
    with torch.no_grad():
        idx, score = plain.gate(x.cuda())
    assert (idx == -1).any().item()
    names = ("htoh4.weight", "htoh4.bias", "h4toh.weight", "h4toh.bias")
    cpu = [torch.cat([dict(e.named_parameters())[n].detach() for e in plain.experts], 0)
           .double().cpu().requires_grad_(True) for n in names]
    x_cpu = x.double().requires_grad_(True)
    want = O.brute_force_moe_mlp(x_cpu, idx.cpu(), score.double().cpu(), *cpu)
    want.backward(dy.double())
    tol = 1e-4 if dt == "f32" else 1e-10
    assert max_rel_err(out, want) <= tol
    assert max_rel_err(xd.grad, x_cpu.grad) <= tol
    for n, ref in zip(names, cpu):
        got = torch.cat([dict(e.named_parameters())[n].grad for e in plain.experts], 0)
        assert max_rel_err(got, ref.grad) <= tol, n


class _NaiveExpert(torch.nn.Module):
    """tests/moe.py: one Linear(d, d)."""

    def __init__(self, d_model):
        super().__init__()
        self.linear = torch.nn.Linear(d_model, d_model)

    def forward(self, x, fec=None):
        return self.linear(x)


class _LinearExpert(torch.nn.Module):
    """tests/moe.py: Linear -> ReLU -> Linear."""

    def __init__(self, d_model):
        super().__init__()
        self.model = torch.nn.Sequential(torch.nn.Linear(d_model, d_model * 2), torch.nn.ReLU(),
                                         torch.nn.Linear(d_model * 2, d_model))

    def forward(self, x, fec=None):
        return self.model(x)


@pytest.mark.parametrize("top_k", [2, 3])
@pytest.mark.parametrize("experts", [[_NaiveExpert] * 4,
                                     [_LinearExpert, _NaiveExpert] * 4])
def test_heterogeneous_expert_modules(top_k, experts):
    """tests/test_numerical.py:405-510 (test_fmoe_experts): a list of different
    ordinary modules; output, input gradient and each expert's summed parameter
    gradient against a per-token evaluation of the same modules."""
    import copy

    from fastmoe_amd import FMoE

    torch.manual_seed(42)
    moe = FMoE(num_expert=None, d_model=16, top_k=top_k, expert=experts).cuda()
    ref_experts = copy.deepcopy(moe.experts)
    x = torch.rand(24, 16, device="cuda")
    a = x.clone().requires_grad_(True)
    out = moe(a)
    out.sum().backward()
    with torch.no_grad():
        idx, score = moe.gate(x)
    b = x.clone().requires_grad_(True)
    rows = []
    for t in range(x.shape[0]):
        acc = 0
        for j in range(top_k):
            acc = acc + score[t, j] * ref_experts[int(idx[t, j])](b[t:t + 1])[0]
        rows.append(acc)
    want = torch.stack(rows)
    want.sum().backward()
    assert max_rel_err(out, want) <= 1e-5

    def grad_sums(mods):
        return torch.stack([torch.stack([p.grad.sum() if p.grad is not None
                                         else torch.zeros((), device="cuda")
                                         for p in m.parameters()]).sum() for m in mods])

    assert max_rel_err(grad_sums(moe.experts), grad_sums(ref_experts)) <= 1e-4
    # the experts' share of the input gradient (the gate's own share comes on top)
    hook = moe.gate.register_forward_hook(lambda m, i, o: (o[0], o[1].detach()))
    try:
        c = x.clone().requires_grad_(True)
        moe(c).sum().backward()
    finally:
        hook.remove()
    assert max_rel_err(c.grad, b.grad) <= 1e-4


def test_module_list_of_fused_expert_class_runs_without_a_host_read():
    """The reference's layout of FMoETransformerMLP -- one _Expert(1, ...) per
    expert -- runs as one grouped call per layer from the device-side segment
    table: same numbers as the fused module, gradients land on each expert's own
    parameters, and no call of the pass synchronises with the host."""
    from fastmoe_amd import FMoETransformerMLP

    torch.manual_seed(3)
    fused = FMoETransformerMLP(6, 64, 128, top_k=2).to(torch.bfloat16).cuda()
    plain = FMoETransformerMLP(6, 64, 128, top_k=2, fused=False).to(torch.bfloat16).cuda()
    plain.load_state_dict(fused.state_dict())
    assert plain._device_side_dispatch() and len(plain.experts) == 6
    x = torch.randn(333, 64, device="cuda", dtype=torch.bfloat16)
    dy = torch.randn_like(x)
    a = x.clone().requires_grad_(True)
    fused(a).backward(dy)
    b = x.clone().requires_grad_(True)
    plain(b).backward(dy)                       # warm-up (tables, attributes)
    for p in plain.parameters():
        p.grad = None
    b.grad = None
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")     # any host synchronisation raises
    try:
        out = plain(b)
        out.backward(dy)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    assert torch.equal(out, fused(x))
    assert torch.equal(b.grad, a.grad)
    for i, e in enumerate(plain.experts):
        assert torch.equal(e.htoh4.weight.grad[0], fused.experts.htoh4.weight.grad[i])
        assert torch.equal(e.h4toh.bias.grad[0], fused.experts.h4toh.bias.grad[i])


def test_fused_experts_are_indexable_like_the_reference_list():
    """Code written against `layer.experts[i]` (fmoe/transformer.py:51-55) keeps
    working on the fused module: views of the stacked parameters."""
    from fastmoe_amd import FMoETransformerMLP

    torch.manual_seed(4)
    layer = FMoETransformerMLP(5, 32, 64, top_k=2).cuda()
    ex = layer.experts
    assert len(ex) == 5 and len(list(ex)) == 5
    assert tuple(ex[1].htoh4.weight.shape) == (1, 64, 32) and tuple(ex[-1].h4toh.bias.shape) == (1, 32)
    assert ex[2].htoh4.weight.data_ptr() == ex.htoh4.weight[2].data_ptr()
    with pytest.raises(IndexError):
        ex[5]
    rows = torch.randn(40, 32, device="cuda")
    counts = torch.tensor([0, 0, 0, 40, 0])
    whole = ex(rows, counts)
    one = ex[3](rows, torch.tensor([40]))
    assert torch.equal(whole, one)
    one.sum().backward()
    assert ex.htoh4.weight.grad[3].any().item() and not ex.htoh4.weight.grad[0].any().item()
    assert sum(p.numel() for p in ex[0].parameters()) == 64 * 32 + 64 + 32 * 64 + 32


class _TwoInputExpert(torch.nn.Module):
    """tests/test_mimo.py:28-62: one fused expert applied to both entries of a
    dict or list input."""

    def __init__(self, num_expert, d_model, d_hidden, device_side):
        super().__init__()
        from fastmoe_amd import FMoELinear

        self.htoh4 = FMoELinear(num_expert, d_model, d_hidden, bias=True)
        self.h4toh = FMoELinear(num_expert, d_hidden, d_model, bias=True)
        # with this attribute FMoE hands over a device-side SegmentTable
        self.accepts_segment_table = device_side

    def _mlp(self, t, fec):
        return self.h4toh(F.gelu(self.htoh4(t, fec)), fec)

    def forward(self, inp, fwd_expert_count):
        if isinstance(inp, dict):
            return {k: self._mlp(v, fwd_expert_count) for k, v in inp.items()}
        return [self._mlp(v, fwd_expert_count) for v in inp]


def _mimo_layer(num_expert, d_model, d_hidden, top_k, device_side):
    from fastmoe_amd import FMoE, NaiveGate

    class Gate(NaiveGate):
        def forward(self, inp, return_all_scores=False):
            first = inp["x"] if isinstance(inp, dict) else inp[0]
            return super().forward(first, return_all_scores)

    class Layer(FMoE):
        def __init__(self):
            super().__init__(num_expert=num_expert, d_model=d_model, gate=Gate, top_k=top_k)
            self.experts = _TwoInputExpert(num_expert, d_model, d_hidden, device_side)

    return Layer()


@pytest.mark.parametrize("device_side", [False, True])
@pytest.mark.parametrize("list_input", [False, True])
@pytest.mark.parametrize("dt", ["f32", "f64", "f16", "bf16"])
@pytest.mark.parametrize("num_expert,top_k", [(4, 2), (8, 3)])
def test_nested_inputs_as_in_the_reference_mimo_suite(num_expert, top_k, dt, list_input,
                                                      device_side):
    """tests/test_mimo.py:100-150 (batch 4, d_model 16, d_hidden 64): a dict or
    list of two tensors goes through the layer; both entries must agree with each
    other (same data) and with the brute force, forward and backward, on the
    reference-shaped route and on the device-side one."""
    dtype = DTYPES[dt]
    torch.manual_seed(42)
    moe = _mimo_layer(num_expert, 16, 64, top_k, device_side)
    with torch.no_grad():
        for p in moe.experts.parameters():
            p.mul_(0).add_(torch.randn(p.shape) * 0.3)
    moe = moe.to(dtype).cuda()
    x = torch.rand(4, 16).to(dtype)
    a = x.cuda().requires_grad_(True)
    b = x.cuda().requires_grad_(True)
    inp = [a, b] if list_input else {"x": a, "y": b}
    out = moe(inp)
    first, second = (out[0], out[1]) if list_input else (out["x"], out["y"])
    assert type(out) is type(inp)
    assert torch.equal(first, second)
    (first.float().sum() + 2 * second.float().sum()).backward()
    with torch.no_grad():
        idx, score = moe.gate(inp)
    ex = moe.experts
    cpu = [t.detach().double().cpu().requires_grad_(True)
           for t in (ex.htoh4.weight, ex.htoh4.bias, ex.h4toh.weight, ex.h4toh.bias)]
    x_cpu = x.double().requires_grad_(True)
    s_cpu = score.double().cpu().requires_grad_(True)
    want = O.brute_force_moe_mlp(x_cpu, idx.cpu(), s_cpu, *cpu)
    (3 * want.sum()).backward()
    tol = {"f32": 1e-4, "f64": 1e-10, "f16": 1e-2, "bf16": 4e-2}[dt]
    assert max_rel_err(first, want) <= tol
    for got, ref in zip((ex.htoh4.weight.grad, ex.htoh4.bias.grad, ex.h4toh.weight.grad,
                         ex.h4toh.bias.grad), cpu):
        assert max_rel_err(got, ref.grad) <= tol
    # the second entry never reaches the gate: its gradient is the experts' share
    # alone, 2/3 of what the oracle's 3 x sum() sends back to x
    assert b.grad is not None and max_rel_err(b.grad, x_cpu.grad * (2.0 / 3.0)) <= tol


def _masked_reference(moe, x, mask, mask_dict):
    """Dense float64 restatement of the masked layer (fmoe/layers.py:240-295): masked
    tokens take no expert; each of their k slots holds mask_dict[mask value] (zeros
    without an entry); the combine weights every slot by the gate's score."""
    from oracle import moe_oracle as O

    with torch.no_grad():
        idx, score = moe.gate(x.cuda())
    idx, score = idx.cpu(), score.double().cpu().reshape(x.shape[0], -1)
    ex = moe.experts
    params = [p.detach().double().cpu().requires_grad_(True)
              for p in (ex.htoh4.weight, ex.htoh4.bias, ex.h4toh.weight, ex.h4toh.bias)]
    xd = x.double().cpu().requires_grad_(True)
    sd = score.clone().requires_grad_(True)
    live_idx = torch.where((mask == 0).view(-1, 1), idx, torch.full_like(idx, -1))
    out = O.brute_force_moe_mlp(xd, live_idx, sd, *params)
    for k, v in mask_dict.items():
        row = sd.sum(dim=1, keepdim=True) * v.double().cpu().view(1, -1)
        out = torch.where((mask == k).view(-1, 1), row, out)
    return out, xd, sd, params


@pytest.mark.parametrize("fused", [True, False])
def test_masked_layer_dispatches_on_the_device(fused):
    """mask / mask_dict (fmoe/layers.py:240-255,270-286) without the reference's
    row deletion: masked tokens lose their slots inside the routing kernels, their
    output rows come from mask_dict, and no call of the pass synchronises with the
    host.  Outputs and gradients against the dense restatement."""
    from fastmoe_amd import FMoETransformerMLP

    torch.manual_seed(11)
    t, d, h, e, k = 257, 64, 96, 5, 2
    mask = torch.zeros(t, dtype=torch.long)
    mask[3::7] = 1          # rows replaced by mask_dict[1]
    mask[5::11] = 2         # rows replaced by mask_dict[2]
    mask[6::13] = 3         # no entry: rows of zeros
    mask_dict = {1: torch.randn(d).cuda(), 2: torch.zeros(d).cuda()}
    moe = FMoETransformerMLP(e, d, h, top_k=k, mask=mask.cuda(), mask_dict=mask_dict,
                             fused=True).cuda()
    if not fused:
        plain = FMoETransformerMLP(e, d, h, top_k=k, mask=mask.cuda(), mask_dict=mask_dict,
                                   fused=False).cuda()
        plain.load_state_dict(moe.state_dict())
    else:
        plain = moe
    assert plain._device_side_dispatch()
    x = torch.randn(t, d)
    dy = torch.randn(t, d)
    a = x.clone().cuda().requires_grad_(True)
    dy_dev = dy.cuda()
    plain(a).backward(dy_dev)                    # warm-up (tables, attributes)
    a.grad = None
    for p in plain.parameters():
        p.grad = None
    # the gate's own path to x is kept out of the comparison: the scores become a leaf
    leaf = {}

    def cut(m, i, o):
        leaf["score"] = o[1].detach().requires_grad_(True)
        return o[0], leaf["score"]
    hook = plain.gate.register_forward_hook(cut)
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")      # any host synchronisation raises
    try:
        out = plain(a)
        out.backward(dy_dev)
    finally:
        torch.cuda.set_sync_debug_mode("default")
        hook.remove()
    want, xd, sd, params = _masked_reference(moe, x, mask, mask_dict)
    want.backward(dy.double())
    assert max_rel_err(out, want) <= 2e-5
    assert not out[mask == 3].any().item() and not out[mask == 2].any().item()
    assert max_rel_err(a.grad, xd.grad) <= 2e-5
    assert not a.grad[mask != 0].any().item()    # masked tokens reach no expert
    if fused:
        got = [moe.experts.htoh4.weight.grad, moe.experts.htoh4.bias.grad,
               moe.experts.h4toh.weight.grad, moe.experts.h4toh.bias.grad]
    else:
        got = [torch.cat([getattr(getattr(m, lin), par).grad for m in plain.experts])
               for lin, par in (("htoh4", "weight"), ("htoh4", "bias"), ("h4toh", "weight"),
                                ("h4toh", "bias"))]
    for g, p in zip(got, params):
        assert max_rel_err(g, p.grad) <= 2e-5
    # the score gradient of a masked token is <dy, its mask_dict row>
    assert max_rel_err(leaf["score"].grad.reshape(t, k), sd.grad) <= 2e-5
    assert leaf["score"].grad.reshape(t, k)[mask == 1].any().item()


def test_list_of_experts_with_hooks_takes_the_reference_route():
    """A forward hook on one module of the list must run: the grouped call on pointer
    tables never calls the modules, so such a list is dispatched the reference's way."""
    from fastmoe_amd import FMoETransformerMLP

    torch.manual_seed(5)
    plain = FMoETransformerMLP(4, 32, 64, top_k=2, fused=False).cuda()
    assert plain._device_side_dispatch()
    calls = []
    h = plain.experts[2].htoh4.register_forward_hook(lambda m, i, o: calls.append(2))
    try:
        assert not plain._device_side_dispatch()
        x = torch.randn(50, 32, device="cuda")
        want = plain(x)
    finally:
        h.remove()
    assert calls and plain._device_side_dispatch()
    assert max_rel_err(plain(x), want) <= 2e-5


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32", "f64"])
def test_pointer_table_ops_give_the_bits_of_the_stacked_call(dt):
    """fmoe_grouped_linear_{fwd,bwd}_ptrs on separately allocated per-expert weights
    against the same call on their concatenation (cuda/parallel_linear.cuh:69-87 takes
    per-expert pointers the same way): identical bits, every product, with and without
    the activation."""
    from fastmoe_amd import fmoe_cuda
    from helpers import DTYPES, randn

    dtype = DTYPES[dt]
    counts = [300, 0, 129, 64, 1, 0, 513]
    e, in_f, out_f = len(counts), 72, 136
    seg = torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32).cuda()
    n = sum(counts)
    x = randn((n, in_f), dtype, 1).cuda()
    dy = randn((n, out_f), dtype, 2).cuda()
    ws = [randn((1, out_f, in_f), dtype, 10 + i, 0.1).cuda() for i in range(e)]
    bs = [randn((1, out_f), dtype, 30 + i).cuda() for i in range(e)]
    w, b = torch.cat(ws), torch.cat(bs)
    wt, bt = fmoe_cuda.pointer_table(ws), fmoe_cuda.pointer_table(bs)
    assert wt.dtype == torch.int64 and wt.tolist() == [t.data_ptr() for t in ws]
    y = fmoe_cuda.grouped_linear_fwd(x, seg, w, b)
    assert torch.equal(fmoe_cuda.grouped_linear_fwd_ptrs(x, seg, wt, bt, out_f), y)
    assert torch.equal(fmoe_cuda.grouped_linear_fwd_ptrs(x, seg, wt, None, out_f),
                       fmoe_cuda.grouped_linear_fwd(x, seg, w, None))
    ya, aa = fmoe_cuda.grouped_linear_fwd(x, seg, w, b, with_gelu=True)
    yb, ab = fmoe_cuda.grouped_linear_fwd_ptrs(x, seg, wt, bt, out_f, with_gelu=True)
    assert torch.equal(ya, yb) and torch.equal(aa, ab)
    for act_pre in (None, randn((n, in_f), dtype, 3).cuda()):
        ga = fmoe_cuda.grouped_linear_bwd(dy, x, seg, w, act_pre=act_pre)
        gb = fmoe_cuda.grouped_linear_bwd_ptrs(dy, x, seg, wt, act_pre=act_pre)
        for p, q in zip(ga, gb):
            assert p.shape == q.shape and torch.equal(p, q)
    only_dx = fmoe_cuda.grouped_linear_bwd_ptrs(dy, x, seg, wt, need_bias=False, need_dw=False)
    assert only_dx[1] is None and only_dx[2] is None
    assert torch.equal(only_dx[0], fmoe_cuda.grouped_linear_bwd(dy, x, seg, w)[0])
