"""Host-side logic that needs no GPU: nested-input helpers, module
construction, checkpoint layouts, gate arithmetic, argument checks."""
import collections

import pytest
import torch

from fastmoe_amd import _tree as tree


def test_tree_map_and_flatten():
    nt = collections.namedtuple("nt", "a b")
    s = {"x": [1, 2, (3, 4)], "y": nt(5, 6)}
    doubled = tree.map_structure(lambda v: v * 2, s)
    assert doubled == {"x": [2, 4, (6, 8)], "y": nt(10, 12)}
    assert tree.flatten(s) == [1, 2, 3, 4, 5, 6]
    assert tree.map_structure(lambda a, b: a + b, [1, {"k": 2}], [10, {"k": 20}]) == [11, {"k": 22}]
    assert tree.flatten(7) == [7]


def test_layer_constructor_mirrors_the_reference():
    from fastmoe_amd import FMoE, FMoELinear, FMoETransformerMLP, NaiveGate

    m = FMoETransformerMLP(num_expert=4, d_model=16, d_hidden=32, top_k=3)
    assert m.experts_fused and m.top_k == 3 and m.num_expert == 4
    assert isinstance(m.gate, NaiveGate) and m.gate.gate.out_features == 4
    assert tuple(m.experts.htoh4.weight.shape) == (4, 32, 16)
    assert tuple(m.experts.h4toh.bias.shape) == (4, 16)
    assert all(getattr(p, "dp_comm") == "none" for p in m.experts.parameters())
    assert all(getattr(p, "dp_comm") == "gate" for p in m.gate.parameters())
    plain = FMoETransformerMLP(num_expert=4, d_model=16, d_hidden=32, fused=False)
    assert not plain.experts_fused and len(plain.experts) == 4
    assert tuple(plain.experts[0].htoh4.weight.shape) == (1, 32, 16)
    lin = FMoELinear(3, 8, 5, bias=False)
    assert lin.bias is None and "num_expert=3" in lin.extra_repr()
    with pytest.raises(NotImplementedError):
        FMoE(num_expert=2, d_model=8, world_size=2)
    listed = FMoE(num_expert=7, d_model=8, expert=[lambda d: torch.nn.Linear(d, d)] * 3)
    assert listed.num_expert == 3 and not listed.experts_fused


def test_checkpoints_convert_between_expert_layouts():
    from fastmoe_amd import FMoETransformerMLP

    torch.manual_seed(0)
    fused = FMoETransformerMLP(num_expert=3, d_model=8, d_hidden=12)
    plain = FMoETransformerMLP(num_expert=3, d_model=8, d_hidden=12, fused=False)
    plain.load_state_dict(fused.state_dict())
    for i in range(3):
        assert torch.equal(plain.experts[i].htoh4.weight[0], fused.experts.htoh4.weight[i])
        assert torch.equal(plain.experts[i].h4toh.bias[0], fused.experts.h4toh.bias[i])
    back = FMoETransformerMLP(num_expert=3, d_model=8, d_hidden=12)
    back.load_state_dict(plain.state_dict())
    assert torch.equal(back.experts.h4toh.weight, fused.experts.h4toh.weight)
    assert torch.equal(back.gate.gate.weight, fused.gate.gate.weight)


def test_naive_gate_is_topk_then_softmax():
    from fastmoe_amd import NaiveGate

    torch.manual_seed(1)
    gate = NaiveGate(8, 6, 1, top_k=2)
    x = torch.randn(10, 8)
    idx, score, logits = gate(x, return_all_scores=True)
    val, ref_idx = torch.topk(gate.gate(x), 2, dim=-1)
    assert torch.equal(torch.sort(idx, 1).values, torch.sort(ref_idx, 1).values)
    assert torch.allclose(score.sum(1), torch.ones(10))
    assert torch.allclose(torch.sort(score, 1).values,
                          torch.sort(torch.softmax(val, -1), 1).values)
    assert gate.has_loss and gate.get_loss() is not None and not gate.has_loss


def test_operator_module_rejects_host_tensors_with_runtime_error():
    from fastmoe_amd import fmoe_cuda

    with pytest.raises(RuntimeError):
        fmoe_cuda.expert_count(torch.zeros(4, dtype=torch.int64),
                               torch.zeros(2, dtype=torch.int32))
    with pytest.raises(RuntimeError):
        fmoe_cuda.local_scatter(torch.zeros(4, 8), torch.zeros(2, dtype=torch.int64))
    with pytest.raises(RuntimeError):
        fmoe_cuda.route(torch.zeros(4, dtype=torch.int64), 2)


def test_install_as_fmoe_cuda_registers_the_module():
    import sys

    import fastmoe_amd

    saved = sys.modules.pop("fmoe_cuda", None)
    try:
        fastmoe_amd.install_as_fmoe_cuda()
        import fmoe_cuda  # noqa: F401

        for name in ("expert_count", "assign_pos", "linear_forward", "linear_backward",
                     "limit_by_capacity", "prune_gate_by_capacity"):
            assert callable(getattr(sys.modules["fmoe_cuda"], name))
    finally:
        sys.modules.pop("fmoe_cuda", None)
        if saved is not None:
            sys.modules["fmoe_cuda"] = saved


def test_bench_workloads_are_seeded_and_shaped():
    import bench

    for name, cfg in bench.CONFIGS.items():
        if cfg["T"] > 8192:
            continue
        logits, idx = bench.make_routing(dict(cfg, name=name))
        logits2, _ = bench.make_routing(dict(cfg, name=name))
        assert torch.equal(logits, logits2)
        assert logits.shape[0] == cfg["T"]
    cfg5 = bench.CONFIGS["cfg5"]
    logits, _ = bench.make_routing(cfg5)
    assert int(torch.isinf(logits[0]).sum()) == 13          # 13 experts never chosen
    work = bench.kernel_work(bench.CONFIGS["cfg2"], 16384)
    assert work["grouped_linear_fwd"] == ("flop", 2.0 * 16384 * 1024 * 4096)
    assert work["local_scatter"][1] == 2.0 * 16384 * 1024 * 2 + 8.0 * 16384
