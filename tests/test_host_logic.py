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


def _descriptor_checker(tmp_path):
    """Compiles the grouped GEMM's descriptor arithmetic (csrc/dma_desc.h) for the
    host and hands back its three functions."""
    import ctypes
    import os
    import subprocess

    from conftest import ROOT

    src = tmp_path / "dma_desc_host.cpp"
    src.write_text(
        '#include "dma_desc.h"\n'
        'extern "C" long long valid_bytes(int kc, int rv, int rs, int ld, int kt) {\n'
        '  return fmoe::dma_valid_bytes(kc != 0, rv, rs, ld, kt); }\n'
        'extern "C" int num_records(long long r) { return fmoe::dma_num_records(r); }\n'
        'extern "C" int ld_ok(long long ld) { return fmoe::dma_ld_supported(ld); }\n')
    so = tmp_path / "dma_desc_host.so"
    subprocess.run(["g++", "-O1", "-shared", "-fPIC", "-I",
                    os.path.join(ROOT, "fastmoe_amd", "csrc"), str(src), "-o", str(so)], check=True)
    lib = ctypes.CDLL(str(so))
    lib.valid_bytes.restype = ctypes.c_longlong
    lib.valid_bytes.argtypes = [ctypes.c_int] * 5
    lib.num_records.argtypes = [ctypes.c_longlong]
    lib.ld_ok.argtypes = [ctypes.c_longlong]
    return lib


def test_gemm_descriptors_survive_experts_beyond_2_to_the_31_bytes(tmp_path):
    """The weight-gradient product walks the rows of one expert as its K index:
    rows x features x 2 bytes passes 2^31 for a long expert.  The byte count must
    stay exact (64-bit) and the descriptor's 32-bit num_records must neither wrap
    nor cut off rows that exist; rows past the end must still read as zeros."""
    lib = _descriptor_checker(tmp_path)
    out_of_range = 0x80000000
    for rows, ld, bk in ((300000, 4096, 32), (75000, 14336, 64), (1 << 20, 16384, 64),
                         (1000, 1024, 32)):
        r_span = min(256, ld)
        total = lib.valid_bytes(0, r_span, r_span, ld, rows)
        assert total == ((rows - 1) * ld + r_span) * 2          # exact, no wrap
        step = bk * ld * 2
        for t in (0, 1, (rows // bk) // 2, rows // bk - 1, rows // bk, rows // bk + 1):
            remaining = total - t * step
            rec = lib.num_records(remaining)
            assert 0 <= rec < out_of_range
            k_left = rows - t * bk
            for k in range(bk):
                first = (k * ld) * 2                             # first pack of K row k
                last = (k * ld + r_span - 8) * 2                 # last valid pack of it
                assert last + 16 < out_of_range
                if k < k_left:
                    assert last + 16 <= rec, (rows, ld, t, k)    # existing rows are readable
                else:
                    assert first >= rec, (rows, ld, t, k)        # rows past the end are not
    # [row][k] operands: 256 rows of the widest supported feature size
    ld = (out_of_range // 512) - 8
    assert lib.ld_ok(ld) and not lib.ld_ok(out_of_range // 512)
    total = lib.valid_bytes(1, 256, 0, ld, ld)
    assert total == (255 * ld + ld) * 2 and lib.num_records(total) == total
    assert lib.num_records(0) == 0 and lib.num_records(-4096) == 0
    assert lib.valid_bytes(0, 256, 256, 4096, 0) == 0            # expert without rows


def test_stale_library_is_detected(tmp_path):
    """A binary built from other sources is told apart without loading it."""
    from fastmoe_amd import _lib, build

    assert build.built_hash(_lib.LIB_PATH) == build.source_hash()
    assert build.source_hash().encode() in _lib.load().fmoe_version()
    fake = tmp_path / "libfmoe_hip.so"
    blob = open(_lib.LIB_PATH, "rb").read()
    marker = build.HASH_MARKER.encode()
    at = blob.find(marker) + len(marker)
    fake.write_bytes(blob[:at] + b"0" * 12 + blob[at + 12:])
    assert build.built_hash(str(fake)) == "0" * 12 != build.source_hash()
