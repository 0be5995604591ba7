"""The routing entry point that allocates nothing (fmoe_route_static) against the
workspace-taking one (fmoe_route), through the C ABI: bit-exact outputs on two
calls in a row, the second on a smaller input (the built-in scratch buffer
still holds the first call's tables), plus the size limit."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import make_gate

pytestmark = pytest.mark.gpu


def _route_both(lib, gate_np, n_expert, stream):
    gate = torch.from_numpy(gate_np).cuda()
    n = gate.numel()

    def outputs():
        # poisoned, so that an entry the call should write and does not shows up
        return (torch.full((n_expert,), -7, dtype=torch.int64, device="cuda"),
                torch.full((n_expert + 1,), -7, dtype=torch.int32, device="cuda"),
                torch.full((n,), -7, dtype=torch.int64, device="cuda"),
                torch.full((n,), -7, dtype=torch.int32, device="cuda"))

    a, b = outputs(), outputs()
    ws_bytes = lib.fmoe_route_workspace_bytes(n, n_expert)
    ws = torch.empty(max(int(ws_bytes), 1), dtype=torch.uint8, device="cuda")
    rc = lib.fmoe_route(gate.data_ptr(), n, n_expert, a[0].data_ptr(), a[1].data_ptr(),
                        a[2].data_ptr(), a[3].data_ptr(), ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, lib.fmoe_last_error()
    rc = lib.fmoe_route_static(gate.data_ptr(), n, n_expert, b[0].data_ptr(), b[1].data_ptr(),
                               b[2].data_ptr(), b[3].data_ptr(), stream)
    assert rc == 0, lib.fmoe_last_error()
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in a], [t.cpu().numpy() for t in b]


def test_route_static_matches_route_on_two_calls_in_a_row():
    from fastmoe_amd import _lib
    from oracle import moe_oracle as O

    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    # config-5 sized first (65536 slots, 128 experts, 13 of them empty, some drops),
    # then a smaller, differently shaped input that reuses the scratch buffer
    cases = [(8192, 8, 128, tuple(range(0, 128, 10)), 0.05, 1),
             (1000, 2, 16, (), 0.2, 2),
             (3, 1, 5, (), 0.0, 3)]
    for n_tokens, top_k, n_expert, empty, drop, seed in cases:
        gate = make_gate(n_tokens, top_k, n_expert, drop=drop, seed=seed, empty=empty)
        want, got = _route_both(lib, gate, n_expert, stream)
        for w, g, name in zip(want, got, ("count", "seg_off", "pos", "inv")):
            assert np.array_equal(w, g), f"{name} differs at {n_tokens}x{top_k}, E={n_expert}"
        # and both agree with the CPU checker where the call defines the result
        pos, count, seg_off, inv = O.route(gate, n_expert)
        assert np.array_equal(got[0], count) and np.array_equal(got[1], seg_off)
        assert np.array_equal(got[2][: len(pos)], pos) and np.array_equal(got[3], inv)


def test_route_static_rejects_sizes_beyond_its_buffer():
    from fastmoe_amd import _lib

    lib = _lib.load()
    n, e = 1 << 24, 4096            # 8192 blocks x 4096 experts x 4 bytes = 128 MiB of tables
    assert lib.fmoe_route_workspace_bytes(n, e) > 4 * 1024 * 1024
    rc = lib.fmoe_route_static(None, n, e, None, None, None, None, None)
    assert rc == -4 and b"route_static" in lib.fmoe_last_error()


def test_route_static_python_wrapper():
    from fastmoe_amd import fmoe_cuda

    gate = torch.from_numpy(make_gate(500, 2, 8, drop=0.1, seed=5)).cuda()
    pos, count, seg, inv = fmoe_cuda.route(gate, 8)
    c2 = torch.empty_like(count)
    s2 = torch.empty_like(seg)
    p2 = torch.zeros_like(pos)
    i2 = torch.empty_like(inv)
    fmoe_cuda.route_static(gate, 8, c2, s2, p2, i2)
    n_valid = int(seg[-1])
    assert torch.equal(c2, count) and torch.equal(s2, seg) and torch.equal(i2, inv)
    assert torch.equal(p2[:n_valid], pos[:n_valid])
