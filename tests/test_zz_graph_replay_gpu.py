"""HIP-graph capture and replay of the whole layer (forward + backward).  Kept
in a file of its own that pytest collects last."""
import pytest
import torch

from test_layer_gpu import _make

pytestmark = pytest.mark.gpu


def test_forward_and_backward_replay_from_a_hip_graph():
    """The fused layer enqueues without reading anything back to the host, so
    forward + backward can be captured once and replayed on new data whose
    routing differs.  Every replay is checked against the eager layer, with
    eager work and synchronisations between the replays."""
    dtype = torch.bfloat16
    moe = _make(8, 128, 256, 2, dtype, seed=5, scale=0.05)
    g = torch.Generator().manual_seed(21)
    xs = [torch.randn(300, 128, generator=g).to(dtype).cuda() for _ in range(4)]
    dys = [torch.randn(300, 128, generator=g).to(dtype).cuda() for _ in range(4)]
    params = list(moe.parameters())

    def eager(x, dy):
        for p in params:
            p.grad = None
        xi = x.clone().requires_grad_(True)
        out = moe(xi)
        out.backward(dy)
        return [out.detach().clone(), xi.grad.clone()] + [p.grad.clone() for p in params]

    want = [eager(x, dy) for x, dy in zip(xs, dys)]    # also warms every kernel up
    static_x = xs[0].clone().requires_grad_(True)
    static_dy = dys[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # warm-up on the capture stream
        for _ in range(2):
            for p in params:
                p.grad = None
            static_x.grad = None
            moe(static_x).backward(static_dy)
    torch.cuda.current_stream().wait_stream(side)
    for p in params:
        p.grad = None
    static_x.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = moe(static_x)
        static_out.backward(static_dy)
    # the tensors the graph writes (eager steps below rebind p.grad to new ones)
    got = [static_out, static_x.grad] + [p.grad for p in params]
    for i in (1, 2, 3, 0, 2):
        with torch.no_grad():
            static_x.copy_(xs[i])
            static_dy.copy_(dys[i])
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(got, want[i]):
            assert torch.equal(a, b)
        _ = eager(xs[(i + 1) % 4], dys[(i + 1) % 4])   # eager work between replays
        torch.cuda.synchronize()


def test_make_graphed_callables_replays_the_layer():
    """fastmoe_amd.graphed (torch.cuda.make_graphed_callables behind the library's
    set-up) captures the layer's forward and backward in two graphs behind an ordinary
    autograd interface.  The graphed layer gives the bits of an eager twin on new data
    with other routings, with eager work and synchronisations between its calls."""
    import copy

    import fastmoe_amd

    dtype = torch.bfloat16
    moe = _make(8, 128, 256, 2, dtype, seed=5, scale=0.05)
    twin = copy.deepcopy(moe)
    g = torch.Generator().manual_seed(22)
    xs = [torch.randn(300, 128, generator=g).to(dtype).cuda() for _ in range(4)]
    dys = [torch.randn(300, 128, generator=g).to(dtype).cuda() for _ in range(4)]

    def run(layer, x, dy):
        params = list(layer.parameters())
        for p in params:
            p.grad = None
        xi = x.clone().requires_grad_(True)
        out = layer(xi)
        out.backward(dy)
        return [out.detach().clone(), xi.grad.clone()] + [p.grad.clone() for p in params]

    want = [run(twin, x, dy) for x, dy in zip(xs, dys)]
    graphed = fastmoe_amd.graphed(moe, xs[0].clone().requires_grad_(True))
    for i in (1, 2, 3, 0, 2):
        got = run(graphed, xs[i], dys[i])
        torch.cuda.synchronize()
        for a, b in zip(got, want[i]):
            assert torch.equal(a, b)
        _ = run(twin, xs[(i + 1) % 4], dys[(i + 1) % 4])
        torch.cuda.synchronize()
