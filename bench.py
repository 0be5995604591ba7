#!/usr/bin/env python3
"""Benchmark of the single-GPU MoE-MLP hot path on one MI355X.

A step is one forward + backward pass of the MoE MLP (route, scatter, two
grouped expert GEMMs with GELU between them, gather fused with the top-k
combine, and the whole backward) over one batch of synthetic input that is
already resident in HBM.  Prints ONE JSON line:

  metric / value      MoE-MLP fwd+bwd tokens/s (whole job, one GPU)
  roofline            the kernel that takes the most time in a step: achieved
                      algorithmic FLOP/s (or bytes/s) per launch, from HIP
                      events recorded around every launch inside the timed
                      region on the stream the kernels run on.  A grouped GEMM
                      is priced against the roofline its own arithmetic puts
                      it under: HBM when every operand and result moved once
                      at 8 TB/s takes longer than its FLOPs at the matrix
                      cores' peak (many short experts on large weights),
                      else MFMA; the other fraction rides along
  cpu_baseline        the CPU checker's brute-force layer (torch fp32 on the
                      host cores) timed on a bounded sample of the same workload
  kernels             per-kernel average time and achieved rate, from an untimed
                      pass with events around every op (the dominant op's entry
                      comes from the timed region)

usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg4]
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import torch  # noqa: E402
import torch.nn.functional as F  # noqa: E402

# T tokens, d d_model, h d_hidden, E experts, k top-k
CONFIGS = {
    "cfg1": dict(T=512, d=128, h=256, E=4, k=2, dtype="f32", x_std=0.02,
                 note="CPU-plumbing case: N(0,0.02) inputs and weights"),
    "cfg2": dict(T=8192, d=1024, h=4096, E=16, k=2, dtype="bf16",
                 note="balanced: gate logits N(0,1)"),
    "cfg3": dict(T=16384, d=2048, h=8192, E=64, k=2, dtype="bf16", zipf=1.2,
                 cap_factor=1.25, note="Zipf(1.2) routing, capacity factor 1.25"),
    "cfg4": dict(T=16384, d=4096, h=14336, E=8, k=2, dtype="bf16",
                 note="Mixtral-sized layer"),
    "cfg5": dict(T=8192, d=2048, h=1408, E=128, k=8, dtype="bf16", n_empty=13,
                 note="fine-grained experts, 13 of 128 empty"),
}
DTYPES = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
PEAK = {"hbm": 8.0e12, "bf16": 2.5e15, "f16": 2.5e15, "f32": 157.3e12}

# Bytes per launch (read + write) that leave L2 towards the Infinity Cache and
# HBM, from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs of this script
# (`--counter-pass`; the commands and per-kernel tables are in
# profiles/moe_step_<config>_hbm_traffic.md), scaled by what the same counters read in
# the same run for the row-scatter kernel, whose traffic is known: FETCH_SIZE x 0.998
# on cfg4 and x 1.035 on cfg2 (applied to cfg1, cfg3 and cfg5 as well, whose scatter
# reads part of its input from L2), WRITE_SIZE x 1.000.  MiB, read + written.  A
# config without an entry for its dominant op makes the run fail: measure, then add.
MiB = 2 ** 20
MEASURED_TRAFFIC = {
    ("cfg1", "grouped_linear_bwd"): (2.68 + 1.25) * MiB,             # dX, dW and bias-gradient kernels
    ("cfg1", "grouped_linear_fwd"): (1.22 + 0.75) * MiB,
    ("cfg1", "grouped_linear_fwd_act"): (1.22 + 0.75) * MiB,
    ("cfg2", "grouped_linear_bwd"): (310.9 + 214.6) * MiB,           # avg of both layers
    ("cfg2", "grouped_linear_fwd"): (172.1 + 32.2) * MiB,
    ("cfg2", "grouped_linear_fwd_act"): (138.6 + 257.0) * MiB,
    ("cfg3", "grouped_linear_bwd"): (2103.5 + 2297.3) * MiB,         # avg of both layers
    ("cfg3", "grouped_linear_fwd"): (1570.1 + 159.4) * MiB,
    ("cfg3", "grouped_linear_fwd_act"): (1570.1 + 159.4 + 127.2 + 253.3) * MiB,  # + activation kernel
    ("cfg4", "grouped_linear_bwd"): (6009.1 + 1517.7) * MiB,         # avg of both layers
    ("cfg4", "grouped_linear_fwd"): (2928.1 + 258.0) * MiB,
    ("cfg4", "grouped_linear_fwd_act"): (2927.0 + 1799.0) * MiB,
    ("cfg5", "grouped_linear_bwd"): (1248.4 + 949.7) * MiB,          # avg of both layers
    ("cfg5", "grouped_linear_fwd"): (815.8 + 217.5) * MiB,
    ("cfg5", "grouped_linear_fwd_act"): (815.8 + 217.5 + 88.5 + 176.0) * MiB,    # + activation kernel
}


def make_routing(cfg: dict, seed: int = 0):
    """(logits [T, E] float32 or None, idx [T, k] int64 or None): the seeded
    synthetic routing of a configuration, generated on the CPU."""
    g = torch.Generator().manual_seed(seed)
    T, E, k = cfg["T"], cfg["E"], cfg["k"]
    if "zipf" in cfg:
        p = torch.arange(1, E + 1, dtype=torch.float64) ** (-cfg["zipf"])
        idx = torch.multinomial((p / p.sum()).expand(T, -1), k, replacement=False,
                                generator=g)
        logits = torch.randn(T, k, generator=g)   # softmax of these gives the scores
        return logits, idx
    logits = torch.randn(T, E, generator=g)
    for e in range(cfg.get("n_empty", 0)):
        logits[:, (e * E) // cfg["n_empty"]] = float("-inf")
    return logits, None


class PresetGate(torch.nn.Module):
    """Gate whose decisions are part of the workload, independent of x: top-k of
    preset logits and the softmax of the k values (the NaiveGate arithmetic,
    fmoe/gates/naive_gate.py:31-38), or preset Zipf choices clipped to the
    capacity by the native limit/prune ops."""

    cfg = None  # set before the layer is constructed

    def __init__(self, d_model, num_expert, world_size, top_k=2):
        super().__init__()
        cfg = PresetGate.cfg
        self.top_k = top_k
        self.num_expert = num_expert
        logits, idx = make_routing(cfg)
        self.logits = torch.nn.Parameter(logits)
        self.register_buffer("idx", idx if idx is not None else torch.zeros(0, dtype=torch.int64))
        self.capacity = None
        if "cap_factor" in cfg:
            self.capacity = math.ceil(cfg["cap_factor"] * cfg["T"] * cfg["k"] / cfg["E"])
        self.dtype = DTYPES[cfg["dtype"]]

    def forward(self, inp):
        if self.idx.numel():
            from fastmoe_amd.gates import limit_by_capacity

            idx = self.idx
            score = F.softmax(self.logits, dim=-1)
            if self.capacity is not None:
                _l, _g, idx = limit_by_capacity(idx, self.num_expert, 1, self.capacity)
        else:
            from fastmoe_amd.functions import topk_softmax

            idx, score = topk_softmax(self.logits, self.top_k)
        return idx, score.to(self.dtype)


def build_layer(cfg: dict, device="cuda", fused=True):
    """The layer with seeded weights, its input and the gradient of its output.
    fused=False builds the reference's expert layout, one module per expert
    (fmoe/transformer.py:51-55), with values from the same generator."""
    from fastmoe_amd import FMoETransformerMLP

    dtype = DTYPES[cfg["dtype"]]
    PresetGate.cfg = cfg
    torch.manual_seed(0)
    layer = FMoETransformerMLP(num_expert=cfg["E"], d_model=cfg["d"], d_hidden=cfg["h"],
                               top_k=cfg["k"], gate=PresetGate, fused=fused)
    g = torch.Generator().manual_seed(1)
    with torch.no_grad():
        for p in layer.experts.parameters():
            p.copy_(torch.randn(p.shape, generator=g) * 0.02)
    gate_logits = layer.gate.logits.data
    layer = layer.to(dtype)
    layer.gate.logits.data = gate_logits          # routing logits stay fp32
    layer = layer.to(device)
    x = (torch.randn(cfg["T"], cfg["d"], generator=g) * cfg.get("x_std", 1.0)).to(dtype)
    dy = torch.randn(cfg["T"], cfg["d"], generator=g).to(dtype)
    return layer, x.to(device), dy.to(device)


def step(layer, x, dy):
    for p in layer.parameters():
        p.grad = None
    x.grad = None
    out = layer(x)
    out.backward(dy)
    return out


def graph_replay(layer, x, dy, cfg, steps):
    """The same step captured once in a HIP graph and replayed `steps` times: the
    layer enqueues without reading anything back, so the capture is legal and the
    replay shows the step without its host-side launch cost."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(layer, x, dy)
    torch.cuda.current_stream().wait_stream(side)
    for p in layer.parameters():
        p.grad = None
    x.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        layer(x).backward(dy)
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    return {"ms_per_step": round(ms, 4), "tokens_per_s": round(cfg["T"] / (ms * 1e-3), 1)}


# ---------------------------------------------------------------- accounting
def kernel_work(cfg: dict, n_valid: int):
    """Algorithmic FLOPs / bytes of ONE launch of each op on this workload."""
    T, d, h, E, k = cfg["T"], cfg["d"], cfg["h"], cfg["E"], cfg["k"]
    s = 4 if cfg["dtype"] == "f32" else 2
    N = T * k
    gemm = 2.0 * n_valid * d * h
    return {
        "grouped_linear_fwd": ("flop", gemm),
        "grouped_linear_fwd_act": ("flop", gemm),        # first layer, gelu from the same tiles
        "grouped_linear_dgrad": ("flop", gemm),
        "grouped_linear_wgrad": ("flop", gemm),
        "grouped_linear_bwd": ("flop", 2.0 * gemm),      # dX and dW in one launch
        # both layers' bias gradients average to (rows*(d+h)/2) elements read
        "grouped_linear_bias_grad": ("byte", n_valid * (d + h) / 2.0 * s),
        "route": ("byte", 8.0 * N + 8.0 * n_valid + 4.0 * N + 8.0 * N),
        "local_scatter": ("byte", 2.0 * n_valid * d * s + 8.0 * n_valid),
        "scatter_tokens": ("byte", T * d * s + n_valid * d * s + 4.0 * N),
        "gather_combine_fwd": ("byte", n_valid * d * s + T * d * s + N * (4 + s)),
        "gather_combine_bwd": ("byte", T * d * s + 2.0 * n_valid * d * s + N * (4 + 2 * s)),
        "scatter_reduce": ("byte", n_valid * d * s + T * d * s + 4.0 * N),
        "expert_count": ("byte", 8.0 * N),
        "topk_softmax_fwd": ("byte", 4.0 * T * E + 12.0 * N),
        "topk_softmax_bwd": ("byte", 4.0 * T * E + 16.0 * N),
        "gelu_fwd": ("byte", 2.0 * n_valid * h * s),
        "gelu_bwd": ("byte", 3.0 * n_valid * h * s),
        "limit_by_capacity": ("byte", 20.0 * E),
        "prune_gate_by_capacity": ("byte", 24.0 * N),
    }


def gemm_bytes(cfg: dict, n_valid: int, e_live: int):
    """Algorithmic HBM bytes of ONE launch of each grouped GEMM: every operand and
    result once.  Experts without rows have no tiles in the forward and dX products
    (their weights are not read); dW writes every expert's gradient, zeros included.
    A workload of many short experts (cfg3: 64 experts of 62-640 rows on 32 MiB
    weights) moves more bytes per FLOP than the matrix-core roofline's ridge, and is
    then to be read against the HBM roofline."""
    d, h, E = cfg["d"], cfg["h"], cfg["E"]
    s = 4 if cfg["dtype"] == "f32" else 2
    rows = n_valid * (d + h) * s          # one activation operand + one result, avg of both layers
    w_live, w_all = e_live * d * h * s, E * d * h * s
    return {
        "grouped_linear_fwd": rows + w_live,
        "grouped_linear_fwd_act": rows + n_valid * h * s + w_live,     # second result: gelu
        "grouped_linear_dgrad": rows + w_live,
        "grouped_linear_wgrad": rows + w_all,
        "grouped_linear_bwd": 1.5 * rows + w_live + w_all,             # dy, x read; dx written
    }


def cpu_baseline(cfg: dict, layer, x, target_seconds: float = 15.0):
    """The CPU checker's brute-force layer (fp32, all host threads) on the first
    S tokens of the workload, S sized for about `target_seconds` of work."""
    from oracle import moe_oracle as O

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    ex = layer.experts
    with torch.no_grad():
        idx_all, score_all = layer.gate(x)
    w = [p.detach().float().cpu() for p in (ex.htoh4.weight, ex.htoh4.bias,
                                            ex.h4toh.weight, ex.h4toh.bias)]

    def run(S):
        xs = x[:S].float().cpu().requires_grad_(True)
        ps = [t.clone().requires_grad_(True) for t in w]
        t0 = time.perf_counter()
        out = O.brute_force_moe_mlp(xs, idx_all[:S].cpu(), score_all[:S].float().cpu(), *ps)
        out.sum().backward()
        return time.perf_counter() - t0

    T = cfg["T"]
    probe = max(64, T // 32)
    run(probe)                                   # warm-up (thread pool, allocator)
    t_probe = run(probe)
    S = int(min(T, max(probe, probe * target_seconds / 3.0 / max(t_probe, 1e-6))))
    t_first = run(S)
    # the small probe overstates the per-token cost (per-expert overheads):
    # rescale once from the first full-size run
    if t_first < target_seconds / 6.0 and S < T:
        S = int(min(T, S * target_seconds / 3.0 / max(t_first, 1e-6)))
        t_first = run(S)
    times = [t_first] + [run(S) for _ in range(2)]
    best = min(times)
    return {
        "value": S / best,
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"first {S} of {T} tokens of {cfg['name']}, fp32 torch on the host, "
                  f"fwd+bwd, best of 3 ({best:.3f} s)",
    }


def yardstick(cfg: dict, layer, seg_off, iters: int = 5):
    """The expert GEMMs of this workload as the BLAS library runs them: torch.mm
    (hipBLASLt) on the same weights and row segments.  Two forms per product and layer:
    `loop`, one call per expert on its own rows (the reference's algorithm,
    cuda/parallel_linear.cuh:55-163, a loop of BLAS calls), and `dense`, ONE call with
    all rows against one expert's weight (no ragged edges, no small problems: what
    the library reaches on this shape at its best).  Untimed leg, for comparison only:
    nothing of the product path runs through it."""
    ex = layer.experts
    dtype = DTYPES[cfg["dtype"]]
    seg = seg_off.cpu().tolist()
    n = seg[-1]
    dev = ex.htoh4.weight.device
    g = torch.Generator(device="cpu").manual_seed(7)
    out = {"what": "torch.mm (hipBLASLt) on this workload's weights and row segments; "
                   "loop = one call per expert (the reference's algorithm), dense = one call, "
                   "all rows x one expert's weight", "products": {}}
    peak = PEAK[cfg["dtype"]]

    def timed(fn):
        for _ in range(2):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        b.synchronize()
        return a.elapsed_time(b) * 1e-3 / iters

    for name, lin in (("layer1", ex.htoh4), ("layer2", ex.h4toh)):
        w = lin.weight.detach()                       # [E, out, in]
        out_f, in_f = w.shape[1], w.shape[2]
        x = (torch.randn(n, in_f, generator=g) * 0.5).to(dtype).to(dev)
        dy = (torch.randn(n, out_f, generator=g) * 0.5).to(dtype).to(dev)
        live = [(e, seg[e], seg[e + 1]) for e in range(len(seg) - 1) if seg[e + 1] > seg[e]]
        flop = 2.0 * n * in_f * out_f
        forms = {
            "fwd": (lambda: [torch.mm(x[a:b], w[e].t()) for e, a, b in live],
                    lambda: torch.mm(x, w[0].t())),
            "dgrad": (lambda: [torch.mm(dy[a:b], w[e]) for e, a, b in live],
                      lambda: torch.mm(dy, w[0])),
            "wgrad": (lambda: [torch.mm(dy[a:b].t(), x[a:b]) for e, a, b in live],
                      lambda: torch.mm(dy.t(), x)),
        }
        for prod, (loop, dense) in forms.items():
            t_loop, t_dense = timed(loop), timed(dense)
            out["products"][f"{name}_{prod}"] = {
                "loop_us": round(t_loop * 1e6, 1),
                "loop_frac_of_peak": round(flop / t_loop / peak, 4),
                "dense_us": round(t_dense * 1e6, 1),
                "dense_frac_of_peak": round(flop / t_dense / peak, 4),
            }
        del x, dy
    p = out["products"]
    for form in ("loop", "dense"):
        tot = sum(v[f"{form}_us"] for v in p.values())
        out[f"{form}_total_us"] = round(tot, 1)
        out[f"{form}_frac_of_peak"] = round(
            12.0 * n * cfg["d"] * cfg["h"] / (tot * 1e-6) / peak, 4)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="cfg4", choices=sorted(CONFIGS),
                    help="workload; the default is the largest single-GPU configuration")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--binding", default="compiled", choices=["compiled", "ctypes"],
                    help="Python binding of the C ABI: the compiled pybind11 extension "
                         "(default) or the ctypes calls (need nothing but the shared "
                         "library, more host time per step); both feed the per-op event hook")
    ap.add_argument("--layout", default="fused", choices=["fused", "list"],
                    help="expert parameters as [E, out, in] tensors (default) or as the "
                         "reference's list of single-expert modules (the kernels then read "
                         "the weights through pointer tables); list implies --no-cpu "
                         "--no-yardstick")
    ap.add_argument("--counter-pass", action="store_true",
                    help="for the rocprofv3 runs that measure roofline.traffic themselves: "
                         "report it as null instead of looking it up")
    ap.add_argument("--no-yardstick", action="store_true",
                    help="skip the untimed torch.mm (hipBLASLt) comparison of the expert GEMMs")
    ap.add_argument("--graph", action="store_true",
                    help="also time the same steps replayed from one HIP graph (extra field)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures ONE GPU: this build has no multi-GPU path "
                 "(world_size is 1); run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (there is no CPU fallback of the hot path)")

    os.environ["FMOE_BINDING"] = args.binding
    from fastmoe_amd import fmoe_cuda

    assert fmoe_cuda.BINDING == args.binding
    cfg = dict(CONFIGS[args.config], name=args.config)
    if args.layout == "list":
        args.no_cpu = args.no_yardstick = True
    layer, x, dy = build_layer(cfg, fused=args.layout == "fused")
    x.requires_grad_(True)

    for _ in range(args.warmup):
        step(layer, x, dy)
    torch.cuda.synchronize()

    with torch.no_grad():
        idx, _ = layer.gate(x)
    n_valid = int((idx >= 0).sum().item())
    work = kernel_work(cfg, n_valid)
    e_live = int(torch.bincount(idx[idx >= 0].flatten(), minlength=cfg["E"]).ne(0).sum().item())
    gbytes = gemm_bytes(cfg, n_valid, e_live)

    def summarise(records, n_steps):
        per = {}
        for name, a, b in records:
            per.setdefault(name, []).append(a.elapsed_time(b))
        out = {}
        for name, ts in per.items():
            avg_ms = sum(ts) / len(ts)
            kind, amount = work.get(name, ("byte", 0.0))
            rate = amount / (avg_ms * 1e-3) if avg_ms > 0 else 0.0
            peak = PEAK[cfg["dtype"]] if kind == "flop" else PEAK["hbm"]
            out[name] = {
                "launches_per_step": len(ts) / n_steps,
                "avg_us": round(avg_ms * 1e3, 2),
                "median_us": round(sorted(ts)[len(ts) // 2] * 1e3, 2),
                "min_us": round(min(ts) * 1e3, 2),
                "total_ms_per_step": round(sum(ts) / n_steps, 4),
                ("tflops" if kind == "flop" else "gbps"):
                    round(rate / (1e12 if kind == "flop" else 1e9), 2),
                "frac_of_peak": round(rate / peak, 4),
            }
            if name in gbytes and avg_ms > 0:
                out[name]["hbm_frac_of_peak"] = round(
                    gbytes[name] / (avg_ms * 1e-3) / PEAK["hbm"], 4)
        return out

    # Untimed survey pass with an event pair around every op: the per-kernel
    # table, and which op takes the largest share of a step.  (Every event pair
    # idles the GPU for a few microseconds, so the timed region below keeps
    # them on that one op only.)
    hooks = True    # both bindings feed the per-op event hook
    survey_steps = min(5, max(1, args.steps))
    records = []
    fmoe_cuda.profile_hook = lambda name, a, b: records.append((name, a, b))
    fmoe_cuda.profile_only = None
    for _ in range(survey_steps if hooks else 0):
        step(layer, x, dy)
    torch.cuda.synchronize()
    kernels = summarise(records, survey_steps)
    dom = max(kernels, key=lambda n: kernels[n]["total_ms_per_step"]) if hooks else None

    # Timed region: exactly --steps steps, events around the dominant op only.
    records = []
    fmoe_cuda.profile_only = {dom}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(layer, x, dy)
    enqueue = time.perf_counter() - t0
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    fmoe_cuda.profile_hook = None
    fmoe_cuda.profile_only = None
    ms_per_step = elapsed * 1e3 / args.steps
    timed = summarise(records, args.steps)
    if hooks:
        kernels[dom] = dict(timed[dom], timed_region=True)
    kind, amount = work[dom] if hooks else ("flop", 0.0)
    avg_s = kernels[dom]["avg_us"] * 1e-6 if hooks else 1.0
    if kind == "flop" and gbytes.get(dom, 0.0) / PEAK["hbm"] > amount / PEAK[cfg["dtype"]]:
        # more HBM time than matrix-core time in the algorithm itself: memory roofline
        roofline = {"kernel": dom, "bound": "hbm", "achieved": round(gbytes[dom] / avg_s / 1e9, 2),
                    "peak": PEAK["hbm"] / 1e9, "unit": "GB/s",
                    "mfma_frac": round(amount / avg_s / PEAK[cfg["dtype"]], 4)}
    elif kind == "flop":
        roofline = {"kernel": dom, "bound": "mfma", "achieved": round(amount / avg_s / 1e12, 2),
                    "peak": PEAK[cfg["dtype"]] / 1e12, "unit": "TFLOP/s"}
        if dom in gbytes:
            roofline["hbm_frac"] = round(gbytes[dom] / avg_s / PEAK["hbm"], 4)
    else:
        roofline = {"kernel": dom, "bound": "hbm", "achieved": round(amount / avg_s / 1e9, 2),
                    "peak": PEAK["hbm"] / 1e9, "unit": "GB/s"}
    roofline["frac"] = round(roofline["achieved"] / roofline["peak"], 4)
    if args.counter_pass:
        roofline["traffic"] = None
    elif (args.config, dom) not in MEASURED_TRAFFIC:
        # a stale or missing entry must not pass silently as "no data"
        sys.exit(f"bench.py: no measured HBM traffic on record for {dom} on {args.config}: "
                 "run the rocprofv3 FETCH_SIZE / WRITE_SIZE passes named in "
                 f"profiles/moe_step_{args.config}_hbm_traffic.md and add the entry to "
                 "MEASURED_TRAFFIC")
    else:
        roofline["traffic"] = round(MEASURED_TRAFFIC[(args.config, dom)])
    roofline["avg_launch_us"] = kernels[dom]["avg_us"] if hooks else None

    result = {
        "metric": "MoE-MLP fwd+bwd tokens/s @1 MI355X",
        "value": round(cfg["T"] / (ms_per_step * 1e-3), 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "host_enqueue_ms_per_step": round(enqueue * 1e3 / args.steps, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": cfg["dtype"],
        "data": "synthetic",
        "binding": args.binding,
        "expert_layout": args.layout,
        "config": {
            "workload": (f"{args.config}: {cfg['T']} tokens, d_model {cfg['d']}, d_hidden "
                         f"{cfg['h']}, {cfg['E']} experts, top-{cfg['k']}, {cfg['dtype']}; "
                         f"{cfg['note']}"),
            "routed_slots": cfg["T"] * cfg["k"],
            "live_slots": n_valid,
            "gemm_flops_per_step": 12.0 * n_valid * cfg["d"] * cfg["h"],
        },
        "gemm_tflops_overall": round(12.0 * n_valid * cfg["d"] * cfg["h"]
                                     / (ms_per_step * 1e-3) / 1e12, 2),
        "roofline": roofline,
        "kernels": kernels,
    }
    # the step's own GEMMs next to the library's, same shapes: the four grouped launches
    gemm_us = sum(kernels[k]["total_ms_per_step"] * 1e3 for k in kernels
                  if k.startswith("grouped_linear"))
    result["gemm_frac_of_peak_step"] = round(
        12.0 * n_valid * cfg["d"] * cfg["h"] / (gemm_us * 1e-6) / PEAK[cfg["dtype"]], 4) \
        if gemm_us > 0 else None
    if not args.no_yardstick:
        from fastmoe_amd.functions import RoutePlan

        with torch.no_grad():
            plan = RoutePlan(idx, cfg["E"])
        result["yardstick"] = yardstick(cfg, layer, plan.segments.seg_off)
    if args.graph:
        result["hip_graph"] = graph_replay(layer, x, dy, cfg, args.steps)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(cfg, layer, x.detach())
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
