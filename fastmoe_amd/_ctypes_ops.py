"""The operators of ``fmoe_cuda`` as ctypes calls into libfmoe_hip.so.

One of the two bindings of the C ABI (the other is the compiled pybind11 extension
built from csrc/fmoe_cuda_ext.cpp); ``fastmoe_amd.fmoe_cuda`` picks one of them and
documents the operator surface.  Same function names, argument order, side effects
and error type (``RuntimeError``) as the pybind11 module in cuda/fmoe_cuda.cpp:104-125
of the reference, on torch's current HIP stream.  It needs nothing but the shared
library.

Every function needs the HIP library and HIP tensors; nothing here computes on the
CPU.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Optional, Tuple

import torch

from . import _lib

_DTYPE = {
    torch.float32: 0,
    torch.float64: 1,
    torch.float16: 2,
    torch.bfloat16: 3,
}

_L = _lib.load()


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _dev(t: torch.Tensor, name: str, dtype=None) -> None:
    _need(isinstance(t, torch.Tensor), f"{name} must be a tensor")
    _need(t.is_cuda, f"{name} must be a CUDA tensor")
    _need(t.is_contiguous(), f"{name} must be contiguous")
    if dtype is not None:
        _need(t.dtype == dtype, f"{name} must have dtype {dtype}, got {t.dtype}")


def _dt(t: torch.Tensor, name: str) -> int:
    _need(t.dtype in _DTYPE, f"{name}: unsupported dtype {t.dtype}")
    return _DTYPE[t.dtype]


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


class _on:
    """Makes the tensor's device current for the duration of a launch."""

    def __init__(self, t: torch.Tensor):
        self.idx = t.device.index
        self.guard = None

    def __enter__(self):
        if self.idx is not None and self.idx != torch.cuda.current_device():
            self.guard = torch.cuda.device(self.idx)
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)


_front = None


def _hook_state():
    """The module that holds `profile_hook` / `profile_only` (fastmoe_amd.fmoe_cuda)."""
    global _front
    if _front is None:
        from . import fmoe_cuda as front

        _front = front
    return _front


class _launch(_on):
    """Device guard plus, when profiling, an event pair around the launches."""

    def __init__(self, t: torch.Tensor, name: str):
        super().__init__(t)
        self.name = name
        self.t = t
        self.ev = None

    def __enter__(self):
        super().__enter__()
        st = _front or _hook_state()
        if st.profile_hook is not None and (st.profile_only is None
                                            or self.name in st.profile_only):
            self.ev = (torch.cuda.Event(enable_timing=True),
                       torch.cuda.Event(enable_timing=True))
            self.ev[0].record(torch.cuda.current_stream(self.t.device))

    def __exit__(self, *exc):
        if self.ev is not None:
            self.ev[1].record(torch.cuda.current_stream(self.t.device))
            _front.profile_hook(self.name, self.ev[0], self.ev[1])
        super().__exit__(*exc)


# Routing workspaces, one per (device, stream): launches on one stream run in order,
# so consecutive calls can share a buffer (it is scratch: nothing in it outlives a
# call).  A stream under graph capture gets a fresh tensor instead, which then
# belongs to the graph's own memory pool.
_ws_cache = {}


def _workspace(numel: int, n_expert: int, device) -> torch.Tensor:
    nbytes = _L.fmoe_route_workspace_bytes(numel, n_expert)
    _need(nbytes >= 0, "route workspace: bad sizes")
    nbytes = max(int(nbytes), 1)
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(nbytes, dtype=torch.uint8, device=device)
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    ws = _ws_cache.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 16), dtype=torch.uint8, device=device)
        _ws_cache[key] = ws
    return ws


# --------------------------------------------------------------------------
# The reference surface (cuda/fmoe_cuda.cpp:117-124)
# --------------------------------------------------------------------------
def expert_count(gate_idx: torch.Tensor, expert_count: torch.Tensor) -> None:
    """expert_count[e] += number of entries of gate_idx equal to e (-1 skipped).

    cuda/local_exchange.cu:22-32."""
    _dev(gate_idx, "gate_idx", torch.int64)
    _dev(expert_count, "expert_count", torch.int32)
    with _launch(gate_idx, "expert_count"):
        _lib.check(
            _L.fmoe_expert_count(gate_idx.data_ptr(), gate_idx.numel(),
                                 expert_count.data_ptr(), expert_count.numel(),
                                 _stream(gate_idx)),
            "expert_count")


def assign_pos(cum_count: torch.Tensor, gate: torch.Tensor, pos: torch.Tensor) -> None:
    """Fills pos from the inclusive cumulative counts; cum_count is left holding
    the exclusive ones.  cuda/local_exchange.cu:5-20."""
    _dev(cum_count, "cum_count", torch.int32)
    _dev(gate, "gate", torch.int64)
    _dev(pos, "pos", torch.int64)
    n, e = gate.numel(), cum_count.numel()
    ws = _workspace(n, e, gate.device)
    with _launch(gate, "assign_pos"):
        _lib.check(
            _L.fmoe_assign_pos(cum_count.data_ptr(), gate.data_ptr(), pos.data_ptr(),
                               n, e, ws.data_ptr(), ws.numel(), _stream(gate)),
            "assign_pos")


def _seg_off_from_counts(expert_count: torch.Tensor, device, rows: Optional[int] = None
                         ) -> torch.Tensor:
    """seg_off (device int32[E+1]) from host or device int64 counts.  With host counts
    and `rows` given, the counts must not claim more rows than the buffers hold (the
    grouped kernels trust seg_off)."""
    _need(expert_count.dtype == torch.int64, "expert_count must be int64")
    e = expert_count.numel()
    if rows is not None and not expert_count.is_cuda:
        _need(bool((expert_count >= 0).all()), "expert_count holds a negative count")
        total = int(expert_count.sum())
        _need(total <= rows, f"expert_count sums to {total} rows, the buffer has {rows}")
    if expert_count.is_cuda:
        seg = torch.zeros(e + 1, dtype=torch.int32, device=device)
        seg[1:] = torch.cumsum(expert_count.reshape(-1), 0)
        return seg
    cnt = expert_count.contiguous()
    seg = torch.empty(e + 1, dtype=torch.int32, device=device)
    _lib.check(
        _L.fmoe_seg_off_from_host_counts(cnt.data_ptr(), e, seg.data_ptr(),
                                         torch.cuda.current_stream(device).cuda_stream),
        "seg_off_from_host_counts")
    return seg


def linear_forward(input_buf: torch.Tensor, expert_count: torch.Tensor,
                   weight: torch.Tensor, bias: Optional[torch.Tensor] = None
                   ) -> torch.Tensor:
    """output[seg_e] = input_buf[seg_e] @ weight[e].T + bias[e].

    expert_count is the reference's host int64 tensor
    (cuda/parallel_linear.cu:5-50); a device tensor is accepted as well."""
    _dev(input_buf, "input_buf")
    _dev(weight, "weight", input_buf.dtype)
    _need(input_buf.dim() == 2, "input_buf must be [rows, in]")
    with _on(input_buf):
        seg = _seg_off_from_counts(expert_count, input_buf.device, input_buf.shape[0])
        return grouped_linear_fwd(input_buf, seg, weight, bias)


def linear_backward(grad_output_buf: torch.Tensor, input_buf: torch.Tensor,
                    expert_count: torch.Tensor, weight: torch.Tensor,
                    bias: Optional[torch.Tensor] = None) -> List[torch.Tensor]:
    """[grad_input, grad_weight, grad_bias]; cuda/parallel_linear.cu:53-96.

    grad_bias is always returned (zeros-shaped [E, out]); without a bias it is
    left unset by the reference and dropped by its caller (fmoe/linear.py:33)."""
    _dev(grad_output_buf, "grad_output_buf")
    _dev(input_buf, "input_buf", grad_output_buf.dtype)
    _need(input_buf.dim() == 2, "input_buf must be [rows, in]")
    with _on(input_buf):
        seg = _seg_off_from_counts(expert_count, input_buf.device, input_buf.shape[0])
        dx, dw, db = grouped_linear_bwd(grad_output_buf, input_buf, seg, weight,
                                        need_bias=True)
    return [dx, dw, db]


def limit_by_capacity(expert_count: torch.Tensor, capacity: torch.Tensor,
                      n_expert: int, n_worker: int) -> torch.Tensor:
    """Granted counts under per-expert capacity; capacity is consumed in place.

    cuda/balancing.cu:9-22."""
    _dev(expert_count, "expert_count", torch.int64)
    _dev(capacity, "capacity", torch.int32)
    _need(expert_count.numel() >= n_expert * n_worker, "expert_count too short")
    _need(capacity.numel() >= n_expert, "capacity too short")
    ack = torch.empty_like(expert_count)
    with _launch(expert_count, "limit_by_capacity"):
        _lib.check(
            _L.fmoe_limit_by_capacity(expert_count.data_ptr(), capacity.data_ptr(),
                                      ack.data_ptr(), n_expert, n_worker,
                                      _stream(expert_count)),
            "limit_by_capacity")
    return ack


def prune_gate_by_capacity(gate_idx: torch.Tensor, expert_count: torch.Tensor,
                           n_expert: int, n_worker: int) -> torch.Tensor:
    """New gate indices with -1 where the expert's budget ran out (earlier
    slots win); expert_count is consumed in place.  cuda/balancing.cu:24-39."""
    _dev(gate_idx, "gate_idx", torch.int64)
    _dev(expert_count, "expert_count", torch.int32)
    _need(expert_count.numel() >= n_expert * n_worker, "expert_count too short")
    new_gate = torch.empty_like(gate_idx)
    n = gate_idx.numel()
    ws = _workspace(n, n_expert * n_worker, gate_idx.device)
    with _launch(gate_idx, "prune_gate_by_capacity"):
        _lib.check(
            _L.fmoe_prune_gate_by_capacity(gate_idx.data_ptr(), new_gate.data_ptr(),
                                           expert_count.data_ptr(), n, n_expert,
                                           n_worker, ws.data_ptr(), ws.numel(),
                                           _stream(gate_idx)),
            "prune_gate_by_capacity")
    return new_gate


# --------------------------------------------------------------------------
# Native dispatch ops named by the reference's Python helpers
# (fmoe/functions.py:78-90)
# --------------------------------------------------------------------------
def local_scatter(inp: torch.Tensor, pos: torch.Tensor, idx_div: int = 1,
                  n_rows_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[r] = inp[pos[r] // idx_div]."""
    _dev(inp, "inp")
    _dev(pos, "pos", torch.int64)
    _need(inp.dim() == 2, "inp must be [rows, d]")
    dt = _dt(inp, "inp")
    n, d = pos.numel(), inp.shape[1]
    out = torch.empty((n, d), dtype=inp.dtype, device=inp.device)
    with _launch(inp, "local_scatter"):
        _lib.check(
            _L.fmoe_local_scatter(inp.data_ptr(), pos.data_ptr(), out.data_ptr(), n, d,
                                  idx_div, _ptr(n_rows_dev), dt, _stream(inp)),
            "local_scatter")
    return out


def scatter_tokens(inp: torch.Tensor, inv: torch.Tensor, top_k: int) -> torch.Tensor:
    """buf[inv[t * top_k + j]] = inp[t] for live slots: local_scatter in token
    order (one read per token row).  Rows of buf no slot maps to are not written."""
    _dev(inp, "inp")
    _dev(inv, "inv", torch.int32)
    _need(inp.dim() == 2, "inp must be [tokens, d]")
    t, d = inp.shape
    _need(inv.numel() == t * top_k, "inv must have tokens * top_k entries")
    out = torch.empty((t * top_k, d), dtype=inp.dtype, device=inp.device)
    with _launch(inp, "scatter_tokens"):
        _lib.check(
            _L.fmoe_scatter_tokens(inp.data_ptr(), inv.data_ptr(), out.data_ptr(), t, top_k, d,
                                   _dt(inp, "inp"), _stream(inp)),
            "scatter_tokens")
    return out


def local_gather(inp: torch.Tensor, pos: torch.Tensor, out_batch_size: int,
                 maybe_overlap: bool = True,
                 n_rows_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """zeros[out_batch_size, d] with row pos[r] set to (or, when rows may
    overlap, incremented by) inp[r]."""
    _dev(inp, "inp")
    _dev(pos, "pos", torch.int64)
    _need(inp.dim() == 2, "inp must be [rows, d]")
    dt = _dt(inp, "inp")
    n, d = pos.numel(), inp.shape[1]
    _need(inp.shape[0] >= n, "inp has fewer rows than pos")
    out = torch.empty((out_batch_size, d), dtype=inp.dtype, device=inp.device)
    if maybe_overlap and inp.dtype not in (torch.float32, torch.float64):
        # half types accumulate in fp32, rounded once at the end
        acc = local_gather(inp.float(), pos, out_batch_size, True, n_rows_dev)
        return acc.to(inp.dtype)
    with _launch(inp, "local_gather"):
        _lib.check(
            _L.fmoe_local_gather(inp.data_ptr(), pos.data_ptr(), out.data_ptr(), n,
                                 out_batch_size, d, _ptr(n_rows_dev),
                                 1 if maybe_overlap else 0, dt, _stream(inp)),
            "local_gather")
    return out


# --------------------------------------------------------------------------
# Fused, synchronisation-free ops
# --------------------------------------------------------------------------
def route(gate: torch.Tensor, n_expert: int, want_inv: bool = True
          ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, Optional[torch.Tensor]]:
    """(pos int64[N], count int64[E], seg_off int32[E+1], inv int32[N]) from the
    gate indices, all on the device, without a device-to-host copy.

    Only the first seg_off[E] entries of pos are written."""
    _dev(gate, "gate", torch.int64)
    n = gate.numel()
    dev = gate.device
    count = torch.empty(n_expert, dtype=torch.int64, device=dev)
    seg = torch.empty(n_expert + 1, dtype=torch.int32, device=dev)
    pos = torch.empty(n, dtype=torch.int64, device=dev)
    inv = torch.empty(n, dtype=torch.int32, device=dev) if want_inv else None
    ws = _workspace(n, n_expert, dev)
    with _launch(gate, "route"):
        _lib.check(
            _L.fmoe_route(gate.data_ptr(), n, n_expert, count.data_ptr(),
                          seg.data_ptr(), pos.data_ptr(), _ptr(inv), ws.data_ptr(),
                          ws.numel(), _stream(gate)),
            "route")
    return pos, count, seg, inv


def route_static(gate: torch.Tensor, n_expert: int, count: torch.Tensor, seg_off: torch.Tensor,
                 pos: torch.Tensor, inv: Optional[torch.Tensor] = None) -> None:
    """`route` into tensors the caller already holds, with the library's built-in
    scratch buffer instead of a workspace: the call itself allocates nothing
    (fmoe_route_static).  count int64[E], seg_off int32[E+1], pos int64[N],
    inv int32[N] or None.  Calls on one GPU share the buffer and must not overlap."""
    _dev(gate, "gate", torch.int64)
    _dev(count, "count", torch.int64)
    _dev(seg_off, "seg_off", torch.int32)
    _dev(pos, "pos", torch.int64)
    n = gate.numel()
    _need(count.numel() == n_expert and seg_off.numel() == n_expert + 1 and pos.numel() >= n,
          "route_static: count[E], seg_off[E+1] and pos[N] expected")
    if inv is not None:
        _dev(inv, "inv", torch.int32)
        _need(inv.numel() >= n, "route_static: inv must have N entries")
    with _launch(gate, "route"):
        _lib.check(
            _L.fmoe_route_static(gate.data_ptr(), n, n_expert, count.data_ptr(),
                                 seg_off.data_ptr(), pos.data_ptr(), _ptr(inv), _stream(gate)),
            "route_static")


def grouped_linear_fwd(x: torch.Tensor, seg_off: torch.Tensor, weight: torch.Tensor,
                       bias: Optional[torch.Tensor] = None, with_gelu: bool = False):
    """y[seg_e] = x[seg_e] @ weight[e].T + bias[e] with device-side seg_off.

    with_gelu: returns (y, gelu(y)), the exact GELU applied to the rounded y, written
    by the same output tiles where the library can (rows behind seg_off[E] are left
    as allocated in both)."""
    _dev(x, "x")
    _dev(weight, "weight", x.dtype)
    _dev(seg_off, "seg_off", torch.int32)
    _need(x.dim() == 2 and weight.dim() == 3, "x must be 2-d and weight 3-d")
    e, out_f, in_f = weight.shape
    _need(x.shape[1] == in_f, f"x has {x.shape[1]} features, weight expects {in_f}")
    _need(seg_off.numel() == e + 1, "seg_off must have E+1 entries")
    if bias is not None:
        _dev(bias, "bias", x.dtype)
        _need(tuple(bias.shape) == (e, out_f), "bias must be [E, out]")
    dt = _dt(x, "x")
    y = torch.empty((x.shape[0], out_f), dtype=x.dtype, device=x.device)
    if with_gelu:
        y_act = torch.empty_like(y)
        with _launch(x, "grouped_linear_fwd_act"):
            _lib.check(
                _L.fmoe_grouped_linear_fwd_act(x.data_ptr(), weight.data_ptr(), _ptr(bias),
                                               seg_off.data_ptr(), y.data_ptr(),
                                               y_act.data_ptr(), x.shape[0], in_f, out_f, e,
                                               dt, _stream(x)),
                "grouped_linear_fwd_act")
        return y, y_act
    with _launch(x, "grouped_linear_fwd"):
        _lib.check(
            _L.fmoe_grouped_linear_fwd(x.data_ptr(), weight.data_ptr(), _ptr(bias),
                                       seg_off.data_ptr(), y.data_ptr(), x.shape[0],
                                       in_f, out_f, e, dt, _stream(x)),
            "grouped_linear_fwd")
    return y


def grouped_linear_bwd(dy: torch.Tensor, x: torch.Tensor, seg_off: torch.Tensor,
                       weight: torch.Tensor, need_bias: bool = True,
                       need_dx: bool = True, need_dw: bool = True,
                       act_pre: Optional[torch.Tensor] = None):
    """(dx, dw, db) of grouped_linear_fwd; entries not asked for are None.

    With act_pre ([rows, in], the pre-activations x = gelu(act_pre) came from) dx
    is the gradient with respect to act_pre: the backward of the activation is
    applied to it, inside the kernel's epilogue where the library can."""
    _dev(dy, "dy")
    _dev(x, "x", dy.dtype)
    _dev(weight, "weight", dy.dtype)
    _dev(seg_off, "seg_off", torch.int32)
    _need(x.dim() == 2 and weight.dim() == 3, "x must be 2-d and weight 3-d")
    e, out_f, in_f = weight.shape
    n = x.shape[0]
    _need(tuple(dy.shape) == (n, out_f), "dy must be [rows, out]")
    _need(x.shape[1] == in_f, "x must be [rows, in]")
    _need(seg_off.numel() == e + 1, "seg_off must have E+1 entries")
    dt = _dt(dy, "dy")
    dx = torch.empty((n, in_f), dtype=dy.dtype, device=dy.device) if need_dx else None
    dw = torch.empty_like(weight) if need_dw else None
    db = torch.empty((e, out_f), dtype=dy.dtype, device=dy.device) if need_bias else None
    # one call: dX and dW go out in one launch where the library can, and on the
    # bf16/f16 matrix-core kernels the bias gradient is summed inside the dW tiles
    name = ("grouped_linear_bwd" if need_dx and need_dw else
            "grouped_linear_dgrad" if need_dx else
            "grouped_linear_wgrad" if need_dw else "grouped_linear_bias_grad")
    if act_pre is not None and need_dx:
        _dev(act_pre, "act_pre", dy.dtype)
        _need(tuple(act_pre.shape) == (n, in_f), "act_pre must be [rows, in]")
        with _launch(dy, name):     # same kernels and FLOPs as without act_pre: same op name
            _lib.check(
                _L.fmoe_grouped_linear_bwd_act(dy.data_ptr(), x.data_ptr(),
                                               weight.data_ptr(), seg_off.data_ptr(),
                                               act_pre.data_ptr(), _ptr(dx), _ptr(dw),
                                               _ptr(db), n, in_f, out_f, e, dt, _stream(dy)),
                name)
    elif need_dx or need_dw or need_bias:
        with _launch(dy, name):
            _lib.check(
                _L.fmoe_grouped_linear_bwd(dy.data_ptr(), x.data_ptr(),
                                           weight.data_ptr(), seg_off.data_ptr(),
                                           _ptr(dx), _ptr(dw), _ptr(db), n, in_f, out_f,
                                           e, dt, _stream(dy)),
                name)
    return dx, dw, db


def pointer_table(tensors) -> torch.Tensor:
    """Device int64[len(tensors)] holding the tensors' data pointers: the w_ptrs /
    bias_ptrs argument of grouped_linear_fwd_ptrs / _bwd_ptrs for experts whose
    parameters are separate allocations.  Filled on torch's current stream without a
    host synchronisation.  All tensors on one GPU, contiguous, 16-byte aligned."""
    tensors = list(tensors)
    _need(len(tensors) >= 1, "pointer_table: no tensors")
    first = tensors[0]
    ptrs = []
    for t in tensors:
        _dev(t, "pointer_table entry", first.dtype)
        _need(t.device == first.device and t.shape == first.shape,
              "pointer_table: tensors must share device and shape")
        _need(t.data_ptr() % 16 == 0, "pointer_table: tensors must be 16-byte aligned")
        ptrs.append(t.data_ptr())
    table = torch.empty(len(ptrs), dtype=torch.int64, device=first.device)
    host = (ctypes.c_void_p * len(ptrs))(*ptrs)
    with _on(first):
        _lib.check(_L.fmoe_pointer_table(host, len(ptrs), table.data_ptr(), _stream(first)),
                   "pointer_table")
    return table


def grouped_linear_fwd_ptrs(x: torch.Tensor, seg_off: torch.Tensor, w_table: torch.Tensor,
                            b_table: Optional[torch.Tensor], out_feat: int,
                            with_gelu: bool = False):
    """grouped_linear_fwd for per-expert weights [1, out, in] (and biases [1, out]) given
    as pointer tables (pointer_table): y, or with with_gelu (y, gelu(y)).  No weight is
    copied."""
    _dev(x, "x")
    _dev(seg_off, "seg_off", torch.int32)
    _dev(w_table, "w_table", torch.int64)
    _need(x.dim() == 2, "x must be [rows, in]")
    e = w_table.numel()
    _need(seg_off.numel() == e + 1, "seg_off must have E+1 entries")
    if b_table is not None:
        _dev(b_table, "b_table", torch.int64)
        _need(b_table.numel() == e, "b_table must have E entries")
    y = torch.empty((x.shape[0], out_feat), dtype=x.dtype, device=x.device)
    y_act = torch.empty_like(y) if with_gelu else None
    with _launch(x, "grouped_linear_fwd_act" if with_gelu else "grouped_linear_fwd"):
        _lib.check(
            _L.fmoe_grouped_linear_fwd_ptrs(x.data_ptr(), w_table.data_ptr(), _ptr(b_table),
                                            seg_off.data_ptr(), y.data_ptr(), _ptr(y_act),
                                            x.shape[0], x.shape[1], out_feat, e, _dt(x, "x"),
                                            _stream(x)),
            "grouped_linear_fwd_ptrs")
    return (y, y_act) if with_gelu else y


def grouped_linear_bwd_ptrs(dy: torch.Tensor, x: torch.Tensor, seg_off: torch.Tensor,
                            w_table: torch.Tensor, need_bias: bool = True, need_dx: bool = True,
                            need_dw: bool = True, act_pre: Optional[torch.Tensor] = None):
    """grouped_linear_bwd for weights given as a pointer table: (dx, dw [E, out, in],
    db [E, out]); the caller hands out dw[e:e+1] / db[e:e+1] as the per-expert gradients."""
    _dev(dy, "dy")
    _dev(x, "x", dy.dtype)
    _dev(seg_off, "seg_off", torch.int32)
    _dev(w_table, "w_table", torch.int64)
    _need(x.dim() == 2 and dy.dim() == 2 and dy.shape[0] == x.shape[0],
          "dy must be [rows, out] and x [rows, in]")
    e, n, in_f, out_f = w_table.numel(), x.shape[0], x.shape[1], dy.shape[1]
    _need(seg_off.numel() == e + 1, "seg_off must have E+1 entries")
    dx = torch.empty((n, in_f), dtype=dy.dtype, device=dy.device) if need_dx else None
    dw = torch.empty((e, out_f, in_f), dtype=dy.dtype, device=dy.device) if need_dw else None
    db = torch.empty((e, out_f), dtype=dy.dtype, device=dy.device) if need_bias else None
    if act_pre is not None and need_dx:
        _dev(act_pre, "act_pre", dy.dtype)
        _need(tuple(act_pre.shape) == (n, in_f), "act_pre must be [rows, in]")
    else:
        act_pre = None
    name = ("grouped_linear_bwd" if need_dx and need_dw else
            "grouped_linear_dgrad" if need_dx else
            "grouped_linear_wgrad" if need_dw else "grouped_linear_bias_grad")
    if need_dx or need_dw or need_bias:
        with _launch(dy, name):
            _lib.check(
                _L.fmoe_grouped_linear_bwd_ptrs(dy.data_ptr(), x.data_ptr(), w_table.data_ptr(),
                                                seg_off.data_ptr(), _ptr(act_pre), _ptr(dx),
                                                _ptr(dw), _ptr(db), n, in_f, out_f, e,
                                                _dt(dy, "dy"), _stream(dy)),
                "grouped_linear_bwd_ptrs")
    return dx, dw, db


def gather_combine_fwd(buf: torch.Tensor, inv: torch.Tensor, score: torch.Tensor,
                       n_tokens: int, top_k: int) -> torch.Tensor:
    """y[t] = sum_j score[t, j] * buf[inv[t*k+j]] (dropped slots contribute 0)."""
    _dev(buf, "buf")
    _dev(inv, "inv", torch.int32)
    _dev(score, "score", buf.dtype)
    _need(inv.numel() == n_tokens * top_k and score.numel() == n_tokens * top_k,
          "inv/score must have n_tokens*top_k entries")
    d = buf.shape[1]
    y = torch.empty((n_tokens, d), dtype=buf.dtype, device=buf.device)
    with _launch(buf, "gather_combine_fwd"):
        _lib.check(
            _L.fmoe_gather_combine_fwd(buf.data_ptr(), inv.data_ptr(), score.data_ptr(),
                                       y.data_ptr(), n_tokens, top_k, d,
                                       _dt(buf, "buf"), _stream(buf)),
            "gather_combine_fwd")
    return y


def gather_combine_bwd(dy: torch.Tensor, buf: torch.Tensor, inv: torch.Tensor,
                       score: torch.Tensor, n_tokens: int, top_k: int
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
    """(dbuf [rows, d] in expert order, dscore [n_tokens, top_k])."""
    _dev(dy, "dy")
    _dev(buf, "buf", dy.dtype)
    _dev(inv, "inv", torch.int32)
    _dev(score, "score", dy.dtype)
    d = buf.shape[1]
    _need(tuple(dy.shape) == (n_tokens, d), "dy must be [n_tokens, d]")
    dbuf = torch.empty_like(buf)
    dscore = torch.empty((n_tokens, top_k), dtype=dy.dtype, device=dy.device)
    with _launch(dy, "gather_combine_bwd"):
        _lib.check(
            _L.fmoe_gather_combine_bwd(dy.data_ptr(), buf.data_ptr(), inv.data_ptr(),
                                       score.data_ptr(), dbuf.data_ptr(),
                                       dscore.data_ptr(), n_tokens, top_k, d,
                                       _dt(dy, "dy"), _stream(dy)),
            "gather_combine_bwd")
    return dbuf, dscore


def scatter_reduce(dbuf: torch.Tensor, inv: torch.Tensor, n_tokens: int,
                   top_k: int) -> torch.Tensor:
    """dx[t] = sum_j dbuf[inv[t*k+j]] over live slots (deterministic order)."""
    _dev(dbuf, "dbuf")
    _dev(inv, "inv", torch.int32)
    _need(inv.numel() == n_tokens * top_k, "inv must have n_tokens*top_k entries")
    d = dbuf.shape[1]
    dx = torch.empty((n_tokens, d), dtype=dbuf.dtype, device=dbuf.device)
    with _launch(dbuf, "scatter_reduce"):
        _lib.check(
            _L.fmoe_scatter_reduce(dbuf.data_ptr(), inv.data_ptr(), dx.data_ptr(),
                                   n_tokens, top_k, d, _dt(dbuf, "dbuf"),
                                   _stream(dbuf)),
            "scatter_reduce")
    return dx


MAX_GATE_TOP_K = 16   # FMOE_MAX_GATE_TOP_K of the C ABI


def topk_softmax_fwd(logits: torch.Tensor, top_k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(idx int64 [T, k], score [T, k]) of logits [T, E]: the k largest logits of
    every token by descending value (equal logits: lower index first) and the
    softmax over them, as naive_gate.py:31-38 computes with torch.topk + softmax."""
    _dev(logits, "logits")
    _need(logits.dim() == 2, "logits must be [tokens, experts]")
    t, e = logits.shape
    idx = torch.empty((t, top_k), dtype=torch.int64, device=logits.device)
    score = torch.empty((t, top_k), dtype=logits.dtype, device=logits.device)
    with _launch(logits, "topk_softmax_fwd"):
        _lib.check(
            _L.fmoe_topk_softmax_fwd(logits.data_ptr(), t, e, top_k, idx.data_ptr(),
                                     score.data_ptr(), _dt(logits, "logits"), _stream(logits)),
            "topk_softmax_fwd")
    return idx, score


def topk_softmax_bwd(dscore: torch.Tensor, score: torch.Tensor, idx: torch.Tensor,
                     n_expert: int) -> torch.Tensor:
    """dlogits [T, E] of topk_softmax_fwd (zero outside the chosen experts)."""
    _dev(dscore, "dscore")
    _dev(score, "score", dscore.dtype)
    _dev(idx, "idx", torch.int64)
    t, k = score.shape
    _need(tuple(dscore.shape) == (t, k) and tuple(idx.shape) == (t, k),
          "dscore, score and idx must all be [tokens, top_k]")
    dlogits = torch.empty((t, n_expert), dtype=score.dtype, device=score.device)
    with _launch(score, "topk_softmax_bwd"):
        _lib.check(
            _L.fmoe_topk_softmax_bwd(dscore.data_ptr(), score.data_ptr(), idx.data_ptr(),
                                     dlogits.data_ptr(), t, n_expert, k,
                                     _dt(score, "score"), _stream(score)),
            "topk_softmax_bwd")
    return dlogits


def _row_len(x: torch.Tensor) -> int:
    return x.shape[-1] if x.dim() >= 1 and x.numel() else 0


def gelu_fwd(x: torch.Tensor, n_rows_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """gelu(x) = 0.5 x (1 + erf(x / sqrt 2)), the torch.nn.GELU() between the two
    expert layers (fmoe/transformer.py:28-30).  `n_rows_dev` (device int32[1]):
    only that many leading rows of x are live; the rest of the result is left
    unwritten."""
    _dev(x, "x")
    _need(x.is_contiguous(), "x must be contiguous")
    y = torch.empty_like(x)
    with _launch(x, "gelu_fwd"):
        _lib.check(_L.fmoe_gelu_fwd(x.data_ptr(), y.data_ptr(), x.numel(), _ptr(n_rows_dev),
                                    _row_len(x), _dt(x, "x"), _stream(x)), "gelu_fwd")
    return y


def gelu_bwd(dy: torch.Tensor, x: torch.Tensor,
             n_rows_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """dy * gelu'(x); `n_rows_dev` as in gelu_fwd."""
    _dev(x, "x")
    _dev(dy, "dy", x.dtype)
    _need(x.is_contiguous() and dy.is_contiguous() and dy.numel() == x.numel(),
          "dy and x must be contiguous and of one size")
    dx = torch.empty_like(x)
    with _launch(x, "gelu_bwd"):
        _lib.check(_L.fmoe_gelu_bwd(dy.data_ptr(), x.data_ptr(), dx.data_ptr(), x.numel(),
                                    _ptr(n_rows_dev), _row_len(x), _dt(x, "x"), _stream(x)),
                   "gelu_bwd")
    return dx


def init(device=None) -> None:
    """One-time set-up of a GPU (the current one by default) on its current stream:
    the activation tables and the address of route_static's buffer (fmoe_init).
    Needed only before capturing a HIP graph whose first call would otherwise do it."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else \
        torch.device(device)
    with torch.cuda.device(dev):
        _lib.check(_L.fmoe_init(torch.cuda.current_stream(dev).cuda_stream), "init")


def set_gemm_path(path: int) -> None:
    """0 = matrix-core kernel where the shape allows (tile shape chosen by the
    library), 1 = scalar kernel only, 2..5 = matrix-core kernel with bf16/f16
    tile configuration 1..4 forced, 6 = automatic with the forward activation as a
    kernel of its own (for tests; the setting belongs to the calling thread)."""
    _lib.check(_L.fmoe_set_gemm_path(path), "set_gemm_path")
