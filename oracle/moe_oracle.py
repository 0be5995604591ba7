"""Python face of the CPU checker.

TEST INFRASTRUCTURE ONLY (used by tests/, the smoke run and the CPU leg of the
benchmark); the product never imports it.

Two parts:
  * numpy wrappers around libfmoe_oracle.so, the plain-C restatement of the
    reference's kernels (see fmoe_oracle.c for the lines each one follows);
  * `brute_force_moe_mlp`, a torch restatement of the dense per-expert MoE MLP
    that the reference's tests use as their oracle (tests/moe.py:30-49),
    differentiated by autograd.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import c_int64, c_void_p

import numpy as np
import torch
import torch.nn.functional as F
from scipy.special import erfc as _erfc

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libfmoe_oracle.so")
_lib = None


def build() -> str:
    """Compiles the C restatement with gcc (seconds)."""
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _SO


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a: np.ndarray) -> c_void_p:
    assert a.flags["C_CONTIGUOUS"]
    return c_void_p(a.ctypes.data)


def _i64(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.int64))


# ------------------------------------------------------------------ routing
def expert_count(gate, n_expert: int, into=None) -> np.ndarray:
    gate = _i64(gate).reshape(-1)
    count = np.zeros(n_expert, np.int32) if into is None else into
    _load().oracle_expert_count(_p(gate), c_int64(gate.size), _p(count), c_int64(n_expert))
    return count


def assign_pos(cum_count: np.ndarray, gate) -> np.ndarray:
    """Returns pos; cum_count (int32, inclusive prefix) is clobbered in place."""
    gate = _i64(gate).reshape(-1)
    assert cum_count.dtype == np.int32
    n_valid = int(cum_count[-1]) if cum_count.size else 0
    pos = np.full(n_valid, -7, np.int64)
    _load().oracle_assign_pos(_p(cum_count), _p(gate), _p(pos), c_int64(gate.size))
    return pos


def route(gate, n_expert: int):
    """(pos, count int64[E], seg_off int32[E+1], inv int32[N]) the way the
    reference's count_by_gate builds them (fmoe/functions.py:28-49)."""
    gate = _i64(gate).reshape(-1)
    count = expert_count(gate, n_expert)
    cum = np.cumsum(count.astype(np.int64)).astype(np.int32)
    seg_off = np.concatenate([[0], cum]).astype(np.int32)
    pos = assign_pos(cum.copy(), gate)
    inv = np.full(gate.size, -1, np.int32)
    inv[pos] = np.arange(pos.size, dtype=np.int32)
    return pos, count.astype(np.int64), seg_off, inv


def limit_by_capacity(ec, cap: np.ndarray, n_expert: int, n_worker: int) -> np.ndarray:
    """Returns eca; cap (int32) is clobbered in place."""
    ec = _i64(ec).reshape(-1)
    assert cap.dtype == np.int32
    eca = np.zeros_like(ec)
    _load().oracle_limit_by_capacity(_p(ec), _p(cap), _p(eca), c_int64(n_expert),
                                     c_int64(n_worker))
    return eca


def prune_gate_by_capacity(gate, ec: np.ndarray, n_bins: int) -> np.ndarray:
    """Returns the pruned gate (same shape); ec (int32) is clobbered in place."""
    g = _i64(gate)
    assert ec.dtype == np.int32
    out = np.empty_like(g)
    _load().oracle_prune_gate_by_capacity(_p(g.reshape(-1)), _p(out.reshape(-1)), _p(ec),
                                          c_int64(g.size), c_int64(n_bins))
    return out


# ----------------------------------------------------------------- dispatch
def local_scatter(inp: np.ndarray, idx, idx_div: int = 1) -> np.ndarray:
    inp = np.ascontiguousarray(inp)
    idx = _i64(idx)
    out = np.empty((idx.size, inp.shape[1]), inp.dtype)
    _load().oracle_local_scatter(_p(inp), _p(idx), _p(out), c_int64(idx.size),
                                 c_int64(inp.shape[1] * inp.itemsize), c_int64(idx_div))
    return out


def local_gather(inp: np.ndarray, pos, out_rows: int) -> np.ndarray:
    inp = np.ascontiguousarray(inp)
    pos = _i64(pos)
    out = np.empty((out_rows, inp.shape[1]), inp.dtype)
    _load().oracle_local_gather(_p(inp), _p(pos), _p(out), c_int64(pos.size),
                                c_int64(out_rows), c_int64(inp.shape[1] * inp.itemsize))
    return out


def local_gather_add(inp: np.ndarray, pos, out_rows: int) -> np.ndarray:
    inp = np.ascontiguousarray(inp, dtype=np.float64)
    pos = _i64(pos)
    out = np.empty((out_rows, inp.shape[1]), np.float64)
    _load().oracle_local_gather_add_f64(_p(inp), _p(pos), _p(out), c_int64(pos.size),
                                        c_int64(out_rows), c_int64(inp.shape[1]))
    return out


def combine(score: np.ndarray, out: np.ndarray) -> np.ndarray:
    score = np.ascontiguousarray(score, dtype=np.float64)
    out = np.ascontiguousarray(out, dtype=np.float64)
    n_tokens, top_k = score.shape
    y = np.empty((n_tokens, out.shape[1]), np.float64)
    _load().oracle_combine_f64(_p(score), _p(out), _p(y), c_int64(n_tokens),
                               c_int64(top_k), c_int64(out.shape[1]))
    return y


# ------------------------------------------------------------- expert GEMMs
def linear_forward(x, w, bias, expert_count) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float64)
    w = np.ascontiguousarray(w, dtype=np.float64)
    cnt = _i64(expert_count)
    e, out_f, in_f = w.shape
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float64)
    y = np.zeros((x.shape[0], out_f), np.float64)
    _load().oracle_linear_forward_f64(_p(x), _p(w), None if b is None else _p(b),
                                      _p(cnt), _p(y), c_int64(in_f), c_int64(out_f),
                                      c_int64(e))
    return y


def linear_backward(dy, x, w, expert_count):
    dy = np.ascontiguousarray(dy, dtype=np.float64)
    x = np.ascontiguousarray(x, dtype=np.float64)
    w = np.ascontiguousarray(w, dtype=np.float64)
    cnt = _i64(expert_count)
    e, out_f, in_f = w.shape
    dx = np.zeros_like(x)
    dw = np.empty_like(w)
    db = np.empty((e, out_f), np.float64)
    _load().oracle_linear_backward_f64(_p(dy), _p(x), _p(w), _p(cnt), _p(dx), _p(dw),
                                       _p(db), c_int64(in_f), c_int64(out_f), c_int64(e))
    return dx, dw, db


# ------------------------------------------------------------------- gate
def topk_softmax(logits: np.ndarray, top_k: int):
    """fmoe/gates/naive_gate.py:31-38: the top_k largest logits of every row and
    the softmax over those values, float64.  torch.topk leaves the order open;
    here: descending logit, equal logits by ascending expert index."""
    logits = np.asarray(logits, dtype=np.float64)
    n_expert = logits.shape[1]
    # stable sort of (-logit) keeps the lower index first among equals
    order = np.argsort(-logits, axis=1, kind="stable")[:, :top_k]
    val = np.take_along_axis(logits, order, axis=1)
    p = np.exp(val - val[:, :1])
    assert top_k <= n_expert
    return order.astype(np.int64), p / p.sum(axis=1, keepdims=True)


def topk_softmax_backward(dscore: np.ndarray, score: np.ndarray, idx: np.ndarray,
                          n_expert: int) -> np.ndarray:
    """Gradient of topk_softmax with respect to the logits: softmax backward on
    the k chosen entries, zero elsewhere."""
    dscore = np.asarray(dscore, dtype=np.float64)
    score = np.asarray(score, dtype=np.float64)
    g = score * (dscore - (dscore * score).sum(axis=1, keepdims=True))
    out = np.zeros((score.shape[0], n_expert))
    np.put_along_axis(out, np.asarray(idx), g, axis=1)
    return out


# ------------------------------------------------------------- activation
def gelu(x: np.ndarray) -> np.ndarray:
    """The torch.nn.GELU() that fmoe/transformer.py:28-30 applies between the two
    expert layers (default of transformer.py:45): x Phi(x), float64.  Phi through
    erfc, which keeps the relative accuracy of the negative tail."""
    x = np.asarray(x, dtype=np.float64)
    return 0.5 * x * _erfc(-x / np.sqrt(2.0))


def gelu_backward(dy: np.ndarray, x: np.ndarray) -> np.ndarray:
    """dy * (Phi(x) + x phi(x)), float64."""
    x = np.asarray(x, dtype=np.float64)
    grad = 0.5 * _erfc(-x / np.sqrt(2.0)) + x * np.exp(-0.5 * x * x) / np.sqrt(2.0 * np.pi)
    return np.asarray(dy, dtype=np.float64) * grad


# ------------------------------------------------------- whole layer (torch)
def brute_force_moe_mlp(inp, gate_idx, gate_score, w1, b1, w2, b2,
                        activation=F.gelu):
    """Dense per-expert evaluation of the MoE MLP, tests/moe.py:30-49: repeat
    every token top_k times, run each expert on the slots whose index equals
    it, write the rows back, then weight and sum each token's k rows with a
    bmm.  Slots with index -1 (dropped) contribute zero.  Differentiable."""
    top_k = gate_idx.shape[1]
    d_model = w2.shape[1]
    x_rep = inp.repeat_interleave(repeats=top_k, dim=0)
    gate_long = gate_idx.long().reshape(-1)
    o = torch.zeros(x_rep.shape[0], d_model, dtype=inp.dtype, device=inp.device)
    for e in range(w1.shape[0]):
        sel = gate_long == e
        if not bool(sel.any()):
            continue
        h = x_rep[sel] @ w1[e].t()
        if b1 is not None:
            h = h + b1[e]
        h = activation(h)
        h = h @ w2[e].t()
        if b2 is not None:
            h = h + b2[e]
        o = _put(o, sel, h)
    score = gate_score.reshape(-1, 1, top_k)
    return torch.bmm(score, o.view(-1, top_k, d_model)).reshape(-1, d_model)


def _put(o, sel, rows):
    """Out-of-place `o[sel] = rows` so autograd tracks it."""
    idx = sel.nonzero(as_tuple=True)[0]
    return o.index_copy(0, idx, rows)
