// Compiled PyTorch binding of libfmoe_hip.so: a pybind11 module named
// `fmoe_cuda`, the drop-in for the reference's extension of that name
// (cuda/fmoe_cuda.cpp:104-125: expert_count, assign_pos, linear_forward,
// linear_backward, limit_by_capacity, prune_gate_by_capacity), plus the
// dispatch and fused operators this package's own layer uses.  It holds no
// kernels: every function checks its tensors, allocates the outputs with torch,
// takes torch's current HIP stream and calls the C ABI of include/fmoe_hip.h.
// A non-zero status becomes a RuntimeError carrying fmoe_last_error().
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <c10/core/DeviceGuard.h>

#include <hip/hip_runtime_api.h>

#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "../../include/fmoe_hip.h"

namespace {

using torch::Tensor;
using OptTensor = c10::optional<Tensor>;

void need(bool cond, const std::string& msg) {
  if (!cond) throw std::runtime_error(msg);
}

void check(int status, const char* what) {
  if (status != 0)
    throw std::runtime_error(std::string(what) + " failed (status " + std::to_string(status) +
                             "): " + fmoe_last_error());
}

void dev(const Tensor& t, const char* name) {
  need(t.defined(), std::string(name) + " must be a tensor");
  need(t.is_cuda(), std::string(name) + " must be a CUDA tensor");
  need(t.is_contiguous(), std::string(name) + " must be contiguous");
}
void dev(const Tensor& t, const char* name, at::ScalarType dtype) {
  dev(t, name);
  need(t.scalar_type() == dtype, std::string(name) + " has the wrong dtype");
}

int dt(const Tensor& t, const char* name) {
  switch (t.scalar_type()) {
    case at::kFloat: return FMOE_F32;
    case at::kDouble: return FMOE_F64;
    case at::kHalf: return FMOE_F16;
    case at::kBFloat16: return FMOE_BF16;
    default: throw std::runtime_error(std::string(name) + ": unsupported dtype");
  }
}

void* stream_of(const Tensor& t) {
  return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

void* ptr(const OptTensor& t) { return t.has_value() && t->defined() ? t->data_ptr() : nullptr; }

// Routing workspace for a call on torch's current stream of `like`'s device.  One
// buffer per (device, stream) is kept and reused: launches on one stream run in
// order, and nothing in the workspace outlives a call.  A stream under graph capture
// gets a fresh tensor instead, which then belongs to the graph's own memory pool.
Tensor workspace(int64_t numel, int64_t n_expert, const Tensor& like) {
  int64_t bytes = fmoe_route_workspace_bytes(numel, (int32_t)n_expert);
  need(bytes >= 0, "route workspace: bad sizes");
  if (bytes < 1) bytes = 1;
  auto opts = like.options().dtype(at::kByte);
  void* stream = stream_of(like);
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing((hipStream_t)stream, &capturing) != hipSuccess ||
      capturing != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return torch::empty({bytes}, opts);
  }
  static std::mutex mu;
  // (never destroyed: at process exit the tensors must not be freed after torch's
  // allocator has gone)
  static auto* cache = new std::map<std::pair<int, void*>, Tensor>();
  std::lock_guard<std::mutex> lock(mu);
  Tensor& ws = (*cache)[{(int)like.device().index(), stream}];
  if (!ws.defined() || ws.numel() < bytes) ws = torch::empty({std::max<int64_t>(bytes, 1 << 16)}, opts);
  return ws;
}

// ---------------------------------------------------------------- reference surface
void expert_count(Tensor gate_idx, Tensor count) {
  dev(gate_idx, "gate_idx", at::kLong);
  dev(count, "expert_count", at::kInt);
  c10::DeviceGuard guard(gate_idx.device());
  check(fmoe_expert_count(gate_idx.data_ptr<int64_t>(), gate_idx.numel(), count.data_ptr<int32_t>(),
                          (int32_t)count.numel(), stream_of(gate_idx)),
        "expert_count");
}

void assign_pos(Tensor cum_count, Tensor gate, Tensor pos) {
  dev(cum_count, "cum_count", at::kInt);
  dev(gate, "gate", at::kLong);
  dev(pos, "pos", at::kLong);
  c10::DeviceGuard guard(gate.device());
  Tensor ws = workspace(gate.numel(), cum_count.numel(), gate);
  check(fmoe_assign_pos(cum_count.data_ptr<int32_t>(), gate.data_ptr<int64_t>(),
                        pos.data_ptr<int64_t>(), gate.numel(), (int32_t)cum_count.numel(),
                        ws.data_ptr(), ws.numel(), stream_of(gate)),
        "assign_pos");
}

// seg_off (device int32[E+1]) from the reference's host int64 counts, or from
// device counts without a host round trip.  With host counts and rows >= 0 the
// counts must not claim more rows than the buffers hold (the grouped kernels trust
// seg_off); the reference assumes the sum equals the row count.
Tensor seg_off_from_counts(const Tensor& expert_count, const Tensor& like, int64_t rows = -1) {
  need(expert_count.scalar_type() == at::kLong, "expert_count must be int64");
  const int64_t e = expert_count.numel();
  if (!expert_count.is_cuda() && rows >= 0) {
    const Tensor c = expert_count.contiguous();
    int64_t total = 0;
    for (int64_t i = 0; i < e; ++i) {
      need(c.data_ptr<int64_t>()[i] >= 0, "expert_count holds a negative count");
      total += c.data_ptr<int64_t>()[i];
    }
    need(total <= rows, "expert_count sums to " + std::to_string(total) + " rows, the buffer has " +
                            std::to_string(rows));
  }
  auto opts = like.options().dtype(at::kInt);
  if (expert_count.is_cuda()) {
    Tensor seg = torch::zeros({e + 1}, opts);
    seg.slice(0, 1).copy_(torch::cumsum(expert_count.reshape({-1}), 0));
    return seg;
  }
  Tensor cnt = expert_count.contiguous();
  Tensor seg = torch::empty({e + 1}, opts);
  check(fmoe_seg_off_from_host_counts(cnt.data_ptr<int64_t>(), e, seg.data_ptr<int32_t>(),
                                      stream_of(like)),
        "seg_off_from_host_counts");
  return seg;
}

Tensor grouped_linear_fwd(Tensor x, Tensor seg_off, Tensor weight, OptTensor bias) {
  dev(x, "x");
  dev(weight, "weight", x.scalar_type());
  dev(seg_off, "seg_off", at::kInt);
  need(x.dim() == 2 && weight.dim() == 3, "x must be 2-d and weight 3-d");
  const int64_t e = weight.size(0), out_f = weight.size(1), in_f = weight.size(2);
  need(x.size(1) == in_f, "x and weight disagree on the input features");
  need(seg_off.numel() == e + 1, "seg_off must have E+1 entries");
  if (bias.has_value() && bias->defined()) {
    dev(*bias, "bias", x.scalar_type());
    need(bias->dim() == 2 && bias->size(0) == e && bias->size(1) == out_f, "bias must be [E, out]");
  }
  c10::DeviceGuard guard(x.device());
  Tensor y = torch::empty({x.size(0), out_f}, x.options());
  check(fmoe_grouped_linear_fwd(x.data_ptr(), weight.data_ptr(), ptr(bias),
                                seg_off.data_ptr<int32_t>(), y.data_ptr(), x.size(0), in_f, out_f,
                                e, dt(x, "x"), stream_of(x)),
        "grouped_linear_fwd");
  return y;
}

// grouped_linear_fwd(..., with_gelu): y, or (y, gelu(y)) from the same launch
py::object grouped_linear_fwd_any(Tensor x, Tensor seg_off, Tensor weight, OptTensor bias,
                                  bool with_gelu) {
  if (!with_gelu) return py::cast(grouped_linear_fwd(x, seg_off, weight, bias));
  dev(x, "x");
  dev(weight, "weight", x.scalar_type());
  dev(seg_off, "seg_off", at::kInt);
  need(x.dim() == 2 && weight.dim() == 3, "x must be 2-d and weight 3-d");
  const int64_t e = weight.size(0), out_f = weight.size(1), in_f = weight.size(2);
  need(x.size(1) == in_f, "x and weight disagree on the input features");
  need(seg_off.numel() == e + 1, "seg_off must have E+1 entries");
  if (bias.has_value() && bias->defined()) {
    dev(*bias, "bias", x.scalar_type());
    need(bias->dim() == 2 && bias->size(0) == e && bias->size(1) == out_f, "bias must be [E, out]");
  }
  c10::DeviceGuard guard(x.device());
  Tensor y = torch::empty({x.size(0), out_f}, x.options());
  Tensor y_act = torch::empty_like(y);
  check(fmoe_grouped_linear_fwd_act(x.data_ptr(), weight.data_ptr(), ptr(bias),
                                    seg_off.data_ptr<int32_t>(), y.data_ptr(), y_act.data_ptr(),
                                    x.size(0), in_f, out_f, e, dt(x, "x"), stream_of(x)),
        "grouped_linear_fwd_act");
  return py::make_tuple(y, y_act);
}

std::tuple<OptTensor, OptTensor, OptTensor> grouped_linear_bwd(Tensor dy, Tensor x, Tensor seg_off,
                                                               Tensor weight, bool need_bias,
                                                               bool need_dx, bool need_dw,
                                                               OptTensor act_pre) {
  dev(dy, "dy");
  dev(x, "x", dy.scalar_type());
  dev(weight, "weight", dy.scalar_type());
  dev(seg_off, "seg_off", at::kInt);
  need(x.dim() == 2 && weight.dim() == 3, "x must be 2-d and weight 3-d");
  const int64_t e = weight.size(0), out_f = weight.size(1), in_f = weight.size(2);
  const int64_t n = x.size(0);
  need(dy.dim() == 2 && dy.size(0) == n && dy.size(1) == out_f, "dy must be [rows, out]");
  need(x.size(1) == in_f, "x must be [rows, in]");
  need(seg_off.numel() == e + 1, "seg_off must have E+1 entries");
  c10::DeviceGuard guard(dy.device());
  OptTensor dx, dw, db;
  if (need_dx) dx = torch::empty({n, in_f}, dy.options());
  if (need_dw) dw = torch::empty_like(weight);
  if (need_bias) db = torch::empty({e, out_f}, dy.options());
  if (act_pre && need_dx) {
    dev(*act_pre, "act_pre", dy.scalar_type());
    need(act_pre->dim() == 2 && act_pre->size(0) == n && act_pre->size(1) == in_f,
         "act_pre must be [rows, in]");
    check(fmoe_grouped_linear_bwd_act(dy.data_ptr(), x.data_ptr(), weight.data_ptr(),
                                      seg_off.data_ptr<int32_t>(), act_pre->data_ptr(), ptr(dx),
                                      ptr(dw), ptr(db), n, in_f, out_f, e, dt(dy, "dy"),
                                      stream_of(dy)),
          "grouped_linear_bwd_act");
  } else if (need_dx || need_dw || need_bias)
    check(fmoe_grouped_linear_bwd(dy.data_ptr(), x.data_ptr(), weight.data_ptr(),
                                  seg_off.data_ptr<int32_t>(), ptr(dx), ptr(dw), ptr(db), n, in_f,
                                  out_f, e, dt(dy, "dy"), stream_of(dy)),
          "grouped_linear_bwd");
  return {dx, dw, db};
}

// Device int64[n] of the tensors' data pointers (see fmoe_pointer_table)
Tensor pointer_table(std::vector<Tensor> tensors) {
  need(!tensors.empty(), "pointer_table: no tensors");
  const Tensor& first = tensors[0];
  std::vector<const void*> ptrs;
  ptrs.reserve(tensors.size());
  for (const Tensor& t : tensors) {
    dev(t, "pointer_table entry", first.scalar_type());
    need(t.device() == first.device() && t.sizes() == first.sizes(),
         "pointer_table: tensors must share device and shape");
    need((uintptr_t)t.data_ptr() % 16 == 0, "pointer_table: tensors must be 16-byte aligned");
    ptrs.push_back(t.data_ptr());
  }
  c10::DeviceGuard guard(first.device());
  Tensor table = torch::empty({(int64_t)ptrs.size()}, first.options().dtype(at::kLong));
  check(fmoe_pointer_table(ptrs.data(), (int64_t)ptrs.size(), (const void**)table.data_ptr(),
                           stream_of(first)),
        "pointer_table");
  return table;
}

py::object grouped_linear_fwd_ptrs(Tensor x, Tensor seg_off, Tensor w_table, OptTensor b_table,
                                   int64_t out_f, bool with_gelu) {
  dev(x, "x");
  dev(seg_off, "seg_off", at::kInt);
  dev(w_table, "w_table", at::kLong);
  need(x.dim() == 2, "x must be [rows, in]");
  const int64_t e = w_table.numel();
  need(seg_off.numel() == e + 1, "seg_off must have E+1 entries");
  if (b_table.has_value() && b_table->defined()) {
    dev(*b_table, "b_table", at::kLong);
    need(b_table->numel() == e, "b_table must have E entries");
  }
  c10::DeviceGuard guard(x.device());
  Tensor y = torch::empty({x.size(0), out_f}, x.options());
  OptTensor y_act;
  if (with_gelu) y_act = torch::empty_like(y);
  check(fmoe_grouped_linear_fwd_ptrs(x.data_ptr(), (const void* const*)w_table.data_ptr(),
                                     (const void* const*)ptr(b_table), seg_off.data_ptr<int32_t>(),
                                     y.data_ptr(), ptr(y_act), x.size(0), x.size(1), out_f, e,
                                     dt(x, "x"), stream_of(x)),
        "grouped_linear_fwd_ptrs");
  if (with_gelu) return py::make_tuple(y, *y_act);
  return py::cast(y);
}

std::tuple<OptTensor, OptTensor, OptTensor> grouped_linear_bwd_ptrs(
    Tensor dy, Tensor x, Tensor seg_off, Tensor w_table, bool need_bias, bool need_dx,
    bool need_dw, OptTensor act_pre) {
  dev(dy, "dy");
  dev(x, "x", dy.scalar_type());
  dev(seg_off, "seg_off", at::kInt);
  dev(w_table, "w_table", at::kLong);
  need(x.dim() == 2 && dy.dim() == 2 && dy.size(0) == x.size(0),
       "dy must be [rows, out] and x [rows, in]");
  const int64_t e = w_table.numel(), n = x.size(0), in_f = x.size(1), out_f = dy.size(1);
  need(seg_off.numel() == e + 1, "seg_off must have E+1 entries");
  c10::DeviceGuard guard(dy.device());
  OptTensor dx, dw, db;
  if (need_dx) dx = torch::empty({n, in_f}, dy.options());
  if (need_dw) dw = torch::empty({e, out_f, in_f}, dy.options());
  if (need_bias) db = torch::empty({e, out_f}, dy.options());
  const bool with_act = act_pre.has_value() && act_pre->defined() && need_dx;
  if (with_act) {
    dev(*act_pre, "act_pre", dy.scalar_type());
    need(act_pre->dim() == 2 && act_pre->size(0) == n && act_pre->size(1) == in_f,
         "act_pre must be [rows, in]");
  }
  if (need_dx || need_dw || need_bias)
    check(fmoe_grouped_linear_bwd_ptrs(dy.data_ptr(), x.data_ptr(),
                                       (const void* const*)w_table.data_ptr(),
                                       seg_off.data_ptr<int32_t>(),
                                       with_act ? act_pre->data_ptr() : nullptr, ptr(dx), ptr(dw),
                                       ptr(db), n, in_f, out_f, e, dt(dy, "dy"), stream_of(dy)),
          "grouped_linear_bwd_ptrs");
  return {dx, dw, db};
}

Tensor linear_forward(Tensor input_buf, Tensor expert_count, Tensor weight, OptTensor bias) {
  dev(input_buf, "input_buf");
  c10::DeviceGuard guard(input_buf.device());
  need(input_buf.dim() == 2, "input_buf must be [rows, in]");
  return grouped_linear_fwd(input_buf, seg_off_from_counts(expert_count, input_buf, input_buf.size(0)),
                            weight, bias);
}

std::vector<Tensor> linear_backward(Tensor grad_output_buf, Tensor input_buf, Tensor expert_count,
                                    Tensor weight, OptTensor /*bias*/) {
  dev(grad_output_buf, "grad_output_buf");
  dev(input_buf, "input_buf", grad_output_buf.scalar_type());
  c10::DeviceGuard guard(input_buf.device());
  need(input_buf.dim() == 2, "input_buf must be [rows, in]");
  auto r = grouped_linear_bwd(grad_output_buf, input_buf,
                              seg_off_from_counts(expert_count, input_buf, input_buf.size(0)),
                              weight, true, true, true, c10::nullopt);
  return {*std::get<0>(r), *std::get<1>(r), *std::get<2>(r)};
}

Tensor limit_by_capacity(Tensor expert_count, Tensor capacity, int64_t n_expert, int64_t n_worker) {
  dev(expert_count, "expert_count", at::kLong);
  dev(capacity, "capacity", at::kInt);
  need(expert_count.numel() >= n_expert * n_worker, "expert_count too short");
  need(capacity.numel() >= n_expert, "capacity too short");
  c10::DeviceGuard guard(expert_count.device());
  Tensor ack = torch::empty_like(expert_count);
  check(fmoe_limit_by_capacity(expert_count.data_ptr<int64_t>(), capacity.data_ptr<int32_t>(),
                               ack.data_ptr<int64_t>(), n_expert, n_worker, stream_of(expert_count)),
        "limit_by_capacity");
  return ack;
}

Tensor prune_gate_by_capacity(Tensor gate_idx, Tensor expert_count, int64_t n_expert,
                              int64_t n_worker) {
  dev(gate_idx, "gate_idx", at::kLong);
  dev(expert_count, "expert_count", at::kInt);
  need(expert_count.numel() >= n_expert * n_worker, "expert_count too short");
  c10::DeviceGuard guard(gate_idx.device());
  Tensor out = torch::empty_like(gate_idx);
  Tensor ws = workspace(gate_idx.numel(), n_expert * n_worker, gate_idx);
  check(fmoe_prune_gate_by_capacity(gate_idx.data_ptr<int64_t>(), out.data_ptr<int64_t>(),
                                    expert_count.data_ptr<int32_t>(), gate_idx.numel(), n_expert,
                                    n_worker, ws.data_ptr(), ws.numel(), stream_of(gate_idx)),
        "prune_gate_by_capacity");
  return out;
}

// ---------------------------------------------------------------- dispatch
Tensor local_scatter(Tensor inp, Tensor pos, int64_t idx_div, OptTensor n_rows_dev) {
  dev(inp, "inp");
  dev(pos, "pos", at::kLong);
  need(inp.dim() == 2, "inp must be [rows, d]");
  c10::DeviceGuard guard(inp.device());
  Tensor out = torch::empty({pos.numel(), inp.size(1)}, inp.options());
  check(fmoe_local_scatter(inp.data_ptr(), pos.data_ptr<int64_t>(), out.data_ptr(), pos.numel(),
                           inp.size(1), idx_div, (const int32_t*)ptr(n_rows_dev), dt(inp, "inp"),
                           stream_of(inp)),
        "local_scatter");
  return out;
}

Tensor scatter_tokens(Tensor inp, Tensor inv, int64_t top_k) {
  dev(inp, "inp");
  dev(inv, "inv", at::kInt);
  need(inp.dim() == 2, "inp must be [tokens, d]");
  need(inv.numel() == inp.size(0) * top_k, "inv must have tokens * top_k entries");
  c10::DeviceGuard guard(inp.device());
  Tensor out = torch::empty({inp.size(0) * top_k, inp.size(1)}, inp.options());
  check(fmoe_scatter_tokens(inp.data_ptr(), inv.data_ptr<int32_t>(), out.data_ptr(), inp.size(0),
                            top_k, inp.size(1), dt(inp, "inp"), stream_of(inp)),
        "scatter_tokens");
  return out;
}

Tensor local_gather(Tensor inp, Tensor pos, int64_t out_batch_size, bool maybe_overlap,
                    OptTensor n_rows_dev) {
  dev(inp, "inp");
  dev(pos, "pos", at::kLong);
  need(inp.dim() == 2, "inp must be [rows, d]");
  need(inp.size(0) >= pos.numel(), "inp has fewer rows than pos");
  if (maybe_overlap && inp.scalar_type() != at::kFloat && inp.scalar_type() != at::kDouble)
    // half types accumulate in fp32, rounded once at the end
    return local_gather(inp.to(at::kFloat), pos, out_batch_size, true, n_rows_dev)
        .to(inp.scalar_type());
  c10::DeviceGuard guard(inp.device());
  Tensor out = torch::empty({out_batch_size, inp.size(1)}, inp.options());
  check(fmoe_local_gather(inp.data_ptr(), pos.data_ptr<int64_t>(), out.data_ptr(), pos.numel(),
                          out_batch_size, inp.size(1), (const int32_t*)ptr(n_rows_dev),
                          maybe_overlap ? 1 : 0, dt(inp, "inp"), stream_of(inp)),
        "local_gather");
  return out;
}

// ---------------------------------------------------------------- fused ops
std::tuple<Tensor, Tensor, Tensor, OptTensor> route(Tensor gate, int64_t n_expert, bool want_inv) {
  dev(gate, "gate", at::kLong);
  c10::DeviceGuard guard(gate.device());
  const int64_t n = gate.numel();
  Tensor count = torch::empty({n_expert}, gate.options());
  Tensor seg = torch::empty({n_expert + 1}, gate.options().dtype(at::kInt));
  Tensor pos = torch::empty({n}, gate.options());
  OptTensor inv;
  if (want_inv) inv = torch::empty({n}, gate.options().dtype(at::kInt));
  Tensor ws = workspace(n, n_expert, gate);
  check(fmoe_route(gate.data_ptr<int64_t>(), n, (int32_t)n_expert, count.data_ptr<int64_t>(),
                   seg.data_ptr<int32_t>(), pos.data_ptr<int64_t>(), (int32_t*)ptr(inv),
                   ws.data_ptr(), ws.numel(), stream_of(gate)),
        "route");
  return {pos, count, seg, inv};
}

void route_static(Tensor gate, int64_t n_expert, Tensor count, Tensor seg_off, Tensor pos,
                  OptTensor inv) {
  dev(gate, "gate", at::kLong);
  dev(count, "count", at::kLong);
  dev(seg_off, "seg_off", at::kInt);
  dev(pos, "pos", at::kLong);
  const int64_t n = gate.numel();
  need(count.numel() == n_expert && seg_off.numel() == n_expert + 1 && pos.numel() >= n,
       "route_static: count[E], seg_off[E+1] and pos[N] expected");
  if (inv.has_value() && inv->defined()) {
    dev(*inv, "inv", at::kInt);
    need(inv->numel() >= n, "route_static: inv must have N entries");
  }
  c10::DeviceGuard guard(gate.device());
  check(fmoe_route_static(gate.data_ptr<int64_t>(), n, (int32_t)n_expert, count.data_ptr<int64_t>(),
                          seg_off.data_ptr<int32_t>(), pos.data_ptr<int64_t>(), (int32_t*)ptr(inv),
                          stream_of(gate)),
        "route_static");
}

Tensor gather_combine_fwd(Tensor buf, Tensor inv, Tensor score, int64_t n_tokens, int64_t top_k) {
  dev(buf, "buf");
  dev(inv, "inv", at::kInt);
  dev(score, "score", buf.scalar_type());
  need(inv.numel() == n_tokens * top_k && score.numel() == n_tokens * top_k,
       "inv/score must have n_tokens*top_k entries");
  c10::DeviceGuard guard(buf.device());
  Tensor y = torch::empty({n_tokens, buf.size(1)}, buf.options());
  check(fmoe_gather_combine_fwd(buf.data_ptr(), inv.data_ptr<int32_t>(), score.data_ptr(),
                                y.data_ptr(), n_tokens, top_k, buf.size(1), dt(buf, "buf"),
                                stream_of(buf)),
        "gather_combine_fwd");
  return y;
}

std::tuple<Tensor, Tensor> gather_combine_bwd(Tensor dy, Tensor buf, Tensor inv, Tensor score,
                                              int64_t n_tokens, int64_t top_k) {
  dev(dy, "dy");
  dev(buf, "buf", dy.scalar_type());
  dev(inv, "inv", at::kInt);
  dev(score, "score", dy.scalar_type());
  need(dy.dim() == 2 && dy.size(0) == n_tokens && dy.size(1) == buf.size(1),
       "dy must be [n_tokens, d]");
  c10::DeviceGuard guard(dy.device());
  Tensor dbuf = torch::empty_like(buf);
  Tensor dscore = torch::empty({n_tokens, top_k}, dy.options());
  check(fmoe_gather_combine_bwd(dy.data_ptr(), buf.data_ptr(), inv.data_ptr<int32_t>(),
                                score.data_ptr(), dbuf.data_ptr(), dscore.data_ptr(), n_tokens,
                                top_k, buf.size(1), dt(dy, "dy"), stream_of(dy)),
        "gather_combine_bwd");
  return {dbuf, dscore};
}

Tensor scatter_reduce(Tensor dbuf, Tensor inv, int64_t n_tokens, int64_t top_k) {
  dev(dbuf, "dbuf");
  dev(inv, "inv", at::kInt);
  need(inv.numel() == n_tokens * top_k, "inv must have n_tokens*top_k entries");
  c10::DeviceGuard guard(dbuf.device());
  Tensor dx = torch::empty({n_tokens, dbuf.size(1)}, dbuf.options());
  check(fmoe_scatter_reduce(dbuf.data_ptr(), inv.data_ptr<int32_t>(), dx.data_ptr(), n_tokens, top_k,
                            dbuf.size(1), dt(dbuf, "dbuf"), stream_of(dbuf)),
        "scatter_reduce");
  return dx;
}

std::tuple<Tensor, Tensor> topk_softmax_fwd(Tensor logits, int64_t top_k) {
  dev(logits, "logits");
  need(logits.dim() == 2, "logits must be [tokens, experts]");
  c10::DeviceGuard guard(logits.device());
  const int64_t t = logits.size(0), e = logits.size(1);
  Tensor idx = torch::empty({t, top_k}, logits.options().dtype(at::kLong));
  Tensor score = torch::empty({t, top_k}, logits.options());
  check(fmoe_topk_softmax_fwd(logits.data_ptr(), t, (int32_t)e, (int32_t)top_k,
                              idx.data_ptr<int64_t>(), score.data_ptr(), dt(logits, "logits"),
                              stream_of(logits)),
        "topk_softmax_fwd");
  return {idx, score};
}

Tensor topk_softmax_bwd(Tensor dscore, Tensor score, Tensor idx, int64_t n_expert) {
  dev(dscore, "dscore");
  dev(score, "score", dscore.scalar_type());
  dev(idx, "idx", at::kLong);
  need(score.dim() == 2 && dscore.sizes() == score.sizes() && idx.sizes() == score.sizes(),
       "dscore, score and idx must all be [tokens, top_k]");
  c10::DeviceGuard guard(score.device());
  Tensor dlogits = torch::empty({score.size(0), n_expert}, score.options());
  check(fmoe_topk_softmax_bwd(dscore.data_ptr(), score.data_ptr(), idx.data_ptr<int64_t>(),
                              dlogits.data_ptr(), score.size(0), (int32_t)n_expert,
                              (int32_t)score.size(1), dt(score, "score"), stream_of(score)),
        "topk_softmax_bwd");
  return dlogits;
}

int64_t row_len(const Tensor& x) { return x.dim() >= 1 && x.numel() ? x.size(-1) : 0; }

Tensor gelu_fwd(Tensor x, OptTensor n_rows_dev) {
  dev(x, "x");
  c10::DeviceGuard guard(x.device());
  Tensor y = torch::empty_like(x);
  check(fmoe_gelu_fwd(x.data_ptr(), y.data_ptr(), x.numel(), (const int32_t*)ptr(n_rows_dev),
                      row_len(x), dt(x, "x"), stream_of(x)),
        "gelu_fwd");
  return y;
}

Tensor gelu_bwd(Tensor dy, Tensor x, OptTensor n_rows_dev) {
  dev(x, "x");
  dev(dy, "dy", x.scalar_type());
  need(dy.numel() == x.numel(), "dy and x must be of one size");
  c10::DeviceGuard guard(x.device());
  Tensor dx = torch::empty_like(x);
  check(fmoe_gelu_bwd(dy.data_ptr(), x.data_ptr(), dx.data_ptr(), x.numel(),
                      (const int32_t*)ptr(n_rows_dev), row_len(x), dt(x, "x"), stream_of(x)),
        "gelu_bwd");
  return dx;
}

void set_gemm_path(int64_t path) { check(fmoe_set_gemm_path((int)path), "set_gemm_path"); }

}  // namespace

PYBIND11_MODULE(fmoe_cuda, m) {
  m.doc() = "MI355X drop-in for FastMoE's fmoe_cuda extension (compiled binding of libfmoe_hip.so)";
  namespace py = pybind11;
  // the reference surface, cuda/fmoe_cuda.cpp:117-124
  m.def("expert_count", &expert_count, "count gate indices");
  m.def("assign_pos", &assign_pos, "assign pos by gate");
  m.def("linear_forward", &linear_forward, py::arg("input_buf"), py::arg("expert_count"),
        py::arg("weight"), py::arg("bias") = py::none());
  m.def("linear_backward", &linear_backward, py::arg("grad_output_buf"), py::arg("input_buf"),
        py::arg("expert_count"), py::arg("weight"), py::arg("bias") = py::none());
  m.def("limit_by_capacity", &limit_by_capacity);
  m.def("prune_gate_by_capacity", &prune_gate_by_capacity);
  // dispatch
  m.def("local_scatter", &local_scatter, py::arg("inp"), py::arg("pos"), py::arg("idx_div") = 1,
        py::arg("n_rows_dev") = py::none());
  m.def("scatter_tokens", &scatter_tokens);
  m.def("local_gather", &local_gather, py::arg("inp"), py::arg("pos"), py::arg("out_batch_size"),
        py::arg("maybe_overlap") = true, py::arg("n_rows_dev") = py::none());
  // fused, synchronisation-free operators
  m.def("route", &route, py::arg("gate"), py::arg("n_expert"), py::arg("want_inv") = true);
  m.def("route_static", &route_static, py::arg("gate"), py::arg("n_expert"), py::arg("count"),
        py::arg("seg_off"), py::arg("pos"), py::arg("inv") = py::none());
  m.def("grouped_linear_fwd", &grouped_linear_fwd_any, py::arg("x"), py::arg("seg_off"),
        py::arg("weight"), py::arg("bias") = py::none(), py::arg("with_gelu") = false);
  m.def("grouped_linear_bwd", &grouped_linear_bwd, py::arg("dy"), py::arg("x"), py::arg("seg_off"),
        py::arg("weight"), py::arg("need_bias") = true, py::arg("need_dx") = true,
        py::arg("need_dw") = true, py::arg("act_pre") = py::none());
  m.def("pointer_table", &pointer_table);
  m.def("grouped_linear_fwd_ptrs", &grouped_linear_fwd_ptrs, py::arg("x"), py::arg("seg_off"),
        py::arg("w_table"), py::arg("b_table"), py::arg("out_feat"),
        py::arg("with_gelu") = false);
  m.def("grouped_linear_bwd_ptrs", &grouped_linear_bwd_ptrs, py::arg("dy"), py::arg("x"),
        py::arg("seg_off"), py::arg("w_table"), py::arg("need_bias") = true,
        py::arg("need_dx") = true, py::arg("need_dw") = true, py::arg("act_pre") = py::none());
  m.def("gather_combine_fwd", &gather_combine_fwd);
  m.def("gather_combine_bwd", &gather_combine_bwd);
  m.def("scatter_reduce", &scatter_reduce);
  m.def("topk_softmax_fwd", &topk_softmax_fwd);
  m.def("topk_softmax_bwd", &topk_softmax_bwd);
  m.def("gelu_fwd", &gelu_fwd, py::arg("x"), py::arg("n_rows_dev") = py::none());
  m.def("gelu_bwd", &gelu_bwd, py::arg("dy"), py::arg("x"), py::arg("n_rows_dev") = py::none());
  m.def("set_gemm_path", &set_gemm_path);
  m.def("_seg_off_from_counts",
        [](Tensor expert_count, py::object device) {
          // `device` may be a torch.device or anything torch.empty accepts
          Tensor like = torch::empty({0}, torch::TensorOptions().device(
                                              py::cast<c10::Device>(device)));
          c10::DeviceGuard guard(like.device());
          return seg_off_from_counts(expert_count, like);
        });
  m.attr("MAX_GATE_TOP_K") = FMOE_MAX_GATE_TOP_K;
  m.attr("binding") = "compiled";
#ifdef FMOE_EXT_SOURCE_HASH
  // digest of this file and of the C ABI header it was compiled against: the loader
  // rebuilds a binary whose digest differs from the sources beside it
  m.attr("source_hash") = "fmoe-ext:" FMOE_EXT_SOURCE_HASH;
#endif
}
