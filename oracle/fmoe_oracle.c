/*
 * CPU restatement of the reference's single-GPU MoE hot path, in plain C.
 *
 * TEST INFRASTRUCTURE ONLY: the checker that tests/, the smoke run and the CPU
 * leg of the benchmark compare the HIP kernels against.  Nothing in the
 * product imports, links or calls it.
 *
 * Every function names the reference lines it follows (paths relative to the
 * reference tree).  Where the reference's result depends on the order in
 * which GPU threads win an atomic, the restatement fixes ONE legal order and
 * says which; the parity tests additionally check the order-free invariants.
 *
 * What pins each function (see tests/test_oracle.py):
 *   expert_count      numpy.bincount
 *   assign_pos        numpy stable argsort; permutation / membership invariants
 *   limit_by_capacity closed form min(ec, cap) at one worker; conservation and
 *                     monotonicity invariants at several
 *   prune_gate        kept_e == min(count_e, cap_e); rank-from-argsort formula
 *   scatter / gather  numpy fancy indexing
 *   combine           numpy einsum
 *   linear fwd / bwd  torch F.linear and torch.autograd per segment; E == 1
 *                     reduces to nn.Linear; empty experts give zero gradients
 */
#include <stdint.h>
#include <string.h>

/* cuda/local_exchange.cuh:36-69: histogram, -1 and out-of-range skipped,
 * accumulated into the caller's buffer. */
void oracle_expert_count(const int64_t* gate, int64_t n, int32_t* count,
                         int64_t n_expert) {
  for (int64_t i = 0; i < n; ++i) {
    int64_t g = gate[i];
    if (g == -1) continue;
    if (g < 0 || g >= n_expert) continue;
    count[g] += 1;
  }
}

/* cuda/local_exchange.cuh:5-16: p = atomicSub(&cum[g], 1); pos[p-1] = idx.
 * Arrival order fixed to DESCENDING idx, which fills every segment in
 * ascending slot order.  cum is left holding the exclusive prefix. */
void oracle_assign_pos(int32_t* cum_count, const int64_t* gate, int64_t* pos,
                       int64_t numel) {
  for (int64_t idx = numel - 1; idx >= 0; --idx) {
    int64_t g = gate[idx];
    if (g > -1) {
      int32_t p = cum_count[g];
      cum_count[g] = p - 1;
      pos[p - 1] = idx;
    }
  }
}

/* cuda/balancing.cuh:5-21 with the launch of :23-30: one thread per (worker,
 * expert); arrival order fixed to ASCENDING worker id. */
void oracle_limit_by_capacity(const int64_t* ec, int32_t* cap, int64_t* eca,
                              int64_t n_expert, int64_t n_worker) {
  for (int64_t eid = 0; eid < n_expert; ++eid) {
    for (int64_t wid = 0; wid < n_worker; ++wid) {
      int32_t proposal = (int32_t)ec[wid * n_expert + eid];
      int32_t cap_left = cap[eid];
      cap[eid] = cap_left - proposal;
      if (cap_left >= proposal) {
        eca[wid * n_expert + eid] = proposal;
      } else if (cap_left >= 0) {
        eca[wid * n_expert + eid] = cap_left;
      } else {
        eca[wid * n_expert + eid] = 0;
      }
    }
  }
}

/* cuda/balancing.cuh:32-45: orig = atomicSub(&ec[g], 1); keep iff orig > 0.
 * Arrival order fixed to ASCENDING slot index.  The reference indexes ec[-1]
 * for an input of -1; here such entries (and any outside [0, n_bins)) pass
 * through unchanged and consume nothing. */
void oracle_prune_gate_by_capacity(const int64_t* gate, int64_t* new_gate,
                                   int32_t* ec, int64_t numel, int64_t n_bins) {
  for (int64_t i = 0; i < numel; ++i) {
    int64_t g = gate[i];
    if (g < 0 || g >= n_bins) {
      new_gate[i] = g;
      continue;
    }
    int32_t orig = ec[g];
    ec[g] = orig - 1;
    new_gate[i] = orig <= 0 ? -1 : g;
  }
}

/* fmoe/functions.py:78-80 after the `pos // top_k` of fmoe/layers.py:49-53:
 * out[r] = inp[idx[r] / idx_div], rows of row_bytes bytes. */
void oracle_local_scatter(const void* inp, const int64_t* idx, void* out,
                          int64_t n_rows, int64_t row_bytes, int64_t idx_div) {
  for (int64_t r = 0; r < n_rows; ++r)
    memcpy((char*)out + r * row_bytes,
           (const char*)inp + (idx[r] / idx_div) * row_bytes, (size_t)row_bytes);
}

/* fmoe/functions.py:83-90 with maybe_overlap=False: zeros, then
 * out[pos[r]] = inp[r]. */
void oracle_local_gather(const void* inp, const int64_t* pos, void* out,
                         int64_t n_rows, int64_t out_rows, int64_t row_bytes) {
  memset(out, 0, (size_t)(out_rows * row_bytes));
  for (int64_t r = 0; r < n_rows; ++r)
    memcpy((char*)out + pos[r] * row_bytes, (const char*)inp + r * row_bytes,
           (size_t)row_bytes);
}

/* fmoe/functions.py:83-90 with maybe_overlap=True (index_add_), double. */
void oracle_local_gather_add_f64(const double* inp, const int64_t* pos,
                                 double* out, int64_t n_rows, int64_t out_rows,
                                 int64_t d) {
  memset(out, 0, (size_t)(out_rows * d) * sizeof(double));
  for (int64_t r = 0; r < n_rows; ++r)
    for (int64_t c = 0; c < d; ++c) out[pos[r] * d + c] += inp[r * d + c];
}

/* fmoe/layers.py:281-295: y[t] = sum_j score[t][j] * out[t*k + j]. */
void oracle_combine_f64(const double* score, const double* out, double* y,
                        int64_t n_tokens, int64_t top_k, int64_t d) {
  for (int64_t t = 0; t < n_tokens; ++t)
    for (int64_t c = 0; c < d; ++c) {
      double s = 0;
      for (int64_t j = 0; j < top_k; ++j)
        s += score[t * top_k + j] * out[(t * top_k + j) * d + c];
      y[t * d + c] = s;
    }
}

/* cuda/parallel_linear.cuh:55-89 (+ bias pre-fill of
 * cuda/parallel_linear.cu:24-25): Y[seg_e] = X[seg_e] W_e^T + b_e, segments
 * of expert_count[e] rows in expert order, experts with no rows skipped. */
void oracle_linear_forward_f64(const double* x, const double* w,
                               const double* bias, const int64_t* expert_count,
                               double* y, int64_t in_feat, int64_t out_feat,
                               int64_t n_expert) {
  int64_t ptr = 0;
  for (int64_t e = 0; e < n_expert; ++e) {
    int64_t cnt = expert_count[e];
    if (cnt == 0) continue;
    const double* we = w + e * in_feat * out_feat;
    for (int64_t r = ptr; r < ptr + cnt; ++r)
      for (int64_t o = 0; o < out_feat; ++o) {
        double s = bias ? bias[e * out_feat + o] : 0.0;
        for (int64_t i = 0; i < in_feat; ++i)
          s += x[r * in_feat + i] * we[o * in_feat + i];
        y[r * out_feat + o] = s;
      }
    ptr += cnt;
  }
}

/* cuda/parallel_linear.cuh:91-163: dX[seg_e] = dY[seg_e] W_e;
 * dW_e = dY[seg_e]^T X[seg_e]; db_e = column sums of dY[seg_e]
 * (column_reduce, :8-53); experts with no rows get zero dW_e and db_e
 * (:115-119). */
void oracle_linear_backward_f64(const double* dy, const double* x,
                                const double* w, const int64_t* expert_count,
                                double* dx, double* dw, double* db,
                                int64_t in_feat, int64_t out_feat,
                                int64_t n_expert) {
  int64_t ptr = 0;
  for (int64_t e = 0; e < n_expert; ++e) {
    int64_t cnt = expert_count[e];
    const double* we = w + e * in_feat * out_feat;
    double* dwe = dw + e * in_feat * out_feat;
    memset(dwe, 0, (size_t)(in_feat * out_feat) * sizeof(double));
    memset(db + e * out_feat, 0, (size_t)out_feat * sizeof(double));
    if (cnt == 0) continue;
    for (int64_t r = ptr; r < ptr + cnt; ++r) {
      for (int64_t i = 0; i < in_feat; ++i) {
        double s = 0;
        for (int64_t o = 0; o < out_feat; ++o)
          s += dy[r * out_feat + o] * we[o * in_feat + i];
        dx[r * in_feat + i] = s;
      }
      for (int64_t o = 0; o < out_feat; ++o) {
        double g = dy[r * out_feat + o];
        db[e * out_feat + o] += g;
        for (int64_t i = 0; i < in_feat; ++i)
          dwe[o * in_feat + i] += g * x[r * in_feat + i];
      }
    }
    ptr += cnt;
  }
}
