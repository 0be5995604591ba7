// Top-k gate on gfx950: the k largest logits of every token and the softmax
// over those k values in one pass, and the matching backward pass.
//
// Replaces the torch.topk + F.softmax pair of fmoe/gates/naive_gate.py:31-38
// (and, in the backward, softmax-backward + zero-fill + scatter).  Results are
// ordered by descending logit; equal logits go to the lower expert index.
//
// A group of lanes shares a token.  Up to 512 experts the group (8 lanes, 32
// above 32 experts) holds all logits in registers and every one of the k
// rounds is a plain arg-max over what is still alive; above that each of 32
// lanes keeps the k best of its share as a sorted list and the rounds pop the
// overall winners.  The arrays are a few hundred KiB at most: the kernels are
// bound by launch latency and instruction count, not by memory.
#include "common.h"

namespace fmoe {

constexpr int kGateThreads = 256;
// Lanes per token of the backward kernel: 8, and 32 from this many experts on.
constexpr int kGateWideFrom = 64;
constexpr int kGateChunk = 8;                       // logits a lane loads before it sorts them

// Order of the candidates: larger logit first, equal logits by expert index.
// A NaN logit ranks above every number (as torch.topk ranks it), so a diverged
// row selects its NaNs and its scores come out as NaN instead of being masked.
template <typename A>
__device__ __forceinline__ bool better(A v, int e, A w, int f) {
  const bool v_nan = v != v, w_nan = w != w;
  if (v_nan || w_nan) return v_nan && (!w_nan || e < f);
  return v > w || (v == w && e < f);
}

template <typename T, int KMAX, int LANES>
__global__ __launch_bounds__(kGateThreads) void topk_softmax_fwd_kernel(
    const T* __restrict__ logits, int64_t n_tokens, int n_expert, int top_k,
    int64_t* __restrict__ idx, T* __restrict__ score) {
  using acc_t = typename Elem<T>::acc_t;
  const int g = threadIdx.x % LANES;
  const int64_t t = (int64_t)blockIdx.x * (kGateThreads / LANES) + threadIdx.x / LANES;
  const bool live = t < n_tokens;
  // local candidates, best first; empty slots hold (-inf, INT_MAX)
  acc_t val[KMAX];
  int id[KMAX];
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    val[j] = -INFINITY;
    id[j] = 0x7fffffff;
  }
  if (live) {
    const T* row = logits + t * n_expert;
    // kGateChunk loads in flight, then their insertions: one memory round trip
    // per chunk instead of one per logit
    for (int e0 = g; e0 < n_expert; e0 += LANES * kGateChunk) {
      T raw[kGateChunk];
#pragma unroll
      for (int u = 0; u < kGateChunk; ++u) {
        const int e = e0 + u * LANES;
        if (e < n_expert) raw[u] = row[e];
      }
#pragma unroll
      for (int u = 0; u < kGateChunk; ++u) {
        int ve = e0 + u * LANES;
        if (ve >= n_expert) break;
        acc_t v = Elem<T>::to_acc(raw[u]);
        // insertion into the sorted list: the displaced entry moves down
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
          if (better(v, ve, val[j], id[j])) {
            const acc_t tv = val[j];
            const int te = id[j];
            val[j] = v;
            id[j] = ve;
            v = tv;
            ve = te;
          }
        }
      }
    }
  }
  // k rounds: the best head of the LANES lists wins and is popped
  acc_t sel[KMAX];
  int sel_id[KMAX];
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    sel[j] = -INFINITY;
    sel_id[j] = 0;
    if (j < top_k) {
      acc_t bv = val[0];
      int be = id[0];
#pragma unroll
      for (int d = 1; d < LANES; d <<= 1) {
        const acc_t ov = __shfl_xor(bv, d, kWave);
        const int oe = __shfl_xor(be, d, kWave);
        if (better(ov, oe, bv, be)) {
          bv = ov;
          be = oe;
        }
      }
      sel[j] = bv;
      sel_id[j] = be;
      if (id[0] == be) {  // this lane held the winner: pop it
#pragma unroll
        for (int q = 0; q + 1 < KMAX; ++q) {
          val[q] = val[q + 1];
          id[q] = id[q + 1];
        }
        val[KMAX - 1] = -INFINITY;
        id[KMAX - 1] = 0x7fffffff;
      }
    }
  }
  if (!live || g != 0) return;
  // softmax over the winners; sel[0] is the largest
  acc_t p[KMAX];
  acc_t sum = 0;
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    p[j] = 0;
    if (j < top_k) {
      p[j] = exp(sel[j] - sel[0]);
      sum += p[j];
    }
  }
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    if (j < top_k) {
      idx[t * top_k + j] = sel_id[j];
      score[t * top_k + j] = Elem<T>::from_acc(p[j] / sum);
    }
  }
}

// Up to 512 experts: the LANES lanes of a token hold ALL its logits in
// registers, C each (element u of lane g is expert LANES u + g), and every
// round takes the best logit still alive: a scan of the lane's C values, a
// shuffle reduction over the group, and the owner retires the winner in a bit
// mask.  No sorted lists to maintain.
template <typename T, int LANES, int C>
__global__ __launch_bounds__(kGateThreads) void topk_softmax_fwd_flat_kernel(
    const T* __restrict__ logits, int64_t n_tokens, int n_expert, int top_k,
    int64_t* __restrict__ idx, T* __restrict__ score) {
  using acc_t = typename Elem<T>::acc_t;
  constexpr int KMAX = FMOE_MAX_GATE_TOP_K;
  static_assert(C <= 32, "one bit per register in the alive mask");
  const int g = threadIdx.x % LANES;
  const int64_t t = (int64_t)blockIdx.x * (kGateThreads / LANES) + threadIdx.x / LANES;
  const bool live = t < n_tokens;
  acc_t v[C];
  uint32_t alive = 0;
#pragma unroll
  for (int u = 0; u < C; ++u) {
    const int e = u * LANES + g;
    v[u] = -INFINITY;
    if (live && e < n_expert) {
      v[u] = Elem<T>::to_acc(logits[t * n_expert + e]);
      alive |= 1u << u;
    }
  }
  acc_t sel[KMAX];
  int sel_id[KMAX];
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    sel[j] = -INFINITY;
    sel_id[j] = 0;
    if (j < top_k) {
      acc_t bv = -INFINITY;
      int be = 0x7fffffff;
#pragma unroll
      for (int u = 0; u < C; ++u) {
        const bool take = ((alive >> u) & 1u) && better(v[u], u * LANES + g, bv, be);
        bv = take ? v[u] : bv;
        be = take ? u * LANES + g : be;
      }
#pragma unroll
      for (int d = 1; d < LANES; d <<= 1) {
        const acc_t ov = __shfl_xor(bv, d, kWave);
        const int oe = __shfl_xor(be, d, kWave);
        const bool take = better(ov, oe, bv, be);
        bv = take ? ov : bv;
        be = take ? oe : be;
      }
      sel[j] = bv;
      sel_id[j] = be;
      if (be % LANES == g) alive &= ~(1u << ((be / LANES) & 31));  // no-op for "none left"
    }
  }
  if (!live || g != 0) return;
  acc_t p[KMAX];
  acc_t sum = 0;
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    p[j] = 0;
    if (j < top_k) {
      p[j] = exp(sel[j] - sel[0]);
      sum += p[j];
    }
  }
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    if (j < top_k) {
      idx[t * top_k + j] = sel_id[j];
      score[t * top_k + j] = Elem<T>::from_acc(p[j] / sum);
    }
  }
}

// dlogits[t][idx[t][j]] = score_j * (dscore_j - sum_i dscore_i * score_i), zero elsewhere.
template <typename T, int KMAX, int LANES>
__global__ __launch_bounds__(kGateThreads) void topk_softmax_bwd_kernel(
    const T* __restrict__ dscore, const T* __restrict__ score,
    const int64_t* __restrict__ idx, T* __restrict__ dlogits, int64_t n_tokens,
    int n_expert, int top_k) {
  using acc_t = typename Elem<T>::acc_t;
  const int g = threadIdx.x % LANES;
  const int64_t t = (int64_t)blockIdx.x * (kGateThreads / LANES) + threadIdx.x / LANES;
  if (t >= n_tokens) return;
  acc_t grad[KMAX];
  int id[KMAX];
  acc_t dot = 0;
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    grad[j] = 0;
    id[j] = -1;
    if (j < top_k) {
      const acc_t s = Elem<T>::to_acc(score[t * top_k + j]);
      const acc_t d = Elem<T>::to_acc(dscore[t * top_k + j]);
      dot += d * s;
      grad[j] = d;
      id[j] = (int)idx[t * top_k + j];
    }
  }
#pragma unroll
  for (int j = 0; j < KMAX; ++j)
    if (j < top_k) grad[j] = Elem<T>::to_acc(score[t * top_k + j]) * (grad[j] - dot);
  T* row = dlogits + t * n_expert;
  for (int e = g; e < n_expert; e += LANES) {
    acc_t v = 0;
#pragma unroll
    for (int j = 0; j < KMAX; ++j)
      if (id[j] == e) v = grad[j];
    row[e] = Elem<T>::from_acc(v);
  }
}

template <typename T, int KMAX>
static int launch_fwd(const void* logits, int64_t n_tokens, int n_expert, int top_k,
                      int64_t* idx, void* score, hipStream_t s) {
  const T* in = (const T*)logits;
  T* out = (T*)score;
#define FMOE_GATE_FLAT(LANES, C)                                                              \
  hipLaunchKernelGGL((topk_softmax_fwd_flat_kernel<T, LANES, C>),                             \
                     dim3(ceil_div(n_tokens, kGateThreads / LANES)), dim3(kGateThreads), 0, s, \
                     in, n_tokens, n_expert, top_k, idx, out)
  // measured at 128 experts, k = 8, 8192 tokens: 32 lanes x 4 registers 15 us,
  // 8 lanes x 16 registers 19 us (one wave per SIMD, nothing to overlap with),
  // the sorted lists 20 us
  if (n_expert <= 16) FMOE_GATE_FLAT(8, 2);
  else if (n_expert <= 32) FMOE_GATE_FLAT(8, 4);
  else if (n_expert <= 64) FMOE_GATE_FLAT(32, 2);
  else if (n_expert <= 128) FMOE_GATE_FLAT(32, 4);
  else if (n_expert <= 256) FMOE_GATE_FLAT(32, 8);
  else if (n_expert <= 512) FMOE_GATE_FLAT(32, 16);
  else
    hipLaunchKernelGGL((topk_softmax_fwd_kernel<T, KMAX, 32>),
                       dim3(ceil_div(n_tokens, kGateThreads / 32)), dim3(kGateThreads), 0, s, in,
                       n_tokens, n_expert, top_k, idx, out);
#undef FMOE_GATE_FLAT
  FMOE_LAUNCH_CHECK("topk_softmax_fwd");
  return FMOE_OK;
}

template <typename T, int KMAX>
static int launch_bwd(const void* dscore, const void* score, const int64_t* idx, void* dlogits,
                      int64_t n_tokens, int n_expert, int top_k, hipStream_t s) {
  if (n_expert >= kGateWideFrom)
    hipLaunchKernelGGL((topk_softmax_bwd_kernel<T, KMAX, 32>),
                       dim3(ceil_div(n_tokens, kGateThreads / 32)), dim3(kGateThreads), 0, s,
                       (const T*)dscore, (const T*)score, idx, (T*)dlogits, n_tokens, n_expert,
                       top_k);
  else
    hipLaunchKernelGGL((topk_softmax_bwd_kernel<T, KMAX, 8>),
                       dim3(ceil_div(n_tokens, kGateThreads / 8)), dim3(kGateThreads), 0, s,
                       (const T*)dscore, (const T*)score, idx, (T*)dlogits, n_tokens, n_expert,
                       top_k);
  FMOE_LAUNCH_CHECK("topk_softmax_bwd");
  return FMOE_OK;
}

static int check_gate(const char* who, int64_t n_tokens, int64_t n_expert, int64_t top_k,
                      int dtype) {
  FMOE_REQUIRE(dtype_size(dtype) != 0, FMOE_ERR_INVALID, "%s: unknown dtype %d", who, dtype);
  FMOE_REQUIRE(n_tokens >= 0 && n_expert >= 1 && top_k >= 1, FMOE_ERR_INVALID,
               "%s: bad sizes tokens=%lld experts=%lld top_k=%lld", who, (long long)n_tokens,
               (long long)n_expert, (long long)top_k);
  FMOE_REQUIRE(top_k <= n_expert, FMOE_ERR_INVALID, "%s: top_k %lld exceeds %lld experts", who,
               (long long)top_k, (long long)n_expert);
  FMOE_REQUIRE(top_k <= FMOE_MAX_GATE_TOP_K, FMOE_ERR_UNSUPPORTED,
               "%s: top_k %lld exceeds FMOE_MAX_GATE_TOP_K (%d)", who, (long long)top_k,
               FMOE_MAX_GATE_TOP_K);
  FMOE_REQUIRE(n_expert < ((int64_t)1 << 31) &&
                   n_tokens < ((int64_t)1 << 31) * (kGateThreads / 32),
               FMOE_ERR_UNSUPPORTED, "%s: size exceeds the index range", who);
  return FMOE_OK;
}

}  // namespace fmoe

using namespace fmoe;

#define FMOE_GATE_DISPATCH(FN, T, ...)                         \
  (top_k <= 2 ? FN<T, 2>(__VA_ARGS__)                          \
              : top_k <= 4 ? FN<T, 4>(__VA_ARGS__)             \
                           : top_k <= 8 ? FN<T, 8>(__VA_ARGS__) : FN<T, 16>(__VA_ARGS__))

extern "C" int fmoe_topk_softmax_fwd(const void* logits, int64_t n_tokens, int32_t n_expert,
                                     int32_t top_k, int64_t* idx, void* score, int dtype,
                                     void* stream) {
  int rc = check_gate("topk_softmax_fwd", n_tokens, n_expert, top_k, dtype);
  if (rc) return rc;
  if (n_tokens == 0) return FMOE_OK;
  FMOE_REQUIRE(logits && idx && score, FMOE_ERR_INVALID, "topk_softmax_fwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case FMOE_F32: return FMOE_GATE_DISPATCH(launch_fwd, float, logits, n_tokens, n_expert, top_k, idx, score, s);
    case FMOE_F64: return FMOE_GATE_DISPATCH(launch_fwd, double, logits, n_tokens, n_expert, top_k, idx, score, s);
    case FMOE_F16: return FMOE_GATE_DISPATCH(launch_fwd, __half, logits, n_tokens, n_expert, top_k, idx, score, s);
    default: return FMOE_GATE_DISPATCH(launch_fwd, __hip_bfloat16, logits, n_tokens, n_expert, top_k, idx, score, s);
  }
}

extern "C" int fmoe_topk_softmax_bwd(const void* dscore, const void* score, const int64_t* idx,
                                     void* dlogits, int64_t n_tokens, int32_t n_expert,
                                     int32_t top_k, int dtype, void* stream) {
  int rc = check_gate("topk_softmax_bwd", n_tokens, n_expert, top_k, dtype);
  if (rc) return rc;
  if (n_tokens == 0) return FMOE_OK;
  FMOE_REQUIRE(dscore && score && idx && dlogits, FMOE_ERR_INVALID,
               "topk_softmax_bwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case FMOE_F32: return FMOE_GATE_DISPATCH(launch_bwd, float, dscore, score, idx, dlogits, n_tokens, n_expert, top_k, s);
    case FMOE_F64: return FMOE_GATE_DISPATCH(launch_bwd, double, dscore, score, idx, dlogits, n_tokens, n_expert, top_k, s);
    case FMOE_F16: return FMOE_GATE_DISPATCH(launch_bwd, __half, dscore, score, idx, dlogits, n_tokens, n_expert, top_k, s);
    default: return FMOE_GATE_DISPATCH(launch_bwd, __hip_bfloat16, dscore, score, idx, dlogits, n_tokens, n_expert, top_k, s);
  }
}
