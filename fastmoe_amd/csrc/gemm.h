// Shared declarations of the grouped expert GEMMs (one launch for all experts).
#pragma once
#include "common.h"

namespace fmoe {

// The three products of an expert linear layer, all over the rows
// [seg_off[e], seg_off[e+1]) of expert e:
//   FWD    Y[seg]  = X[seg]  * W_e^T (+ b_e)   M = rows, N = out,  K = in
//   DGRAD  dX[seg] = dY[seg] * W_e             M = rows, N = in,   K = out
//   WGRAD  dW_e    = dY[seg]^T * X[seg]        M = out,  N = in,   K = rows
enum GemmMode { GEMM_FWD = 0, GEMM_DGRAD = 1, GEMM_WGRAD = 2,
                // FWD with GemmArgs::act_out: a kernel of its own inside the bf16
                // matrix-core family (callers pass GEMM_FWD and set act_out)
                GEMM_FWD_ACT = 3,
                // DGRAD with GemmArgs::act_pre, likewise (callers pass GEMM_DGRAD)
                GEMM_DGRAD_ACT = 4 };
constexpr bool is_fwd(int mode) { return mode == GEMM_FWD || mode == GEMM_FWD_ACT; }
constexpr bool is_dgrad(int mode) { return mode == GEMM_DGRAD || mode == GEMM_DGRAD_ACT; }

struct GemmArgs {
  const void* a;        // FWD: x      DGRAD: dy     WGRAD: dy
  const void* b;        // FWD: w      DGRAD: w      WGRAD: x
  void* c;              // FWD: y      DGRAD: dx     WGRAD: dw
  const void* bias;     // FWD: b [E, out] added to y, may be null.  WGRAD on the bf16/f16
                        // matrix-core kernels: if not null, the [E, out] bias gradient
                        // (column sums of dy per expert), WRITTEN by the launch
  const int32_t* seg_off;
  int64_t n_rows;       // rows allocated in the row-major activations
  int in_feat;
  int out_feat;
  int n_expert;
  int tile;             // 0 = choose the tile shape automatically, 1..4 = force one
  // DGRAD on the bf16 matrix-core kernel only: if not null, dx = (dy W) * gelu'(act_pre)
  // with act_pre [n_rows, in_feat] the pre-activations behind the layer's input,
  // and act_table the device table of gelu'(-|x|) (gelu_bwd_table()).
  const void* act_pre = nullptr;
  const float* act_table = nullptr;
  // FWD on the bf16 matrix-core kernel only: if not null, act_out [n_rows, out_feat]
  // receives gelu(y) next to y, through act_fwd_table, the device table of gelu(x)
  // by 16-bit pattern of x (gelu_fwd_table()).
  void* act_out = nullptr;
  const uint16_t* act_fwd_table = nullptr;
  // Experts whose parameters are separate allocations (the reference keeps one module
  // per expert, fmoe/transformer.py:51-55, and its GEMM loop takes per-expert pointers,
  // cuda/parallel_linear.cuh:69-87): DEVICE arrays of n_expert device pointers.  When
  // w_table is not null, expert e's weight in FWD and DGRAD is w_table[e]
  // ([out_feat, in_feat]) instead of b + e * out_feat * in_feat; when bias_table is
  // not null, its forward bias is bias_table[e] ([out_feat]) instead of bias + e * out_feat.
  const void* const* w_table = nullptr;
  const void* const* bias_table = nullptr;
};

// Expert e's part of a per-expert operand: from the pointer table when there is one,
// else `stride` elements per expert into the contiguous array (null if neither).
// `e` is uniform over the workgroup, so this is scalar work.
template <typename P>
__device__ __forceinline__ const P* expert_operand(const void* base, const void* const* table,
                                                   int e, int64_t stride) {
  if (table) return (const P*)table[e];
  return base ? (const P*)base + e * stride : nullptr;
}

// *p for a p that may come out of such a pointer table.  A pointer read from memory
// has no known address space, and a plain load through it would be a flat load (it
// waits on two counters and can reach LDS); this one says that p is global memory.
template <int kBytes> struct BitsOf;
template <> struct BitsOf<2> { typedef uint16_t type; };
template <> struct BitsOf<4> { typedef uint32_t type; };
template <> struct BitsOf<8> { typedef uint64_t type; };
template <typename V>
__device__ __forceinline__ V load_global(const void* p) {
  typedef typename BitsOf<sizeof(V)>::type bits_t;
  const bits_t b = *(__attribute__((address_space(1))) const bits_t*)p;
  return __builtin_bit_cast(V, b);
}

// The part of the gelu'(-|x|) table the fused DGRAD epilogue keeps in LDS: the
// bf16 patterns of 2^-28 <= |x| < 16, 4096 floats at a fixed place behind the
// largest staged output tile (256 rows of 256 + 8 elements).  Arguments outside
// (zeros, denormals, |x| >= 16, infinities, NaNs) are rare in pre-activations
// and take the full table in memory.
constexpr int kActTabFirst = 0x3180, kActTabCount = 0x1000;
constexpr int kActTabBytes = kActTabCount * 4;
constexpr int kActTabLdsOffset = 256 * (256 + 8) * 2;   // bytes from the start of LDS

// Device table of gelu'(-|x|) for a 16-bit dtype, built on first use (act.hip).
int gelu_bwd_table(int dtype, hipStream_t s, const float** table);
// Device table of gelu(x) by the 16-bit pattern of x (65536 results of the dtype).
int gelu_fwd_table(int dtype, hipStream_t s, const uint16_t** table);

// Virtual row-tile index space of the scalar kernel: expert e owns the tiles
// from seg_off[e] / BM + e on (the starts are strictly increasing, so tiles
// that belong to nobody simply exit); n_rows / BM + n_expert bounds their number.
inline int virtual_row_tiles(int64_t n_rows, int n_expert, int bm) {
  return (int)(n_rows / bm) + n_expert;
}

// Scalar (non-matrix-core) grouped GEMM for any dtype and any shape.
int launch_gemm_simt(int mode, const GemmArgs& g, int dtype, hipStream_t s);

// bf16 / f16 grouped GEMM on the matrix cores.  Returns FMOE_ERR_UNSUPPORTED
// without launching when the shape does not fit (callers then use the scalar
// kernel).
bool gemm_mfma_supported(int mode, const GemmArgs& g, int dtype);
int launch_gemm_mfma(int mode, const GemmArgs& g, int dtype, hipStream_t s);
// dX (gd: a = dY, b = W, c = dX) and dW (gw: a = dY, b = X, c = dW) of one
// grouped linear, in one launch where the tile shapes allow it.
int launch_gemm_mfma_bwd(const GemmArgs& gd, const GemmArgs& gw, int dtype, hipStream_t s);

// f32 / f64 grouped GEMM on the matrix cores, for 4-element-aligned shapes.
bool gemm_mfma_wide_supported(int mode, const GemmArgs& g, int dtype);
int launch_gemm_mfma_wide(int mode, const GemmArgs& g, int dtype, hipStream_t s);

}  // namespace fmoe
