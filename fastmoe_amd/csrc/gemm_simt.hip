// Scalar grouped GEMM: every dtype (f32, f64, f16, bf16) and every shape,
// including feature sizes that are not multiples of the matrix-core tiles.
// It is the path for feature sizes that are not multiples of 8 (f32/f64: 4)
// and for unaligned bases; everything else runs on the MFMA kernels.
//
// 64x64 output tile per 256-thread block, 16-deep K slices staged in LDS in
// the accumulation type, 4x4 register tile per thread.  Operand roles follow
// cuda/parallel_linear.cuh:69-87,124-147 of the reference.
#include "gemm.h"

namespace fmoe {

constexpr int SBM = 64, SBN = 64, SBK = 16, STHREADS = 256;

template <typename T, int MODE>
__global__ __launch_bounds__(STHREADS) void gemm_simt_kernel(GemmArgs g) {
  using acc_t = typename Elem<T>::acc_t;
  __shared__ acc_t As[SBK][SBM + 4];
  __shared__ acc_t Bs[SBK][SBN + 4];
  __shared__ int s_expert;

  const int tid = threadIdx.x;
  const int in_f = g.in_feat, out_f = g.out_feat;
  int e, m_tile;
  if (MODE == GEMM_WGRAD) {
    e = blockIdx.z;
    m_tile = blockIdx.y;
  } else {
    // find the expert that owns virtual row tile blockIdx.y
    const int v = blockIdx.y;
    if (tid == 0) {
      int lo = 0, hi = g.n_expert - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (g.seg_off[mid] / SBM + mid <= v) lo = mid; else hi = mid - 1;
      }
      s_expert = lo;
    }
    __syncthreads();
    e = s_expert;
    m_tile = v - (g.seg_off[e] / SBM + e);
  }
  const int64_t row0 = g.seg_off[e];
  const int cnt = g.seg_off[e + 1] - g.seg_off[e];

  // C[M,N] = A[M,K] * B[K,N] with element strides (sam, sak), (sbk, sbn)
  int M, N, K;
  int64_t sam, sak, sbk, sbn, ldc;
  const T *A, *B;
  T* C;
  if (MODE == GEMM_FWD) {
    M = cnt; N = out_f; K = in_f;
    A = (const T*)g.a + row0 * in_f;                 sam = in_f;  sak = 1;
    B = expert_operand<T>(g.b, g.w_table, e, (int64_t)out_f * in_f); sbk = 1;     sbn = in_f;
    C = (T*)g.c + row0 * out_f;                      ldc = out_f;
  } else if (MODE == GEMM_DGRAD) {
    M = cnt; N = in_f; K = out_f;
    A = (const T*)g.a + row0 * out_f;                sam = out_f; sak = 1;
    B = expert_operand<T>(g.b, g.w_table, e, (int64_t)out_f * in_f); sbk = in_f;  sbn = 1;
    C = (T*)g.c + row0 * in_f;                       ldc = in_f;
  } else {
    M = out_f; N = in_f; K = cnt;
    A = (const T*)g.a + row0 * out_f;                sam = 1;     sak = out_f;
    B = (const T*)g.b + row0 * in_f;                 sbk = in_f;  sbn = 1;
    C = (T*)g.c + (int64_t)e * out_f * in_f;         ldc = in_f;
  }
  const int m0 = m_tile * SBM, n0 = blockIdx.x * SBN;
  if (m0 >= M || n0 >= N) return;  // block-uniform

  const int tx = tid % 16, ty = tid / 16;
  acc_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0;

  for (int k0 = 0; k0 < K; k0 += SBK) {
#pragma unroll
    for (int i = 0; i < (SBM * SBK) / STHREADS; ++i) {
      const int q = tid + i * STHREADS;
      int m, k;
      if (sak == 1) { k = q % SBK; m = q / SBK; } else { m = q % SBM; k = q / SBM; }
      acc_t v = 0;
      if (m0 + m < M && k0 + k < K)
        v = Elem<T>::to_acc(A[(int64_t)(m0 + m) * sam + (int64_t)(k0 + k) * sak]);
      As[k][m] = v;
    }
#pragma unroll
    for (int i = 0; i < (SBN * SBK) / STHREADS; ++i) {
      const int q = tid + i * STHREADS;
      int n, k;
      if (sbk == 1) { k = q % SBK; n = q / SBK; } else { n = q % SBN; k = q / SBN; }
      acc_t v = 0;
      if (n0 + n < N && k0 + k < K)
        v = Elem<T>::to_acc(B[(int64_t)(k0 + k) * sbk + (int64_t)(n0 + n) * sbn]);
      Bs[k][n] = v;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < SBK; ++kk) {
      acc_t a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }

  const T* bias = MODE == GEMM_FWD ? expert_operand<T>(g.bias, g.bias_table, e, out_f) : nullptr;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      acc_t v = acc[i][j];
      if (bias) v += Elem<T>::to_acc(load_global<T>(bias + n));
      C[(int64_t)m * ldc + n] = Elem<T>::from_acc(v);
    }
  }
}

template <typename T>
static int launch_simt_t(int mode, const GemmArgs& g, hipStream_t s) {
  const int in_f = g.in_feat, out_f = g.out_feat;
  if (mode == GEMM_WGRAD) {
    dim3 grid(ceil_div(in_f, SBN), ceil_div(out_f, SBM), g.n_expert);
    FMOE_REQUIRE(grid.y <= 65535 && grid.z <= 65535, FMOE_ERR_UNSUPPORTED,
                 "grouped GEMM: grid too large");
    hipLaunchKernelGGL((gemm_simt_kernel<T, GEMM_WGRAD>), grid, dim3(STHREADS), 0,
                       s, g);
  } else {
    const int vt = virtual_row_tiles(g.n_rows, g.n_expert, SBM);
    const int N = mode == GEMM_FWD ? out_f : in_f;
    dim3 grid(ceil_div(N, SBN), vt, 1);
    FMOE_REQUIRE(grid.y <= 65535, FMOE_ERR_UNSUPPORTED,
                 "grouped GEMM: too many row tiles (%d)", vt);
    if (mode == GEMM_FWD)
      hipLaunchKernelGGL((gemm_simt_kernel<T, GEMM_FWD>), grid, dim3(STHREADS), 0,
                         s, g);
    else
      hipLaunchKernelGGL((gemm_simt_kernel<T, GEMM_DGRAD>), grid, dim3(STHREADS),
                         0, s, g);
  }
  FMOE_LAUNCH_CHECK("gemm_simt");
  return FMOE_OK;
}

int launch_gemm_simt(int mode, const GemmArgs& g, int dtype, hipStream_t s) {
  switch (dtype) {
    case FMOE_F32: return launch_simt_t<float>(mode, g, s);
    case FMOE_F64: return launch_simt_t<double>(mode, g, s);
    case FMOE_F16: return launch_simt_t<__half>(mode, g, s);
    case FMOE_BF16: return launch_simt_t<__hip_bfloat16>(mode, g, s);
    default: return set_error(FMOE_ERR_INVALID, "grouped GEMM: unknown dtype %d", dtype);
  }
}

}  // namespace fmoe
