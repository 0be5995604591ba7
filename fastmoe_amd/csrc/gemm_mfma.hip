// Grouped expert GEMM on the gfx950 matrix cores (bf16 / f16 in, fp32
// accumulate): one launch covers every expert, with ragged row counts taken
// from a device-side seg_off table, so empty experts cost nothing and no host
// synchronisation is needed.
//
// Block tile BM x BN x BK with WM x WN wave64s; every wave owns a
// (BM/WM) x (BN/WN) patch as a grid of 32x32 accumulators fed by
// v_mfma_f32_32x32x16_{bf16,f16}.  Operand tiles go global -> registers -> LDS
// (double buffered) as 16-byte packs:
//   * an operand whose K index is contiguous in memory is stored [row][BK]
//     with the 16-byte pack index XOR-swizzled by the row, and a lane reads
//     its 8 consecutive K values with one ds_read_b128;
//   * an operand whose K index is the strided one (W in DGRAD, both operands
//     in WGRAD) is stored as it arrives, [k][row], and read back transposed.
// Loads are predicated per 16-byte pack and zero-filled, so partial tiles in
// M, N and K need no separate kernel.
//
// Operand roles follow cuda/parallel_linear.cuh:69-87,124-147 of the
// reference; the per-expert cuBLAS loop there becomes a tile index space.
#include "gemm.h"

namespace fmoe {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

template <typename T> struct Mma;
template <> struct Mma<__hip_bfloat16> {
  __device__ static __forceinline__ f32x16_t run(uint4 a, uint4 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
        __builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
};
template <> struct Mma<__half> {
  __device__ static __forceinline__ f32x16_t run(uint4 a, uint4 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
};

constexpr int kTrPad = 8;  // elements of padding per [k] row of a transposed tile

// One operand tile of R rows (the M or N index) by BK: how it is fetched,
// where it lands in LDS and how a wave reads its MFMA fragment back.
// KC == true : memory is [row][k] (k contiguous), LDS is [row][BK] swizzled.
// KC == false: memory is [k][row] (row contiguous), LDS is [k][R + kTrPad].
template <int R, int BK, int NT, bool KC>
struct OperandTile {
  static constexpr int kChunks = R * BK / 8;
  static constexpr int kPerThread = kChunks / NT;
  static_assert(kChunks % NT == 0, "tile must split evenly over the threads");
  static constexpr int kCpr = KC ? BK / 8 : R / 8;  // 16-byte packs per LDS row
  static constexpr int kLdsElems = KC ? R * BK : BK * (R + kTrPad);

  __device__ static __forceinline__ int swz(int row) {
    return (row ^ (row >> 3)) & (BK / 8 - 1);
  }

  uint4 regs[kPerThread];

  // base points at element (row 0, k 0) of the operand for this problem;
  // ld is the stride of the non-contiguous index; limits are exclusive.
  __device__ __forceinline__ void fetch(const uint16_t* base, int64_t ld, int r0,
                                        int k0, int r_limit, int k_limit, int tid) {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int q = tid + i * NT;
      const int major = q / kCpr, minor = (q % kCpr) * 8;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (KC) {
        const int r = r0 + major, k = k0 + minor;
        if (r < r_limit && k < k_limit)
          v = *reinterpret_cast<const uint4*>(base + (int64_t)r * ld + k);
      } else {
        const int k = k0 + major, r = r0 + minor;
        if (k < k_limit && r < r_limit)
          v = *reinterpret_cast<const uint4*>(base + (int64_t)k * ld + r);
      }
      regs[i] = v;
    }
  }

  __device__ __forceinline__ void stash(uint16_t* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < kPerThread; ++i) {
      const int q = tid + i * NT;
      const int major = q / kCpr, minor = q % kCpr;
      int off;
      if (KC) off = major * BK + ((minor ^ swz(major)) * 8);
      else off = major * (R + kTrPad) + minor * 8;
      *reinterpret_cast<uint4*>(lds + off) = regs[i];
    }
  }

  // fragment of the 32-row sub-tile starting at `row32` for K step `kk`
  // (16 values of K): lane l gets row row32 + l%32, K values 8*(l/32) .. +7.
  __device__ static __forceinline__ uint4 frag(const uint16_t* lds, int row32,
                                               int kk, int lane) {
    const int r = row32 + (lane & 31);
    const int half = lane >> 5;
    if (KC) {
      const int chunk = kk * 2 + half;
      return *reinterpret_cast<const uint4*>(lds + r * BK + ((chunk ^ swz(r)) * 8));
    } else {
      const uint16_t* p = lds + (kk * 16 + half * 8) * (R + kTrPad) + r;
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = p[(2 * j) * (R + kTrPad)];
        const uint32_t hi = p[(2 * j + 1) * (R + kTrPad)];
        w[j] = lo | (hi << 16);
      }
      return make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
};

template <typename T, int BM, int BN, int BK, int WM, int WN, int MODE>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mfma_kernel(GemmArgs g,
                                                                int tiles_n,
                                                                int tiles_m) {
  constexpr int NT = WM * WN * 64;
  constexpr bool A_KC = MODE != GEMM_WGRAD;
  constexpr bool B_KC = MODE == GEMM_FWD;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BK % 16 == 0, "tile shape");
  using ATile = OperandTile<BM, BK, NT, A_KC>;
  using BTile = OperandTile<BN, BK, NT, B_KC>;

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  // [A buffer 0][A buffer 1][B buffer 0][B buffer 1]
  uint16_t* const lds_a = smem;
  uint16_t* const lds_b = smem + 2 * ATile::kLdsElems;
  __shared__ int s_expert;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / WN, wave_n = wave % WN;
  const int in_f = g.in_feat, out_f = g.out_feat;

  // ---- which tile is this block?
  const int pid = blockIdx.x;
  const int n_tile = pid % tiles_n;
  int e, m_tile;
  if (MODE == GEMM_WGRAD) {
    m_tile = (pid / tiles_n) % tiles_m;
    e = pid / (tiles_n * tiles_m);
  } else {
    const int v = pid / tiles_n;  // virtual row tile
    if (tid == 0) s_expert = -1;
    __syncthreads();
    for (int x = tid; x < g.n_expert; x += NT) {
      const int so = g.seg_off[x];
      const int c = g.seg_off[x + 1] - so;
      const int vs = so / BM + x;
      if (v >= vs && v < vs + (c + BM - 1) / BM) s_expert = x;
    }
    __syncthreads();
    e = s_expert;
    if (e < 0) return;  // nobody owns this virtual tile
    m_tile = v - (g.seg_off[e] / BM + e);
  }
  e = __builtin_amdgcn_readfirstlane(e);
  m_tile = __builtin_amdgcn_readfirstlane(m_tile);
  const int row0 = g.seg_off[e];
  const int cnt = g.seg_off[e + 1] - row0;

  int M, N, K;
  int64_t lda, ldb, ldc;
  const uint16_t *A, *B;
  T* C;
  if (MODE == GEMM_FWD) {
    M = cnt; N = out_f; K = in_f;
    A = (const uint16_t*)g.a + (int64_t)row0 * in_f;        lda = in_f;
    B = (const uint16_t*)g.b + (int64_t)e * out_f * in_f;   ldb = in_f;
    C = (T*)g.c + (int64_t)row0 * out_f;                    ldc = out_f;
  } else if (MODE == GEMM_DGRAD) {
    M = cnt; N = in_f; K = out_f;
    A = (const uint16_t*)g.a + (int64_t)row0 * out_f;       lda = out_f;
    B = (const uint16_t*)g.b + (int64_t)e * out_f * in_f;   ldb = in_f;
    C = (T*)g.c + (int64_t)row0 * in_f;                     ldc = in_f;
  } else {
    M = out_f; N = in_f; K = cnt;
    A = (const uint16_t*)g.a + (int64_t)row0 * out_f;       lda = out_f;
    B = (const uint16_t*)g.b + (int64_t)row0 * in_f;        ldb = in_f;
    C = (T*)g.c + (int64_t)e * out_f * in_f;                ldc = in_f;
  }
  const int m0 = m_tile * BM, n0 = n_tile * BN;
  if (m0 >= M || n0 >= N) return;

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  ATile ta;
  BTile tb;
  const int k_tiles = (K + BK - 1) / BK;
  if (k_tiles > 0) {
    ta.fetch(A, lda, m0, 0, M, K, tid);
    tb.fetch(B, ldb, n0, 0, N, K, tid);
    ta.stash(lds_a, tid);
    tb.stash(lds_b, tid);
  }
  __syncthreads();

  for (int kt = 0; kt < k_tiles; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < k_tiles;
    if (more) {
      ta.fetch(A, lda, m0, (kt + 1) * BK, M, K, tid);
      tb.fetch(B, ldb, n0, (kt + 1) * BK, N, K, tid);
    }
    const uint16_t* la = lds_a + cur * ATile::kLdsElems;
    const uint16_t* lb = lds_b + cur * BTile::kLdsElems;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      uint4 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        fa[i] = ATile::frag(la, wave_m * (BM / WM) + i * 32, kk, lane);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        fb[j] = BTile::frag(lb, wave_n * (BN / WN) + j * 32, kk, lane);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = Mma<T>::run(fa[i], fb[j], acc[i][j]);
    }
    if (more) {
      ta.stash(lds_a + (cur ^ 1) * ATile::kLdsElems, tid);
      tb.stash(lds_b + (cur ^ 1) * BTile::kLdsElems, tid);
    }
    __syncthreads();
  }

  // ---- epilogue: accumulator r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32]
  const T* bias = (MODE == GEMM_FWD && g.bias)
                      ? (const T*)g.bias + (int64_t)e * out_f : nullptr;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + wave_n * (BN / WN) + j * 32 + (lane & 31);
    if (n >= N) continue;
    const float bv = bias ? Elem<T>::to_acc(bias[n]) : 0.f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int mb = m0 + wave_m * (BM / WM) + i * 32 + 4 * (lane >> 5);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = mb + 8 * (r / 4) + (r % 4);
        if (m < M) C[(int64_t)m * ldc + n] = Elem<T>::from_acc(acc[i][j][r] + bv);
      }
    }
  }
}

// ------------------------------------------------------------------ host side
template <typename T, int BM, int BN, int BK, int WM, int WN, int MODE>
static int launch_cfg(const GemmArgs& g, hipStream_t s) {
  constexpr int NT = WM * WN * 64;
  using ATile = OperandTile<BM, BK, NT, MODE != GEMM_WGRAD>;
  using BTile = OperandTile<BN, BK, NT, MODE == GEMM_FWD>;
  constexpr size_t lds_bytes = 2 * (ATile::kLdsElems + BTile::kLdsElems) * sizeof(uint16_t);
  auto kern = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, MODE>;
  static bool configured = false;  // attribute is per function, set once
  if (!configured) {
    FMOE_HIP_CHECK(hipFuncSetAttribute((const void*)kern,
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes));
    configured = true;
  }
  int tiles_n, tiles_m;
  int64_t blocks;
  if (MODE == GEMM_WGRAD) {
    tiles_n = ceil_div(g.in_feat, BN);
    tiles_m = ceil_div(g.out_feat, BM);
    blocks = (int64_t)tiles_n * tiles_m * g.n_expert;
  } else {
    tiles_n = ceil_div(MODE == GEMM_FWD ? g.out_feat : g.in_feat, BN);
    tiles_m = virtual_row_tiles(g.n_rows, g.n_expert, BM);
    blocks = (int64_t)tiles_n * tiles_m;
  }
  FMOE_REQUIRE(blocks < ((int64_t)1 << 31), FMOE_ERR_UNSUPPORTED,
               "grouped GEMM: too many tiles");
  if (blocks == 0) return FMOE_OK;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(NT), lds_bytes, s, g,
                     tiles_n, tiles_m);
  FMOE_LAUNCH_CHECK("gemm_mfma");
  return FMOE_OK;
}

template <typename T, int MODE>
static int launch_mode(const GemmArgs& g, hipStream_t s) {
  // large tiles when the average expert fills them, small ones otherwise
  bool large;
  if (MODE == GEMM_WGRAD) large = g.in_feat >= 1024 && g.out_feat >= 1024;
  else large = g.n_rows / g.n_expert >= 768;
  if (large) return launch_cfg<T, 256, 256, 64, 2, 2, MODE>(g, s);
  return launch_cfg<T, 128, 128, 64, 2, 2, MODE>(g, s);
}

template <typename T>
static int launch_t(int mode, const GemmArgs& g, hipStream_t s) {
  switch (mode) {
    case GEMM_FWD: return launch_mode<T, GEMM_FWD>(g, s);
    case GEMM_DGRAD: return launch_mode<T, GEMM_DGRAD>(g, s);
    default: return launch_mode<T, GEMM_WGRAD>(g, s);
  }
}

bool gemm_mfma_supported(int mode, const GemmArgs& g, int dtype) {
  (void)mode;
  if (dtype != FMOE_BF16 && dtype != FMOE_F16) return false;
  if (g.in_feat % 8 != 0 || g.out_feat % 8 != 0) return false;
  if (((uintptr_t)g.a | (uintptr_t)g.b | (uintptr_t)g.c) % 16 != 0) return false;
  return true;
}

int launch_gemm_mfma(int mode, const GemmArgs& g, int dtype, hipStream_t s) {
  if (!gemm_mfma_supported(mode, g, dtype))
    return set_error(FMOE_ERR_UNSUPPORTED, "grouped GEMM: shape not MFMA-aligned");
  if (dtype == FMOE_BF16) return launch_t<__hip_bfloat16>(mode, g, s);
  return launch_t<__half>(mode, g, s);
}

}  // namespace fmoe
