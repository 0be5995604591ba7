// f32 / f64 grouped GEMM on the matrix cores (v_mfma_f32_32x32x2_f32,
// v_mfma_f64_16x16x4_f64): the full-precision half of the reference's dtype
// dispatch (cuda/parallel_linear.cu:33,76 -> cublasSgemm / cublasDgemm,
// cuda/utils/cublas_wrapper.h:51-90).
//
// These MFMAs run at 1/16 (f32) and 1/32 (f64) of the bf16 rate, so one K slice
// of a 128x128 tile keeps the matrix cores busy for microseconds and a plain
// design is enough: global -> registers -> LDS with two LDS stages of 16 values
// of K, one barrier per slice, and several blocks per CU (four for f32: their
// stages fill the 160 KB of LDS exactly; two for f64) so that one block's barrier and LDS writes hide behind the
// others' MFMAs.  Operand roles and the ragged rows are those of the
// bf16 kernel (gemm.h); the row tiles of an expert are found as in the scalar
// kernel (virtual_row_tiles).
//
// Both operand layouts are copied into LDS as they come, pack by pack: operands
// whose rows are contiguous in memory (W in DGRAD, both in WGRAD) as [k][row],
// K-contiguous ones (X and W in FWD, dY in DGRAD) as [row][k].  The MFMA takes
// one value of K per lane; the lanes pick their values so that a [row][k]
// operand is read as one 4-element pack per four MFMA rounds and a [k][row]
// operand as single values of the same K (see the K loop).
#include "gemm.h"

namespace fmoe {
namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef double f64x4_t __attribute__((ext_vector_type(4)));

constexpr int kWideTile = 128;     // output tile is kWideTile x kWideTile
constexpr int kWideThreads = 256;  // 2 x 2 waves of 64 x 64

template <typename F> struct WideMma;
template <> struct WideMma<float> {
  static constexpr int kBlk = 32;   // rows / columns of one MFMA block
  static constexpr int kAcc = 16;   // accumulators per lane and block
  static constexpr int kBK = 16;    // values of K per LDS slice
  static constexpr int kPad = 4;    // row padding of the LDS image, in elements
  static constexpr int kWaves = 4;      // waves per SIMD the registers are budgeted for
  static constexpr bool kSwap = true;   // feed (B, A): a lane then owns runs of 4 columns
  using acc_t = f32x16_t;
  typedef float vec_t __attribute__((ext_vector_type(4)));             // 16-byte pack
  static __device__ __forceinline__ acc_t run(float a, float b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
};
template <> struct WideMma<double> {
  static constexpr int kBlk = 16;
  static constexpr int kAcc = 4;
  static constexpr int kBK = 16;
  static constexpr int kPad = 2;
  static constexpr int kWaves = 2;
  static constexpr bool kSwap = false;  // a lane owns one column, 16 lanes a row segment
  using acc_t = f64x4_t;
  typedef double vec_t __attribute__((ext_vector_type(4), aligned(16)));  // two 16-byte packs
  static __device__ __forceinline__ acc_t run(double a, double b, acc_t c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
};

// Elements of one operand slice in LDS: [k][row] rows of kWideTile + kPad, or
// [row][k] rows of kBK values + 16 bytes (whichever is larger, so that either
// layout fits).
template <typename F>
constexpr int wide_operand_elems() {
  constexpr int by_k = WideMma<F>::kBK * (kWideTile + WideMma<F>::kPad);
  constexpr int by_row = kWideTile * (WideMma<F>::kBK + 16 / (int)sizeof(F));
  return by_k > by_row ? by_k : by_row;
}
template <typename F>
constexpr size_t wide_lds_bytes() {
  return (size_t)2 * 2 * wide_operand_elems<F>() * sizeof(F);
}

template <typename F, int MODE>
__global__ __launch_bounds__(kWideThreads, (WideMma<F>::kWaves)) void gemm_wide_kernel(GemmArgs g) {
  using Mma = WideMma<F>;
  constexpr int BK = Mma::kBK, BLK = Mma::kBlk, LD = kWideTile + Mma::kPad;
  constexpr int LDK = BK + 16 / (int)sizeof(F);   // row length of a [row][k] image
  constexpr int kOperand = wide_operand_elems<F>();
  // K values one MFMA round of 4 covers: a lane holds 4 consecutive ones
  constexpr int kGroup = 4 * (64 / BLK);
  static_assert(BK % kGroup == 0, "slices are whole groups of K");
  constexpr int kVecs = BK * kWideTile / 4 / kWideThreads;   // packs per thread and operand
  constexpr int TB = 64 / BLK;                // MFMA blocks per wave and direction
  constexpr bool A_KC = MODE != GEMM_WGRAD;   // operand is K-contiguous in memory
  constexpr bool B_KC = MODE == GEMM_FWD;
  using Vec4 = typename Mma::vec_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  F* smem = reinterpret_cast<F*>(smem_raw);   // [stage][A | B][k][row]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wave_m = wave >> 1, wave_n = wave & 1;
  const int in_f = g.in_feat, out_f = g.out_feat;
  int e, m_tile;
  if (MODE == GEMM_WGRAD) {
    e = blockIdx.z;
    m_tile = blockIdx.y;
  } else {
    // the expert that owns virtual row tile blockIdx.y (every thread searches:
    // the loads are uniform, and LDS is left to the operand stages)
    const int v = blockIdx.y;
    int lo = 0, hi = g.n_expert - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (g.seg_off[mid] / kWideTile + mid <= v) lo = mid; else hi = mid - 1;
    }
    e = lo;
    m_tile = v - (g.seg_off[e] / kWideTile + e);
  }
  const int64_t row0 = g.seg_off[e];
  const int cnt = g.seg_off[e + 1] - g.seg_off[e];

  int M, N, K, lda, ldb, ldc;
  const F *A, *B;
  F* C;
  if (MODE == GEMM_FWD) {
    M = cnt; N = out_f; K = in_f;
    A = (const F*)g.a + row0 * in_f;                 lda = in_f;
    B = expert_operand<F>(g.b, g.w_table, e, (int64_t)out_f * in_f); ldb = in_f;
    C = (F*)g.c + row0 * out_f;                      ldc = out_f;
  } else if (MODE == GEMM_DGRAD) {
    M = cnt; N = in_f; K = out_f;
    A = (const F*)g.a + row0 * out_f;                lda = out_f;
    B = expert_operand<F>(g.b, g.w_table, e, (int64_t)out_f * in_f); ldb = in_f;
    C = (F*)g.c + row0 * in_f;                       ldc = in_f;
  } else {
    M = out_f; N = in_f; K = cnt;
    A = (const F*)g.a + row0 * out_f;                lda = out_f;
    B = (const F*)g.b + row0 * in_f;                 ldb = in_f;
    C = (F*)g.c + (int64_t)e * out_f * in_f;         ldc = in_f;
  }
  const int m0 = m_tile * kWideTile, n0 = blockIdx.x * kWideTile;
  if (m0 >= M || n0 >= N) return;  // the same for the whole block
  const int m_valid = min(kWideTile, M - m0), n_valid = min(kWideTile, N - n0);
  const F* a_base = A_KC ? A + (int64_t)m0 * lda : A + m0;
  const F* b_base = B_KC ? B + (int64_t)n0 * ldb : B + n0;

  // Slice [k0, k0 + BK) of one operand into registers; rows past `valid` and
  // values of K past the end arrive as zeros.  K-contiguous operands need K to
  // be a multiple of 4, the others `valid` (a feature size) to be one.
  auto fetch = [&](Vec4* r, const F* base, int ld, auto kc_tag, int valid, int k0) {
    constexpr bool kc = decltype(kc_tag)::value;
#pragma unroll
    for (int u = 0; u < kVecs; ++u) {
      const int idx = tid + u * kWideThreads;
      bool ok;
      const F* p;
      if (kc) {
        const int row = idx / (BK / 4), kq = idx % (BK / 4);
        ok = row < valid && k0 + 4 * kq < K;
        p = base + (int64_t)row * ld + k0 + 4 * kq;
      } else {
        const int k = idx / (kWideTile / 4), q = idx % (kWideTile / 4);
        ok = k0 + k < K && 4 * q < valid;
        p = base + (int64_t)(k0 + k) * ld + 4 * q;
      }
      r[u] = 0;
      if (ok) r[u] = *reinterpret_cast<const Vec4*>(p);
    }
  };
  auto stash = [&](const Vec4* r, F* dst, auto kc_tag) {
    constexpr bool kc = decltype(kc_tag)::value;
#pragma unroll
    for (int u = 0; u < kVecs; ++u) {
      const int idx = tid + u * kWideThreads;
      if (kc) {
        const int row = idx / (BK / 4), kq = idx % (BK / 4);
        *reinterpret_cast<Vec4*>(dst + row * LDK + 4 * kq) = r[u];
      } else {
        const int k = idx / (kWideTile / 4), q = idx % (kWideTile / 4);
        *reinterpret_cast<Vec4*>(dst + k * LD + 4 * q) = r[u];
      }
    }
  };
  using a_kc = std::integral_constant<bool, A_KC>;
  using b_kc = std::integral_constant<bool, B_KC>;

  // f32: acc[i][j] holds the TRANSPOSE of block (i, j) of C (the MFMA is fed
  // (B value, A value)): a lane owns row lane % 32 and runs of 4 consecutive
  // columns, which leave as one 16-byte store each.  f64: block (i, j) itself.
  typename Mma::acc_t acc[TB][TB];
#pragma unroll
  for (int i = 0; i < TB; ++i)
#pragma unroll
    for (int j = 0; j < TB; ++j)
#pragma unroll
      for (int r = 0; r < Mma::kAcc; ++r) acc[i][j][r] = 0;

  Vec4 ra[kVecs], rb[kVecs];
  const int k_tiles = (K + BK - 1) / BK;
  if (k_tiles > 0) {
    fetch(ra, a_base, lda, a_kc{}, m_valid, 0);
    fetch(rb, b_base, ldb, b_kc{}, n_valid, 0);
    stash(ra, smem, a_kc{});
    stash(rb, smem + kOperand, b_kc{});
  }
  __syncthreads();
  const int lr = lane % BLK, lk = lane / BLK;
  for (int kt = 0; kt < k_tiles; ++kt) {
    const F* as = smem + (kt & 1) * 2 * kOperand;
    const F* bs = as + kOperand;
    const bool more = kt + 1 < k_tiles;
    if (more) {  // in flight while this slice is multiplied
      fetch(ra, a_base, lda, a_kc{}, m_valid, (kt + 1) * BK);
      fetch(rb, b_base, ldb, b_kc{}, n_valid, (kt + 1) * BK);
    }
    // The MFMA wants, per lane, one value of K out of 64 / BLK; WHICH value of the
    // slice that is only has to agree between the two operands.  Lane group lk
    // takes k = 4 lk + c in round c of a group of kGroup values, so that a
    // [row][k] operand is read as one 4-element pack per 4 rounds.
#pragma unroll
    for (int s = 0; s < BK / kGroup; ++s) {
      Vec4 a[TB], b[TB];
      const int k4 = s * kGroup + 4 * lk;
#pragma unroll
      for (int i = 0; i < TB; ++i) {
        const int row = wave_m * 64 + i * BLK + lr;
        if (A_KC) a[i] = *reinterpret_cast<const Vec4*>(as + row * LDK + k4);
        else
#pragma unroll
          for (int c = 0; c < 4; ++c) a[i][c] = as[(k4 + c) * LD + row];
      }
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        const int row = wave_n * 64 + j * BLK + lr;
        if (B_KC) b[j] = *reinterpret_cast<const Vec4*>(bs + row * LDK + k4);
        else
#pragma unroll
          for (int c = 0; c < 4; ++c) b[j][c] = bs[(k4 + c) * LD + row];
      }
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int i = 0; i < TB; ++i)
#pragma unroll
          for (int j = 0; j < TB; ++j)
            acc[i][j] = Mma::kSwap ? Mma::run(b[j][c], a[i][c], acc[i][j])
                                   : Mma::run(a[i][c], b[j][c], acc[i][j]);
    }
    if (more) {
      // the other stage was last read in iteration kt - 1, which every wave
      // left through the barrier below
      F* next = smem + ((kt + 1) & 1) * 2 * kOperand;
      stash(ra, next, a_kc{});
      stash(rb, next + kOperand, b_kc{});
    }
    __syncthreads();
  }

  const F* bias = MODE == GEMM_FWD ? expert_operand<F>(g.bias, g.bias_table, e, out_f) : nullptr;
  if constexpr (Mma::kSwap) {
    // 32x32 block, operands swapped: accumulator r of a lane is row lane % 32,
    // column 8 * (r / 4) + 4 * (lane / 32) + r % 4
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      const int m = m0 + wave_m * 64 + i * BLK + lr;
#pragma unroll
      for (int j = 0; j < TB; ++j) {
#pragma unroll
        for (int q = 0; q < Mma::kAcc / 4; ++q) {
          const int n = n0 + wave_n * 64 + j * BLK + 8 * q + 4 * lk;
          if (m < M && n < N) {  // N is a multiple of 4
            Vec4 o;
#pragma unroll
            for (int c = 0; c < 4; ++c) o[c] = acc[i][j][4 * q + c] + (bias ? load_global<F>(bias + n + c) : (F)0);
            *reinterpret_cast<Vec4*>(C + (int64_t)m * ldc + n) = o;
          }
        }
      }
    }
  } else {
    // 16x16 block: accumulator r of a lane is row 4 * r + lane / 16, column
    // lane % 16; 16 lanes store 128 contiguous bytes of a row
#pragma unroll
    for (int j = 0; j < TB; ++j) {
      const int n = n0 + wave_n * 64 + j * BLK + lr;
      const F bv = bias && n < N ? load_global<F>(bias + n) : (F)0;
#pragma unroll
      for (int i = 0; i < TB; ++i) {
#pragma unroll
        for (int r = 0; r < Mma::kAcc; ++r) {
          const int m = m0 + wave_m * 64 + i * BLK + 4 * r + lk;
          if (m < M && n < N) C[(int64_t)m * ldc + n] = acc[i][j][r] + bv;
        }
      }
    }
  }
}

template <typename F, int MODE>
int launch_wide_mode(const GemmArgs& g, hipStream_t s) {
  constexpr size_t lds = wide_lds_bytes<F>();
  static_assert(2 * lds <= 160 * 1024, "at least two blocks per gfx950 CU");
  auto kern = gemm_wide_kernel<F, MODE>;
  FMOE_SET_DYNAMIC_LDS_ONCE(kern, lds);
  dim3 grid;
  if (MODE == GEMM_WGRAD) {
    grid = dim3(ceil_div(g.in_feat, kWideTile), ceil_div(g.out_feat, kWideTile), g.n_expert);
    FMOE_REQUIRE(grid.y <= 65535 && grid.z <= 65535, FMOE_ERR_UNSUPPORTED,
                 "grouped GEMM: grid too large");
  } else {
    const int vt = virtual_row_tiles(g.n_rows, g.n_expert, kWideTile);
    grid = dim3(ceil_div(MODE == GEMM_FWD ? g.out_feat : g.in_feat, kWideTile), vt, 1);
    FMOE_REQUIRE(grid.y <= 65535, FMOE_ERR_UNSUPPORTED,
                 "grouped GEMM: too many row tiles (%d)", vt);
  }
  hipLaunchKernelGGL(kern, grid, dim3(kWideThreads), lds, s, g);
  FMOE_LAUNCH_CHECK("gemm_wide");
  return FMOE_OK;
}

template <typename F>
int launch_wide_t(int mode, const GemmArgs& g, hipStream_t s) {
  switch (mode) {
    case GEMM_FWD: return launch_wide_mode<F, GEMM_FWD>(g, s);
    case GEMM_DGRAD: return launch_wide_mode<F, GEMM_DGRAD>(g, s);
    default: return launch_wide_mode<F, GEMM_WGRAD>(g, s);
  }
}

}  // namespace

// Measured against the scalar kernel's 64x64 tiles, the matrix cores win or tie
// from 16 tiles up, so size does not enter the choice.
bool gemm_mfma_wide_supported(int mode, const GemmArgs& g, int dtype) {
  (void)mode;
  if (dtype != FMOE_F32 && dtype != FMOE_F64) return false;
  if (g.in_feat % 4 != 0 || g.out_feat % 4 != 0) return false;
  if (((uintptr_t)g.a | (uintptr_t)g.b | (uintptr_t)g.c) % 16 != 0) return false;
  return true;
}

int launch_gemm_mfma_wide(int mode, const GemmArgs& g, int dtype, hipStream_t s) {
  if (!gemm_mfma_wide_supported(mode, g, dtype))
    return set_error(FMOE_ERR_UNSUPPORTED, "grouped GEMM: shape not MFMA-aligned");
  if (dtype == FMOE_F32) return launch_wide_t<float>(mode, g, s);
  return launch_wide_t<double>(mode, g, s);
}

}  // namespace fmoe
