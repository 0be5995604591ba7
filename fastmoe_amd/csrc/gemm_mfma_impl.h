// Grouped expert GEMM on the gfx950 matrix cores (bf16 / f16 in, fp32
// accumulate): one launch covers every expert, with ragged row counts taken
// from a device-side seg_off table, so empty experts cost nothing and no host
// synchronisation is needed.
//
// Block tile BM x BN x BK with WM x WN wave64s; every wave owns a
// (BM/WM) x (BN/WN) patch as a grid of 16x16 accumulators fed by
// v_mfma_f32_16x16x32_{bf16,f16}: on random data the chip is power-limited, and
// this shape sustains about 16% more FLOP/s than 32x32x16 at the same power
// (2.07 vs 1.78 PFLOP/s for a loop of MFMAs alone).
//
// Operand tiles go from HBM/L2 straight into LDS with buffer_load_dwordx4 ...
// lds (no staging registers): one wave instruction fills 1 KiB of LDS, lane l
// writing bytes [16 l, 16 l + 16).  Which 16-byte pack of the tile a lane
// fetches is chosen so that the pack lands where the bank-conflict-free read
// pattern expects it:
//   * K contiguous in memory (X, dY as the A operand, W in FWD): LDS is
//     [row][BK]; pack index XOR ((row ^ row/8) & 7); a lane reads its 8
//     consecutive K values with one ds_read_b128.
//   * K strided in memory (W in DGRAD, both operands in WGRAD): LDS is
//     [k][rows] as it arrives; 32-byte segment index XOR 2 (k & 3); fragments
//     come back through ds_read_b64_tr_b16, which transposes 16-bit elements
//     across groups of 16 lanes.
// Out-of-range packs (ragged M, N or K edges) are pointed beyond the buffer
// descriptor's num_records and arrive as zeros, so there are no edge kernels
// and no branches in the load path.
//
// Two pipelines: four LDS stages of 32 values of K (two K-slices in flight while
// one feeds the MFMAs, one barrier per slice), or two stages of 64 values with
// the barrier in front of the last K step (whole 128-byte lines for
// K-contiguous operands).
//
// The rows of an expert are cut into BM-row tiles plus, for a remainder of at
// most BM / 2 rows, one 64- or 128-row tile that costs a fraction of a BM tile,
// so a few rows past a multiple of BM do not cost a whole tile; a last column
// tile (or last row tile of dW) that is at most half full runs as a half-size
// tile.  Tiles are dealt to the workgroups in an XCD-aware patch order.
//
// Operand roles follow cuda/parallel_linear.cuh:69-87,124-147 of the
// reference; the per-expert cuBLAS loop there becomes a tile index space.
#pragma once
#include <type_traits>
#include <algorithm>
#include <utility>

#include "dma_desc.h"
#include "gemm.h"

namespace fmoe {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N - 1>{}): a loop
// whose counter is a compile-time constant inside the body.
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

typedef __attribute__((ext_vector_type(16))) float f32x16_t;
// 32x32x16: for the products whose operands need the transposing LDS read (two
// instructions per fragment); there the 16-cycle MFMAs leave too few issue
// slots between them, and the 32-cycle shape is the faster one.
template <typename T> struct Mma32;
template <> struct Mma32<__hip_bfloat16> {
  __device__ static __forceinline__ f32x16_t run(uint4 a, uint4 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
        __builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
};
template <> struct Mma32<__half> {
  __device__ static __forceinline__ f32x16_t run(uint4 a, uint4 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
};

// s + the two 16-bit values packed in `pair`, in fp32 (v_dot2 against (1, 1)).
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
template <typename T> struct ColSum;
template <> struct ColSum<__hip_bfloat16> {
  __device__ static __forceinline__ float add(uint32_t pair, float s) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pair),
                                           __builtin_bit_cast(bf16x2_t, 0x3f803f80u), s, false);
  }
};
template <> struct ColSum<__half> {
  __device__ static __forceinline__ float add(uint32_t pair, float s) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, pair),
                                  __builtin_bit_cast(f16x2_t, 0x3c003c00u), s, false);
  }
};

// dy * gelu'(x) for the two 16-bit values packed in h (dy) and p (x), rounded to
// the storage type: what the separate activation kernel computes from its table
// of gelu'(-|x|) (positive x: 1 - the entry).
template <typename T> struct PackPair;
template <> struct PackPair<__hip_bfloat16> {
  __device__ static __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
  __device__ static __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
  __device__ static __forceinline__ uint32_t pack(float a, float b) {
    return (uint32_t)__bfloat16_as_ushort(__float2bfloat16(a)) |
           ((uint32_t)__bfloat16_as_ushort(__float2bfloat16(b)) << 16);
  }
};
// f16 has 10 mantissa bits (eight times the table entries in the same range): not
// fused, the entry point runs the separate kernel for it
template <> struct PackPair<__half> {
  __device__ static __forceinline__ float lo(uint32_t) { return 0.f; }
  __device__ static __forceinline__ float hi(uint32_t) { return 0.f; }
  __device__ static __forceinline__ uint32_t pack(float, float) { return 0u; }
};
// Fast form: `tab` is the slice of the table in LDS, valid for patterns whose
// index (pattern without sign - kActTabFirst) is below kActTabCount.  The OR of
// all indices goes into `seen`: a bit at or above kActTabCount's says that some
// argument was outside and the result must be recomputed by the slow form.  `tab`
// is typed as an LDS pointer, so the read with such an index is an LDS instruction
// whatever the compiler makes of the code around it: outside the slice it returns
// whatever is there, or zero, and never faults (a flat load could).
typedef __attribute__((address_space(3))) const float* lds_float_ptr_t;
typedef __attribute__((address_space(3))) const uint16_t* lds_u16_ptr_t;
template <typename T>
__device__ __forceinline__ uint32_t gelu_bwd_pair_fast(uint32_t h, uint32_t p, lds_float_ptr_t tab,
                                                       uint32_t& seen) {
  const uint32_t i0 = (p & 0x7fffu) - kActTabFirst, i1 = ((p >> 16) & 0x7fffu) - kActTabFirst;
  seen |= i0 | i1;
  const float n0 = tab[i0], n1 = tab[i1];
  const float d0 = (p & 0x8000u) ? n0 : 1.f - n0;
  const float d1 = ((int32_t)p < 0) ? n1 : 1.f - n1;
  return PackPair<T>::pack(PackPair<T>::lo(h) * d0, PackPair<T>::hi(h) * d1);
}
// Slow form: any argument, from the full table in memory.
template <typename T>
__device__ __forceinline__ uint32_t gelu_bwd_pair_any(uint32_t h, uint32_t p,
                                                      const float* full_tab) {
  const float n0 = full_tab[p & 0x7fffu], n1 = full_tab[(p >> 16) & 0x7fffu];
  const float d0 = (p & 0x8000u) ? n0 : 1.f - n0;
  const float d1 = ((int32_t)p < 0) ? n1 : 1.f - n1;
  return PackPair<T>::pack(PackPair<T>::lo(h) * d0, PackPair<T>::hi(h) * d1);
}

template <typename T> struct Mma;
template <> struct Mma<__hip_bfloat16> {
  __device__ static __forceinline__ f32x4_t run(uint4 a, uint4 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(
        __builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
};
template <> struct Mma<__half> {
  __device__ static __forceinline__ f32x4_t run(uint4 a, uint4 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
};

constexpr uint32_t kOutOfRange = kDmaOutOfRange;  // beyond any num_records used here
constexpr int kRsrcFlags = 0x00020000;         // raw buffer, 32-bit data format

// One operand tile of R rows (the M or N index) by BK values of K.
// KC == true : memory is [row][k] (k contiguous), LDS is [row][BK].
// KC == false: memory is [k][row] (row contiguous), LDS is [k][R].
//
// A wave copies kPerWave consecutive 1 KiB blocks of the tile per K-slice, one
// buffer_load_dwordx4 ... lds each.
template <int R, int BK, int NW, bool KC>
struct DmaTile {
  static constexpr int kBytes = R * BK * 2;
  static constexpr int kBlocks = kBytes / 1024;     // one wave instruction each
  static constexpr int kPerWave = kBlocks / NW;
  static_assert(kBlocks % NW == 0 && kPerWave >= 1, "tile must split evenly");
  static_assert(KC || R >= 128, "the [k][rows] swizzle permutes 8 segments of 16 rows");
  static_assert(BK == 64 || BK == 32, "swizzles below assume 128- or 64-byte [row][BK] rows");
  static constexpr int kRowPacks = R / 8;           // packs per [k] row (KC == false)
  static constexpr int kKPacks = BK / 8;            // packs per [row] row (KC == true)

  // XOR applied to the pack index of a [row][BK] row.  Chosen by timing
  // ds_read_b128 with four waves reading at once, over all XOR maps that are
  // linear in the row's bits: these two serve both fragment shapes at the full
  // LDS rate (16 rows x 4 packs per instruction for the 16x16x32 MFMA, 32 rows x
  // 2 packs for 32x32x16); without them the reads take two to four times as long.
  __device__ static __forceinline__ int row_swizzle(int row) {
    return BK == 64 ? ((row >> 1) & 7) : (((row >> 4) & 1) | (((row >> 2) & 1) << 1));
  }
  // K offset (elements) inside the slice of the pack lane `lane` copies in
  // block b (KC only).
  __device__ static __forceinline__ int pack_k(int b, int lane) {
    const int row = b * (64 / kKPacks) + lane / kKPacks;
    return ((lane % kKPacks) ^ row_swizzle(row)) * 8;
  }

  // per lane: byte offset of this lane's pack in each of the wave's blocks
  uint32_t voff[kPerWave];
  // per wave (scalar registers)
  i32x4_t rsrc;       // buffer descriptor of the current slice; num_records ends the valid data
  int64_t remaining;  // bytes from the slice origin to the end of the valid data (can pass 2^31)
  int step;           // bytes between consecutive slices
  int k_left;         // K values from the slice start to the end of K

  // origin: element (row 0, k 0) of the tile; ld: elements between rows (KC)
  // or between consecutive k (not KC); r_valid rows and k_total values of K
  // exist; r_span = valid elements along the contiguous index of a [k] row.
  __device__ __forceinline__ void init(const uint16_t* origin, int wave, int lane,
                                       int ld, int r_valid, int r_span, int k_total) {
#pragma unroll
    for (int i = 0; i < kPerWave; ++i) {
      const int b = wave * kPerWave + i;
      if (KC) {
        const int row = b * (64 / kKPacks) + lane / kKPacks;
        voff[i] = (uint32_t)(row * ld + pack_k(b, lane)) * 2u;
      } else {
        const int k = b * (64 / kRowPacks) + lane / kRowPacks;
        // 32-byte segment ^ (2 (k & 3) + bit 3 of k), in 16-byte packs
        const int rc = (lane % kRowPacks) ^ ((k & 3) << 2) ^ (((k >> 3) & 1) << 1);
        voff[i] = rc * 8 < r_valid ? (uint32_t)(k * ld + rc * 8) * 2u : kOutOfRange;
      }
    }
    // everything past the ragged edge is beyond num_records and reads as zero
    const int64_t bytes = dma_valid_bytes(KC, r_valid, r_span, ld, k_total);
    remaining = ((int64_t)__builtin_amdgcn_readfirstlane((int)(bytes >> 32)) << 32) |
                (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)bytes);
    step = __builtin_amdgcn_readfirstlane((KC ? BK : BK * ld) * 2);
    k_left = k_total;
    const uint64_t p = (uint64_t)origin;
    rsrc[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    rsrc[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(p >> 32) & 0xffff);  // stride 0
    rsrc[2] = dma_num_records(remaining);
    rsrc[3] = kRsrcFlags;
    mask_k_tail(wave, lane);
  }

  // [row][k] memory cannot end a row early through num_records: in the one
  // slice that holds the end of K, the packs past it are pointed out of range
  // for good (the slices after it are empty anyway).
  __device__ __forceinline__ void mask_k_tail(int wave, int lane) {
    if (KC && k_left < BK) {
#pragma unroll
      for (int i = 0; i < kPerWave; ++i)
        if (pack_k(wave * kPerWave + i, lane) >= k_left) voff[i] = kOutOfRange;
    }
  }

  // Moves on to the next K-slice (a slice past the end of K reads all zeros).
  __device__ __forceinline__ void advance(int wave, int lane) {
    // 48-bit base: the carry into bits 32..47 cannot reach the stride field
    const uint64_t p = (((uint64_t)(uint32_t)rsrc[1] << 32) | (uint32_t)rsrc[0]) + (uint32_t)step;
    rsrc[0] = (int)(uint32_t)p;
    rsrc[1] = (int)(uint32_t)(p >> 32);
    remaining -= step;
    rsrc[2] = dma_num_records(remaining);
    k_left -= BK;
    mask_k_tail(wave, lane);
  }

  // Copy instruction i of this wave for the current slice, into the tile at
  // LDS byte address `tile_lds`.
  //
  // Written as inline assembly on purpose: the compiler then neither knows
  // that LDS is being written nor counts the loads in vmcnt, so it does not
  // put a full vmcnt(0) wait in front of every LDS read of the OTHER stages.
  // The kernel waits for a slice explicitly and publishes it with a barrier
  // before anyone reads it.
  __device__ __forceinline__ void issue(int i, uint32_t tile_lds, int wave) const {
    const uint32_t dst = tile_lds + (uint32_t)(wave * kPerWave + i) * 1024u;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(dst), "v"(voff[i]), "s"(rsrc) : "memory", "m0");
  }

  // MFMA fragment of the 16-row sub-tile starting at `row16`, K step `ks`
  // (32 values of K): lane l holds row row16 + l%16, K values 8*(l/16) .. +7.
  __device__ static __forceinline__ uint4 frag(const uint16_t* lds, int row16,
                                               int ks, int lane) {
    if (KC) {
      const int r = row16 + (lane & 15);
      const int pack = (ks * 4 + (lane >> 4)) ^ row_swizzle(r);
      return *reinterpret_cast<const uint4*>(lds + r * BK + pack * 8);
    } else {
      // ds_read_b64_tr_b16: within 16 lanes, lane i supplies the address of
      // elements [k + i/4][m + 4*(i%4) .. +3] and receives [k .. k+3][m + i].
      const int k = ks * 32 + 8 * (lane >> 4) + ((lane & 15) >> 2);
      const int m = row16 + 4 * (lane & 3);
      // 32-byte segments; a 64-bit read is served 32 lanes at a time, i.e. two
      // groups of 16 lanes whose k differ by 8, 4 k-rows each, all in one
      // segment: XOR with 2 (k & 3) + bit 3 of k puts those 8 chunks into 8
      // different segments of a 256-byte bank row
      const int seg = (m >> 4) ^ ((k & 3) << 1) ^ ((k >> 3) & 1), within = m & 15;
      const uint16_t* p = lds + k * R + seg * 16 + within;
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4_t*)(p));
      const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4_t*)(p + 4 * R));
      uint4 out;
      const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
      out.x = l2.x; out.y = l2.y; out.z = h2.x; out.w = h2.y;
      return out;
    }
  }

  // MFMA fragment of the 32-row sub-tile starting at `row32`, K step `kk`
  // (16 values of K): lane l holds row row32 + l%32, K values 8*(l/32) .. +7.
  __device__ static __forceinline__ uint4 frag32(const uint16_t* lds, int row32,
                                               int kk, int lane) {
    if (KC) {
      const int r = row32 + (lane & 31);
      const int pack = (kk * 2 + (lane >> 5)) ^ row_swizzle(r);
      return *reinterpret_cast<const uint4*>(lds + r * BK + pack * 8);
    } else {
      // ds_read_b64_tr_b16: within 16 lanes, lane i supplies the address of
      // elements [k + i/4][m + 4*(i%4) .. +3] and receives [k .. k+3][m + i].
      const int k = kk * 16 + 8 * (lane >> 5) + ((lane & 15) >> 2);
      const int m = row32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
      // 32-byte segments; a 64-bit read is served 32 lanes at a time, i.e. 4 k-rows
      // x 2 segments: XOR with 2 (k & 3) puts those 8 chunks into 8 different
      // segments of a 256-byte bank row (bit 3 of k, constant here, serves frag())
      const int seg = (m >> 4) ^ ((k & 3) << 1) ^ ((k >> 3) & 1), within = m & 15;
      const uint16_t* p = lds + k * R + seg * 16 + within;
      const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4_t*)(p));
      const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4_t*)(p + 4 * R));
      uint4 out;
      const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
      out.x = l2.x; out.y = l2.y; out.z = h2.x; out.w = h2.y;
      return out;
    }
  }
};

// Tiles one XCD works on between two refills of its 32 CUs.
constexpr int kXcdRun = 32;

// Patch order over a rows x cols grid of tiles: bands of 16 rows, cut into
// blocks of 8 columns, cut into patches of 4 rows that are walked column by
// column.  32 consecutive numbers are a 4x8 patch (12 operand tiles for 32
// products), 256 consecutive ones a 16x16 region.  Ragged edges shrink the
// band, block or patch; the order stays a bijection.
// (The three sizes can be set at build time, for measurements of other walks: on the
// 16384-token, 4096 -> 14336, 8-expert layer a forward launch pulls 2.87 GiB through L2
// with 4 x 8 patches, 2.86 GiB with 8 x 4 and 4.19 GiB with 2 x 16.)
#ifndef FMOE_PATCH_ROWS
#define FMOE_PATCH_ROWS 4
#define FMOE_PATCH_COLS 8
#define FMOE_BAND_ROWS 16
#endif
__device__ __forceinline__ void tile_order(int t, int rows, int cols, int& row, int& col) {
  constexpr int kBand = FMOE_BAND_ROWS, kCols = FMOE_PATCH_COLS, kRows = FMOE_PATCH_ROWS;
  const int band = t / (kBand * cols);
  int r = t % (kBand * cols);
  const int band_rows = min(kBand, rows - band * kBand);
  const int blk = r / (band_rows * kCols);
  r %= band_rows * kCols;
  const int blk_cols = min(kCols, cols - blk * kCols);
  const int patch = r / (kRows * blk_cols);
  r %= kRows * blk_cols;
  const int patch_rows = min(kRows, band_rows - patch * kRows);
  row = band * kBand + patch * kRows + r % patch_rows;
  col = blk * kCols + r / patch_rows;
}

// Where a tile sits in the rows of its expert.
struct TileRows {
  int e;        // expert
  int m0;       // first row of the tile inside the expert
  int row0;     // first row of the expert
  int cnt;      // rows of the expert
};

// One output tile: rows [m0, m0 + BM) of expert e's row range (WGRAD: of its
// out_feat x in_feat gradient) by columns [n_origin, + BN); `where` names
// the expert, m0 and the expert's rows.
template <typename T, int BM, int BN, int BK, int WM, int WN, int NS, int MODE>
__device__ __forceinline__ void gemm_tile16(const GemmArgs& g, uint16_t* smem, TileRows where,
                                          int n_origin) {
  constexpr int NW = WM * WN;
  constexpr int NT = NW * 64;
  constexpr bool A_KC = MODE != GEMM_WGRAD;
  constexpr bool B_KC = is_fwd(MODE);
  constexpr int TM = BM / WM / 16, TN = BN / WN / 16;   // 16x16 blocks of a wave
  static_assert(BM % (WM * 16) == 0 && BN % (WN * 16) == 0 && BK % 32 == 0, "tile shape");
  static_assert((NS >= 4 && NS <= 8) || (NS == 2 && BK == 64), "LDS stages");
  using ATile = DmaTile<BM, BK, NW, A_KC>;
  using BTile = DmaTile<BN, BK, NW, B_KC>;
  constexpr int kStageBytes = ATile::kBytes + BTile::kBytes;
  constexpr int kStageElems = kStageBytes / 2;
  constexpr int kLoads = ATile::kPerWave + BTile::kPerWave;  // per wave per slice
  static_assert(NS == 2 || kLoads * (NS - 3) < 64, "vmcnt is a 6-bit counter");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave / WN, wave_n = wave % WN;
  const int in_f = g.in_feat, out_f = g.out_feat;
  const int e = __builtin_amdgcn_readfirstlane(where.e);
  const int row0 = __builtin_amdgcn_readfirstlane(where.row0);
  const int cnt = __builtin_amdgcn_readfirstlane(where.cnt);

  int M, N, K, lda, ldb, ldc;
  const uint16_t *A, *B;
  T* C;
  if (is_fwd(MODE)) {
    M = cnt; N = out_f; K = in_f;
    A = (const uint16_t*)g.a + (int64_t)row0 * in_f;        lda = in_f;
    B = expert_operand<uint16_t>(g.b, g.w_table, e, (int64_t)out_f * in_f); ldb = in_f;
    C = (T*)g.c + (int64_t)row0 * out_f;                    ldc = out_f;
  } else if (is_dgrad(MODE)) {
    M = cnt; N = in_f; K = out_f;
    A = (const uint16_t*)g.a + (int64_t)row0 * out_f;       lda = out_f;
    B = expert_operand<uint16_t>(g.b, g.w_table, e, (int64_t)out_f * in_f); ldb = in_f;
    C = (T*)g.c + (int64_t)row0 * in_f;                     ldc = in_f;
  } else {
    M = out_f; N = in_f; K = cnt;
    A = (const uint16_t*)g.a + (int64_t)row0 * out_f;       lda = out_f;
    B = (const uint16_t*)g.b + (int64_t)row0 * in_f;        ldb = in_f;
    C = (T*)g.c + (int64_t)e * out_f * in_f;                ldc = in_f;
  }
  const int m0 = __builtin_amdgcn_readfirstlane(where.m0);
  const int n0 = __builtin_amdgcn_readfirstlane(n_origin);
  if (m0 >= M || n0 >= N) return;
  const int m_valid = min(BM, M - m0), n_valid = min(BN, N - n0);

  const uint32_t lds_base = (uint32_t)(size_t)(lds_ptr_t)smem;
  ATile ta;
  BTile tb;
  ta.init(A_KC ? A + (int64_t)m0 * lda : A + m0, wave, lane, lda, m_valid, M - m0, K);
  tb.init(B_KC ? B + (int64_t)n0 * ldb : B + n0, wave, lane, ldb, n_valid, N - n0, K);

  // j-th copy instruction of this wave for the current slice (A tile's first)
  auto issue_load = [&](int j, uint32_t stage_lds) {
    if (j < ATile::kPerWave) ta.issue(j, stage_lds, wave);
    else tb.issue(j - ATile::kPerWave, stage_lds + ATile::kBytes, wave);
  };

  // acc[i][j] holds the TRANSPOSE of the 16x16 block (i, j) of C: the MFMA is
  // fed (B fragment, A fragment), so a lane ends up with 4 consecutive columns
  // of one row of C and can store them as 8 bytes.
  f32x4_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

  constexpr int KS = BK / 32;                    // K steps (32 values of K) per slice
  constexpr int kPerStep = TM * TN;              // MFMAs per K step
  constexpr int kMmaPerSlice = KS * kPerStep;
  static_assert(TM + TN <= kPerStep, "interleaving plan");
  static_assert(NW == 4, "one copy of the K loop per wave");
  const int k_tiles = (K + BK - 1) / BK;
  // fragments of the K step being multiplied and, filled meanwhile, of the next
  uint4 fa[2][TM], fb[2][TN];

  // K step `ks` of a slice whose first K step uses fragment buffer `par`: its
  // MFMAs, with the TM + TN LDS reads of the next K step's fragments dealt
  // evenly between them in the order of their first use (B0, A0, B1.., A1..),
  // so the LDS sees a steady stream and every read has half a K step to land.
  // (ks and par arrive as integral_constant tags: every register index below is
  // a constant of the instantiation.)  after_mfma(q) is the caller's hook for
  // its copy instructions.
  auto k_step = [&](auto ks_tag, auto par_tag, auto bunch_tag, const uint16_t* la,
                    const uint16_t* lb, const uint16_t* la_next, const uint16_t* lb_next,
                    auto&& after_mfma) {
    constexpr int ks = decltype(ks_tag)::value, par = decltype(par_tag)::value;
    // bunched: read r right behind MFMA r, so that all are on their way early
    constexpr bool bunched = decltype(bunch_tag)::value;
    constexpr int cur = (par + ks) & 1;
    constexpr bool wraps = ks + 1 == KS;
    const uint16_t* pa = wraps ? la_next : la;
    const uint16_t* pb = wraps ? lb_next : lb;
    constexpr int ks_pre = wraps ? 0 : ks + 1;
    constexpr int n_reads = TM + TN;
    static_for<kPerStep>([&](auto q_tag) {
      constexpr int q = decltype(q_tag)::value, i = q / TN, j = q % TN;
      acc[i][j] = Mma<T>::run(fb[cur][j], fa[cur][i], acc[i][j]);
      // read r sits behind MFMA r * kPerStep / n_reads (or behind MFMA r)
      constexpr int r = bunched ? q : (q * n_reads + kPerStep - 1) / kPerStep;
      if constexpr (r < n_reads && (bunched || r * kPerStep / n_reads == q)) {
        if constexpr (r == 0)
          fb[cur ^ 1][0] = BTile::frag(pb, wave_n * (BN / WN), ks_pre, lane);
        else if constexpr (r == 1)
          fa[cur ^ 1][0] = ATile::frag(pa, wave_m * (BM / WM), ks_pre, lane);
        else if constexpr (r < TN + 1)
          fb[cur ^ 1][r - 1] = BTile::frag(pb, wave_n * (BN / WN) + (r - 1) * 16, ks_pre, lane);
        else
          fa[cur ^ 1][r - TN] = ATile::frag(pa, wave_m * (BM / WM) + (r - TN) * 16, ks_pre, lane);
      }
      after_mfma(q_tag);
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  if constexpr (NS == 2) {
    // ---- two stages of 64 values of K, two barriers per slice
    //
    // A [row][k] operand then moves whole 128-byte lines (half as many L2
    // requests as 64-byte pieces of rows).  Iteration kt runs the two K steps
    // of slice kt out of registers filled one K step ahead:
    //   * the first K step reads the fragments of the second one right away, one
    //     read behind each of its first MFMAs.  When they have landed the stage of
    //     slice kt is not needed any more; the waves say so at the first barrier
    //     (behind MFMA kFreeAt - 1) and start copying slice kt+2 into it;
    //   * the copies are dealt over the rest of the slice, one copy of the block
    //     every (kCopyEnd - kFreeAt) / (4 kLoads) MFMAs: the CU's one address unit
    //     takes about 20 cycles per copy (52 bytes per cycle measured), so the 64
    //     copies of a 256 x 256 slice keep it busy for 60 % of the slice's MFMA
    //     time and must not be packed into one K step, where the waves would wait
    //     at every copy for the unit to take it;
    //   * the second barrier, in front of the last K step, publishes slice kt+1
    //     (copied during the slice before, landed by now); the last K step reads
    //     the first fragments of slice kt+1 between its MFMAs.
    static_assert(KS == 2, "two K steps per slice");
    // first MFMA of a slice behind which copies may go, and the MFMA the last
    // one has gone before (the slice has 2 * kPerStep MFMAs)
    constexpr int kFreeAt = TM + TN + 8, kCopyEnd = 2 * kPerStep - 4;
    static_assert(kFreeAt < kPerStep && kLoads <= kCopyEnd - kFreeAt,
                  "at most one copy per MFMA of a wave");
#pragma unroll
    for (int j = 0; j < kLoads; ++j) issue_load(j, lds_base);
    ta.advance(wave, lane);
    tb.advance(wave, lane);
#pragma unroll
    for (int j = 0; j < kLoads; ++j) issue_load(j, lds_base + kStageBytes);
    ta.advance(wave, lane);
    tb.advance(wave, lane);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads) : "memory");
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[0][i] = ATile::frag(smem, wave_m * (BM / WM) + i * 16, 0, lane);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[0][j] = BTile::frag(smem + ATile::kBytes / 2, wave_n * (BN / WN) + j * 16, 0, lane);

    // MFMA (counted through the slice) behind which copy c of the wave in
    // position `phase` goes: the 4 * kLoads copies of the block are dealt evenly
    // over MFMAs kFreeAt .. kCopyEnd - 1, one wave after the other.
    auto k_loop = [&](auto phase_tag) {
      constexpr int kPhase = decltype(phase_tag)::value;
      // copies of this wave issued before MFMA n of the slice
      auto issued_before = [](int n) constexpr {
        int cnt = 0;
        for (int c = 0; c < kLoads; ++c)
          if (kFreeAt + (c * NW + kPhase) * (kCopyEnd - kFreeAt) / (kLoads * NW) < n) ++cnt;
        return cnt;
      };
      for (int kt = 0; kt < k_tiles; ++kt) {
        const int stage = kt & 1;
        const uint32_t cur_lds = lds_base + (uint32_t)stage * kStageBytes;
        const uint16_t* la = smem + stage * kStageElems;
        const uint16_t* lb = la + ATile::kBytes / 2;
        const uint16_t* la_next = smem + (stage ^ 1) * kStageElems;
        const uint16_t* lb_next = la_next + ATile::kBytes / 2;
        static_for<KS>([&](auto ks_tag) {
          constexpr int ks = decltype(ks_tag)::value;
          if constexpr (ks == KS - 1) {
            // slice kt+1 is needed from here on: everything but the copies of slice
            // kt+2 issued so far has landed
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(issued_before(kPerStep)) : "memory");
            __syncthreads();
          }
          k_step(ks_tag, std::integral_constant<int, 0>{},
                 std::integral_constant<bool, ks == 0>{}, la, lb, la_next, lb_next,
                 [&](auto q_tag) {
            constexpr int n = ks * kPerStep + decltype(q_tag)::value;
            if constexpr (n == kFreeAt - 1) {
              // the fragments of the slice's last K step are in registers (or on
              // their way: wait for them): once every wave says so, the stage is free
              __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
              __syncthreads();
            }
            if constexpr (n >= kFreeAt && n < kCopyEnd) {
              constexpr int c = issued_before(n);   // the next copy to issue
              if constexpr (c < kLoads &&
                            kFreeAt + (c * NW + kPhase) * (kCopyEnd - kFreeAt) / (kLoads * NW) == n)
                issue_load(c, cur_lds);
            }
          });
          if constexpr (ks == KS - 1) {  // slice kt+2 is issued in full
            ta.advance(wave, lane);
            tb.advance(wave, lane);
          }
        });
      }
    };
    switch (wave) {
      case 0: k_loop(std::integral_constant<int, 0>{}); break;
      case 1: k_loop(std::integral_constant<int, 1>{}); break;
      case 2: k_loop(std::integral_constant<int, 2>{}); break;
      default: k_loop(std::integral_constant<int, 3>{}); break;
    }
  } else {
    // ---- software pipeline over the K-slices (NS LDS stages, NS >= 4)
    //
    // At the top of iteration kt: slices kt and kt+1 are visible to every wave,
    // slice kt+2 is in flight, the MFMA fragments of its first K step are
    // already in registers, and the stage of slice kt-1 is free.  The iteration
    //   * issues the copy of slice kt+NS-1 into that free stage, one copy
    //     instruction at a time between the MFMAs,
    //   * runs the MFMAs of slice kt, reading the fragments of the next K step
    //     between them; the last one prefetches the first fragments of slice
    //     kt+1, so the MFMA pipe does not drain at the barrier,
    //   * waits until its own share of slice kt+2 has landed and meets the other
    //     waves at the barrier, which publishes slice kt+2 and frees stage kt.
    // Slices past the end of K are zero-filled dummies; nothing is conditional.
    //
    // The barrier releases the waves of a block together, and a copy instruction
    // keeps the CU's one address unit busy for some 16 cycles: if every wave put
    // its copies behind the same MFMAs, each would queue behind the others and
    // hold up its own MFMAs.  The loop therefore exists once per wave (`phase`),
    // with the copy instructions of wave w behind MFMAs that no other wave uses;
    // and, a slice of 32 being ONE K step, once per parity of the slice number,
    // which names the fragment buffer in use.
    static_assert(kLoads <= kMmaPerSlice, "at most one copy per MFMA");
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) {
#pragma unroll
      for (int j = 0; j < kLoads; ++j) issue_load(j, lds_base + s * kStageBytes);
      ta.advance(wave, lane);
      tb.advance(wave, lane);
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 3) * kLoads) : "memory");
    __syncthreads();

#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[0][i] = ATile::frag(smem, wave_m * (BM / WM) + i * 16, 0, lane);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[0][j] = BTile::frag(smem + ATile::kBytes / 2, wave_n * (BN / WN) + j * 16, 0, lane);

    // one K-slice held by `stage`; parity_tag names the buffer of its first K step
    auto slice = [&](auto phase_tag, auto parity_tag, int stage) {
      constexpr int kPhase = decltype(phase_tag)::value;
      const int stage_next = stage + 1 == NS ? 0 : stage + 1;
      const int stage_free = stage == 0 ? NS - 1 : stage - 1;
      const uint32_t free_lds = lds_base + (uint32_t)stage_free * kStageBytes;
      const uint16_t* la = smem + stage * kStageElems;
      const uint16_t* lb = la + ATile::kBytes / 2;
      const uint16_t* la_next = smem + stage_next * kStageElems;
      const uint16_t* lb_next = la_next + ATile::kBytes / 2;
      static_for<KS>([&](auto ks_tag) {
        k_step(ks_tag, parity_tag, std::false_type{}, la, lb, la_next, lb_next, [&](auto q_tag) {
          // copy instruction c of phase p sits behind MFMA
          // (c * NW + p) * kMmaPerSlice / (kLoads * NW) of the slice
          constexpr int n = decltype(ks_tag)::value * kPerStep + decltype(q_tag)::value;
          constexpr int c0 = (n * kLoads * NW - kPhase * kMmaPerSlice + NW * kMmaPerSlice - 1) /
                             (NW * kMmaPerSlice);
          constexpr int c = c0 < 0 ? 0 : c0;
          if constexpr (c < kLoads && (c * NW + kPhase) * kMmaPerSlice / (kLoads * NW) == n)
            issue_load(c, free_lds);
        });
      });
      ta.advance(wave, lane);
      tb.advance(wave, lane);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 3) * kLoads) : "memory");
      __syncthreads();
      return stage_next;
    };
    auto k_loop = [&](auto phase_tag) {
      int stage = 0;
      if constexpr (KS % 2 == 1) {
        // two slices per trip, so that the buffer parity is fixed in the code
        int kt = 0;
        for (; kt + 1 < k_tiles; kt += 2) {
          stage = slice(phase_tag, std::integral_constant<int, 0>{}, stage);
          stage = slice(phase_tag, std::integral_constant<int, 1>{}, stage);
        }
        if (kt < k_tiles) stage = slice(phase_tag, std::integral_constant<int, 0>{}, stage);
      } else {
        for (int kt = 0; kt < k_tiles; ++kt)
          stage = slice(phase_tag, std::integral_constant<int, 0>{}, stage);
      }
    };
    switch (wave) {
      case 0: k_loop(std::integral_constant<int, 0>{}); break;
      case 1: k_loop(std::integral_constant<int, 1>{}); break;
      case 2: k_loop(std::integral_constant<int, 2>{}); break;
      default: k_loop(std::integral_constant<int, 3>{}); break;
    }
  }
  // The zero-filled dummy slices are still landing in LDS: let them finish,
  // then the whole LDS allocation is free to stage the output tile.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // ---- epilogue: accumulator r of lane l is
  //      C[m = l%16][n = 4*(l/16) + r] of its 16x16 block.
  // The tile goes through LDS (row-major, rows padded by 16 bytes so that the
  // 8-byte writes of 16 rows x 2 column groups, the 32 lanes served together,
  // spread over the banks) and leaves as 16-byte packs: one wave instruction
  // then stores whole 512-byte row segments.
  const T* bias = is_fwd(MODE) ? expert_operand<T>(g.bias, g.bias_table, e, out_f) : nullptr;
  struct alignas(8) Out4 { T v[4]; };
  constexpr int kLdc = BN + 8;   // elements per staged row
  T* stage_c = reinterpret_cast<T*>(smem);
  // (only the forward product has a bias; elsewhere the sums are rounded as they
  // are: adding a zero would cost an instruction per value, which the compiler may
  // not drop because of -0.  ONE code path: two variants of this loop made the
  // register allocator shuffle the accumulators inside the K loop.)
  constexpr bool kBias = is_fwd(MODE);
  float bv[TN][4];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
#pragma unroll
    for (int c = 0; c < 4; ++c) bv[j][c] = 0.f;
    if constexpr (kBias) {
      const int col = wave_n * (BN / WN) + j * 16 + 4 * (lane >> 4);
      if (bias && n0 + col < N) {
        const Out4 b4 = load_global<Out4>(bias + n0 + col);
#pragma unroll
        for (int c = 0; c < 4; ++c) bv[j][c] = Elem<T>::to_acc(b4.v[c]);
      }
    }
  }
  // block (i, j) of the wave's accumulators, rounded, into the staged tile
  auto stage_block = [&](auto i_tag, auto j_tag) {
    constexpr int i = decltype(i_tag)::value, j = decltype(j_tag)::value;
    const int col = wave_n * (BN / WN) + j * 16 + 4 * (lane >> 4);
    const int row = wave_m * (BM / WM) + i * 16 + (lane & 15);
    Out4 o;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      o.v[c] = Elem<T>::from_acc(kBias ? acc[i][j][c] + bv[j][c] : acc[i][j][c]);
    *reinterpret_cast<Out4*>(stage_c + row * kLdc + col) = o;
  };
  // every thread moves one fixed 16-byte column pack of every kRowsPerStep-th row
  constexpr int kRowPacks = BN / 8;                  // 16-byte packs per tile row
  constexpr int kRowsPerStep = NT / kRowPacks;
  constexpr int kSteps = BM / kRowsPerStep;
  static_assert(NT % kRowPacks == 0 && BM % kRowsPerStep == 0 && kSteps <= 32,
                "output tile must split evenly over the threads");
  const int pk = tid % kRowPacks, r0 = tid / kRowPacks;
  const T* sp = stage_c + r0 * kLdc + pk * 8;
  // Rows past the expert's last one are cut off by the buffer descriptor (the
  // bytes of this tile end with the last valid row), so the loop carries no
  // per-row condition; a pack past the last column (N is a multiple of 8: a pack
  // is all in or all out) gets an offset no descriptor reaches.
  const __amdgpu_buffer_rsrc_t c_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(C + (int64_t)m0 * ldc + n0), (short)0, ((m_valid - 1) * ldc + n_valid) * 2,
      kRsrcFlags);
  const int c_off = n0 + pk * 8 < N ? (r0 * ldc + pk * 8) * 2 : (int)kOutOfRange;
  // FWD with the activation fused in (g.act_out): the tile is written twice, as it
  // is (the pre-activations the backward needs) and through the table of
  // gelu(x) for 16-bit x, whose slice for 2^-28 <= |x| < 16 (both signs, 8192
  // results) sits in LDS behind the staged tile; a pack with an argument outside
  // that range (zeros, denormals, |x| >= 16, infinities, NaNs) is looked up in the
  // full table in memory.
  constexpr bool fuse_fwd = MODE == GEMM_FWD_ACT;
  // (behind this instantiation's own staged tile: a small tile shape then needs little
  // LDS and two of its workgroups fit a CU)
  constexpr int kTabOffset = BM * kLdc * 2;
  static_assert(kTabOffset % 16 == 0 && kTabOffset <= kActTabLdsOffset, "place of the table");
  uint16_t* fwd_tab_w = smem + kTabOffset / 2;
  const lds_u16_ptr_t fwd_tab = (lds_u16_ptr_t)fwd_tab_w;
  static_assert((kActTabBytes / 16) % NT == 0, "the table splits evenly over the threads");
  constexpr int kTabPerThread = kActTabBytes / 16 / NT;
  i32x4_t tab_regs[kTabPerThread];
#pragma unroll
  for (int i = 0; i < kTabPerThread; ++i) tab_regs[i] = i32x4_t{0, 0, 0, 0};
  __amdgpu_buffer_rsrc_t a_rsrc = c_rsrc;
  if constexpr (fuse_fwd) {
    // 16-byte piece L of the slice: 8 results from pattern 0x3180 + 8 L on, the
    // second half of the pieces from 0xB180 on (the negative arguments)
    constexpr int kHalfPieces = kActTabBytes / 16 / 2;
#pragma unroll
    for (int i = 0; i < kTabPerThread; ++i) {
      const int piece = tid + i * NT;
      const int first = piece < kHalfPieces ? kActTabFirst + 8 * piece
                                            : 0x8000 + kActTabFirst + 8 * (piece - kHalfPieces);
      tab_regs[i] = *reinterpret_cast<const i32x4_t*>(g.act_fwd_table + first);
    }
    a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void*)((T*)g.act_out + (int64_t)row0 * ldc + (int64_t)m0 * ldc + n0), (short)0,
        ((m_valid - 1) * ldc + n_valid) * 2, kRsrcFlags);
  }
  // gelu of the 8 values of a pack
  auto act_of = [&](i32x4_t pre) -> i32x4_t {
    i32x4_t out;
    uint32_t seen = 0;
#pragma unroll
    for (int wd = 0; wd < 4; ++wd) {
      const uint32_t pw = (uint32_t)pre[wd];
      const uint32_t t0 = (pw & 0x7fffu) - kActTabFirst, t1 = ((pw >> 16) & 0x7fffu) - kActTabFirst;
      seen |= t0 | t1;
      const uint32_t r0v = fwd_tab[t0 | ((pw >> 3) & 0x1000u)];
      const uint32_t r1v = fwd_tab[t1 | ((pw >> 19) & 0x1000u)];
      out[wd] = (int)(r0v | (r1v << 16));
    }
    if (__builtin_amdgcn_ballot_w64(seen >= (uint32_t)kActTabCount) != 0) {
#pragma unroll
      for (int wd = 0; wd < 4; ++wd) {
        const uint32_t pw = (uint32_t)pre[wd];
        out[wd] = (int)((uint32_t)g.act_fwd_table[pw & 0xffffu] |
                        ((uint32_t)g.act_fwd_table[pw >> 16] << 16));
      }
    }
    return out;
  };
  // The upper half of every wave's rows is staged while the packs of the lower
  // half are on their way out: the stores leave at the address unit's pace (about
  // 30 cycles per wave instruction), the staging is conversion work for the vector
  // unit, and a wave that issued them back to back would sit at the stores.
  constexpr int kBand = BM / WM / kRowsPerStep;      // store steps per band of wave rows
  constexpr bool kOverlap = TM % 2 == 0 && (BM / WM) % (2 * kRowsPerStep) == 0;
  if constexpr (kOverlap) {
    constexpr int kHalf = kSteps / 2, kBlocks = TM / 2 * TN;
    // store step of the s-th pack of half h
    auto step_of = [](int h, int s2) constexpr {
      return s2 / (kBand / 2) * kBand + h * (kBand / 2) + s2 % (kBand / 2);
    };
    static_for<kBlocks>([&](auto b_tag) {
      constexpr int b = decltype(b_tag)::value;
      stage_block(std::integral_constant<int, b % (TM / 2)>{}, std::integral_constant<int, b / (TM / 2)>{});
    });
    if constexpr (fuse_fwd) {
#pragma unroll
      for (int i = 0; i < kTabPerThread; ++i)
        reinterpret_cast<i32x4_t*>(fwd_tab_w)[tid + i * NT] = tab_regs[i];
    }
    __syncthreads();
    // Every pack gets registers of its own: a store holds its data registers
    // until memory has acknowledged it, so a register reused for a later pack
    // would make that pack wait for a full store round trip.
    i32x4_t v[kSteps], w[kHalf];
#pragma unroll
    for (int s2 = 0; s2 < kHalf; ++s2)
      v[s2] = *reinterpret_cast<const i32x4_t*>(sp + step_of(0, s2) * kRowsPerStep * kLdc);
    static_for<kHalf>([&](auto s_tag) {
      constexpr int s2 = decltype(s_tag)::value;
      __builtin_amdgcn_raw_buffer_store_b128(
          v[s2], c_rsrc, c_off + step_of(0, s2) * kRowsPerStep * ldc * 2, 0, 0);
      if constexpr (fuse_fwd) {
        w[s2] = act_of(v[s2]);
        __builtin_amdgcn_raw_buffer_store_b128(
            w[s2], a_rsrc, c_off + step_of(0, s2) * kRowsPerStep * ldc * 2, 0, 0);
      }
      constexpr int b_lo = s2 * kBlocks / kHalf, b_hi = (s2 + 1) * kBlocks / kHalf;
      static_for<b_hi - b_lo>([&](auto d_tag) {
        constexpr int b = b_lo + decltype(d_tag)::value;
        stage_block(std::integral_constant<int, TM / 2 + b % (TM / 2)>{},
                    std::integral_constant<int, b / (TM / 2)>{});
      });
      __builtin_amdgcn_sched_barrier(0);
    });
    __syncthreads();
#pragma unroll
    for (int s2 = 0; s2 < kHalf; ++s2)
      v[kHalf + s2] = *reinterpret_cast<const i32x4_t*>(sp + step_of(1, s2) * kRowsPerStep * kLdc);
#pragma unroll
    for (int s2 = 0; s2 < kHalf; ++s2) {
      __builtin_amdgcn_raw_buffer_store_b128(
          v[kHalf + s2], c_rsrc, c_off + step_of(1, s2) * kRowsPerStep * ldc * 2, 0, 0);
      if constexpr (fuse_fwd) {
        w[s2] = act_of(v[kHalf + s2]);
        __builtin_amdgcn_raw_buffer_store_b128(
            w[s2], a_rsrc, c_off + step_of(1, s2) * kRowsPerStep * ldc * 2, 0, 0);
      }
    }
  } else {
    static_for<TM * TN>([&](auto b_tag) {
      constexpr int b = decltype(b_tag)::value;
      stage_block(std::integral_constant<int, b % TM>{}, std::integral_constant<int, b / TM>{});
    });
    if constexpr (fuse_fwd) {
#pragma unroll
      for (int i = 0; i < kTabPerThread; ++i)
        reinterpret_cast<i32x4_t*>(fwd_tab_w)[tid + i * NT] = tab_regs[i];
    }
    __syncthreads();
    i32x4_t v[kSteps], w[kSteps];
#pragma unroll
    for (int u = 0; u < kSteps; ++u)
      v[u] = *reinterpret_cast<const i32x4_t*>(sp + u * kRowsPerStep * kLdc);
#pragma unroll
    for (int u = 0; u < kSteps; ++u) {
      __builtin_amdgcn_raw_buffer_store_b128(v[u], c_rsrc, c_off + u * kRowsPerStep * ldc * 2, 0,
                                             0);
      if constexpr (fuse_fwd) {
        w[u] = act_of(v[u]);
        __builtin_amdgcn_raw_buffer_store_b128(w[u], a_rsrc, c_off + u * kRowsPerStep * ldc * 2,
                                               0, 0);
      }
    }
  }
}


// gemm_tile() with 32x32x16 MFMAs (the wave's patch as a grid of 32x32
// accumulators): used for DGRAD and WGRAD.
template <typename T, int BM, int BN, int BK, int WM, int WN, int NS, int MODE>
__device__ __forceinline__ void gemm_tile32(const GemmArgs& g, uint16_t* smem, TileRows where,
                                          int n_origin) {
  constexpr int NW = WM * WN;
  constexpr int NT = NW * 64;
  constexpr bool A_KC = MODE != GEMM_WGRAD;
  constexpr bool B_KC = is_fwd(MODE);
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BK % 16 == 0, "tile shape");
  static_assert((NS >= 4 && NS <= 8) || (NS == 2 && BK == 64), "LDS stages");
  using ATile = DmaTile<BM, BK, NW, A_KC>;
  using BTile = DmaTile<BN, BK, NW, B_KC>;
  constexpr int kStageBytes = ATile::kBytes + BTile::kBytes;
  constexpr int kStageElems = kStageBytes / 2;
  constexpr int kLoads = ATile::kPerWave + BTile::kPerWave;  // per wave per slice
  static_assert(NS == 2 || kLoads * (NS - 3) < 64, "vmcnt is a 6-bit counter");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave / WN, wave_n = wave % WN;
  const int in_f = g.in_feat, out_f = g.out_feat;
  const int e = __builtin_amdgcn_readfirstlane(where.e);
  const int row0 = __builtin_amdgcn_readfirstlane(where.row0);
  const int cnt = __builtin_amdgcn_readfirstlane(where.cnt);

  int M, N, K, lda, ldb, ldc;
  const uint16_t *A, *B;
  T* C;
  if (is_fwd(MODE)) {
    M = cnt; N = out_f; K = in_f;
    A = (const uint16_t*)g.a + (int64_t)row0 * in_f;        lda = in_f;
    B = expert_operand<uint16_t>(g.b, g.w_table, e, (int64_t)out_f * in_f); ldb = in_f;
    C = (T*)g.c + (int64_t)row0 * out_f;                    ldc = out_f;
  } else if (is_dgrad(MODE)) {
    M = cnt; N = in_f; K = out_f;
    A = (const uint16_t*)g.a + (int64_t)row0 * out_f;       lda = out_f;
    B = expert_operand<uint16_t>(g.b, g.w_table, e, (int64_t)out_f * in_f); ldb = in_f;
    C = (T*)g.c + (int64_t)row0 * in_f;                     ldc = in_f;
  } else {
    M = out_f; N = in_f; K = cnt;
    A = (const uint16_t*)g.a + (int64_t)row0 * out_f;       lda = out_f;
    B = (const uint16_t*)g.b + (int64_t)row0 * in_f;        ldb = in_f;
    C = (T*)g.c + (int64_t)e * out_f * in_f;                ldc = in_f;
  }
  const int m0 = __builtin_amdgcn_readfirstlane(where.m0);
  const int n0 = __builtin_amdgcn_readfirstlane(n_origin);
  if (m0 >= M || n0 >= N) return;
  const int m_valid = min(BM, M - m0), n_valid = min(BN, N - n0);

  const uint32_t lds_base = (uint32_t)(size_t)(lds_ptr_t)smem;
  ATile ta;
  BTile tb;
  ta.init(A_KC ? A + (int64_t)m0 * lda : A + m0, wave, lane, lda, m_valid, M - m0, K);
  tb.init(B_KC ? B + (int64_t)n0 * ldb : B + n0, wave, lane, ldb, n_valid, N - n0, K);

  // j-th copy instruction of this wave for the current slice (A tile's first)
  auto issue_load = [&](int j, uint32_t stage_lds) {
    if (j < ATile::kPerWave) ta.issue(j, stage_lds, wave);
    else tb.issue(j - ATile::kPerWave, stage_lds + ATile::kBytes, wave);
  };

  // acc[i][j] holds the TRANSPOSE of the 32x32 block (i, j) of C: the MFMA is
  // fed (B fragment, A fragment), so a lane ends up with 4 consecutive columns
  // of one row of C per group of 4 accumulators and can store them as 8 bytes.
  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // WGRAD tiles of the first column also sum the columns of their A operand
  // (dY of this expert): the bias gradient, fp32, one v_dot2 per pair of values.
  // g.bias then points at the [E, out_feat] gradient.
  const bool colsum = MODE == GEMM_WGRAD && g.bias != nullptr && n0 == 0;
  float cs[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) cs[i] = 0.f;
  auto add_colsum = [&](const uint4 (&frags)[TM]) {
    if (MODE == GEMM_WGRAD && colsum) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        cs[i] = ColSum<T>::add(frags[i].x, cs[i]);
        cs[i] = ColSum<T>::add(frags[i].y, cs[i]);
        cs[i] = ColSum<T>::add(frags[i].z, cs[i]);
        cs[i] = ColSum<T>::add(frags[i].w, cs[i]);
      }
    }
  };

  constexpr int KK = BK / 16;                    // MFMA K steps per slice
  constexpr int kMmaPerSlice = KK * TM * TN;
  static_assert(KK % 2 == 0, "fragment double buffer is indexed by the parity of the K step");
  static_assert(NS != 2 || TM + TN <= TM * TN, "interleaving plan of the two-stage loop");
  static_assert(NW == 4, "one copy of the K loop per wave");
  const int k_tiles = (K + BK - 1) / BK;
  uint4 fa[2][TM], fb[2][TN];

  if constexpr (NS == 2) {
    // ---- two stages of 64 values of K, one barrier per slice
    //
    // A [row][k] operand then moves whole 128-byte lines (half as many L2
    // requests as 64-byte pieces of rows).  Iteration kt runs the four K steps
    // of slice kt; the barrier sits in front of the LAST K step:
    //   * K steps 0..2 read their fragments from slice kt's stage; by the
    //     barrier every wave has read all of it, so the stage is free, and has
    //     waited for its share of slice kt+1, so that slice is published;
    //   * K step 3 prefetches the first fragments of slice kt+1 and starts the
    //     copy of slice kt+2 into the freed stage; K step 0 of the next
    //     iteration issues the second half of that copy.  The copy then has K
    //     steps 1 and 2 (32 MFMAs) to land.
    constexpr int kHalf = kLoads / 2;
    static_assert(kLoads % 2 == 0, "the copy of a slice is issued in two halves");
#pragma unroll
    for (int j = 0; j < kLoads; ++j) issue_load(j, lds_base);
    ta.advance(wave, lane);
    tb.advance(wave, lane);
#pragma unroll
    for (int j = 0; j < kHalf; ++j) issue_load(j, lds_base + kStageBytes);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kHalf) : "memory");
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[0][i] = ATile::frag32(smem, wave_m * (BM / WM) + i * 32, 0, lane);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[0][j] = BTile::frag32(smem + ATile::kBytes / 2, wave_n * (BN / WN) + j * 32, 0, lane);

    auto k_loop = [&](auto phase_tag) {
      constexpr int kPhase = decltype(phase_tag)::value;
      constexpr int kPerStep = TM * TN;           // MFMAs per K step
      for (int kt = 0; kt < k_tiles; ++kt) {
        const int stage = kt & 1;
        const uint32_t cur_lds = lds_base + (uint32_t)stage * kStageBytes;
        const uint32_t other_lds = lds_base + (uint32_t)(stage ^ 1) * kStageBytes;
        const uint16_t* la = smem + stage * kStageElems;
        const uint16_t* lb = la + ATile::kBytes / 2;
        const uint16_t* la_next = smem + (stage ^ 1) * kStageElems;
        const uint16_t* lb_next = la_next + ATile::kBytes / 2;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          if (kk == KK - 1) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): my reads of this stage are done
            __syncthreads();
          }
          const int cur = kk & 1;
          const uint16_t* pa = kk + 1 < KK ? la : la_next;
          const uint16_t* pb = kk + 1 < KK ? lb : lb_next;
          const int kk_pre = kk + 1 < KK ? kk + 1 : 0;
#pragma unroll
          for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
              acc[i][j] = Mma32<T>::run(fb[cur][j], fa[cur][i], acc[i][j]);
              const int q = i * TN + j;
              if (q < TM)
                fa[cur ^ 1][q] = ATile::frag32(pa, wave_m * (BM / WM) + q * 32, kk_pre, lane);
              else if (q < TM + TN)
                fb[cur ^ 1][q - TM] =
                    BTile::frag32(pb, wave_n * (BN / WN) + (q - TM) * 32, kk_pre, lane);
              // copy instruction c of a half sits behind MFMA
              // (c * NW + phase) * kPerStep / (kHalf * NW) of its K step
              if (kk == 0 || kk == KK - 1) {
#pragma unroll
                for (int c = 0; c < kHalf; ++c)
                  if ((c * NW + kPhase) * kPerStep / (kHalf * NW) == q) {
                    if (kk == 0) issue_load(kHalf + c, other_lds);  // rest of slice kt+1
                    else issue_load(c, cur_lds);                    // start of slice kt+2
                  }
              }
              __builtin_amdgcn_sched_barrier(0);
            }
          }
          add_colsum(fa[cur]);
          if (kk == 0) {  // slice kt+1 is issued in full: move on to slice kt+2
            ta.advance(wave, lane);
            tb.advance(wave, lane);
          }
        }
      }
    };
    switch (wave) {
      case 0: k_loop(std::integral_constant<int, 0>{}); break;
      case 1: k_loop(std::integral_constant<int, 1>{}); break;
      case 2: k_loop(std::integral_constant<int, 2>{}); break;
      default: k_loop(std::integral_constant<int, 3>{}); break;
    }
  } else {
    // ---- software pipeline over the K-slices (NS LDS stages, NS >= 4)
    //
    // At the top of iteration kt: slices kt and kt+1 are visible to every wave,
    // slice kt+2 is in flight, the MFMA fragments of (kt, K step 0) are already
    // in registers, and the stage of slice kt-1 is free.  The iteration
    //   * issues the copy of slice kt+NS-1 into that free stage, one copy
    //     instruction at a time between the MFMAs,
    //   * runs the MFMAs of slice kt, reading the fragments of the next K step
    //     one LDS read behind each MFMA; the last K step prefetches the first
    //     fragments of slice kt+1, so the MFMA pipe does not drain at the barrier,
    //   * waits until its own share of slice kt+2 has landed and meets the other
    //     waves at the barrier, which publishes slice kt+2 and frees stage kt.
    // Slices past the end of K are zero-filled dummies; nothing is conditional.
    //
    // The barrier releases the waves of a block together, and a copy instruction
    // keeps the CU's one address unit busy for some 16 cycles: if every wave put
    // its copies behind the same MFMAs, each would queue behind the others and
    // hold up its own MFMAs.  The loop therefore exists once per wave (`phase`),
    // with the copy instructions of wave w behind MFMAs that no other wave uses.
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) {
#pragma unroll
      for (int j = 0; j < kLoads; ++j) issue_load(j, lds_base + s * kStageBytes);
      ta.advance(wave, lane);
      tb.advance(wave, lane);
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 3) * kLoads) : "memory");
    __syncthreads();

#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[0][i] = ATile::frag32(smem, wave_m * (BM / WM) + i * 32, 0, lane);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[0][j] = BTile::frag32(smem + ATile::kBytes / 2, wave_n * (BN / WN) + j * 32, 0, lane);

    auto k_loop = [&](auto phase_tag) {
      constexpr int kPhase = decltype(phase_tag)::value;
      int stage = 0;
      for (int kt = 0; kt < k_tiles; ++kt) {
        const int stage_next = stage + 1 == NS ? 0 : stage + 1;
        const int stage_free = stage == 0 ? NS - 1 : stage - 1;
        const uint32_t free_lds = lds_base + (uint32_t)stage_free * kStageBytes;
        const uint16_t* la = smem + stage * kStageElems;
        const uint16_t* lb = la + ATile::kBytes / 2;
        const uint16_t* la_next = smem + stage_next * kStageElems;
        const uint16_t* lb_next = la_next + ATile::kBytes / 2;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
          const int cur = kk & 1;
          const uint16_t* pa = kk + 1 < KK ? la : la_next;
          const uint16_t* pb = kk + 1 < KK ? lb : lb_next;
          const int kk_pre = kk + 1 < KK ? kk + 1 : 0;
#pragma unroll
          for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
              acc[i][j] = Mma32<T>::run(fb[cur][j], fa[cur][i], acc[i][j]);
              const int q = i * TN + j;
              if (q < TM)
                fa[cur ^ 1][q] = ATile::frag32(pa, wave_m * (BM / WM) + q * 32, kk_pre, lane);
              else if (q < TM + TN)
                fb[cur ^ 1][q - TM] =
                    BTile::frag32(pb, wave_n * (BN / WN) + (q - TM) * 32, kk_pre, lane);
              // copy instruction c of phase p sits behind MFMA
              // (c * NW + p) * kMmaPerSlice / (kLoads * NW)
              const int n = kk * TM * TN + q;
#pragma unroll
              for (int c = 0; c < kLoads; ++c)
                if ((c * NW + kPhase) * kMmaPerSlice / (kLoads * NW) == n) issue_load(c, free_lds);
              __builtin_amdgcn_sched_barrier(0);
            }
          }
          // narrow wave tiles have fewer MFMAs per K step than fragments to read
#pragma unroll
          for (int q = TM * TN; q < TM + TN; ++q) {
            if (q < TM)
              fa[cur ^ 1][q] = ATile::frag32(pa, wave_m * (BM / WM) + q * 32, kk_pre, lane);
            else
              fb[cur ^ 1][q - TM] =
                  BTile::frag32(pb, wave_n * (BN / WN) + (q - TM) * 32, kk_pre, lane);
          }
          add_colsum(fa[cur]);
        }
        ta.advance(wave, lane);
        tb.advance(wave, lane);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 3) * kLoads) : "memory");
        __syncthreads();
        stage = stage_next;
      }
    };
    switch (wave) {
      case 0: k_loop(std::integral_constant<int, 0>{}); break;
      case 1: k_loop(std::integral_constant<int, 1>{}); break;
      case 2: k_loop(std::integral_constant<int, 2>{}); break;
      default: k_loop(std::integral_constant<int, 3>{}); break;
    }
  }
  // The zero-filled dummy slices are still landing in LDS: let them finish,
  // then the whole LDS allocation is free to stage the output tile.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // column sums: lanes l and l + 32 hold the two K halves of row l % 32
  if (MODE == GEMM_WGRAD && colsum) {
    T* db = (T*)const_cast<void*>(g.bias) + (int64_t)e * out_f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const float total = cs[i] + __shfl_xor(cs[i], 32, 64);
      const int m = m0 + wave_m * (BM / WM) + i * 32 + (lane & 31);
      if (wave_n == 0 && lane < 32 && m < M) db[m] = Elem<T>::from_acc(total);
    }
  }

  // ---- epilogue: accumulator r of lane l is
  //      C[m = l%32][n = 8*(r/4) + 4*(l/32) + r%4] of its 32x32 block.
  // The tile goes through LDS (row-major, rows padded by 16 bytes so that the
  // 8-byte writes of 32 rows spread over the banks) and leaves as 16-byte packs:
  // one wave instruction then stores whole 512-byte row segments.
  const T* bias = is_fwd(MODE) ? expert_operand<T>(g.bias, g.bias_table, e, out_f) : nullptr;
  struct alignas(8) Out4 { T v[4]; };
  constexpr int kLdc = BN + 8;   // elements per staged row
  T* stage_c = reinterpret_cast<T*>(smem);
  // DGRAD with the activation's backward fused in: the slice of the gelu' table
  // goes into LDS behind the staged tile (its loads fly during the staging)
  constexpr bool fuse_act = MODE == GEMM_DGRAD_ACT;
  constexpr int kTabOffset = BM * kLdc * 2;   // behind this instantiation's own staged tile
  static_assert(kTabOffset % 16 == 0 && kTabOffset <= kActTabLdsOffset, "place of the table");
  float* act_tab_w = reinterpret_cast<float*>(smem + kTabOffset / 2);
  const lds_float_ptr_t act_tab = (lds_float_ptr_t)act_tab_w;
  // (an even split: a guarded load into the array would put it into scratch
  // memory, one load and one wait at a time)
  static_assert((kActTabCount / 4) % NT == 0, "the table splits evenly over the threads");
  constexpr int kTabPerThread = kActTabCount / 4 / NT;
  i32x4_t tab_regs[kTabPerThread];
#pragma unroll
  for (int i = 0; i < kTabPerThread; ++i) tab_regs[i] = i32x4_t{0, 0, 0, 0};
  if constexpr (fuse_act) {
    const i32x4_t* src = reinterpret_cast<const i32x4_t*>(g.act_table + kActTabFirst);
#pragma unroll
    for (int i = 0; i < kTabPerThread; ++i) tab_regs[i] = src[tid + i * NT];
  }
  // (only the forward product has a bias; elsewhere the sums are rounded as they
  // are: adding a zero would cost an instruction per value, which the compiler may
  // not drop because of -0)
  constexpr bool kBias = is_fwd(MODE);
  // 4 columns of block (i, j), column group q, rounded, into the staged tile
  auto stage_block = [&](auto i_tag, auto j_tag, auto q_tag) {
    constexpr int i = decltype(i_tag)::value, j = decltype(j_tag)::value;
    constexpr int q = decltype(q_tag)::value;
    const int col = wave_n * (BN / WN) + j * 32 + 8 * q + 4 * (lane >> 5);
    const int row = wave_m * (BM / WM) + i * 32 + (lane & 31);
    float bv[4] = {0.f, 0.f, 0.f, 0.f};
    if constexpr (kBias) {
      if (bias && n0 + col < N) {
        const Out4 b4 = load_global<Out4>(bias + n0 + col);
#pragma unroll
        for (int c = 0; c < 4; ++c) bv[c] = Elem<T>::to_acc(b4.v[c]);
      }
    }
    Out4 o;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      o.v[c] = Elem<T>::from_acc(kBias ? acc[i][j][4 * q + c] + bv[c] : acc[i][j][4 * q + c]);
    *reinterpret_cast<Out4*>(stage_c + row * kLdc + col) = o;
  };
  // blocks [lo, hi) of the wave in the order (j, q, i): i runs over rows [i_lo, i_lo + n_i)
  auto stage_blocks = [&](auto ilo_tag, auto ni_tag, auto lo_tag, auto hi_tag) {
    constexpr int i_lo = decltype(ilo_tag)::value, n_i = decltype(ni_tag)::value;
    constexpr int lo = decltype(lo_tag)::value, hi = decltype(hi_tag)::value;
    static_for<hi - lo>([&](auto d_tag) {
      constexpr int b = lo + decltype(d_tag)::value;
      stage_block(std::integral_constant<int, i_lo + b % n_i>{},
                  std::integral_constant<int, b / n_i / 4>{},
                  std::integral_constant<int, b / n_i % 4>{});
    });
  };
  // every thread moves one fixed 16-byte column pack of every kRowsPerStep-th row
  constexpr int kRowPacks = BN / 8;                  // 16-byte packs per tile row
  constexpr int kRowsPerStep = NT / kRowPacks;
  constexpr int kSteps = BM / kRowsPerStep;
  static_assert(NT % kRowPacks == 0 && BM % kRowsPerStep == 0 && kSteps <= 32,
                "output tile must split evenly over the threads");
  const int pk = tid % kRowPacks, r0 = tid / kRowPacks;
  const T* sp = stage_c + r0 * kLdc + pk * 8;
  // Rows past the expert's last one are cut off by the buffer descriptor (the
  // bytes of this tile end with the last valid row), so the loop carries no
  // per-row condition.
  const __amdgpu_buffer_rsrc_t c_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(C + (int64_t)m0 * ldc + n0), (short)0, ((m_valid - 1) * ldc + n_valid) * 2,
      kRsrcFlags);
  const int c_off = (r0 * ldc + pk * 8) * 2;
  // The upper half of every wave's rows is staged while the packs of the lower
  // half are on their way out (see gemm_tile16); with the activation's backward
  // fused in, the whole tile is staged first.
  constexpr int kBand = BM / WM / kRowsPerStep;      // store steps per band of wave rows
  constexpr bool kOverlap = TM % 2 == 0 && (BM / WM) % (2 * kRowsPerStep) == 0;
  constexpr int kHalfRows = kOverlap ? TM / 2 : TM;  // row blocks staged before the first barrier
  constexpr int kBlocksLo = kHalfRows * TN * 4, kBlocksHi = (TM - kHalfRows) * TN * 4;
  stage_blocks(std::integral_constant<int, 0>{}, std::integral_constant<int, kHalfRows>{},
               std::integral_constant<int, 0>{}, std::integral_constant<int, kBlocksLo>{});
  if constexpr (fuse_act) {
#pragma unroll
    for (int i = 0; i < kTabPerThread; ++i)
      reinterpret_cast<i32x4_t*>(act_tab_w)[tid + i * NT] = tab_regs[i];
  }
  if constexpr (kOverlap) {
    if constexpr (!fuse_act) {
      constexpr int kHalf = kSteps / 2;
      // store step of the s-th pack of half h
      auto step_of = [](int h, int s2) constexpr {
        return s2 / (kBand / 2) * kBand + h * (kBand / 2) + s2 % (kBand / 2);
      };
      const int c_off_v = n0 + pk * 8 < N ? c_off : (int)kOutOfRange;  // N is a multiple of 8
      __syncthreads();
      // Every pack gets registers of its own: a store holds its data registers
      // until memory has acknowledged it.
      i32x4_t v[kSteps];
#pragma unroll
      for (int s2 = 0; s2 < kHalf; ++s2)
        v[s2] = *reinterpret_cast<const i32x4_t*>(sp + step_of(0, s2) * kRowsPerStep * kLdc);
      static_for<kHalf>([&](auto s_tag) {
        constexpr int s2 = decltype(s_tag)::value;
        __builtin_amdgcn_raw_buffer_store_b128(
            v[s2], c_rsrc, c_off_v + step_of(0, s2) * kRowsPerStep * ldc * 2, 0, 0);
        stage_blocks(std::integral_constant<int, kHalfRows>{},
                     std::integral_constant<int, TM - kHalfRows>{},
                     std::integral_constant<int, s2 * kBlocksHi / kHalf>{},
                     std::integral_constant<int, (s2 + 1) * kBlocksHi / kHalf>{});
        __builtin_amdgcn_sched_barrier(0);
      });
      __syncthreads();
#pragma unroll
      for (int s2 = 0; s2 < kHalf; ++s2)
        v[kHalf + s2] =
            *reinterpret_cast<const i32x4_t*>(sp + step_of(1, s2) * kRowsPerStep * kLdc);
#pragma unroll
      for (int s2 = 0; s2 < kHalf; ++s2)
        __builtin_amdgcn_raw_buffer_store_b128(
            v[kHalf + s2], c_rsrc, c_off_v + step_of(1, s2) * kRowsPerStep * ldc * 2, 0, 0);
      return;
    }
    stage_blocks(std::integral_constant<int, kHalfRows>{},
                 std::integral_constant<int, TM - kHalfRows>{}, std::integral_constant<int, 0>{},
                 std::integral_constant<int, kBlocksHi>{});
  }
  __syncthreads();
  if constexpr (fuse_act) {
    // dx = dH * gelu'(pre): the staged dH (already rounded to the storage type,
    // as a separate activation kernel would read it) times the table value of
    // the matching pre-activation pack, fetched through a descriptor with the
    // tile's own bounds (a pack outside reads as zeros and its store is dropped).
    if (n0 + pk * 8 < N) {
      const __amdgpu_buffer_rsrc_t p_rsrc = __builtin_amdgcn_make_buffer_rsrc(
          (void*)((const T*)g.act_pre + ((int64_t)row0 + m0) * ldc + n0), (short)0,
          ((m_valid - 1) * ldc + n_valid) * 2, kRsrcFlags);
      constexpr int kChunk = kSteps < 8 ? kSteps : 8;
      constexpr int kChunks = kSteps / kChunk;
      static_assert(kSteps % kChunk == 0, "chunks of the fused epilogue");
      // the pre-activation packs of chunk c + 1 are in flight while chunk c is worked on
      i32x4_t pv[2][kChunk];
      auto load_pre = [&](auto c_tag) {
        constexpr int c = decltype(c_tag)::value;
#pragma unroll
        for (int u = 0; u < kChunk; ++u)
          pv[c & 1][u] = __builtin_amdgcn_raw_buffer_load_b128(
              p_rsrc, c_off + (c * kChunk + u) * kRowsPerStep * ldc * 2, 0, 0);
      };
      load_pre(std::integral_constant<int, 0>{});
      static_for<kChunks>([&](auto c_tag) {
        constexpr int c = decltype(c_tag)::value;
        if constexpr (c + 1 < kChunks) load_pre(std::integral_constant<int, c + 1>{});
        i32x4_t hv[kChunk], ov[kChunk];
#pragma unroll
        for (int u = 0; u < kChunk; ++u)
          hv[u] = *reinterpret_cast<const i32x4_t*>(sp + (c * kChunk + u) * kRowsPerStep * kLdc);
        uint32_t seen = 0;
#pragma unroll
        for (int u = 0; u < kChunk; ++u)
#pragma unroll
          for (int wd = 0; wd < 4; ++wd)
            ov[u][wd] = (int)gelu_bwd_pair_fast<T>((uint32_t)hv[u][wd], (uint32_t)pv[c & 1][u][wd],
                                                   act_tab, seen);
        if (__builtin_amdgcn_ballot_w64(seen >= (uint32_t)kActTabCount) != 0) {
#pragma unroll
          for (int u = 0; u < kChunk; ++u)
#pragma unroll
            for (int wd = 0; wd < 4; ++wd)
              ov[u][wd] = (int)gelu_bwd_pair_any<T>((uint32_t)hv[u][wd],
                                                    (uint32_t)pv[c & 1][u][wd], g.act_table);
        }
#pragma unroll
        for (int u = 0; u < kChunk; ++u)
          __builtin_amdgcn_raw_buffer_store_b128(
              ov[u], c_rsrc, c_off + (c * kChunk + u) * kRowsPerStep * ldc * 2, 0, 0);
      });
    }
    return;
  }
  if (n0 + pk * 8 < N) {  // N is a multiple of 8: a pack is all in or all out
    // Every pack gets registers of its own: a store holds its data registers
    // until memory has acknowledged it, so a register reused for a later pack
    // would make that pack wait for a full store round trip.
    i32x4_t v[kSteps];
#pragma unroll
    for (int u = 0; u < kSteps; ++u)
      v[u] = *reinterpret_cast<const i32x4_t*>(sp + u * kRowsPerStep * kLdc);
#pragma unroll
    for (int u = 0; u < kSteps; ++u)
      __builtin_amdgcn_raw_buffer_store_b128(v[u], c_rsrc, c_off + u * kRowsPerStep * ldc * 2, 0,
                                             0);
  }
}

// The MFMA shape of a product: 16x16x32 where both operands are read from LDS
// with plain 16-byte reads (FWD: 187 other instructions per 128 MFMAs), 32x32x16
// where an operand needs the transposing read.  Measured on the cfg-4 shapes:
// FWD 1.29-1.31 vs 1.24-1.26 PFLOP/s with 16x16x32, DGRAD 1.21 vs 1.35 and
// WGRAD 1.24 vs 1.27 the other way round.
#ifndef FMOE_MFMA16_MODES
#define FMOE_MFMA16_MODES ((1 << GEMM_FWD) | (1 << GEMM_FWD_ACT))
#endif
template <typename T, int BM, int BN, int BK, int WM, int WN, int NS, int MODE>
__device__ __forceinline__ void gemm_tile(const GemmArgs& g, uint16_t* smem, TileRows where,
                                          int n_origin) {
  if constexpr ((FMOE_MFMA16_MODES >> MODE) & 1)
    gemm_tile16<T, BM, BN, BK, WM, WN, NS, MODE>(g, smem, where, n_origin);
  else
    gemm_tile32<T, BM, BN, BK, WM, WN, NS, MODE>(g, smem, where, n_origin);
}

// Remainder tiles (see the kernels below): 64 rows (the 4 waves side by side,
// K slices of 32 in 6 LDS stages: a slice is a quarter of the MFMA work of a
// 256-row one, so its copies need more slices of lead to cover the memory
// latency) or 128 rows (2 x 2 waves, 4 stages).
constexpr int kSmallRows = 64;
constexpr int kSmallBK = 32;
constexpr int kSmallStages = 6;

// Whether tile shape BM x BN (4 waves) has a remainder shape kSmallRows x BN
// (the 4 waves side by side) that the pipeline's interleaving plan accepts.
template <int BM, int BN, int MODE>
constexpr bool has_small_tiles() {
  constexpr int tm = kSmallRows / 32, tn = BN / 4 / 32;   // in 32x32 blocks, the tighter case
  return MODE != GEMM_WGRAD && BM > kSmallRows && BN % 128 == 0 && tm + tn <= tm * tn;
}

// How expert rows are cut into tiles: `full` tiles of BM rows from row 0 on
// and, for a remainder of at most BM / 2 rows, one remainder tile (`small` is
// 0 or 1) of 64 rows, or of 128 rows when the remainder is longer than 64;
// a remainder above BM / 2 rows takes one more BM tile.  Remainder tiles cost
// about 0.45 (64 rows) and 0.6 (128 rows) of a 256-row tile.
template <int BM, bool SMALL>
__device__ __forceinline__ void cut_rows(int cnt, int& full, int& small) {
  if (!SMALL) {
    full = (cnt + BM - 1) / BM;
    small = 0;
    return;
  }
  full = cnt / BM;
  const int rem = cnt - full * BM;
  small = rem > 0 && rem <= BM / 2;
  if (rem > BM / 2) ++full;
}

// Runs a BM x BN tile, or the half-width / half-height tile that covers it when
// at most half of its columns (any product) or of its rows (WGRAD: the rows of
// dW are out_feat) exist: a feature size of, say, 1408 = 5.5 x 256 then pays
// for 5.6 tiles instead of 6.
template <typename T, int BM, int BN, int BK, int WM, int WN, int NS, int MODE>
__device__ __forceinline__ void edge_aware_tile(const GemmArgs& g, uint16_t* smem, TileRows where,
                                                int n_tile) {
  const int n0 = n_tile * BN;
  if constexpr (BM == 256 && BN == 256 && WM == 2 && WN == 2) {
    const int n_total = is_fwd(MODE) ? g.out_feat : g.in_feat;
    if (n_total - n0 <= BN / 2) {
      gemm_tile<T, BM, BN / 2, BK, WM, WN, NS, MODE>(g, smem, where, n0);
      return;
    }
    if (MODE == GEMM_WGRAD && g.out_feat - where.m0 <= BM / 2) {
      gemm_tile<T, BM / 2, BN, 32, WM, WN, 4, MODE>(g, smem, where, n0);
      return;
    }
  }
  gemm_tile<T, BM, BN, BK, WM, WN, NS, MODE>(g, smem, where, n0);
}

// A remainder tile streams its whole weight strip (BN columns x K) through one
// CU for 64 rows of output, at the rate of that CU's address unit (~52 bytes per
// cycle): when a launch has so few of them that they would leave most CUs idle
// (at most kNarrowMax; cfg 2 has 32 to 128 behind 1024 full tiles) they are cut
// into narrower ones, 64 columns for FWD and 128 for DGRAD (whose weight tile is
// [k][columns] and needs 128 of them for its LDS layout): four or two times as
// many CUs then share the streaming.  It pays from K = 2048 on (measured on the
// cfg-2 shapes from cold caches: K = 4096 forward 209 -> 180 us, dX 199 -> 182 us;
// at K = 1024 the fixed cost of four times as many tiles eats the gain).
// Their K slices hold 64 values: a narrow tile has 4 to 16 MFMAs per wave and K step,
// and with slices of 32 its K loop ran at the pace of the per-slice barrier and wait
// rather than of its copies (measured on the cfg-2 shapes with +-3 % ragged experts:
// forward K = 4096 136 -> 128 us, dX K = 4096 151 -> 143 us, fused backward 325 ->
// 311 us; nothing changes where no narrow tiles run).
// (Making every remainder tile narrow, whatever their number, was measured and dropped:
// level on the cfg-2 and cfg-5 shapes, 5-17 % slower on the cfg-3 ones, where 128-row
// remainders behind capacity-capped experts would stream their rows two or four times.)
constexpr int kNarrowMax = 128;
constexpr int kNarrowMinK = 2048;
constexpr int kNarrowBK = 64;
constexpr int kNarrowStages = 5;   // of a 64-row narrow tile (three slices of 64 in flight)
template <int BM, int BN, int MODE>
constexpr int narrow_factor() {
  return (BM == 256 && BN == 256 && MODE != GEMM_WGRAD) ? (is_fwd(MODE) ? 4 : 2) : 1;
}

// LDS bytes the remainder tiles of a BM x BN kernel need for their pipelines (their
// staged output tiles are smaller than the main tile's): the 64- and 128-row tiles
// of full width and, where the product has them, the narrow ones.
template <int BM, int BN, int MODE>
constexpr size_t remainder_lds_bytes() {
  if (!has_small_tiles<BM, BN, MODE>()) return 0;
  size_t need = (size_t)kSmallStages * (kSmallRows + BN) * kSmallBK * 2;
  if (BM >= 4 * kSmallRows)
    need = std::max(need, (size_t)4 * (2 * kSmallRows + BN) * kSmallBK * 2);
  constexpr int kF = narrow_factor<BM, BN, MODE>();
  if (kF > 1) {
    need = std::max(need, (size_t)4 * (2 * kSmallRows + BN / kF) * kNarrowBK * 2);
    need = std::max(need, (size_t)kNarrowStages * (kSmallRows + BN / kF) * kNarrowBK * 2);
  }
  return need;
}

// Runs the remainder tile at rows [where.m0, where.cnt) of its expert; n_tile
// counts columns in units of BN, or of BN / narrow_factor for narrow tiles.
template <typename T, int BM, int BN, int MODE>
__device__ __forceinline__ void remainder_tile(const GemmArgs& g, uint16_t* smem, TileRows where,
                                               int n_tile, bool narrow) {
  constexpr int kF = narrow_factor<BM, BN, MODE>();
  if constexpr (kF > 1) {
    if (narrow) {
      constexpr int NB = BN / kF;
      if (where.cnt - where.m0 > kSmallRows)
        gemm_tile<T, 2 * kSmallRows, NB, kNarrowBK, 2, 2, 4, MODE>(g, smem, where, n_tile * NB);
      else
        gemm_tile<T, kSmallRows, NB, kNarrowBK, 2, 2, kNarrowStages, MODE>(g, smem, where,
                                                                         n_tile * NB);
      return;
    }
  }
  if constexpr (BM >= 4 * kSmallRows) {
    if (where.cnt - where.m0 > kSmallRows) {
      gemm_tile<T, 2 * kSmallRows, BN, kSmallBK, 2, 2, 4, MODE>(g, smem, where, n_tile * BN);
      return;
    }
  }
  gemm_tile<T, kSmallRows, BN, kSmallBK, 1, 4, kSmallStages, MODE>(g, smem, where, n_tile * BN);
}

// Position of a workgroup in the order in which tiles are handed out.
// The hardware gives consecutive workgroup ids to the 8 XCDs in turn, and each
// XCD has its own L2.  The live tiles are numbered 0..live-1 so that
// neighbours share operands (tile_order()); XCD x takes the runs
// [256 j + 32 x, +32) of that numbering (shorter runs when there are fewer than
// 256 tiles), one run per round of its 32 CUs, so the blocks that share an L2
// work on a 4x8 patch and the whole chip on a 16x16 one.  Blocks past the live
// range sit at the end of the launch order and exit at once (idle blocks
// interleaved with live ones were measured to delay live blocks of the same
// XCD by a whole tile time).
__device__ __forceinline__ int tile_number(int pid, int live) {
  const int run = max(1, min(kXcdRun, (live + 7) >> 3));  // fewer than 256 tiles: spread them
  const int slot = pid >> 3;                      // position in this XCD's queue
  return (slot / run) * (8 * run) + (pid & 7) * run + slot % run;
}

// Inclusive prefix sum over the 64 lanes of a wave with data-parallel-primitive
// moves (no trips through the LDS crossbar: every workgroup runs this before its
// first copy): shifts by 1, 2, 4, 8 inside each row of 16 lanes, then lane 15 of
// rows 0 and 2 added to rows 1 and 3, then lane 31 added to rows 2 and 3.  A lane
// without a source, or outside the row mask, adds the 0 passed as the old value.
__device__ __forceinline__ int wave_inclusive_sum(int x) {
  x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false);  // row_shr:1
  x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false);  // row_shr:2
  x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false);  // row_shr:4
  x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false);  // row_shr:8
  x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false);  // row_bcast:15
  x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false);  // row_bcast:31
  return x;
}

// Row tiles of a ragged product.  The BM-row tiles of all experts are numbered
// first, one expert after the other, the remainder tiles behind them.
//
// Up to 64 experts: lane x of EVERY wave cuts the rows of expert x and a wave
// scan turns the counts into first-tile numbers, so no LDS and no barrier are
// involved and the owner of a tile is read from its lane.  More experts: each
// thread cuts the rows of a contiguous run of experts, the scan runs over the
// whole block through LDS, and the thread whose run contains a given row tile
// walks the run to find its owner.
template <int BM, bool SMALL, int NW>
struct RowTiles {
  bool by_lane;            // the up-to-64-experts scheme
  int x_lo, x_hi;          // this thread's run of experts
  int mine_f, mine_s;      // BM-row / remainder tiles in the run
  int first_f, first_s;    // number of the run's first tile of either kind
  int rows_f, rows_s;      // totals over all experts
  int my_row0, my_cnt;     // by_lane: the expert of this lane

  // May contain a __syncthreads(); s_wave_sum has 2 * NW entries.
  __device__ __forceinline__ void scan(const int32_t* seg_off, int n_expert, int* s_wave_sum) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    by_lane = n_expert <= 64;
    mine_f = mine_s = 0;
    if (by_lane) {
      x_lo = lane;
      x_hi = lane < n_expert ? lane + 1 : lane;
      my_row0 = my_cnt = 0;
      if (lane < n_expert) {
        my_row0 = seg_off[lane];
        my_cnt = seg_off[lane + 1] - my_row0;
        cut_rows<BM, SMALL>(my_cnt, mine_f, mine_s);
      }
    } else {
      const int per_thread = (n_expert + NW * 64 - 1) / (NW * 64);
      x_lo = min(tid * per_thread, n_expert);
      x_hi = min(x_lo + per_thread, n_expert);
      for (int x = x_lo; x < x_hi; ++x) {
        int f, sm;
        cut_rows<BM, SMALL>(seg_off[x + 1] - seg_off[x], f, sm);
        mine_f += f;
        mine_s += sm;
      }
    }
    // inclusive scans inside the wave
    const int incl_f = wave_inclusive_sum(mine_f);
    const int incl_s = SMALL ? wave_inclusive_sum(mine_s) : 0;
    first_f = incl_f - mine_f;
    first_s = incl_s - mine_s;
    if (by_lane) {
      rows_f = __builtin_amdgcn_readlane(incl_f, 63);
      rows_s = __builtin_amdgcn_readlane(incl_s, 63);
      return;
    }
    if (lane == 63) {
      s_wave_sum[wave] = incl_f;
      s_wave_sum[NW + wave] = incl_s;
    }
    __syncthreads();
    rows_f = rows_s = 0;
#pragma unroll
    for (int w2 = 0; w2 < NW; ++w2) {
      const int wf = s_wave_sum[w2], ws = s_wave_sum[NW + w2];
      if (w2 < wave) {
        first_f += wf;
        first_s += ws;
      }
      rows_f += wf;
      rows_s += ws;
    }
  }

  // Owner of row tile v (of the remainder kind if `small`), v below the total
  // of its kind.  s_out has 4 entries; may contain a __syncthreads().
  __device__ __forceinline__ TileRows find(const int32_t* seg_off, int v, bool small,
                                           int* s_out) const {
    const int first = small ? first_s : first_f, mine = small ? mine_s : mine_f;
    const bool own = v >= first && v < first + mine;
    TileRows t;
    if (by_lane) {
      const int owner = __ffsll((unsigned long long)__ballot(own)) - 1;  // exactly one lane
      const int at = __builtin_amdgcn_readlane(first, owner);
      const int f = __builtin_amdgcn_readlane(mine_f, owner);
      t.e = owner;
      t.m0 = small ? f * BM : (v - at) * BM;
      t.row0 = __builtin_amdgcn_readlane(my_row0, owner);
      t.cnt = __builtin_amdgcn_readlane(my_cnt, owner);
      return t;
    }
    if (own) {
      int at = first;
      for (int x = x_lo; x < x_hi; ++x) {
        const int r0 = seg_off[x], c = seg_off[x + 1] - r0;
        int f, sm;
        cut_rows<BM, SMALL>(c, f, sm);
        const int tx = small ? sm : f;
        if (v < at + tx) {
          s_out[0] = x;
          s_out[1] = small ? f * BM : (v - at) * BM;
          s_out[2] = r0;
          s_out[3] = c;
          break;
        }
        at += tx;
      }
    }
    __syncthreads();
    t.e = s_out[0];
    t.m0 = s_out[1];
    t.row0 = s_out[2];
    t.cnt = s_out[3];
    return t;
  }
};

// One of the three products.
template <typename T, int BM, int BN, int BK, int WM, int WN, int NS, int MODE>
__global__ __launch_bounds__(WM * WN * 64) void gemm_mfma_kernel(GemmArgs g,
                                                                int tiles_n,
                                                                int tiles_m) {
  constexpr int NW = WM * WN;
  constexpr bool kSmall = has_small_tiles<BM, BN, MODE>();
  static_assert(!kSmall || NW == 4, "remainder tiles put 4 waves side by side");
  extern __shared__ __attribute__((aligned(1024))) uint16_t smem[];  // [stage][A | B]
  __shared__ int s_owner[4], s_wave_sum[2 * NW];

  const int pid = blockIdx.x;
  if (MODE == GEMM_WGRAD) {
    const int live = tiles_n * tiles_m * g.n_expert;
    const int t = tile_number(pid, live);
    if (t >= live) return;
    int m_tile, n_tile;
    tile_order(t % (tiles_n * tiles_m), tiles_m, tiles_n, m_tile, n_tile);
    const int e = t / (tiles_n * tiles_m);
    const int row0 = g.seg_off[e];
    edge_aware_tile<T, BM, BN, BK, WM, WN, NS, MODE>(
        g, smem, {e, m_tile * BM, row0, g.seg_off[e + 1] - row0}, n_tile);
    return;
  }
  RowTiles<BM, kSmall, NW> rows;
  rows.scan(g.seg_off, g.n_expert, s_wave_sum);
  constexpr int kF = kSmall ? narrow_factor<BM, BN, MODE>() : 1;
  const int wide_s = rows.rows_s * tiles_n;
  const bool narrow = kF > 1 && wide_s <= kNarrowMax &&
                      (is_fwd(MODE) ? g.in_feat : g.out_feat) >= kNarrowMinK;
  const int cols_s = narrow ? tiles_n * kF : tiles_n;
  const int live_f = rows.rows_f * tiles_n, live = live_f + rows.rows_s * cols_s;
  if (live == 0) return;
  const int t = tile_number(pid, live);
  if (t >= live) return;  // the same for the whole block
  const bool small = t >= live_f;  // BM-row tiles start first: they take longer
  int v, n_tile;
  if (small) tile_order(t - live_f, rows.rows_s, cols_s, v, n_tile);
  else tile_order(t, rows.rows_f, tiles_n, v, n_tile);
  const TileRows where = rows.find(g.seg_off, v, small, s_owner);
  if constexpr (kSmall) {
    if (small) {
      remainder_tile<T, BM, BN, MODE>(g, smem, where, n_tile, narrow);
      return;
    }
  }
  edge_aware_tile<T, BM, BN, BK, WM, WN, NS, MODE>(g, smem, where, n_tile);
}

// Both gradient products of one grouped linear in one launch: the BM-row
// tiles of dX = dY W first, then the tiles of dW = dY^T X and the remainder
// tiles of dX, whichever of the two kinds takes longer first (`small_first`).
// The tail of one product overlaps the head of the next instead of leaving CUs
// idle between two launches.  gd / gw are the arguments the two products
// would get on their own.
template <typename T, int BM, int BN, int BK, int WM, int WN, int NS, bool ACT>
__global__ __launch_bounds__(WM * WN * 64) void gemm_bwd_kernel(GemmArgs gd, GemmArgs gw,
                                                               int tiles_n_d, int tiles_n_w,
                                                               int tiles_m_w, int small_first) {
  constexpr int NW = WM * WN;
  // dX with gelu' of the pre-activations applied in its tiles (gd.act_pre), or plain
  constexpr int DMODE = ACT ? GEMM_DGRAD_ACT : GEMM_DGRAD;
  constexpr bool kSmall = has_small_tiles<BM, BN, DMODE>();
  static_assert(!kSmall || NW == 4, "remainder tiles put 4 waves side by side");
  extern __shared__ __attribute__((aligned(1024))) uint16_t smem[];
  __shared__ int s_owner[4], s_wave_sum[2 * NW];

  RowTiles<BM, kSmall, NW> rows;
  rows.scan(gd.seg_off, gd.n_expert, s_wave_sum);
  constexpr int kF = kSmall ? narrow_factor<BM, BN, DMODE>() : 1;
  const bool narrow = kF > 1 && rows.rows_s * tiles_n_d <= kNarrowMax &&
                      gd.out_feat >= kNarrowMinK;
  const int cols_s = narrow ? tiles_n_d * kF : tiles_n_d;
  const int live_d = rows.rows_f * tiles_n_d, live_s = rows.rows_s * cols_s;
  const int per_expert_w = tiles_n_w * tiles_m_w;
  const int live_w = per_expert_w * gw.n_expert;
  const int live = live_d + live_w + live_s;
  if (live == 0) return;
  const int t = tile_number(blockIdx.x, live);
  if (t >= live) return;  // the same for the whole block
  // [0, live_d): dX tiles; then the dW range and the remainder range
  const int w_begin = live_d + (small_first ? live_s : 0);
  const int s_begin = live_d + (small_first ? 0 : live_w);
  if (t >= w_begin && t < w_begin + live_w) {
    const int tw = t - w_begin;
    int m_tile, n_tile;
    tile_order(tw % per_expert_w, tiles_m_w, tiles_n_w, m_tile, n_tile);
    const int e = tw / per_expert_w;
    const int row0 = gw.seg_off[e];
    edge_aware_tile<T, BM, BN, BK, WM, WN, NS, GEMM_WGRAD>(
        gw, smem, {e, m_tile * BM, row0, gw.seg_off[e + 1] - row0}, n_tile);
    return;
  }
  const bool small = t >= live_d;
  int v, n_tile;
  if (small) tile_order(t - s_begin, rows.rows_s, cols_s, v, n_tile);
  else tile_order(t, rows.rows_f, tiles_n_d, v, n_tile);
  const TileRows where = rows.find(gd.seg_off, v, small, s_owner);
  if constexpr (kSmall) {
    if (small) {
      remainder_tile<T, BM, BN, DMODE>(gd, smem, where, n_tile, narrow);
      return;
    }
  }
  edge_aware_tile<T, BM, BN, BK, WM, WN, NS, DMODE>(gd, smem, where, n_tile);
}

// ------------------------------------------------------------------ host side
template <typename T, int BM, int BN, int BK, int WM, int WN, int NS, int MODE>
static int launch_cfg(const GemmArgs& g, hipStream_t s) {
  constexpr int NW = WM * WN;
  constexpr int NT = NW * 64;
  using ATile = DmaTile<BM, BK, NW, MODE != GEMM_WGRAD>;
  using BTile = DmaTile<BN, BK, NW, is_fwd(MODE)>;
  constexpr size_t pipe_bytes = NS * (ATile::kBytes + BTile::kBytes);
  // staged output tile (+ the activation table slice of a fused epilogue behind it)
  constexpr size_t out_bytes = (size_t)BM * (BN + 8) * 2 +
      (MODE == GEMM_DGRAD_ACT || MODE == GEMM_FWD_ACT ? (size_t)kActTabBytes : 0);
  constexpr size_t small_bytes = remainder_lds_bytes<BM, BN, MODE>();
  constexpr size_t big_bytes = pipe_bytes > out_bytes ? pipe_bytes : out_bytes;
  constexpr size_t lds_bytes = big_bytes > small_bytes ? big_bytes : small_bytes;
  static_assert(lds_bytes + 1024 <= 160 * 1024, "LDS budget of a gfx950 CU");
  constexpr size_t lds_max = lds_bytes;
  constexpr size_t lds_launch = lds_max;
  auto kern = gemm_mfma_kernel<T, BM, BN, BK, WM, WN, NS, MODE>;
  FMOE_SET_DYNAMIC_LDS_ONCE(kern, lds_max);
  int tiles_n, tiles_m;
  int64_t blocks;
  if (MODE == GEMM_WGRAD) {
    tiles_n = ceil_div(g.in_feat, BN);
    tiles_m = ceil_div(g.out_feat, BM);
    blocks = (int64_t)tiles_n * tiles_m * g.n_expert;
  } else {
    tiles_n = ceil_div(is_fwd(MODE) ? g.out_feat : g.in_feat, BN);
    // at most n_rows / BM whole tiles plus, per expert, one more BM tile or
    // one remainder tile
    tiles_m = (int)(g.n_rows / BM) + g.n_expert;
    blocks = (int64_t)tiles_n * tiles_m;
    // room for the narrow form of up to kNarrowMax remainder tiles
    if (has_small_tiles<BM, BN, MODE>())
      blocks += (int64_t)(narrow_factor<BM, BN, MODE>() - 1) *
                std::min<int64_t>((int64_t)tiles_n * g.n_expert, kNarrowMax);
  }
  blocks = ceil_div(blocks, 8 * kXcdRun) * (8 * kXcdRun);  // whole runs for all 8 XCDs
  FMOE_REQUIRE(blocks < ((int64_t)1 << 31), FMOE_ERR_UNSUPPORTED,
               "grouped GEMM: too many tiles");
  if (blocks == 0) return FMOE_OK;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(NT), lds_launch, s, g,
                     tiles_n, tiles_m);
  FMOE_LAUNCH_CHECK("gemm_mfma");
  return FMOE_OK;
}

// Tile shape by a small cost model: blocks run in rounds over the CUs that
// take a block at a time (256 CUs; live tiles come first in launch order, so a
// round is really 256 wide), a tile costs a fixed prologue/epilogue
// plus a per-K-slice time that depends on its shape (measured microseconds).
// The shape with the least estimated time wins; `g.tile` overrides the choice
// for tuning (1..3 = the three shapes, 4 = 256x256 with two stages of 64).
// Ragged experts add at most one partial tile each, which the estimate ignores.
template <int MODE>
static int pick_tile(const GemmArgs& g) {
  if (g.tile >= 1 && g.tile <= 4) return g.tile;
  const int64_t N = is_fwd(MODE) ? g.out_feat : g.in_feat;
  const int64_t K = MODE == GEMM_WGRAD ? g.n_rows / g.n_expert
                                       : (is_fwd(MODE) ? g.in_feat : g.out_feat);
  auto cost = [&](int bm, int bn, double us_per_slice, int blocks_per_cu) -> double {
    const int64_t tiles = MODE == GEMM_WGRAD
        ? (int64_t)g.n_expert * ceil_div(g.out_feat, bm) * ceil_div(g.in_feat, bn)
        : (int64_t)ceil_div(g.n_rows, bm) * ceil_div(N, bn);
    const int64_t slots = 256 * blocks_per_cu;
    const double rounds = (double)((tiles + slots - 1) / slots);
    return rounds * (8.0 + (double)ceil_div(K, 32) * us_per_slice * blocks_per_cu);
  };
  const double c1 = cost(256, 256, 0.78, 1), c2 = cost(128, 256, 0.45, 1),
               c3 = cost(128, 128, 0.27, 2);
  return c1 <= c2 && c1 <= c3 ? 1 : (c2 <= c3 ? 2 : 3);
}

template <typename T, int MODE>
static int launch_mode(const GemmArgs& g, hipStream_t s) {
  switch (pick_tile<MODE>(g)) {
    case 1:
      // A [row][k] operand (both in FWD, dY in DGRAD) moves whole 128-byte
      // lines with K slices of 64: measured 7-8% faster for FWD, 2% for DGRAD;
      // WGRAD, with two [k][row] operands, is level with four stages of 32.
      if constexpr (MODE != GEMM_WGRAD) return launch_cfg<T, 256, 256, 64, 2, 2, 2, MODE>(g, s);
      else return launch_cfg<T, 256, 256, 32, 2, 2, 4, MODE>(g, s);
    case 2: return launch_cfg<T, 128, 256, 32, 2, 2, 4, MODE>(g, s);
    case 4: return launch_cfg<T, 256, 256, 64, 2, 2, 2, MODE>(g, s);
    default: return launch_cfg<T, 128, 128, 32, 2, 2, 4, MODE>(g, s);
  }
}

template <typename T>
static int launch_t(int mode, const GemmArgs& g, hipStream_t s) {
  switch (mode) {
    case GEMM_FWD:
      if constexpr (std::is_same<T, __hip_bfloat16>::value) {
        if (g.act_out) return launch_mode<T, GEMM_FWD_ACT>(g, s);
      }
      FMOE_REQUIRE(g.act_out == nullptr, FMOE_ERR_UNSUPPORTED,
                   "grouped GEMM: the fused activation is a bf16 kernel");
      return launch_mode<T, GEMM_FWD>(g, s);
    case GEMM_DGRAD:
      if constexpr (std::is_same<T, __hip_bfloat16>::value) {
        if (g.act_pre) return launch_mode<T, GEMM_DGRAD_ACT>(g, s);
      }
      FMOE_REQUIRE(g.act_pre == nullptr, FMOE_ERR_UNSUPPORTED,
                   "grouped GEMM: the fused activation is a bf16 kernel");
      return launch_mode<T, GEMM_DGRAD>(g, s);
    default: return launch_mode<T, GEMM_WGRAD>(g, s);
  }
}

// dX and dW of one linear in one launch of 256x256 tiles, K slices of BK in NS stages.
template <typename T, int BK, int NS, bool ACT = false>
static int launch_bwd_fused(const GemmArgs& gd, const GemmArgs& gw, hipStream_t s) {
  constexpr int BM = 256, BN = 256, WM = 2, WN = 2, NT = WM * WN * 64;
  constexpr size_t pipe_bytes = (size_t)NS * (BM + BN) * BK * 2;
  constexpr size_t out_bytes = (size_t)kActTabLdsOffset + kActTabBytes;
  constexpr size_t small_bytes = remainder_lds_bytes<BM, BN, GEMM_DGRAD>();
  constexpr size_t big_bytes = pipe_bytes > out_bytes ? pipe_bytes : out_bytes;
  constexpr size_t lds_bytes = big_bytes > small_bytes ? big_bytes : small_bytes;
  static_assert(lds_bytes + 1024 <= 160 * 1024, "LDS budget of a gfx950 CU");
  if (gd.act_pre) {
    if constexpr (std::is_same<T, __hip_bfloat16>::value) {
      if (!ACT) return launch_bwd_fused<T, BK, NS, true>(gd, gw, s);
    } else {
      FMOE_REQUIRE(false, FMOE_ERR_UNSUPPORTED,
                   "grouped GEMM: the fused activation is a bf16 kernel");
    }
  }
  auto kern = gemm_bwd_kernel<T, BM, BN, BK, WM, WN, NS, ACT>;
  FMOE_SET_DYNAMIC_LDS_ONCE(kern, lds_bytes);
  const int tiles_n_d = ceil_div(gd.in_feat, BN);
  const int tiles_n_w = ceil_div(gw.in_feat, BN), tiles_m_w = ceil_div(gw.out_feat, BM);
  int64_t blocks = (int64_t)tiles_n_d * (gd.n_rows / BM + (int64_t)gd.n_expert) +
                   (int64_t)tiles_n_w * tiles_m_w * gw.n_expert +
                   (int64_t)(narrow_factor<BM, BN, GEMM_DGRAD>() - 1) *
                       std::min<int64_t>((int64_t)tiles_n_d * gd.n_expert, kNarrowMax);
  blocks = ceil_div(blocks, 8 * kXcdRun) * (8 * kXcdRun);
  FMOE_REQUIRE(blocks < ((int64_t)1 << 31), FMOE_ERR_UNSUPPORTED,
               "grouped GEMM: too many tiles");
  // a remainder tile walks out_feat values of K at about 0.4 us per 32, a dW
  // tile the rows of one expert at about 0.78 us per 32 (measured)
  const int small_first =
      0.4 * gd.out_feat > 0.78 * (double)(gd.n_rows / gd.n_expert) ? 1 : 0;
  hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(NT), lds_bytes, s, gd, gw, tiles_n_d,
                     tiles_n_w, tiles_m_w, small_first);
  FMOE_LAUNCH_CHECK("gemm_bwd");
  return FMOE_OK;
}

// dX and dW in one launch when both products would use the 256x256 tiles
// anyway; otherwise one launch each.
template <typename T>
static int launch_bwd_t(const GemmArgs& gd, const GemmArgs& gw, hipStream_t s) {
  const int pd = pick_tile<GEMM_DGRAD>(gd), pw = pick_tile<GEMM_WGRAD>(gw);
  if (pd == 4 && pw == 4) return launch_bwd_fused<T, 64, 2>(gd, gw, s);  // forced
  if (pd != 1 || pw != 1) {
    const int rc = launch_t<T>(GEMM_DGRAD, gd, s);
    return rc ? rc : launch_mode<T, GEMM_WGRAD>(gw, s);
  }
  // K slices of 64 in two stages measured 2-3% faster than four stages of 32
  // when dW's K (the rows of an expert) is long, 2% slower at ~500 rows
  if (gd.tile != 1 && gd.n_rows / gd.n_expert >= 1024)
    return launch_bwd_fused<T, 64, 2>(gd, gw, s);
  return launch_bwd_fused<T, 32, 4>(gd, gw, s);
}

// The two entry points of this file, one instantiation per element type: each is
// compiled in a translation unit of its own (gemm_mfma_bf16.hip, gemm_mfma_f16.hip),
// and gemm_mfma.hip picks the one for the call's dtype.
template <typename T>
int launch_gemm_mfma_typed(int mode, const GemmArgs& g, hipStream_t s) {
  return launch_t<T>(mode, g, s);
}
template <typename T>
int launch_gemm_mfma_bwd_typed(const GemmArgs& gd, const GemmArgs& gw, hipStream_t s) {
  return launch_bwd_t<T>(gd, gw, s);
}

}  // namespace fmoe
