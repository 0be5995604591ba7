// Byte arithmetic of the buffer descriptors that bound the grouped GEMM's
// global -> LDS copies.  Kept apart from the kernels (and free of GPU types) so
// that a host compiler can build it for a unit check of the large-shape cases.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define FMOE_HOST_DEVICE __host__ __device__
#else
#define FMOE_HOST_DEVICE
#endif

namespace fmoe {

// Offsets at or above this value are never inside a descriptor used here: a
// copy pointed there returns zeros.
constexpr uint32_t kDmaOutOfRange = 0x80000000u;

// Bytes from element (row 0, k 0) of an operand tile to the end of its valid
// data, for 2-byte elements.
//   k_contig : memory is [row][k], `ld` elements between rows, r_valid rows of
//              k_total values each;
//   otherwise: memory is [k][row], `ld` elements between consecutive k, k_total
//              rows of which r_span elements are valid.
// In the weight-gradient product k_total is the row count of an expert, so the
// result can pass 2^31 (e.g. 300000 rows x 4096 features): it is a 64-bit count.
FMOE_HOST_DEVICE inline int64_t dma_valid_bytes(bool k_contig, int r_valid, int r_span, int ld,
                                                int k_total) {
  if (k_total <= 0) return 0;
  return k_contig ? ((int64_t)(r_valid - 1) * ld + k_total) * 2
                  : ((int64_t)(k_total - 1) * ld + r_span) * 2;
}

// num_records field for `remaining` valid bytes.  Offsets inside one K-slice of
// a tile stay below 2^31 - 512 (256 rows of at most (2^31 - 512) / 512
// elements), so a count beyond 2^31 - 1 is clamped without cutting off anything
// the slice can address, and still lies below kDmaOutOfRange.
FMOE_HOST_DEVICE inline int32_t dma_num_records(int64_t remaining) {
  if (remaining <= 0) return 0;
  return remaining > 0x7fffffffLL ? 0x7fffffff : (int32_t)remaining;
}

// Largest feature size (elements between rows) the tile-relative 32-bit offsets
// allow: 256 rows x ld x 2 bytes must stay below kDmaOutOfRange.
FMOE_HOST_DEVICE inline bool dma_ld_supported(int64_t ld) {
  return ld * 512 < (int64_t)kDmaOutOfRange;
}

}  // namespace fmoe
