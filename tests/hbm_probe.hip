// Memory-system ceilings for the row movers' access patterns (scatter, gather-combine
// and their backward passes move whole rows of 2-8 KiB with a fixed ratio of rows read
// to rows written).  Independent of the library: every wave reads R pieces of 2 or 4 KiB
// (consecutive, or through a random permutation, as rows in expert order are), XORs them
// and writes W pieces; nothing else happens in the kernel.  What these loops reach is
// what the memory system gives that read:write mix, and the library's kernels are to be
// read against it.  The 2 GiB source is eight times the last-level cache; the 256 MiB
// run shows the same loops when the data stays in that cache.
//
// A second set of loops only stores: 256 x 256 tiles of 2-byte elements (256 row
// segments of 512 bytes at the row pitch of a gradient matrix, every thread one 16-byte
// pack of every eighth row: the store pattern of the grouped GEMM's output tiles), one
// tile per workgroup, against the same bytes stored as one 128 KiB run per workgroup.
// They give the time below which no kernel that writes such tiles can go.
//
//   hipcc --offload-arch=gfx950 -O3 tests/hbm_probe.hip -o /tmp/hbm_probe && /tmp/hbm_probe
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#define CK(x)                                                                  \
  do {                                                                         \
    hipError_t e_ = (x);                                                       \
    if (e_ != hipSuccess) {                                                    \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);    \
      exit(1);                                                                 \
    }                                                                          \
  } while (0)

typedef unsigned int pack_t __attribute__((ext_vector_type(4)));   // 16 bytes

// One wave per group: reads R pieces of U KiB (piece ids from idx, or consecutive),
// writes W pieces of U KiB (consecutive).  W == 0: reads only (a store that never
// happens keeps the loads alive).
template <int U, int R, int W>
__global__ void __launch_bounds__(256) mover(const pack_t* __restrict__ src,
                                             const int* __restrict__ idx,
                                             pack_t* __restrict__ dst, long n_groups) {
  const int lane = threadIdx.x & 63;
  const long g = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (g >= n_groups) return;
  pack_t p[R][U];
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const long piece = idx ? (long)idx[g * R + j] : g * R + j;
#pragma unroll
    for (int u = 0; u < U; ++u) p[j][u] = src[piece * (64 * U) + u * 64 + lane];
  }
  pack_t acc[U];
#pragma unroll
  for (int u = 0; u < U; ++u) acc[u] = p[0][u];
#pragma unroll
  for (int j = 1; j < R; ++j)
#pragma unroll
    for (int u = 0; u < U; ++u) acc[u] ^= p[j][u];
  if (W > 0) {
#pragma unroll
    for (int w = 0; w < W; ++w)
#pragma unroll
      for (int u = 0; u < U; ++u) dst[(g * W + w) * (64 * U) + u * 64 + lane] = acc[u] + w;
  } else {
    pack_t a = acc[0];
#pragma unroll
    for (int u = 1; u < U; ++u) a ^= acc[u];
    if (a.x == 0x12345678u && a.y == 0x9abcdef0u && a.z == 77u) dst[lane] = a;
  }
}

// One workgroup stores one tile: tiles_n tiles side by side, pitch = tiles_n * 512 bytes
// (tiles_n == 0: the tile as one run of 128 KiB).
__global__ void __launch_bounds__(256) tile_writer(char* __restrict__ dst, int tiles_n,
                                                   long pitch) {
  const int tid = threadIdx.x, pk = tid % 32, r0 = tid / 32;
  const long t = blockIdx.x;
  char* base = tiles_n == 0 ? dst + t * 131072
                            : dst + (t / tiles_n) * 256 * pitch + (t % tiles_n) * 512;
  const long row_bytes = tiles_n == 0 ? 512 : pitch;
  const pack_t v = {(unsigned)tid, (unsigned)t, 7u, 9u};
#pragma unroll
  for (int u = 0; u < 32; ++u)
    *reinterpret_cast<pack_t*>(base + (long)(u * 8 + r0) * row_bytes + pk * 16) = v;
}

static void run_tiles(const char* what, char* dst, long dst_bytes, int tiles_n) {
  const long pitch = tiles_n == 0 ? 512 : (long)tiles_n * 512;
  const long tiles = dst_bytes / 131072;
  // whole rows of tiles only, and nothing past the allocation
  if (tiles_n != 0 && tiles % tiles_n != 0) { printf("tile grid does not fit\n"); exit(1); }
  const long last = tiles_n == 0 ? tiles * 131072 : (tiles / tiles_n) * 256 * pitch;
  if (last > dst_bytes) { printf("tile grid past the allocation\n"); exit(1); }
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  for (int i = 0; i < 3; ++i) tile_writer<<<(int)tiles, 256>>>(dst, tiles_n, pitch);
  CK(hipEventRecord(a));
  const int iters = 20;
  for (int i = 0; i < iters; ++i) tile_writer<<<(int)tiles, 256>>>(dst, tiles_n, pitch);
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  const double us = ms * 1e3 / iters;
  printf("| %-40s | %5ld | %8.1f | %5.2f | %.3f | %5.2f |\n", what, tiles, us,
         tiles * 131072.0 / us * 1e-6, tiles * 131072.0 / us * 1e-6 / 8.0, us / (tiles / 256.0));
  fflush(stdout);
}

template <int U, int R, int W>
static void run(const char* what, const pack_t* src, const int* idx, pack_t* dst, long bytes) {
  const long piece = 1024L * U;
  const long n_groups = bytes / piece / R;
  const int grid = (int)((n_groups + 3) / 4);
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  for (int i = 0; i < 3; ++i) mover<U, R, W><<<grid, 256>>>(src, idx, dst, n_groups);
  CK(hipEventRecord(a));
  const int iters = 20;
  for (int i = 0; i < iters; ++i) mover<U, R, W><<<grid, 256>>>(src, idx, dst, n_groups);
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  const double us = ms * 1e3 / iters;
  const double moved = (double)n_groups * (R + W) * piece;
  printf("| %-46s | %d:%d | %6.0f | %8.1f | %5.2f | %.3f |\n", what, R, W, moved / 1048576.0, us,
         moved / us * 1e-6, moved / us * 1e-6 / 8.0);
  fflush(stdout);
}

int main() {
  const long big = 2048L << 20;
  pack_t *src, *dst;
  int* idx;
  CK(hipMalloc(&src, big));
  CK(hipMalloc(&dst, big));
  CK(hipMemset(src, 1, big));
  CK(hipMemset(dst, 0, big));
  std::vector<int> perm(big / 2048);
  CK(hipMalloc(&idx, perm.size() * sizeof(int)));
  std::mt19937 rng(1);
  auto permute = [&](long n) {
    for (long i = 0; i < n; ++i) perm[i] = (int)i;
    std::shuffle(perm.begin(), perm.begin() + n, rng);
    CK(hipMemcpy(idx, perm.data(), n * sizeof(int), hipMemcpyHostToDevice));
  };
  for (long bytes : {256L << 20, 2048L << 20}) {
    printf("\nsource of %ld MiB\n\n", bytes >> 20);
    printf("| pattern | reads:writes | MiB moved | us | TB/s | of 8 TB/s |\n|---|---|---|---|---|---|\n");
    run<2, 8, 0>("consecutive 2 KiB pieces, reads only", src, nullptr, dst, bytes);
    run<2, 1, 1>("consecutive 2 KiB pieces, copy", src, nullptr, dst, bytes);
    permute(bytes / 2048);
    run<2, 8, 0>("permuted 2 KiB pieces, reads only", src, idx, dst, bytes);
    run<2, 1, 1>("permuted 2 KiB pieces, copy (row scatter)", src, idx, dst, bytes);
    run<2, 2, 1>("permuted 2 KiB, 2 reads per write (combine k=2)", src, idx, dst, bytes);
    run<2, 3, 2>("permuted 2 KiB, 3 reads per 2 writes (combine bwd)", src, idx, dst, bytes);
    run<2, 8, 1>("permuted 2 KiB, 8 reads per write (combine k=8)", src, idx, dst, bytes);
    permute(bytes / 4096);
    run<4, 4, 0>("permuted 4 KiB pieces, reads only", src, idx, dst, bytes);
    run<4, 1, 1>("permuted 4 KiB pieces, copy (row scatter)", src, idx, dst, bytes);
    run<4, 2, 1>("permuted 4 KiB, 2 reads per write (combine k=2)", src, idx, dst, bytes);
    run<4, 3, 2>("permuted 4 KiB, 3 reads per 2 writes (combine bwd)", src, idx, dst, bytes);
    run<4, 8, 1>("permuted 4 KiB, 8 reads per write (combine k=8)", src, idx, dst, bytes);
  }
  printf("\nstores only, 256 x 256 tiles of 2-byte elements, one tile per workgroup\n\n");
  printf("| pattern | tiles | us | TB/s | of 8 TB/s | us per round of 256 tiles |\n|---|---|---|---|---|---|\n");
  run_tiles("128 KiB runs", (char*)dst, big, 0);
  run_tiles("tile rows at a pitch of 16 KiB (8192 columns)", (char*)dst, big, 32);
  run_tiles("tile rows at a pitch of 4 KiB (2048 columns)", (char*)dst, big, 8);
  run_tiles("tile rows at a pitch of 8 KiB (4096 columns)", (char*)dst, big, 16);
  return 0;
}
