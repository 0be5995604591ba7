// Row-moving kernels of the MoE dispatch on gfx950: scatter of token rows into
// expert order, gather back, the gather fused with the top-k weighted combine,
// its backward, and the deterministic scatter backward.
//
// All of them are HBM-bound.  One wave64 owns one row (or one token) at a time
// and moves it in 16-byte packs, so a wave issues 1 KiB per load instruction
// and consecutive lanes touch consecutive addresses.
//
// Semantics follow fmoe/functions.py:78-193 and fmoe/layers.py:281-295 of the
// reference.
#include "common.h"

namespace fmoe {

constexpr int kDispThreads = 256;
constexpr int kDispWaves = kDispThreads / kWave;
constexpr int kMaxGrid = 256 * 32;  // enough resident waves for 256 CUs

__device__ __forceinline__ int64_t live_rows(int64_t n_rows,
                                             const int32_t* n_rows_dev) {
  if (n_rows_dev == nullptr) return n_rows;
  const int64_t v = *n_rows_dev;
  return v < n_rows ? v : n_rows;
}

// ------------------------------------------------------------- plain copies
// V is an unsigned type of the widest size that divides a row.
template <typename V>
__global__ __launch_bounds__(kDispThreads) void scatter_rows_kernel(
    const V* __restrict__ inp, const int64_t* __restrict__ idx,
    V* __restrict__ out, int64_t n_rows, int64_t row_vecs, uint32_t idx_div,
    const int32_t* __restrict__ n_rows_dev) {
  const int64_t live = live_rows(n_rows, n_rows_dev);
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * kDispWaves + threadIdx.x / kWave;
  const int64_t n_waves = (int64_t)gridDim.x * kDispWaves;
  for (int64_t r = wave; r < live; r += n_waves) {
    int64_t src = idx[r];
    if (idx_div > 1) src = (int64_t)((uint32_t)src / idx_div);
    const V* s = inp + src * row_vecs;
    V* d = out + r * row_vecs;
    int64_t c = lane;
    for (; c + 3 * kWave < row_vecs; c += 4 * kWave) {
      const V a0 = s[c], a1 = s[c + kWave], a2 = s[c + 2 * kWave],
              a3 = s[c + 3 * kWave];
      d[c] = a0;
      d[c + kWave] = a1;
      d[c + 2 * kWave] = a2;
      d[c + 3 * kWave] = a3;
    }
    for (; c < row_vecs; c += kWave) d[c] = s[c];
  }
}

// out[pos[r]] = inp[r]  (rows of out not hit keep what they hold)
template <typename V>
__global__ __launch_bounds__(kDispThreads) void place_rows_kernel(
    const V* __restrict__ inp, const int64_t* __restrict__ pos,
    V* __restrict__ out, int64_t n_rows, int64_t out_rows, int64_t row_vecs,
    const int32_t* __restrict__ n_rows_dev) {
  const int64_t live = live_rows(n_rows, n_rows_dev);
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * kDispWaves + threadIdx.x / kWave;
  const int64_t n_waves = (int64_t)gridDim.x * kDispWaves;
  for (int64_t r = wave; r < live; r += n_waves) {
    const int64_t dst = pos[r];
    if (dst < 0 || dst >= out_rows) continue;
    const V* s = inp + r * row_vecs;
    V* d = out + dst * row_vecs;
    int64_t c = lane;
    for (; c + 3 * kWave < row_vecs; c += 4 * kWave) {
      const V a0 = s[c], a1 = s[c + kWave], a2 = s[c + 2 * kWave],
              a3 = s[c + 3 * kWave];
      d[c] = a0;
      d[c + kWave] = a1;
      d[c + 2 * kWave] = a2;
      d[c + 3 * kWave] = a3;
    }
    for (; c < row_vecs; c += kWave) d[c] = s[c];
  }
}

// A fill kernel rather than hipMemsetAsync, so the call can sit in a HIP graph.
__global__ __launch_bounds__(kDispThreads) void zero_fill_kernel(
    uint4* __restrict__ p16, int64_t n16, unsigned char* __restrict__ tail,
    int64_t n_tail) {
  const int64_t stride = (int64_t)gridDim.x * kDispThreads;
  const int64_t t = (int64_t)blockIdx.x * kDispThreads + threadIdx.x;
  const uint4 z = make_uint4(0, 0, 0, 0);
  for (int64_t i = t; i < n16; i += stride) p16[i] = z;
  for (int64_t i = t; i < n_tail; i += stride) tail[i] = 0;
}

// out[pos[r]] += inp[r] with device float atomics (f32 / f64 only).
template <typename T>
__global__ __launch_bounds__(kDispThreads) void add_rows_kernel(
    const T* __restrict__ inp, const int64_t* __restrict__ pos,
    T* __restrict__ out, int64_t n_rows, int64_t out_rows, int64_t d,
    const int32_t* __restrict__ n_rows_dev) {
  const int64_t live = live_rows(n_rows, n_rows_dev);
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * kDispWaves + threadIdx.x / kWave;
  const int64_t n_waves = (int64_t)gridDim.x * kDispWaves;
  for (int64_t r = wave; r < live; r += n_waves) {
    const int64_t dst = pos[r];
    if (dst < 0 || dst >= out_rows) continue;
    for (int64_t c = lane; c < d; c += kWave)
      atomicAdd(&out[dst * d + c], inp[r * d + c]);
  }
}

// Value held by lane j (wave-uniform j), readable also when lane j itself is
// masked off in the current branch: v_readlane ignores EXEC.
__device__ __forceinline__ int32_t lane_value(int32_t v, int j) {
  return __builtin_amdgcn_readlane(v, j);
}
__device__ __forceinline__ float lane_value(float v, int j) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), j));
}
__device__ __forceinline__ double lane_value(double v, int j) {
  const long long b = __double_as_longlong(v);
  const int lo = __builtin_amdgcn_readlane((int)(b & 0xffffffffLL), j);
  const int hi = __builtin_amdgcn_readlane((int)(b >> 32), j);
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// ------------------------------------------------ gather fused with combine
// y[t] = sum_j score[t,j] * buf[inv[t,j]]; score == nullptr means weight 1
// (the scatter backward).  VEC elements per lane per step (16 bytes, or 1).
//
// SPLIT waves share a token, each taking a contiguous 1/SPLIT of the row, and a
// lane has UNROLL packs of a source row in flight.  The host picks both so
// that a wave holds 2 to 4 packs per lane of each row: measured on rows of
// 8 KiB, one wave per token reaches 0.60-0.66 of the HBM peak, four waves 0.75+;
// short rows (2 KiB) do best with one wave and 2 packs per lane.
template <typename T, int VEC, int SPLIT, int UNROLL>
__global__ __launch_bounds__(kDispThreads) void combine_fwd_kernel(
    const T* __restrict__ buf, const int32_t* __restrict__ inv,
    const T* __restrict__ score, T* __restrict__ y, int64_t n_tokens, int top_k,
    int64_t d) {
  using acc_t = typename Elem<T>::acc_t;
  struct alignas(sizeof(T) * VEC) Pk { T v[VEC]; };
  constexpr int kTokPerBlock = kDispWaves / SPLIT;
  const int lane = threadIdx.x & (kWave - 1);
  const int w = threadIdx.x / kWave;
  const int part = w % SPLIT;
  const int64_t row_vecs = d / VEC;
  // packs [c_begin, c_end) of the row are this wave's
  const int64_t per_part = (row_vecs + SPLIT * kWave - 1) / (SPLIT * kWave) * kWave;
  const int64_t c_begin = part * per_part;
  const int64_t c_end = c_begin + per_part < row_vecs ? c_begin + per_part : row_vecs;
  const int64_t n_groups = (n_tokens + kTokPerBlock - 1) / kTokPerBlock;
  for (int64_t tg = blockIdx.x; tg < n_groups; tg += gridDim.x) {
    const int64_t t = tg * kTokPerBlock + w / SPLIT;
    if (t >= n_tokens) continue;
    // lane j keeps the row and weight of slot j
    int32_t my_r = -1;
    acc_t my_s = 0;
    if (lane < top_k) {
      my_r = inv[t * top_k + lane];
      my_s = score ? Elem<T>::to_acc(score[t * top_k + lane]) : (acc_t)1;
    }
    // UNROLL packs per lane per step: all their loads are issued before the
    // first is used
    for (int64_t c0 = c_begin + lane; c0 < c_end; c0 += kWave * UNROLL) {
      acc_t acc[UNROLL][VEC];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[u][v] = 0;
      for (int j = 0; j < top_k; ++j) {
        // lanes beyond the row's last pack are not in this loop, so a
        // shuffle could not read them; lane_value can
        const int32_t r = lane_value(my_r, j);
        const acc_t s = lane_value(my_s, j);
        if (r < 0) continue;
        const T* src = buf + (int64_t)r * d;
        Pk p[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const int64_t c = c0 + (int64_t)u * kWave;
          if (c < c_end) p[u] = *reinterpret_cast<const Pk*>(src + c * VEC);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
          for (int v = 0; v < VEC; ++v) acc[u][v] += s * Elem<T>::to_acc(p[u].v[v]);
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int64_t c = c0 + (int64_t)u * kWave;
        if (c < c_end) {
          Pk o;
#pragma unroll
          for (int v = 0; v < VEC; ++v) o.v[v] = Elem<T>::from_acc(acc[u][v]);
          *reinterpret_cast<Pk*>(y + t * d + c * VEC) = o;
        }
      }
    }
  }
}

// dbuf[inv[i]] = score[i] * dy[i/k];  dscore[i] = <dy[i/k], buf[inv[i]]>
// The SPLIT waves of a token meet in LDS with their parts of the dot products
// (summed in a fixed order: the result does not depend on timing).
template <typename T, int VEC, int SPLIT, int UNROLL>
__global__ __launch_bounds__(kDispThreads) void combine_bwd_kernel(
    const T* __restrict__ dy, const T* __restrict__ buf,
    const int32_t* __restrict__ inv, const T* __restrict__ score,
    T* __restrict__ dbuf, T* __restrict__ dscore, int64_t n_tokens, int top_k,
    int64_t d) {
  using acc_t = typename Elem<T>::acc_t;
  struct alignas(sizeof(T) * VEC) Pk { T v[VEC]; };
  constexpr int kTokPerBlock = kDispWaves / SPLIT;
  __shared__ acc_t part_dot[SPLIT > 1 ? kDispWaves : 1][SPLIT > 1 ? kWave : 1];
  const int lane = threadIdx.x & (kWave - 1);
  const int w = threadIdx.x / kWave;
  const int part = w % SPLIT;
  const int64_t row_vecs = d / VEC;
  const int64_t per_part = (row_vecs + SPLIT * kWave - 1) / (SPLIT * kWave) * kWave;
  const int64_t c_begin = part * per_part;
  const int64_t c_end = c_begin + per_part < row_vecs ? c_begin + per_part : row_vecs;
  const int64_t n_groups = (n_tokens + kTokPerBlock - 1) / kTokPerBlock;
  for (int64_t tg = blockIdx.x; tg < n_groups; tg += gridDim.x) {
    const int64_t t = tg * kTokPerBlock + w / SPLIT;
    const bool live = t < n_tokens;
    int32_t my_r = -1;
    acc_t my_s = 0;
    if (live && lane < top_k) {
      my_r = inv[t * top_k + lane];
      my_s = Elem<T>::to_acc(score[t * top_k + lane]);
    }
    acc_t my_dot = 0;   // lane j ends up holding this wave's part of slot j's dot product
    for (int j = 0; j < top_k; ++j) {
      const int32_t r = lane_value(my_r, j);
      const acc_t s = lane_value(my_s, j);
      acc_t dot = 0;
      if (r >= 0) {
        for (int64_t c0 = c_begin + lane; c0 < c_end; c0 += kWave * UNROLL) {
          Pk g[UNROLL], o[UNROLL];
#pragma unroll
          for (int u = 0; u < UNROLL; ++u) {
            const int64_t c = c0 + (int64_t)u * kWave;
            if (c < c_end) {
              g[u] = *reinterpret_cast<const Pk*>(dy + t * d + c * VEC);
              o[u] = *reinterpret_cast<const Pk*>(buf + (int64_t)r * d + c * VEC);
            }
          }
#pragma unroll
          for (int u = 0; u < UNROLL; ++u) {
            const int64_t c = c0 + (int64_t)u * kWave;
            if (c < c_end) {
              Pk wv;
#pragma unroll
              for (int v = 0; v < VEC; ++v) {
                const acc_t gv = Elem<T>::to_acc(g[u].v[v]);
                dot += gv * Elem<T>::to_acc(o[u].v[v]);
                wv.v[v] = Elem<T>::from_acc(s * gv);
              }
              *reinterpret_cast<Pk*>(dbuf + (int64_t)r * d + c * VEC) = wv;
            }
          }
        }
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1)
          dot += __shfl_xor(dot, off, kWave);
      }
      if (lane == j) my_dot = dot;
    }
    if (SPLIT == 1) {
      if (live && lane < top_k) dscore[t * top_k + lane] = Elem<T>::from_acc(my_dot);
    } else {
      part_dot[w][lane] = my_dot;
      __syncthreads();
      if (live && part == 0 && lane < top_k) {
        acc_t total = 0;
#pragma unroll
        for (int q = 0; q < SPLIT; ++q) total += part_dot[w + q][lane];
        dscore[t * top_k + lane] = Elem<T>::from_acc(total);
      }
      __syncthreads();
    }
  }
}

// out[inv[t * k + j]] = inp[t] for every live slot of token t: the scatter in
// token order.  A token row is read once and written k times, where the
// row-ordered scatter reads it k times at k distant moments (with k = 8 most of
// those reads miss L2).  One wave per token; lane j < k holds the row of slot j.
template <typename V>
__global__ __launch_bounds__(kDispThreads) void scatter_tokens_kernel(
    const V* __restrict__ inp, const int32_t* __restrict__ inv, V* __restrict__ out,
    int64_t n_tokens, int top_k, int64_t row_vecs) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (int64_t)blockIdx.x * kDispWaves + threadIdx.x / kWave;
  const int64_t n_waves = (int64_t)gridDim.x * kDispWaves;
  for (int64_t t = wave; t < n_tokens; t += n_waves) {
    const int32_t my_r = lane < top_k ? inv[t * top_k + lane] : -1;
    const V* s = inp + t * row_vecs;
    for (int64_t c0 = lane; c0 < row_vecs; c0 += 4 * kWave) {
      V a[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (c0 + u * kWave < row_vecs) a[u] = s[c0 + u * kWave];
      for (int j = 0; j < top_k; ++j) {
        const int32_t r = lane_value(my_r, j);
        if (r < 0) continue;  // dropped slot (the same for the whole wave)
        V* d = out + (int64_t)r * row_vecs;
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (c0 + u * kWave < row_vecs) d[c0 + u * kWave] = a[u];
      }
    }
  }
}

// ----------------------------------------------------------------- host side
static int grid_for_rows(int64_t rows) {
  int64_t blocks = (rows + kDispWaves - 1) / kDispWaves;
  if (blocks < 1) blocks = 1;
  if (blocks > kMaxGrid) blocks = kMaxGrid;
  return (int)blocks;
}

static inline bool aligned(const void* p, size_t a) {
  return ((uintptr_t)p % a) == 0;
}

// widest unit (16/8/4/2 bytes) dividing the row and aligned at both bases
static int copy_unit(const void* a, const void* b, int64_t row_bytes) {
  const int units[4] = {16, 8, 4, 2};
  for (int u : units)
    if (row_bytes % u == 0 && aligned(a, u) && aligned(b, u)) return u;
  return 1;
}

// How many waves share a token (SPLIT) and how many packs of a row a lane has
// in flight (UNROLL) for rows of `row_vecs` packs: 2 to 4 packs per lane per wave.
static void combine_shape(int64_t row_vecs, int* split, int* unroll) {
  *split = row_vecs >= 8 * kWave ? 4 : (row_vecs >= 4 * kWave ? 2 : 1);
  const int64_t per_lane = (row_vecs + *split * kWave - 1) / (*split * kWave);
  *unroll = per_lane >= 4 ? 4 : (per_lane >= 2 ? 2 : 1);
}

static int grid_for_groups(int64_t n_tokens, int split) {
  const int per_block = kDispWaves / split;
  int64_t blocks = (n_tokens + per_block - 1) / per_block;
  if (blocks < 1) blocks = 1;
  if (blocks > kMaxGrid * 4) blocks = kMaxGrid * 4;
  return (int)blocks;
}

#define FMOE_COMBINE_DISPATCH(KERNEL, ...)                                               \
  do {                                                                                   \
    if (!vec) {                                                                          \
      hipLaunchKernelGGL((KERNEL<T, 1, 1, 4>), dim3(grid_for_groups(n_tokens, 1)),       \
                         dim3(kDispThreads), 0, s, __VA_ARGS__);                         \
      break;                                                                             \
    }                                                                                    \
    int split, unroll;                                                                   \
    combine_shape(d / kVec, &split, &unroll);                                            \
    const dim3 grid(grid_for_groups(n_tokens, split));                                   \
    if (split == 4 && unroll == 4)                                                       \
      hipLaunchKernelGGL((KERNEL<T, kVec, 4, 4>), grid, dim3(kDispThreads), 0, s, __VA_ARGS__); \
    else if (split == 4)                                                                 \
      hipLaunchKernelGGL((KERNEL<T, kVec, 4, 2>), grid, dim3(kDispThreads), 0, s, __VA_ARGS__); \
    else if (split == 2 && unroll == 4)                                                  \
      hipLaunchKernelGGL((KERNEL<T, kVec, 2, 4>), grid, dim3(kDispThreads), 0, s, __VA_ARGS__); \
    else if (split == 2)                                                                 \
      hipLaunchKernelGGL((KERNEL<T, kVec, 2, 2>), grid, dim3(kDispThreads), 0, s, __VA_ARGS__); \
    else if (unroll == 4)                                                                \
      hipLaunchKernelGGL((KERNEL<T, kVec, 1, 4>), grid, dim3(kDispThreads), 0, s, __VA_ARGS__); \
    else if (unroll == 2)                                                                \
      hipLaunchKernelGGL((KERNEL<T, kVec, 1, 2>), grid, dim3(kDispThreads), 0, s, __VA_ARGS__); \
    else                                                                                 \
      hipLaunchKernelGGL((KERNEL<T, kVec, 1, 1>), grid, dim3(kDispThreads), 0, s, __VA_ARGS__); \
  } while (0)

template <typename T>
static int launch_combine_fwd(const void* buf, const int32_t* inv,
                              const void* score, void* y, int64_t n_tokens,
                              int top_k, int64_t d, hipStream_t s) {
  constexpr int kVec = 16 / sizeof(T);
  const bool vec = d % kVec == 0 && aligned(buf, 16) && aligned(y, 16);
  FMOE_COMBINE_DISPATCH(combine_fwd_kernel, (const T*)buf, inv, (const T*)score, (T*)y, n_tokens,
                        top_k, d);
  FMOE_LAUNCH_CHECK("combine_fwd");
  return FMOE_OK;
}

template <typename T>
static int launch_combine_bwd(const void* dy, const void* buf,
                              const int32_t* inv, const void* score, void* dbuf,
                              void* dscore, int64_t n_tokens, int top_k,
                              int64_t d, hipStream_t s) {
  constexpr int kVec = 16 / sizeof(T);
  const bool vec = d % kVec == 0 && aligned(buf, 16) && aligned(dy, 16) &&
                   aligned(dbuf, 16);
  FMOE_COMBINE_DISPATCH(combine_bwd_kernel, (const T*)dy, (const T*)buf, inv, (const T*)score,
                        (T*)dbuf, (T*)dscore, n_tokens, top_k, d);
  FMOE_LAUNCH_CHECK("combine_bwd");
  return FMOE_OK;
}

static int zero_fill(void* p, int64_t bytes, hipStream_t s) {
  if (bytes <= 0) return FMOE_OK;
  // p comes from an allocator that aligns to >= 16; fall back to bytes if not
  int64_t n16 = aligned(p, 16) ? bytes / 16 : 0;
  int64_t n_tail = bytes - n16 * 16;
  int64_t work = n16 > n_tail ? n16 : n_tail;
  int64_t blocks = (work + kDispThreads - 1) / kDispThreads;
  if (blocks > kMaxGrid) blocks = kMaxGrid;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(zero_fill_kernel, dim3((int)blocks), dim3(kDispThreads), 0,
                     s, (uint4*)p, n16, (unsigned char*)p + n16 * 16, n_tail);
  FMOE_LAUNCH_CHECK("zero_fill");
  return FMOE_OK;
}

}  // namespace fmoe

using namespace fmoe;

extern "C" int fmoe_local_scatter(const void* inp, const int64_t* idx, void* out,
                                  int64_t n_rows, int64_t d, int64_t idx_div,
                                  const int32_t* n_rows_dev, int dtype,
                                  void* stream) {
  const int64_t es = (int64_t)dtype_size(dtype);
  FMOE_REQUIRE(es != 0, FMOE_ERR_INVALID, "local_scatter: unknown dtype %d", dtype);
  FMOE_REQUIRE(n_rows >= 0 && d >= 0 && idx_div >= 1, FMOE_ERR_INVALID,
               "local_scatter: bad sizes rows=%lld d=%lld div=%lld",
               (long long)n_rows, (long long)d, (long long)idx_div);
  FMOE_REQUIRE(idx_div < ((int64_t)1 << 31), FMOE_ERR_UNSUPPORTED,
               "local_scatter: idx_div too large");
  if (n_rows == 0 || d == 0) return FMOE_OK;
  FMOE_REQUIRE(inp && idx && out, FMOE_ERR_INVALID, "local_scatter: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const int64_t row_bytes = d * es;
  const int grid = grid_for_rows(n_rows);
  const uint32_t div = (uint32_t)idx_div;
  switch (copy_unit(inp, out, row_bytes)) {
    case 16:
      hipLaunchKernelGGL(scatter_rows_kernel<uint4>, dim3(grid), dim3(kDispThreads),
                         0, s, (const uint4*)inp, idx, (uint4*)out, n_rows,
                         row_bytes / 16, div, n_rows_dev);
      break;
    case 8:
      hipLaunchKernelGGL(scatter_rows_kernel<uint64_t>, dim3(grid),
                         dim3(kDispThreads), 0, s, (const uint64_t*)inp, idx,
                         (uint64_t*)out, n_rows, row_bytes / 8, div, n_rows_dev);
      break;
    case 4:
      hipLaunchKernelGGL(scatter_rows_kernel<uint32_t>, dim3(grid),
                         dim3(kDispThreads), 0, s, (const uint32_t*)inp, idx,
                         (uint32_t*)out, n_rows, row_bytes / 4, div, n_rows_dev);
      break;
    default:
      hipLaunchKernelGGL(scatter_rows_kernel<uint16_t>, dim3(grid),
                         dim3(kDispThreads), 0, s, (const uint16_t*)inp, idx,
                         (uint16_t*)out, n_rows, row_bytes / 2, div, n_rows_dev);
      break;
  }
  FMOE_LAUNCH_CHECK("local_scatter");
  return FMOE_OK;
}

extern "C" int fmoe_scatter_tokens(const void* inp, const int32_t* inv, void* out,
                                   int64_t n_tokens, int64_t top_k, int64_t d, int dtype,
                                   void* stream) {
  const int64_t es = (int64_t)dtype_size(dtype);
  FMOE_REQUIRE(es != 0, FMOE_ERR_INVALID, "scatter_tokens: unknown dtype %d", dtype);
  FMOE_REQUIRE(n_tokens >= 0 && d >= 0 && top_k >= 1, FMOE_ERR_INVALID,
               "scatter_tokens: bad sizes tokens=%lld d=%lld top_k=%lld", (long long)n_tokens,
               (long long)d, (long long)top_k);
  FMOE_REQUIRE(top_k <= kWave, FMOE_ERR_UNSUPPORTED, "scatter_tokens: top_k %lld exceeds %d",
               (long long)top_k, kWave);
  if (n_tokens == 0 || d == 0) return FMOE_OK;
  FMOE_REQUIRE(inp && inv && out, FMOE_ERR_INVALID, "scatter_tokens: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const int64_t row_bytes = d * es;
  const int grid = grid_for_rows(n_tokens);
  switch (copy_unit(inp, out, row_bytes)) {
    case 16:
      hipLaunchKernelGGL(scatter_tokens_kernel<uint4>, dim3(grid), dim3(kDispThreads), 0, s,
                         (const uint4*)inp, inv, (uint4*)out, n_tokens, (int)top_k,
                         row_bytes / 16);
      break;
    case 8:
      hipLaunchKernelGGL(scatter_tokens_kernel<uint64_t>, dim3(grid), dim3(kDispThreads), 0, s,
                         (const uint64_t*)inp, inv, (uint64_t*)out, n_tokens, (int)top_k,
                         row_bytes / 8);
      break;
    case 4:
      hipLaunchKernelGGL(scatter_tokens_kernel<uint32_t>, dim3(grid), dim3(kDispThreads), 0, s,
                         (const uint32_t*)inp, inv, (uint32_t*)out, n_tokens, (int)top_k,
                         row_bytes / 4);
      break;
    default:
      hipLaunchKernelGGL(scatter_tokens_kernel<uint16_t>, dim3(grid), dim3(kDispThreads), 0, s,
                         (const uint16_t*)inp, inv, (uint16_t*)out, n_tokens, (int)top_k,
                         row_bytes / 2);
      break;
  }
  FMOE_LAUNCH_CHECK("scatter_tokens");
  return FMOE_OK;
}

extern "C" int fmoe_local_gather(const void* inp, const int64_t* pos, void* out,
                                 int64_t n_rows, int64_t out_rows, int64_t d,
                                 const int32_t* n_rows_dev, int overlap,
                                 int dtype, void* stream) {
  const int64_t es = (int64_t)dtype_size(dtype);
  FMOE_REQUIRE(es != 0, FMOE_ERR_INVALID, "local_gather: unknown dtype %d", dtype);
  FMOE_REQUIRE(n_rows >= 0 && out_rows >= 0 && d >= 0, FMOE_ERR_INVALID,
               "local_gather: negative size");
  FMOE_REQUIRE(!overlap || dtype == FMOE_F32 || dtype == FMOE_F64,
               FMOE_ERR_UNSUPPORTED,
               "local_gather: overlapping rows need f32 or f64");
  if (out_rows == 0 || d == 0) return FMOE_OK;
  FMOE_REQUIRE(out != nullptr, FMOE_ERR_INVALID, "local_gather: null output");
  hipStream_t s = (hipStream_t)stream;
  int rc = zero_fill(out, out_rows * d * es, s);
  if (rc) return rc;
  if (n_rows == 0) return FMOE_OK;
  FMOE_REQUIRE(inp && pos, FMOE_ERR_INVALID, "local_gather: null pointer");
  const int grid = grid_for_rows(n_rows);
  if (overlap) {
    if (dtype == FMOE_F32)
      hipLaunchKernelGGL(add_rows_kernel<float>, dim3(grid), dim3(kDispThreads), 0,
                         s, (const float*)inp, pos, (float*)out, n_rows, out_rows,
                         d, n_rows_dev);
    else
      hipLaunchKernelGGL(add_rows_kernel<double>, dim3(grid), dim3(kDispThreads),
                         0, s, (const double*)inp, pos, (double*)out, n_rows,
                         out_rows, d, n_rows_dev);
    FMOE_LAUNCH_CHECK("local_gather(add)");
    return FMOE_OK;
  }
  const int64_t row_bytes = d * es;
  switch (copy_unit(inp, out, row_bytes)) {
    case 16:
      hipLaunchKernelGGL(place_rows_kernel<uint4>, dim3(grid), dim3(kDispThreads),
                         0, s, (const uint4*)inp, pos, (uint4*)out, n_rows,
                         out_rows, row_bytes / 16, n_rows_dev);
      break;
    case 8:
      hipLaunchKernelGGL(place_rows_kernel<uint64_t>, dim3(grid),
                         dim3(kDispThreads), 0, s, (const uint64_t*)inp, pos,
                         (uint64_t*)out, n_rows, out_rows, row_bytes / 8,
                         n_rows_dev);
      break;
    case 4:
      hipLaunchKernelGGL(place_rows_kernel<uint32_t>, dim3(grid),
                         dim3(kDispThreads), 0, s, (const uint32_t*)inp, pos,
                         (uint32_t*)out, n_rows, out_rows, row_bytes / 4,
                         n_rows_dev);
      break;
    default:
      hipLaunchKernelGGL(place_rows_kernel<uint16_t>, dim3(grid),
                         dim3(kDispThreads), 0, s, (const uint16_t*)inp, pos,
                         (uint16_t*)out, n_rows, out_rows, row_bytes / 2,
                         n_rows_dev);
      break;
  }
  FMOE_LAUNCH_CHECK("local_gather");
  return FMOE_OK;
}

static int check_combine(const char* who, int64_t n_tokens, int64_t top_k,
                         int64_t d, int dtype) {
  FMOE_REQUIRE(dtype_size(dtype) != 0, FMOE_ERR_INVALID, "%s: unknown dtype %d",
               who, dtype);
  FMOE_REQUIRE(n_tokens >= 0 && d >= 0, FMOE_ERR_INVALID, "%s: negative size", who);
  FMOE_REQUIRE(top_k >= 1 && top_k <= kWave, FMOE_ERR_UNSUPPORTED,
               "%s: top_k %lld outside [1, 64]", who, (long long)top_k);
  return FMOE_OK;
}

extern "C" int fmoe_gather_combine_fwd(const void* buf, const int32_t* inv,
                                       const void* score, void* y,
                                       int64_t n_tokens, int64_t top_k,
                                       int64_t d, int dtype, void* stream) {
  int rc = check_combine("gather_combine_fwd", n_tokens, top_k, d, dtype);
  if (rc) return rc;
  if (n_tokens == 0 || d == 0) return FMOE_OK;
  FMOE_REQUIRE(inv && score && y, FMOE_ERR_INVALID,
               "gather_combine_fwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case FMOE_F32: return launch_combine_fwd<float>(buf, inv, score, y, n_tokens, (int)top_k, d, s);
    case FMOE_F64: return launch_combine_fwd<double>(buf, inv, score, y, n_tokens, (int)top_k, d, s);
    case FMOE_F16: return launch_combine_fwd<__half>(buf, inv, score, y, n_tokens, (int)top_k, d, s);
    default: return launch_combine_fwd<__hip_bfloat16>(buf, inv, score, y, n_tokens, (int)top_k, d, s);
  }
}

extern "C" int fmoe_scatter_reduce(const void* dbuf, const int32_t* inv, void* dx,
                                   int64_t n_tokens, int64_t top_k, int64_t d,
                                   int dtype, void* stream) {
  int rc = check_combine("scatter_reduce", n_tokens, top_k, d, dtype);
  if (rc) return rc;
  if (n_tokens == 0 || d == 0) return FMOE_OK;
  FMOE_REQUIRE(inv && dx, FMOE_ERR_INVALID, "scatter_reduce: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case FMOE_F32: return launch_combine_fwd<float>(dbuf, inv, nullptr, dx, n_tokens, (int)top_k, d, s);
    case FMOE_F64: return launch_combine_fwd<double>(dbuf, inv, nullptr, dx, n_tokens, (int)top_k, d, s);
    case FMOE_F16: return launch_combine_fwd<__half>(dbuf, inv, nullptr, dx, n_tokens, (int)top_k, d, s);
    default: return launch_combine_fwd<__hip_bfloat16>(dbuf, inv, nullptr, dx, n_tokens, (int)top_k, d, s);
  }
}

extern "C" int fmoe_gather_combine_bwd(const void* dy, const void* buf,
                                       const int32_t* inv, const void* score,
                                       void* dbuf, void* dscore,
                                       int64_t n_tokens, int64_t top_k,
                                       int64_t d, int dtype, void* stream) {
  int rc = check_combine("gather_combine_bwd", n_tokens, top_k, d, dtype);
  if (rc) return rc;
  if (n_tokens == 0) return FMOE_OK;
  FMOE_REQUIRE(dy && inv && score && dscore, FMOE_ERR_INVALID,
               "gather_combine_bwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case FMOE_F32: return launch_combine_bwd<float>(dy, buf, inv, score, dbuf, dscore, n_tokens, (int)top_k, d, s);
    case FMOE_F64: return launch_combine_bwd<double>(dy, buf, inv, score, dbuf, dscore, n_tokens, (int)top_k, d, s);
    case FMOE_F16: return launch_combine_bwd<__half>(dy, buf, inv, score, dbuf, dscore, n_tokens, (int)top_k, d, s);
    default: return launch_combine_bwd<__hip_bfloat16>(dy, buf, inv, score, dbuf, dscore, n_tokens, (int)top_k, d, s);
  }
}
