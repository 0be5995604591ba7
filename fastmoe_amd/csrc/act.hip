// GELU (the exact, erf-based one) between the two expert layers, forward and
// backward: the `activation` call of fmoe/transformer.py:28-30 when the module
// is torch.nn.GELU(), the default of FMoETransformerMLP (transformer.py:45).
//
// For 16-bit types the function has 65536 possible arguments, and 160 KB of
// LDS per CU hold the whole table: forward is one 2-byte LDS read per element
// (gelu(x), computed once per GPU in double precision and rounded once),
// backward one 4-byte read (gelu'(-|x|) in f32, which keeps the digits of the
// small values in the negative tail; gelu'(x) = 1 - gelu'(-x)) and one
// multiplication.  That leaves both passes HBM-bound, where evaluating erf
// per element (some 25 VALU instructions) does not.  f32 / f64 evaluate
// 0.5 x (1 + erf(x / sqrt 2)) directly.
#include <math.h>

#include <mutex>

#include "common.h"

namespace fmoe {
namespace {

constexpr int kActThreads = 1024;        // one block per CU (its LDS holds a table)
constexpr int kActUnroll = 4;            // 16-byte packs in flight per thread
constexpr int kTabFwd = 65536;           // entries: every 16-bit pattern
constexpr int kTabBwd = 32768;           // entries: every pattern without its sign bit

// One copy per GPU; [0] = bf16, [1] = f16.
__device__ uint16_t g_gelu_fwd_tab[2][kTabFwd];
__device__ float g_gelu_bwd_tab[2][kTabBwd];

__device__ __forceinline__ double bits_to_double(int which, uint16_t b) {
  if (which == 0) return (double)__uint_as_float((uint32_t)b << 16);
  return (double)__half2float(__ushort_as_half(b));
}
__device__ __forceinline__ uint16_t float_to_bits(int which, float v) {
  if (which == 0) return __bfloat16_as_ushort(__float2bfloat16(v));
  return __half_as_ushort(__float2half(v));
}

// gelu(x) = x Phi(x), gelu'(x) = Phi(x) + x phi(x); Phi through erfc so that the
// negative tail keeps its relative accuracy.
__device__ __forceinline__ double gelu_f64(double x) { return 0.5 * x * erfc(-x * M_SQRT1_2); }
__device__ __forceinline__ double gelu_grad_f64(double x) {
  return 0.5 * erfc(-x * M_SQRT1_2) + x * exp(-0.5 * x * x) * 0.3989422804014327;
}

__global__ void gelu_table_kernel() {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= kTabFwd) return;
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    const double x = bits_to_double(which, (uint16_t)i);
    g_gelu_fwd_tab[which][i] = float_to_bits(which, (float)gelu_f64(x));
    if (i < kTabBwd) g_gelu_bwd_tab[which][i] = (float)gelu_grad_f64(-x);
  }
}

// Elements that need work: all n, or the first *n_rows_dev rows of row_len when
// the caller knows that the rows behind them are dead (slots dropped by a
// capacity limit leave such rows at the end of the expert-ordered buffers).
__device__ __forceinline__ int64_t live_elems(int64_t n, const int32_t* n_rows_dev,
                                              int64_t row_len) {
  if (n_rows_dev == nullptr) return n;
  const int64_t live = (int64_t)*n_rows_dev * row_len;
  return live < n ? live : n;
}

// ---- 16-bit types: table in LDS ------------------------------------------
// x, y: n_packs 16-byte packs of 8 elements.
__global__ __launch_bounds__(kActThreads) void gelu_fwd_lut_kernel(
    const uint4* __restrict__ x, uint4* __restrict__ y, int64_t n_packs, int which,
    const int32_t* __restrict__ n_rows_dev, int64_t row_packs) {
  n_packs = live_elems(n_packs, n_rows_dev, row_packs);
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  uint16_t* lut = reinterpret_cast<uint16_t*>(lds_raw);
  {
    const uint4* src = reinterpret_cast<const uint4*>(g_gelu_fwd_tab[which]);
    uint4* dst = reinterpret_cast<uint4*>(lut);
    for (int i = threadIdx.x; i < kTabFwd * 2 / 16; i += kActThreads) dst[i] = src[i];
  }
  __syncthreads();
  const int64_t stride = (int64_t)gridDim.x * kActThreads;
  for (int64_t p0 = (int64_t)blockIdx.x * kActThreads + threadIdx.x; p0 < n_packs;
       p0 += stride * kActUnroll) {
    uint4 v[kActUnroll];
#pragma unroll
    for (int u = 0; u < kActUnroll; ++u)
      if (p0 + u * stride < n_packs) v[u] = x[p0 + u * stride];
#pragma unroll
    for (int u = 0; u < kActUnroll; ++u) {
      if (p0 + u * stride >= n_packs) continue;
      uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
      for (int c = 0; c < 4; ++c)
        w[c] = (uint32_t)lut[w[c] & 0xffffu] | ((uint32_t)lut[w[c] >> 16] << 16);
      y[p0 + u * stride] = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(kActThreads) void gelu_bwd_lut_kernel(
    const uint4* __restrict__ dy, const uint4* __restrict__ x, uint4* __restrict__ dx,
    int64_t n_packs, int which, const int32_t* __restrict__ n_rows_dev, int64_t row_packs) {
  n_packs = live_elems(n_packs, n_rows_dev, row_packs);
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  float* lut = reinterpret_cast<float*>(lds_raw);
  {
    const uint4* src = reinterpret_cast<const uint4*>(g_gelu_bwd_tab[which]);
    uint4* dst = reinterpret_cast<uint4*>(lut);
    for (int i = threadIdx.x; i < kTabBwd * 4 / 16; i += kActThreads) dst[i] = src[i];
  }
  __syncthreads();
  struct alignas(16) Pk { T v[8]; };
  const int64_t stride = (int64_t)gridDim.x * kActThreads;
  for (int64_t p0 = (int64_t)blockIdx.x * kActThreads + threadIdx.x; p0 < n_packs;
       p0 += stride * kActUnroll) {
    uint4 vx[kActUnroll];
    Pk vg[kActUnroll];
#pragma unroll
    for (int u = 0; u < kActUnroll; ++u)
      if (p0 + u * stride < n_packs) {
        vx[u] = x[p0 + u * stride];
        vg[u] = *reinterpret_cast<const Pk*>(dy + p0 + u * stride);
      }
#pragma unroll
    for (int u = 0; u < kActUnroll; ++u) {
      if (p0 + u * stride >= n_packs) continue;
      const uint32_t w[4] = {vx[u].x, vx[u].y, vx[u].z, vx[u].w};
      Pk o;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const uint32_t b = (c & 1) ? w[c >> 1] >> 16 : w[c >> 1] & 0xffffu;
        const float d = lut[b & 0x7fffu];
        o.v[c] = Elem<T>::from_acc(Elem<T>::to_acc(vg[u].v[c]) * ((b & 0x8000u) ? d : 1.f - d));
      }
      *reinterpret_cast<Pk*>(dx + p0 + u * stride) = o;
    }
  }
}

// ---- 16-bit tails and unaligned buffers: the same tables, from memory ------
__global__ void gelu_fwd_tab_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                    int64_t n, int which) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = g_gelu_fwd_tab[which][x[i]];
}
template <typename T>
__global__ void gelu_bwd_tab_kernel(const T* __restrict__ dy, const uint16_t* __restrict__ x,
                                    T* __restrict__ dx, int64_t n, int which) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint32_t b = x[i];
  const float d = g_gelu_bwd_tab[which][b & 0x7fffu];
  dx[i] = Elem<T>::from_acc(Elem<T>::to_acc(dy[i]) * ((b & 0x8000u) ? d : 1.f - d));
}

// ---- f32 / f64: direct evaluation ---------------------------------------------
__device__ __forceinline__ float gelu_direct(float x) {
  return 0.5f * x * (1.f + erff(x * 0.70710678118654752f));
}
__device__ __forceinline__ double gelu_direct(double x) { return gelu_f64(x); }
__device__ __forceinline__ float gelu_grad_direct(float x) {
  return 0.5f * (1.f + erff(x * 0.70710678118654752f)) +
         x * expf(-0.5f * x * x) * 0.3989422804014327f;
}
__device__ __forceinline__ double gelu_grad_direct(double x) { return gelu_grad_f64(x); }

template <typename T>
__global__ void gelu_fwd_direct_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n,
                                       const int32_t* __restrict__ n_rows_dev,
                                       int64_t row_len) {
  n = live_elems(n, n_rows_dev, row_len);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    y[i] = gelu_direct(x[i]);
}
template <typename T>
__global__ void gelu_bwd_direct_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                       T* __restrict__ dx, int64_t n,
                                       const int32_t* __restrict__ n_rows_dev,
                                       int64_t row_len) {
  n = live_elems(n, n_rows_dev, row_len);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
    dx[i] = dy[i] * gelu_grad_direct(x[i]);
}

// ---- host side ------------------------------------------------------------
constexpr int kMaxDevices = 64;
std::mutex g_setup_mutex;          // guards everything below
bool g_tables_built[kMaxDevices];
bool g_lds_configured = false;
int g_cu_count[kMaxDevices];

// Builds the tables of the current device the first time a 16-bit call reaches
// it, on `s`, and waits for them: from then on any stream may read them.  A
// first call under stream capture is refused (the tables would exist only once
// the graph has been replayed): run one eager call before capturing.
int ensure_tables(hipStream_t s, int* cu_count) {
  int dev = 0;
  FMOE_HIP_CHECK(hipGetDevice(&dev));
  FMOE_REQUIRE(dev >= 0 && dev < kMaxDevices, FMOE_ERR_UNSUPPORTED, "gelu: device %d", dev);
  std::lock_guard<std::mutex> lock(g_setup_mutex);
  if (!g_tables_built[dev]) {
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    FMOE_HIP_CHECK(hipStreamIsCapturing(s, &capture));
    FMOE_REQUIRE(capture == hipStreamCaptureStatusNone, FMOE_ERR_UNSUPPORTED,
                 "gelu: the first 16-bit call on a device builds its tables and cannot be "
                 "captured into a graph; make one eager call first");
    FMOE_HIP_CHECK(hipDeviceGetAttribute(&g_cu_count[dev], hipDeviceAttributeMultiprocessorCount,
                                         dev));
    hipLaunchKernelGGL(gelu_table_kernel, dim3(kTabFwd / 256), dim3(256), 0, s);
    FMOE_LAUNCH_CHECK("gelu_table");
    FMOE_HIP_CHECK(hipStreamSynchronize(s));
    g_tables_built[dev] = true;
  }
  if (!g_lds_configured) {
    FMOE_HIP_CHECK(hipFuncSetAttribute((const void*)gelu_fwd_lut_kernel,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kTabFwd * 2));
    FMOE_HIP_CHECK(hipFuncSetAttribute((const void*)gelu_bwd_lut_kernel<__hip_bfloat16>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kTabBwd * 4));
    FMOE_HIP_CHECK(hipFuncSetAttribute((const void*)gelu_bwd_lut_kernel<__half>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kTabBwd * 4));
    g_lds_configured = true;
  }
  *cu_count = g_cu_count[dev];
  return FMOE_OK;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

// Blocks for the table kernels: one per CU, fewer when there is less work than
// one pass of the chip.
inline int lut_blocks(int64_t n_packs, int cu_count) {
  const int64_t need = (n_packs + kActThreads * kActUnroll - 1) / (kActThreads * kActUnroll);
  return (int)(need < cu_count ? (need < 1 ? 1 : need) : cu_count);
}

inline int direct_blocks(int64_t n) {
  const int64_t b = (n + 255) / 256;
  return (int)(b > 256 * 32 ? 256 * 32 : b);
}

}  // namespace

// Device address of the gelu'(-|x|) table of a 16-bit dtype (32768 floats,
// indexed by the bit pattern without its sign), built on first use.
int gelu_bwd_table(int dtype, hipStream_t s, const float** table) {
  int cus = 0;
  const int rc = ensure_tables(s, &cus);
  if (rc) return rc;
  float* base = nullptr;
  FMOE_HIP_CHECK(hipGetSymbolAddress((void**)&base, HIP_SYMBOL(g_gelu_bwd_tab)));
  *table = base + (dtype == FMOE_BF16 ? 0 : kTabBwd);
  return FMOE_OK;
}

// Device address of the gelu(x) table of a 16-bit dtype (65536 results, indexed
// by the bit pattern of x), built on first use.
int gelu_fwd_table(int dtype, hipStream_t s, const uint16_t** table) {
  int cus = 0;
  const int rc = ensure_tables(s, &cus);
  if (rc) return rc;
  uint16_t* base = nullptr;
  FMOE_HIP_CHECK(hipGetSymbolAddress((void**)&base, HIP_SYMBOL(g_gelu_fwd_tab)));
  *table = base + (dtype == FMOE_BF16 ? 0 : kTabFwd);
  return FMOE_OK;
}

}  // namespace fmoe

using namespace fmoe;

// The live-row hint is used when whole rows are 16-byte packs; otherwise every
// element is processed (dead rows hold finite garbage or zeros, never read).
static bool rows_are_packs(const int32_t* n_rows_dev, int64_t row_len, int64_t n, int dtype) {
  return n_rows_dev != nullptr && row_len > 0 && n % row_len == 0 &&
         (row_len * (int64_t)dtype_size(dtype)) % 16 == 0;
}

extern "C" int fmoe_gelu_fwd(const void* x, void* y, int64_t n, const int32_t* n_rows_dev,
                             int64_t row_len, int dtype, void* stream) {
  FMOE_REQUIRE(dtype_size(dtype) != 0, FMOE_ERR_INVALID, "gelu_fwd: unknown dtype %d", dtype);
  FMOE_REQUIRE(n >= 0, FMOE_ERR_INVALID, "gelu_fwd: bad size %lld", (long long)n);
  if (n == 0) return FMOE_OK;
  FMOE_REQUIRE(x && y, FMOE_ERR_INVALID, "gelu_fwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (!rows_are_packs(n_rows_dev, row_len, n, dtype)) n_rows_dev = nullptr;
  if (dtype == FMOE_F32 || dtype == FMOE_F64) {
    if (dtype == FMOE_F32)
      hipLaunchKernelGGL(gelu_fwd_direct_kernel<float>, dim3(direct_blocks(n)), dim3(256), 0, s,
                         (const float*)x, (float*)y, n, n_rows_dev, row_len);
    else
      hipLaunchKernelGGL(gelu_fwd_direct_kernel<double>, dim3(direct_blocks(n)), dim3(256), 0, s,
                         (const double*)x, (double*)y, n, n_rows_dev, row_len);
    FMOE_LAUNCH_CHECK("gelu_fwd");
    return FMOE_OK;
  }
  int cus = 0;
  const int rc = ensure_tables(s, &cus);
  if (rc) return rc;
  const int which = dtype == FMOE_BF16 ? 0 : 1;
  const int64_t n_packs = aligned16(x) && aligned16(y) ? n / 8 : 0;
  if (n_packs > 0)
    hipLaunchKernelGGL(gelu_fwd_lut_kernel, dim3(lut_blocks(n_packs, cus)), dim3(kActThreads),
                       kTabFwd * 2, s, (const uint4*)x, (uint4*)y, n_packs, which, n_rows_dev,
                       row_len / 8);
  const int64_t done = n_packs * 8, rest = n - done;
  if (rest > 0)
    hipLaunchKernelGGL(gelu_fwd_tab_kernel, dim3((unsigned)((rest + 255) / 256)),
                       dim3(256), 0, s, (const uint16_t*)x + done, (uint16_t*)y + done, rest,
                       which);
  FMOE_LAUNCH_CHECK("gelu_fwd");
  return FMOE_OK;
}

extern "C" int fmoe_gelu_bwd(const void* dy, const void* x, void* dx, int64_t n,
                             const int32_t* n_rows_dev, int64_t row_len, int dtype,
                             void* stream) {
  FMOE_REQUIRE(dtype_size(dtype) != 0, FMOE_ERR_INVALID, "gelu_bwd: unknown dtype %d", dtype);
  FMOE_REQUIRE(n >= 0, FMOE_ERR_INVALID, "gelu_bwd: bad size %lld", (long long)n);
  if (n == 0) return FMOE_OK;
  FMOE_REQUIRE(dy && x && dx, FMOE_ERR_INVALID, "gelu_bwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (!rows_are_packs(n_rows_dev, row_len, n, dtype)) n_rows_dev = nullptr;
  if (dtype == FMOE_F32 || dtype == FMOE_F64) {
    if (dtype == FMOE_F32)
      hipLaunchKernelGGL(gelu_bwd_direct_kernel<float>, dim3(direct_blocks(n)), dim3(256), 0, s,
                         (const float*)dy, (const float*)x, (float*)dx, n, n_rows_dev, row_len);
    else
      hipLaunchKernelGGL(gelu_bwd_direct_kernel<double>, dim3(direct_blocks(n)), dim3(256), 0, s,
                         (const double*)dy, (const double*)x, (double*)dx, n, n_rows_dev,
                         row_len);
    FMOE_LAUNCH_CHECK("gelu_bwd");
    return FMOE_OK;
  }
  int cus = 0;
  const int rc = ensure_tables(s, &cus);
  if (rc) return rc;
  const int which = dtype == FMOE_BF16 ? 0 : 1;
  const int64_t n_packs = aligned16(dy) && aligned16(x) && aligned16(dx) ? n / 8 : 0;
  const int64_t done = n_packs * 8, rest = n - done;
  if (dtype == FMOE_BF16) {
    if (n_packs > 0)
      hipLaunchKernelGGL(gelu_bwd_lut_kernel<__hip_bfloat16>, dim3(lut_blocks(n_packs, cus)),
                         dim3(kActThreads), kTabBwd * 4, s, (const uint4*)dy, (const uint4*)x,
                         (uint4*)dx, n_packs, which, n_rows_dev, row_len / 8);
    if (rest > 0)
      hipLaunchKernelGGL(gelu_bwd_tab_kernel<__hip_bfloat16>,
                         dim3((unsigned)((rest + 255) / 256)), dim3(256), 0, s,
                         (const __hip_bfloat16*)dy + done, (const uint16_t*)x + done,
                         (__hip_bfloat16*)dx + done, rest, which);
  } else {
    if (n_packs > 0)
      hipLaunchKernelGGL(gelu_bwd_lut_kernel<__half>, dim3(lut_blocks(n_packs, cus)),
                         dim3(kActThreads), kTabBwd * 4, s, (const uint4*)dy, (const uint4*)x,
                         (uint4*)dx, n_packs, which, n_rows_dev, row_len / 8);
    if (rest > 0)
      hipLaunchKernelGGL(gelu_bwd_tab_kernel<__half>, dim3((unsigned)((rest + 255) / 256)),
                         dim3(256), 0, s, (const __half*)dy + done, (const uint16_t*)x + done,
                         (__half*)dx + done, rest, which);
  }
  FMOE_LAUNCH_CHECK("gelu_bwd");
  return FMOE_OK;
}
