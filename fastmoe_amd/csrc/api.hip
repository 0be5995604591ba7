// C ABI glue: error text, the expert-linear entry points (kernel selection,
// bias gradient) and the host-count upload.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

#include <algorithm>

#include "gemm.h"

namespace fmoe {

static thread_local char g_err[512] = "";
// What fmoe_set_gemm_path() selected, per calling thread (a testing aid; every
// thread starts with the automatic choice).
static thread_local int g_gemm_path = 0;   // 0 = automatic, 1 = scalar kernel only
static thread_local int g_tile = 0;        // 1..4 = one MFMA tile configuration forced
static thread_local bool g_fuse_fwd_act = true;  // false: the forward activation stays a kernel

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// ------------------------------------------------------------ bias gradient
// db[e][c] = sum over the rows of expert e of dy[r][c], fp32 accumulation
// (fp64 for doubles).  Block = 16 column groups x 16 row lanes; a thread adds
// VEC adjacent columns of every 16th row, four independent rows in flight per
// step, then the 16 row lanes meet in LDS.  HBM-bound: reads dy once.
constexpr int kBgCols = 16, kBgRows = 16, kBgUnroll = 4;
template <typename T, int VEC>
__global__ __launch_bounds__(kBgCols * kBgRows) void bias_grad_kernel(
    const T* __restrict__ dy, const int32_t* __restrict__ seg_off,
    T* __restrict__ db, int out_feat) {
  using acc_t = typename Elem<T>::acc_t;
  struct alignas(sizeof(T) * VEC) Pk { T v[VEC]; };
  __shared__ acc_t part[kBgRows][kBgCols * VEC + 1];
  const int e = blockIdx.y;
  const int cx = threadIdx.x % kBgCols, ry = threadIdx.x / kBgCols;
  const int c0 = (blockIdx.x * kBgCols + cx) * VEC;
  const int r_begin = seg_off[e], r_end = seg_off[e + 1];
  acc_t acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = 0;
  if (c0 < out_feat) {
    const T* col = dy + c0;
    int r = r_begin + ry;
    for (; r + (kBgUnroll - 1) * kBgRows < r_end; r += kBgUnroll * kBgRows) {
      Pk p[kBgUnroll];
#pragma unroll
      for (int u = 0; u < kBgUnroll; ++u)
        p[u] = *reinterpret_cast<const Pk*>(col + (int64_t)(r + u * kBgRows) * out_feat);
#pragma unroll
      for (int u = 0; u < kBgUnroll; ++u)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] += Elem<T>::to_acc(p[u].v[v]);
    }
    for (; r < r_end; r += kBgRows) {
      const Pk p = *reinterpret_cast<const Pk*>(col + (int64_t)r * out_feat);
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] += Elem<T>::to_acc(p.v[v]);
    }
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) part[ry][cx * VEC + v] = acc[v];
  __syncthreads();
  for (int c = threadIdx.x; c < kBgCols * VEC; c += kBgCols * kBgRows) {
    acc_t s = 0;
#pragma unroll
    for (int y = 0; y < kBgRows; ++y) s += part[y][c];
    const int col = blockIdx.x * kBgCols * VEC + c;
    if (col < out_feat) db[(int64_t)e * out_feat + col] = Elem<T>::from_acc(s);
  }
}

template <typename T>
static int launch_bias_grad(const void* dy, const int32_t* seg_off, void* db,
                            int out_feat, int n_expert, hipStream_t s) {
  constexpr int kVec = 16 / sizeof(T);
  const bool vec = out_feat % kVec == 0 && ((uintptr_t)dy % 16) == 0;
  if (vec) {
    dim3 grid(ceil_div(out_feat, kBgCols * kVec), n_expert);
    hipLaunchKernelGGL((bias_grad_kernel<T, kVec>), grid, dim3(kBgCols * kBgRows), 0, s,
                       (const T*)dy, seg_off, (T*)db, out_feat);
  } else {
    dim3 grid(ceil_div(out_feat, kBgCols), n_expert);
    hipLaunchKernelGGL((bias_grad_kernel<T, 1>), grid, dim3(kBgCols * kBgRows), 0, s,
                       (const T*)dy, seg_off, (T*)db, out_feat);
  }
  FMOE_LAUNCH_CHECK("bias_grad");
  return FMOE_OK;
}

// ------------------------------------------------------- host-count upload
struct OffChunk { int32_t v[512]; };
__global__ void write_offsets_kernel(OffChunk c, int32_t* dst, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = c.v[i];
}

static int check_linear(const char* who, int64_t n_rows, int64_t in_feat,
                        int64_t out_feat, int64_t n_expert, int dtype) {
  FMOE_REQUIRE(dtype_size(dtype) != 0, FMOE_ERR_INVALID, "%s: unknown dtype %d",
               who, dtype);
  FMOE_REQUIRE(n_rows >= 0 && in_feat >= 1 && out_feat >= 1 && n_expert >= 1,
               FMOE_ERR_INVALID,
               "%s: bad sizes rows=%lld in=%lld out=%lld experts=%lld", who,
               (long long)n_rows, (long long)in_feat, (long long)out_feat,
               (long long)n_expert);
  FMOE_REQUIRE(n_rows < ((int64_t)1 << 31) && in_feat < ((int64_t)1 << 31) &&
                   out_feat < ((int64_t)1 << 31) && n_expert <= 65535,
               FMOE_ERR_UNSUPPORTED, "%s: size exceeds the int32 index range", who);
  return FMOE_OK;
}

static int run_gemm(int mode, const GemmArgs& g, int dtype, hipStream_t s) {
  if (g_gemm_path == 0 && gemm_mfma_supported(mode, g, dtype))
    return launch_gemm_mfma(mode, g, dtype, s);
  if (g_gemm_path == 0 && gemm_mfma_wide_supported(mode, g, dtype))
    return launch_gemm_mfma_wide(mode, g, dtype, s);
  return launch_gemm_simt(mode, g, dtype, s);
}

}  // namespace fmoe

using namespace fmoe;

#ifndef FMOE_SOURCE_HASH
#define FMOE_SOURCE_HASH "unknown"
#endif
// the build script puts a digest of the sources behind the "fmoe-src:" marker, so
// that a loader can tell a library built from other sources without loading it
extern "C" const char* fmoe_version(void) {
  return "fastmoe_amd 0.2 (gfx950) fmoe-src:" FMOE_SOURCE_HASH;
}
extern "C" const char* fmoe_last_error(void) { return g_err; }

// One-time set-up of the current GPU, all of which the entry points otherwise do
// at their first call: the address of fmoe_route_static's built-in buffer and the
// activation tables of the 16-bit kernels (built on `stream`, waited for).
extern "C" int fmoe_init(void* stream) {
  int rc = route_static_init();
  if (rc) return rc;
  const uint16_t* fwd = nullptr;
  const float* bwd = nullptr;
  rc = gelu_fwd_table(FMOE_BF16, (hipStream_t)stream, &fwd);
  if (rc) return rc;
  return gelu_bwd_table(FMOE_BF16, (hipStream_t)stream, &bwd);
}

extern "C" int fmoe_set_gemm_path(int path) {
  FMOE_REQUIRE(path >= 0 && path <= 6, FMOE_ERR_INVALID, "gemm path must be 0..6");
  // 2..5: matrix-core kernel with tile configuration 1..4 forced; 6: automatic, but
  // the forward activation runs as a kernel of its own behind the GEMM
  g_gemm_path = path == 1 ? 1 : 0;
  g_tile = path >= 2 && path <= 5 ? path - 1 : 0;
  g_fuse_fwd_act = path != 6;
  return FMOE_OK;
}

extern "C" int fmoe_seg_off_from_host_counts(const int64_t* expert_count_host,
                                             int64_t n_expert, int32_t* seg_off,
                                             void* stream) {
  FMOE_REQUIRE(expert_count_host && seg_off && n_expert >= 1, FMOE_ERR_INVALID,
               "seg_off_from_host_counts: bad arguments");
  hipStream_t s = (hipStream_t)stream;
  // offsets travel as kernel arguments: no staging copy, nothing to keep alive
  int64_t run = 0;
  int64_t done = 0;  // entries of seg_off already written
  OffChunk chunk;
  int fill = 0;
  for (int64_t e = 0; e <= n_expert; ++e) {
    FMOE_REQUIRE(run >= 0 && run < ((int64_t)1 << 31), FMOE_ERR_INVALID,
                 "seg_off_from_host_counts: counts negative or too large");
    chunk.v[fill++] = (int32_t)run;
    if (e < n_expert) {
      FMOE_REQUIRE(expert_count_host[e] >= 0, FMOE_ERR_INVALID,
                   "seg_off_from_host_counts: negative count for expert %lld",
                   (long long)e);
      run += expert_count_host[e];
    }
    if (fill == 512 || e == n_expert) {
      hipLaunchKernelGGL(write_offsets_kernel, dim3(2), dim3(256), 0, s, chunk,
                         seg_off + done, fill);
      FMOE_LAUNCH_CHECK("write_offsets");
      done += fill;
      fill = 0;
    }
  }
  return FMOE_OK;
}

// Forward of the grouped linear layer, with the weights (and the bias) as one
// [E, ...] array or as tables of per-expert pointers, and optionally the activation
// behind it: y_act = gelu(y) from the same tiles where the bf16 matrix-core kernel
// runs, by the activation kernel over y otherwise.
static int linear_fwd(const char* who, const void* x, const void* w, const void* const* w_table,
                      const void* bias, const void* const* bias_table, const int32_t* seg_off,
                      void* y, void* y_act, bool want_act, int64_t n_rows, int64_t in_feat,
                      int64_t out_feat, int64_t n_expert, int dtype, void* stream) {
  int rc = check_linear(who, n_rows, in_feat, out_feat, n_expert, dtype);
  if (rc) return rc;
  if (n_rows == 0) return FMOE_OK;
  FMOE_REQUIRE(x && (w || w_table) && seg_off && y && (y_act || !want_act), FMOE_ERR_INVALID,
               "%s: null pointer", who);
  hipStream_t s = (hipStream_t)stream;
  GemmArgs g{x, w, y, bias, seg_off, n_rows, (int)in_feat, (int)out_feat, (int)n_expert, g_tile};
  g.w_table = w_table;
  g.bias_table = bias_table;
  if (!want_act) return run_gemm(GEMM_FWD, g, dtype, s);
  // Worth it from about 768 rows per expert on (measured: 12 % of GEMM + activation
  // kernel at 1024 rows per expert, 5 % at 4096, level at 512, where half of the tiles
  // are remainder tiles that pay the table and the second store for few rows); a
  // forced tile shape (tests, tuning) takes the fused tiles at any size.
  const bool fused = dtype == FMOE_BF16 && g_gemm_path == 0 && (uintptr_t)y_act % 16 == 0 &&
                     g_fuse_fwd_act && (g_tile != 0 || n_rows >= 768 * n_expert) &&
                     gemm_mfma_supported(GEMM_FWD, g, dtype);
  if (fused) {
    rc = gelu_fwd_table(dtype, s, &g.act_fwd_table);
    if (rc) return rc;
    g.act_out = y_act;
    return launch_gemm_mfma(GEMM_FWD, g, dtype, s);
  }
  rc = run_gemm(GEMM_FWD, g, dtype, s);
  if (rc) return rc;
  return fmoe_gelu_fwd(y, y_act, n_rows * out_feat, seg_off + n_expert, out_feat, dtype, stream);
}

extern "C" int fmoe_grouped_linear_fwd(const void* x, const void* w,
                                       const void* bias, const int32_t* seg_off,
                                       void* y, int64_t n_rows, int64_t in_feat,
                                       int64_t out_feat, int64_t n_expert,
                                       int dtype, void* stream) {
  return linear_fwd("grouped_linear_fwd", x, w, nullptr, bias, nullptr, seg_off, y, nullptr,
                    false, n_rows, in_feat, out_feat, n_expert, dtype, stream);
}

extern "C" int fmoe_grouped_linear_fwd_act(const void* x, const void* w, const void* bias,
                                           const int32_t* seg_off, void* y, void* y_act,
                                           int64_t n_rows, int64_t in_feat, int64_t out_feat,
                                           int64_t n_expert, int dtype, void* stream) {
  return linear_fwd("grouped_linear_fwd_act", x, w, nullptr, bias, nullptr, seg_off, y, y_act,
                    true, n_rows, in_feat, out_feat, n_expert, dtype, stream);
}

extern "C" int fmoe_grouped_linear_fwd_ptrs(const void* x, const void* const* w_ptrs,
                                            const void* const* bias_ptrs,
                                            const int32_t* seg_off, void* y, void* y_act,
                                            int64_t n_rows, int64_t in_feat, int64_t out_feat,
                                            int64_t n_expert, int dtype, void* stream) {
  return linear_fwd("grouped_linear_fwd_ptrs", x, nullptr, w_ptrs, nullptr, bias_ptrs, seg_off, y,
                    y_act, y_act != nullptr, n_rows, in_feat, out_feat, n_expert, dtype, stream);
}

// A device array of pointers from a host array, written by a small kernel that
// carries the values as its arguments: no staging copy, nothing to keep alive, no
// host synchronisation.
struct PtrChunk { const void* v[256]; };
__global__ void write_pointers_kernel(PtrChunk c, const void** dst, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = c.v[i];
}

extern "C" int fmoe_pointer_table(const void* const* host_ptrs, int64_t n, const void** table,
                                  void* stream) {
  FMOE_REQUIRE(host_ptrs && table && n >= 1, FMOE_ERR_INVALID, "pointer_table: bad arguments");
  hipStream_t s = (hipStream_t)stream;
  for (int64_t done = 0; done < n; done += 256) {
    PtrChunk chunk;
    const int fill = (int)std::min<int64_t>(256, n - done);
    for (int i = 0; i < fill; ++i) chunk.v[i] = host_ptrs[done + i];
    hipLaunchKernelGGL(write_pointers_kernel, dim3(1), dim3(256), 0, s, chunk, table + done, fill);
    FMOE_LAUNCH_CHECK("write_pointers");
  }
  return FMOE_OK;
}

// Backward of the grouped linear layer; with act_pre, dx is further multiplied
// by gelu'(act_pre): inside the DGRAD tiles' epilogue where the bf16 matrix-core
// kernel runs, by the activation kernel over dx otherwise.
static int linear_bwd(const void* dy, const void* x, const void* w, const void* const* w_table,
                      const int32_t* seg_off,
                      const void* act_pre, void* dx, void* dw, void* dbias, int64_t n_rows,
                      int64_t in_feat, int64_t out_feat, int64_t n_expert, int dtype,
                      void* stream) {
  int rc = check_linear("grouped_linear_bwd", n_rows, in_feat, out_feat, n_expert, dtype);
  if (rc) return rc;
  FMOE_REQUIRE(seg_off != nullptr, FMOE_ERR_INVALID,
               "grouped_linear_bwd: seg_off is null");
  FMOE_REQUIRE(n_rows == 0 || dy != nullptr, FMOE_ERR_INVALID,
               "grouped_linear_bwd: dy is null");
  hipStream_t s = (hipStream_t)stream;
  // The bf16/f16 matrix-core kernel sums the columns of dY inside its dW tiles;
  // every other kernel leaves the bias gradient to the reduction kernel below.
  GemmArgs gw{dy, x, dw, nullptr, seg_off, n_rows, (int)in_feat, (int)out_feat, (int)n_expert, g_tile};
  const bool mfma_w = dw && g_gemm_path == 0 && (n_rows == 0 || x != nullptr) &&
                      gemm_mfma_supported(GEMM_WGRAD, gw, dtype);
  if (mfma_w && dbias) {
    gw.bias = dbias;
    dbias = nullptr;  // comes out of the dW launch
  }
  GemmArgs gd{dy, w, dx, nullptr, seg_off, n_rows, (int)in_feat, (int)out_feat, (int)n_expert, g_tile};
  gd.w_table = w_table;
  void* const dx_out = dx;
  const bool act_fused = act_pre && dx && n_rows > 0 && dtype == FMOE_BF16 && g_gemm_path == 0 &&
                         (uintptr_t)act_pre % 16 == 0 && gemm_mfma_supported(GEMM_DGRAD, gd, dtype);
  if (act_fused) {
    rc = gelu_bwd_table(dtype, s, &gd.act_table);
    if (rc) return rc;
    gd.act_pre = act_pre;
  }
  if (dx && dw && n_rows > 0 && g_gemm_path == 0) {
    FMOE_REQUIRE((w != nullptr || w_table != nullptr) && x != nullptr, FMOE_ERR_INVALID,
                 "grouped_linear_bwd: w or x is null");
    if (gemm_mfma_supported(GEMM_DGRAD, gd, dtype) && mfma_w) {
      rc = launch_gemm_mfma_bwd(gd, gw, dtype, s);
      if (rc) return rc;
      dx = nullptr;  // both products are under way
      dw = nullptr;
    }
  }
  if (dx && n_rows > 0) {
    FMOE_REQUIRE(w != nullptr || w_table != nullptr, FMOE_ERR_INVALID,
                 "grouped_linear_bwd: w is null");
    rc = run_gemm(GEMM_DGRAD, gd, dtype, s);
    if (rc) return rc;
  }
  if (dw) {
    // runs also for n_rows == 0: experts without rows get zero gradients
    FMOE_REQUIRE(n_rows == 0 || x != nullptr, FMOE_ERR_INVALID,
                 "grouped_linear_bwd: x is null");
    rc = run_gemm(GEMM_WGRAD, gw, dtype, s);
    if (rc) return rc;
  }
  if (dbias) {
    switch (dtype) {
      case FMOE_F32: rc = launch_bias_grad<float>(dy, seg_off, dbias, (int)out_feat, (int)n_expert, s); break;
      case FMOE_F64: rc = launch_bias_grad<double>(dy, seg_off, dbias, (int)out_feat, (int)n_expert, s); break;
      case FMOE_F16: rc = launch_bias_grad<__half>(dy, seg_off, dbias, (int)out_feat, (int)n_expert, s); break;
      default: rc = launch_bias_grad<__hip_bfloat16>(dy, seg_off, dbias, (int)out_feat, (int)n_expert, s); break;
    }
    if (rc) return rc;
  }
  if (act_pre && !act_fused && dx_out && n_rows > 0)
    // rows of experts only: the device-side row total is the table's last entry
    return fmoe_gelu_bwd(dx_out, act_pre, dx_out, n_rows * in_feat, seg_off + n_expert, in_feat,
                         dtype, stream);
  return FMOE_OK;
}

extern "C" int fmoe_grouped_linear_bwd(const void* dy, const void* x,
                                       const void* w, const int32_t* seg_off,
                                       void* dx, void* dw, void* dbias,
                                       int64_t n_rows, int64_t in_feat,
                                       int64_t out_feat, int64_t n_expert,
                                       int dtype, void* stream) {
  return linear_bwd(dy, x, w, nullptr, seg_off, nullptr, dx, dw, dbias, n_rows, in_feat,
                    out_feat, n_expert, dtype, stream);
}

extern "C" int fmoe_grouped_linear_bwd_act(const void* dy, const void* x,
                                           const void* w, const int32_t* seg_off,
                                           const void* act_pre, void* dx, void* dw,
                                           void* dbias, int64_t n_rows, int64_t in_feat,
                                           int64_t out_feat, int64_t n_expert,
                                           int dtype, void* stream) {
  FMOE_REQUIRE(act_pre != nullptr || n_rows == 0 || dx == nullptr, FMOE_ERR_INVALID,
               "grouped_linear_bwd_act: act_pre is null");
  return linear_bwd(dy, x, w, nullptr, seg_off, act_pre, dx, dw, dbias, n_rows, in_feat,
                    out_feat, n_expert, dtype, stream);
}

extern "C" int fmoe_grouped_linear_bwd_ptrs(const void* dy, const void* x,
                                            const void* const* w_ptrs, const int32_t* seg_off,
                                            const void* act_pre, void* dx, void* dw,
                                            void* dbias, int64_t n_rows, int64_t in_feat,
                                            int64_t out_feat, int64_t n_expert,
                                            int dtype, void* stream) {
  FMOE_REQUIRE(w_ptrs != nullptr || dx == nullptr || n_rows == 0, FMOE_ERR_INVALID,
               "grouped_linear_bwd_ptrs: w_ptrs is null");
  return linear_bwd(dy, x, nullptr, w_ptrs, seg_off, act_pre, dx, dw, dbias, n_rows, in_feat,
                    out_feat, n_expert, dtype, stream);
}
