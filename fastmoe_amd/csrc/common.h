// Shared host/device helpers for the gfx950 MoE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <mutex>

#include "../../include/fmoe_hip.h"

namespace fmoe {

constexpr int kWave = 64;  // CDNA wavefront width

// Records the text returned by fmoe_last_error() and hands back `code`.
int set_error(int code, const char* fmt, ...);

// Per-GPU set-up of fmoe_route_static (route.hip), part of fmoe_init().
int route_static_init();

inline int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

#define FMOE_REQUIRE(cond, code, ...)                 \
  do {                                                \
    if (!(cond)) return ::fmoe::set_error((code), __VA_ARGS__); \
  } while (0)

#define FMOE_HIP_CHECK(expr)                                              \
  do {                                                                    \
    hipError_t _e = (expr);                                               \
    if (_e != hipSuccess)                                                 \
      return ::fmoe::set_error(FMOE_ERR_HIP, "%s failed: %s (%s:%d)", #expr, \
                               hipGetErrorString(_e), __FILE__, __LINE__); \
  } while (0)

// Launch check: reports configuration errors of the launch just issued.
#define FMOE_LAUNCH_CHECK(name)                                            \
  do {                                                                     \
    hipError_t _e = hipGetLastError();                                     \
    if (_e != hipSuccess)                                                  \
      return ::fmoe::set_error(FMOE_ERR_HIP, "launch of %s failed: %s", name, \
                               hipGetErrorString(_e));                     \
  } while (0)

// Raises a kernel's dynamic-LDS limit once per process (the attribute belongs to
// the function); safe when several host threads make their first call at once.
#define FMOE_SET_DYNAMIC_LDS_ONCE(kern, bytes)                                          \
  do {                                                                                  \
    static std::once_flag _once;                                                        \
    static hipError_t _once_err = hipSuccess;                                           \
    std::call_once(_once, [&] {                                                         \
      _once_err = hipFuncSetAttribute((const void*)(kern),                              \
                                      hipFuncAttributeMaxDynamicSharedMemorySize,       \
                                      (int)(bytes));                                    \
    });                                                                                 \
    FMOE_HIP_CHECK(_once_err);                                                          \
  } while (0)

inline size_t dtype_size(int dtype) {
  switch (dtype) {
    case FMOE_F32: return 4;
    case FMOE_F64: return 8;
    case FMOE_F16: return 2;
    case FMOE_BF16: return 2;
    default: return 0;
  }
}

// ---- element traits: storage type, accumulation type, conversions ----------
template <typename T> struct Elem;
template <> struct Elem<float> {
  using acc_t = float;
  __device__ static inline float to_acc(float v) { return v; }
  __device__ static inline float from_acc(float v) { return v; }
};
template <> struct Elem<double> {
  using acc_t = double;
  __device__ static inline double to_acc(double v) { return v; }
  __device__ static inline double from_acc(double v) { return v; }
};
template <> struct Elem<__half> {
  using acc_t = float;
  __device__ static inline float to_acc(__half v) { return __half2float(v); }
  __device__ static inline __half from_acc(float v) { return __float2half(v); }
};
template <> struct Elem<__hip_bfloat16> {
  using acc_t = float;
  __device__ static inline float to_acc(__hip_bfloat16 v) {
    return __bfloat162float(v);
  }
  __device__ static inline __hip_bfloat16 from_acc(float v) {
    return __float2bfloat16(v);  // round to nearest even
  }
};

// 16-byte pack of T, the unit every row-moving kernel loads and stores.
template <typename T> struct alignas(16) Pack16 {
  static constexpr int kN = 16 / sizeof(T);
  T v[kN];
};

}  // namespace fmoe
