// Shared host/device helpers for libmedvision_hip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/medvision_hip.h"

namespace mv {

// ---- error reporting -------------------------------------------------------------------
char *last_error_buffer();
int fail(int status, const char *fmt, ...);

#define MV_REQUIRE(cond, ...)                                         \
  do {                                                                \
    if (!(cond)) return ::mv::fail(MV_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

#define MV_HIP_CHECK(expr)                                                                 \
  do {                                                                                     \
    hipError_t e__ = (expr);                                                               \
    if (e__ != hipSuccess)                                                                 \
      return ::mv::fail(MV_HIP_ERROR, "%s failed: %s", #expr, hipGetErrorString(e__));     \
  } while (0)

inline int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MV_HIP_ERROR, "%s launch failed: %s", what, hipGetErrorString(e));
  return MV_OK;
}

// ---- storage types ---------------------------------------------------------------------
// Storage T in {float, __half, __hip_bfloat16, double}; arithmetic type Acc<T> is float except
// for double.
template <typename T> struct Acc { using type = float; };
template <> struct Acc<double> { using type = double; };

template <typename T> __device__ __forceinline__ typename Acc<T>::type load(const T *p) {
  return static_cast<typename Acc<T>::type>(*p);
}
template <> __device__ __forceinline__ float load<__half>(const __half *p) { return __half2float(*p); }
template <> __device__ __forceinline__ float load<__hip_bfloat16>(const __hip_bfloat16 *p) {
  // bf16 -> fp32 is a 16-bit shift
  return __uint_as_float(static_cast<unsigned>(*reinterpret_cast<const unsigned short *>(p)) << 16);
}

template <typename T> __device__ __forceinline__ T store_cast(typename Acc<T>::type v) {
  return static_cast<T>(v);
}
template <> __device__ __forceinline__ __half store_cast<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ __hip_bfloat16 store_cast<__hip_bfloat16>(float v) {
  return __float2bfloat16(v);
}

// Run `fn.template operator()<T>()` for the storage type named by `dtype`.
#define MV_DISPATCH(dtype, ...)                                                       \
  switch (dtype) {                                                                    \
    case MV_F32: { using T = float; __VA_ARGS__; break; }                             \
    case MV_F16: { using T = __half; __VA_ARGS__; break; }                            \
    case MV_BF16: { using T = __hip_bfloat16; __VA_ARGS__; break; }                   \
    case MV_F64: { using T = double; __VA_ARGS__; break; }                            \
    default: return ::mv::fail(MV_INVALID_ARGUMENT, "unknown dtype %d", (int)(dtype)); \
  }

inline size_t dtype_size(int dtype) {
  switch (dtype) {
    case MV_F32: case MV_I32: return 4;
    case MV_F16: case MV_BF16: return 2;
    case MV_F64: return 8;
  }
  return 0;
}

// fp32 / fp64 hardware atomics (global_atomic_add_f32 / _f64).  Device memory handed to this
// library is ordinary coarse-grained hipMalloc memory, for which these are safe.
__device__ __forceinline__ void atomic_add(float *p, float v) { unsafeAtomicAdd(p, v); }
__device__ __forceinline__ void atomic_add(double *p, double v) { unsafeAtomicAdd(p, v); }

constexpr int kWave = 64;

// Workgroup ids are dealt round-robin to the 8 XCDs, each with an L2 of its own.  This renumbering
// hands every XCD one contiguous eighth of a grid's x range (the ids beyond the last multiple of 8
// keep their place), so that workgroups sharing an L2 work on neighbouring data.
__device__ __forceinline__ unsigned xcd_contiguous(unsigned id, unsigned count) {
  const unsigned per_xcd = count / 8;
  return id < per_xcd * 8 ? (id % 8) * per_xcd + id / 8 : id;
}

}  // namespace mv
