// Shared host/device helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "cuda_mace_hip.h"

namespace cm {

constexpr int kWave = 64;

// ---- host side -------------------------------------------------------------------------------
void set_error(const char *fmt, ...);  // defined in error.cpp; stores a thread-local message

inline hipStream_t as_stream(cm_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Checks the launch that was just enqueued; returns CM_OK or CM_ELAUNCH.
inline int check_launch(const char *what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(err));
    return CM_ELAUNCH;
  }
  return CM_OK;
}

#define CM_REQUIRE(cond, ...)      \
  do {                             \
    if (!(cond)) {                 \
      cm::set_error(__VA_ARGS__);  \
      return CM_EINVAL;            \
    }                              \
  } while (0)

// ---- device side -----------------------------------------------------------------------------
// l(m) = floor(sqrt(m)) for m in 0..15 without a sqrt.
__device__ __forceinline__ constexpr int l_of_m(int m) { return m == 0 ? 0 : (m < 4 ? 1 : (m < 9 ? 2 : 3)); }

// Orders LDS traffic of one wavefront: stores issued before are visible to loads issued after.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Native 4-wide float vector: arithmetic operators act elementwise, scalars broadcast.
typedef float f4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f4 zero4() { return f4{0.f, 0.f, 0.f, 0.f}; }
__device__ __forceinline__ f4 ld4(const float *p) { return *reinterpret_cast<const f4 *>(p); }
__device__ __forceinline__ void st4(float *p, f4 v) { *reinterpret_cast<f4 *>(p) = v; }
// Non-temporal variants for data that is touched exactly once.
__device__ __forceinline__ f4 ld4_stream(const float *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const f4 *>(p));
}
__device__ __forceinline__ void st4_stream(float *p, f4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<f4 *>(p));
}
__device__ __forceinline__ float hsum4(f4 a) { return (a.x + a.y) + (a.z + a.w); }
// a . b as one multiply and three fused multiply-adds
__device__ __forceinline__ float dot4(f4 a, f4 b) { return fmaf(a.w, b.w, fmaf(a.z, b.z, fmaf(a.y, b.y, a.x * b.x))); }
__device__ __forceinline__ f4 shfl_down4(f4 v, int delta) {
  f4 r;
  r.x = __shfl_down(v.x, delta);
  r.y = __shfl_down(v.y, delta);
  r.z = __shfl_down(v.z, delta);
  r.w = __shfl_down(v.w, delta);
  return r;
}

}  // namespace cm
