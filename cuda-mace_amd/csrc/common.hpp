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

// Compute units of the current device (256 on the part this library is written for; also the answer when the query
// fails), read once per device.
inline int device_compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

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

// Exclusive scan over n values by ONE workgroup of THREADS threads: emit(k, prefix_before_k, value_k) is called once for
// every k, and the total is returned in every thread.  Global memory is touched in whole lines only: the values are
// staged into LDS kStage at a time with consecutive threads on consecutive values, a thread scans a contiguous run of the
// staged values (runs of odd length, so that the threads of a wave start in different banks), the prefixes go back to
// LDS, and emit is called with consecutive threads on consecutive k.  (A thread that walks its run in global memory
// touches a line of its own per access: 75 000 single-word transactions from one compute unit, 40-70 us for 25 000 to
// 32 000 values, against a few here.)  stage: kStage values of LDS, part: THREADS values of LDS.
template <int THREADS, int kStage, typename Acc, class Load, class Emit>
__device__ __forceinline__ Acc workgroup_exclusive_scan(int n, Acc *stage, Acc *part, Load load, Emit emit) {
  const int t = threadIdx.x;
  Acc carry = 0;
  for (int base = 0; base < n; base += kStage) {
    const int cnt = min(kStage, n - base);
    __syncthreads();  // the previous stage has been emitted
    for (int i = t; i < cnt; i += THREADS) stage[i] = static_cast<Acc>(load(base + i));
    __syncthreads();
    const int per = ((cnt + THREADS - 1) / THREADS) | 1;
    const int lo = min(t * per, cnt), hi = min(lo + per, cnt);
    Acc sum = 0;
    for (int i = lo; i < hi; ++i) sum += stage[i];
    part[t] = sum;
    __syncthreads();
    for (int d = 1; d < THREADS; d <<= 1) {
      const Acc v = t >= d ? part[t - d] : Acc(0);
      __syncthreads();
      part[t] += v;
      __syncthreads();
    }
    Acc run = carry + part[t] - sum;  // exclusive prefix of this thread's run
    for (int i = lo; i < hi; ++i) {
      const Acc v = stage[i];
      stage[i] = run;  // emit gets the value back as the difference of neighbouring prefixes
      run += v;
    }
    __syncthreads();
    // value_k = prefix_{k+1} - prefix_k (the last one of the stage from the stage's total)
    const Acc stage_total = carry + part[THREADS - 1];
    for (int i = t; i < cnt; i += THREADS) {
      const Acc before = stage[i];
      const Acc after = i + 1 < cnt ? stage[i + 1] : stage_total;
      emit(base + i, before, after - before);
    }
    carry = stage_total;
  }
  return carry;
}

// The vector of edge e in fp64: pos[b[e]] - pos[a[e]] + shift[e], atom n being row rows[n] of pos when a row map is given;
// zero when either index lies outside the node range.  The one definition every kernel that forms an edge vector uses,
// so that all of them arrive at the same bits.
__device__ __forceinline__ void edge_vector_f64(const double *__restrict__ pos, const int32_t *__restrict__ a,
                                                const int32_t *__restrict__ b, const double *__restrict__ shifts,
                                                const int32_t *__restrict__ rows, int64_t e, int nnodes, double (&v)[3]) {
  const int ia = a[e], ib = b[e];
  v[0] = v[1] = v[2] = 0.0;
  if (static_cast<unsigned>(ia) < static_cast<unsigned>(nnodes) && static_cast<unsigned>(ib) < static_cast<unsigned>(nnodes)) {
    const int ra = rows ? rows[ia] : ia, rb = rows ? rows[ib] : ib;
#pragma unroll
    for (int k = 0; k < 3; ++k) v[k] = pos[3 * rb + k] - pos[3 * ra + k] + shifts[3 * e + k];
  }
}

// Edge range [e0, e1) of a node as read from caller-provided CSR offsets, forced into [0, nedges] with e0 <= e1: offsets
// derived from an unsorted or out-of-range receiver list then name a wrong but addressable range instead of memory
// outside the edge arrays.
__host__ __device__ __forceinline__ void clamp_edge_range(int &e0, int &e1, int64_t nedges) {
  const int ne = static_cast<int>(nedges);
  e0 = e0 < 0 ? 0 : (e0 > ne ? ne : e0);
  e1 = e1 < e0 ? e0 : (e1 > ne ? ne : e1);
}

// Tile `tile` of `tile_rows` consecutive positions of the grouped node order (tiles do not straddle groups; without
// groups, of the plain node order): its group g, first position pos0 and the end of its group; false when there is no
// such tile.  Called by all threads of a workgroup with the same arguments (whole waves).  Up to 64 groups are
// searched with one load per lane and a prefix sum over the lanes (a loop over the groups is a chain of dependent loads:
// microseconds at the head of a kernel that runs for ten).
__device__ __forceinline__ bool locate_group_tile(const int32_t *__restrict__ group_offsets, int ngroups, int nnodes, int tile,
                                                  int tile_rows, int &g, int &pos0, int &gend) {
  g = 0, pos0 = 0, gend = nnodes;
  if (!group_offsets) {
    pos0 = tile * tile_rows;
    return pos0 < nnodes;
  }
  if (ngroups <= kWave) {
    const int lane = threadIdx.x % kWave;
    const int lo = lane < ngroups ? group_offsets[lane] : 0, hi = lane < ngroups ? group_offsets[lane + 1] : 0;
    const int tiles = (hi - lo + tile_rows - 1) / tile_rows;
    int upto = tiles;  // inclusive prefix sum over the lanes
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int v = __shfl_up(upto, d);
      if (lane >= d) upto += v;
    }
    const unsigned long long owners = __ballot(tile < upto);
    if (owners == 0) return false;
    g = __ffsll(static_cast<long long>(owners)) - 1;
    const int first = __shfl(upto - tiles, g);
    pos0 = __shfl(lo, g) + (tile - first) * tile_rows;
    gend = __shfl(hi, g);
    return true;
  }
  for (g = 0; g < ngroups; ++g) {
    const int lo = group_offsets[g], hi = group_offsets[g + 1];
    const int tiles = (hi - lo + tile_rows - 1) / tile_rows;
    if (tile < tiles) {
      pos0 = lo + tile * tile_rows;
      gend = hi;
      return true;
    }
    tile -= tiles;
  }
  return false;
}

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
// Three-wide variant for channel counts that fill the wave with three channels per lane (96, 192).  Loads and stores
// are 12 bytes at 4-byte alignment.
typedef float f3 __attribute__((ext_vector_type(3)));

template <int V>
struct VecOf;
template <>
struct VecOf<4> {
  using type = f4;
};
template <>
struct VecOf<3> {
  using type = f3;
};

// Five- and seven-wide variants for 160 and 224 channels on 32 lanes (strided channel ownership only: there is no
// 20- or 28-byte access).
typedef float f5 __attribute__((ext_vector_type(5)));
typedef float f7 __attribute__((ext_vector_type(7)));
template <>
struct VecOf<5> {
  using type = f5;
};
template <>
struct VecOf<7> {
  using type = f7;
};

template <class T>
__device__ __forceinline__ T zerov();
template <>
__device__ __forceinline__ f5 zerov<f5>() {
  return f5{0.f, 0.f, 0.f, 0.f, 0.f};
}
template <>
__device__ __forceinline__ f7 zerov<f7>() {
  return f7{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
}
template <>
__device__ __forceinline__ f4 zerov<f4>() {
  return zero4();
}
template <>
__device__ __forceinline__ f3 zerov<f3>() {
  return f3{0.f, 0.f, 0.f};
}

template <class T>
__device__ __forceinline__ T ldv(const float *p);
template <>
__device__ __forceinline__ f4 ldv<f4>(const float *p) {
  return ld4(p);
}
template <>
__device__ __forceinline__ f3 ldv<f3>(const float *p) {
  return f3{p[0], p[1], p[2]};
}
template <class T>
__device__ __forceinline__ T ldv_stream(const float *p);
template <>
__device__ __forceinline__ f4 ldv_stream<f4>(const float *p) {
  return ld4_stream(p);
}
template <>
__device__ __forceinline__ f3 ldv_stream<f3>(const float *p) {
  return f3{__builtin_nontemporal_load(p), __builtin_nontemporal_load(p + 1), __builtin_nontemporal_load(p + 2)};
}
__device__ __forceinline__ void stv(float *p, f4 v) { st4(p, v); }
__device__ __forceinline__ void stv(float *p, f3 v) {
  p[0] = v.x;
  p[1] = v.y;
  p[2] = v.z;
}
__device__ __forceinline__ void stv_stream(float *p, f4 v) { st4_stream(p, v); }
__device__ __forceinline__ void stv_stream(float *p, f3 v) {
  __builtin_nontemporal_store(v.x, p);
  __builtin_nontemporal_store(v.y, p + 1);
  __builtin_nontemporal_store(v.z, p + 2);
}
__device__ __forceinline__ float hsumv(f4 a) { return hsum4(a); }
__device__ __forceinline__ float hsumv(f3 a) { return (a.x + a.y) + a.z; }
__device__ __forceinline__ float dotv(f4 a, f4 b) { return dot4(a, b); }
__device__ __forceinline__ float dotv(f3 a, f3 b) { return fmaf(a.z, b.z, fmaf(a.y, b.y, a.x * b.x)); }

__device__ __forceinline__ f4 shfl_down4(f4 v, int delta) {
  f4 r;
  r.x = __shfl_down(v.x, delta);
  r.y = __shfl_down(v.y, delta);
  r.z = __shfl_down(v.z, delta);
  r.w = __shfl_down(v.w, delta);
  return r;
}
__device__ __forceinline__ f4 shfl_downv(f4 v, int delta) { return shfl_down4(v, delta); }
__device__ __forceinline__ f3 shfl_downv(f3 v, int delta) {
  return f3{__shfl_down(v.x, delta), __shfl_down(v.y, delta), __shfl_down(v.z, delta)};
}
__device__ __forceinline__ f5 shfl_downv(f5 v, int delta) {
  f5 r;
#pragma unroll
  for (int i = 0; i < 5; ++i) r[i] = __shfl_down(v[i], delta);
  return r;
}
__device__ __forceinline__ f7 shfl_downv(f7 v, int delta) {
  f7 r;
#pragma unroll
  for (int i = 0; i < 7; ++i) r[i] = __shfl_down(v[i], delta);
  return r;
}

}  // namespace cm
