// Pieces shared by the message-passing kernels (tabulated-radial and spline-fused variants).
#pragma once

#include "common.hpp"

namespace cm {
namespace mp {

constexpr int kChunk = 64;  // edges whose Y / sender values are staged in LDS at a time

constexpr int pow2ceil(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

template <int C, bool STRIDED = false>
struct Cfg {
  // channels per lane: four (one 16-byte access per row), except where three fill the lanes exactly (96 -> 32 lanes,
  // 192 -> 64 lanes) and four would leave a quarter of them idle; kernels that own strided channels (see below) also
  // run 160 and 224 channels on 32 full lanes, five and seven channels each
  static constexpr int V = (C == 96 || C == 192) ? 3 : (STRIDED && C == 160) ? 5 : (STRIDED && C == 224) ? 7 : 4;
  static constexpr int LPE = C / V;          // lanes that carry one edge
  static constexpr int SW = pow2ceil(LPE);   // slot width in lanes (power of two)
  static constexpr int EPW = kWave / SW;     // edges in flight per wave
  using vec = typename VecOf<V>::type;
  static_assert(C % 32 == 0 && C >= 32 && C <= 256 && C % V == 0, "channel count");

  // Which channels a lane owns.  Contiguous: V cl .. V cl + V - 1 (one 16-byte access per row for V = 4, a 12-byte one
  // for V = 3).  STRIDED (V != 4): cl, cl + LPE, cl + 2 LPE, ..., so that each of the V dword accesses of a wave
  // covers a contiguous run of the row: a 12-byte access per lane costs the vector-memory path as much as a 16-byte
  // one, which the kernels that are bound by that path (the forward ones) feel (measured 15 % at 96 and 192 channels),
  // while the backward kernels, bound by instruction issue, are 3 % faster with the single wider access.  Rows in memory
  // are plain channel order either way, so every kernel chooses for itself.  off(cl) is the first channel of lane cl,
  // ES the distance between the lane's channels.
  static constexpr bool kStrided = STRIDED && V != 4;
  static constexpr int ES = kStrided ? LPE : 1;
  __device__ static __forceinline__ int off(int cl) { return kStrided ? cl : V * cl; }
  __device__ static __forceinline__ vec ld(const float *p) {
    if constexpr (V == 4) {
      return ld4(p);
    } else {
      vec r;
#pragma unroll
      for (int i = 0; i < V; ++i) r[i] = p[i * ES];
      return r;
    }
  }
  __device__ static __forceinline__ vec ld_stream(const float *p) {
    if constexpr (V == 4) {
      return ld4_stream(p);
    } else {
      vec r;
#pragma unroll
      for (int i = 0; i < V; ++i) r[i] = __builtin_nontemporal_load(p + i * ES);
      return r;
    }
  }
  __device__ static __forceinline__ void st(float *p, vec v) {
    if constexpr (V == 4) {
      st4(p, v);
    } else {
#pragma unroll
      for (int i = 0; i < V; ++i) p[i * ES] = v[i];
    }
  }
  __device__ static __forceinline__ void st_stream(float *p, vec v) {
    if constexpr (V == 4) {
      st4_stream(p, v);
    } else {
#pragma unroll
      for (int i = 0; i < V; ++i) __builtin_nontemporal_store(v[i], p + i * ES);
    }
  }
};

// Stages Y[0:16, base:base+cnt] (transposed to [edge][16]) and sender[base:base+cnt] in LDS.
__device__ __forceinline__ void stage_chunk(const float *__restrict__ Y, const int32_t *__restrict__ sender,
                                            int64_t nedges, int base, int cnt, int lane, float *sY,
                                            int *sS) {
  if (lane < cnt) {
    const int64_t e = base + lane;
    sS[lane] = sender[e];
    f4 y[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      y[q].x = Y[(4 * q + 0) * nedges + e];
      y[q].y = Y[(4 * q + 1) * nedges + e];
      y[q].z = Y[(4 * q + 2) * nedges + e];
      y[q].w = Y[(4 * q + 3) * nedges + e];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) *reinterpret_cast<f4 *>(sY + lane * 16 + 4 * q) = y[q];
  }
}

// Value of `v` in the lane selected by a DPP control word (data-parallel-primitive operand swizzle of the VALU: no LDS
// round trip).  0xB1 / 0x4E: quad_perm [1,0,3,2] / [2,3,0,1], i.e. lane ^ 1 / lane ^ 2; 0x124 / 0x128: rotate right by
// 4 / 8 within each row of 16 lanes.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

// Sums p[m] over the SW lanes of a slot.  Butterfly with halving: after the exchange over lane
// bit b each lane keeps half of its values, so 16 values cost 8+4+2+1 exchanges instead of 16*4.
// The 12 exchanges over lane bits 0 and 1 stay inside a quad and go through DPP; the rest through ds_bpermute.
// Returns, in every lane, the total for m = bitrev4(cl & 15) (SW >= 16), or for SW == 8 the two
// totals m = bitrev3(cl) * 2 + {0, 1} in p[0], p[1].
template <int SW>
__device__ __forceinline__ void slot_reduce16(float (&p)[16], int cl) {
  static_assert(SW >= 8, "slot width");
  {
    const bool hi = cl & 1;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float keep = hi ? p[8 + k] : p[k];
      const float send = hi ? p[k] : p[8 + k];
      p[k] = keep + dpp_move<0xB1>(send);
    }
  }
  {
    const bool hi = cl & 2;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float keep = hi ? p[4 + k] : p[k];
      const float send = hi ? p[k] : p[4 + k];
      p[k] = keep + dpp_move<0x4E>(send);
    }
  }
  {
    const bool hi = cl & 4;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const float keep = hi ? p[2 + k] : p[k];
      const float send = hi ? p[k] : p[2 + k];
      p[k] = keep + __shfl_xor(send, 4);
    }
  }
  if constexpr (SW >= 16) {
    const bool hi = cl & 8;
    const float keep = hi ? p[1] : p[0];
    const float send = hi ? p[0] : p[1];
    p[0] = keep + __shfl_xor(send, 8);
  }
  if constexpr (SW >= 32) p[0] += __shfl_xor(p[0], 16);
  if constexpr (SW >= 64) p[0] += __shfl_xor(p[0], 32);
}

// Plain sum of one value over the SW lanes of a slot; every lane gets the total.  Inside a row of 16 lanes: quad sums,
// then rotations by 4 and 8 (all DPP); across rows: ds_bpermute.
template <int SW>
__device__ __forceinline__ float slot_sum(float v) {
  static_assert(SW >= 8, "slot width");
  v += dpp_move<0xB1>(v);
  v += dpp_move<0x4E>(v);
  if constexpr (SW >= 16) {
    v += dpp_move<0x124>(v);
    v += dpp_move<0x128>(v);
  } else {
    v += __shfl_xor(v, 4);
  }
#pragma unroll
  for (int off = 16; off < SW; off <<= 1) v += __shfl_xor(v, off);
  return v;
}

// Which m a lane (position cl in its slot) holds after slot_reduce16, SW >= 16.
__device__ __forceinline__ int reduced_index16(int cl) {
  return ((cl & 1) << 3) | ((cl & 2) << 1) | ((cl & 4) >> 1) | ((cl & 8) >> 3);
}

// Writes the reduced gY values of edge j into the LDS tile sGY[m][kChunk].
template <int SW>
__device__ __forceinline__ void store_reduced16(const float (&p)[16], int cl, int j, float *sGY) {
  if constexpr (SW >= 16) {
    if (cl < 16) sGY[reduced_index16(cl) * kChunk + j] = p[0];
  } else {
    const int m0 = (((cl & 1) << 2) | (cl & 2) | ((cl & 4) >> 2)) * 2;
    sGY[m0 * kChunk + j] = p[0];
    sGY[(m0 + 1) * kChunk + j] = p[1];
  }
}

// Sender pass of the backward, shared by both variants (defined in mp.hip).
int launch_sender_pass(int channels, const float *gXe, const int32_t *perm, const int32_t *offsets, int64_t nnodes,
                       int64_t nedges, float *gX, hipStream_t st);

}  // namespace mp
}  // namespace cm

#define CM_DISPATCH_C(channels, CALL)                 \
  switch (channels) {                                 \
    case 32: { constexpr int C_ = 32; CALL; } break;   \
    case 64: { constexpr int C_ = 64; CALL; } break;   \
    case 96: { constexpr int C_ = 96; CALL; } break;   \
    case 128: { constexpr int C_ = 128; CALL; } break; \
    case 160: { constexpr int C_ = 160; CALL; } break; \
    case 192: { constexpr int C_ = 192; CALL; } break; \
    case 224: { constexpr int C_ = 224; CALL; } break; \
    case 256: { constexpr int C_ = 256; CALL; } break; \
    default: break;                                   \
  }
