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

template <int C, bool STRIDED = false, bool WIDE = false>
struct Cfg {
  // channels per lane: four (one 16-byte access per row), except where three fill the lanes exactly (96 -> 32 lanes,
  // 192 -> 64 lanes) and four would leave a quarter of them idle; kernels that own strided channels (see below) also
  // run 160 and 224 channels on 32 full lanes, five and seven channels each
  // WIDE: always four (one 16-byte access per lane and row, some lanes idle at 96 and 192 channels): for kernels that
  // only stream rows, where three dword accesses per row cost the vector-memory path three times the line look-ups
  static constexpr int V = WIDE ? 4 : (C == 96 || C == 192) ? 3 : (STRIDED && C == 160) ? 5 : (STRIDED && C == 224) ? 7 : 4;
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

// Sums p[m] over the SW lanes of a slot.  Butterfly with halving: after the exchange over one lane bit each lane keeps
// half of its values, so 16 values cost 8+4+2+1 exchanges instead of 16*4.
//
// SW >= 32: the two widest stages run over lane bits 3 and 2 as DPP adds whose write is masked by bank (a bank is four
// consecutive lanes of a row of 16, so those two bits select banks): "lanes with the bit clear take p[k] + partner's
// p[k], lanes with the bit set take p[h+k] + partner's p[h+k]" is two instructions per pair and needs no select
// (written as inline assembly because the masked form keeps the destination's other lanes, which the DPP builtin
// cannot express; the s_nop covers the two wait states a DPP read needs after a VALU write of the same register).
// The stage over lane bit 4 swaps rows of 16 lanes between the two registers of a pair (v_permlane16_swap) and adds;
// lane bit 0 goes through a quad permutation with selects, and lane bit 1 (and bit 5 for 64-lane slots) is a plain
// sum.  Every lane ends with the total for m = reduced_index16(cl) in p[0].
//
// SW == 16 / 8: the stages over lane bits 0 and 1 stay inside a quad and go through DPP; the rest through
// ds_bpermute.  Result: m = bitrev4(cl) in p[0] (SW == 16), or the two totals m = bitrev3(cl) * 2 + {0, 1} in p[0], p[1].
template <int SW>
__device__ __forceinline__ void slot_reduce16(float (&p)[16], int cl) {
  static_assert(SW >= 8, "slot width");
  if constexpr (SW >= 32) {
    asm volatile(
        "s_nop 1\n\t"
        "v_add_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %1, %1, %1 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %2, %2, %2 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %3, %3, %3 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %4, %4, %4 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %5, %5, %5 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %6, %6, %6 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %7, %7, %7 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        "v_add_f32_dpp %0, %8, %8 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %1, %9, %9 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %2, %10, %10 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %3, %11, %11 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %4, %12, %12 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %5, %13, %13 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %6, %14, %14 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        "v_add_f32_dpp %7, %15, %15 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
        // lane bit 2: lanes of banks 0 and 2 read four lanes up (rotate right by 12), banks 1 and 3 four lanes down
        "v_add_f32_dpp %0, %0, %0 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %1, %1, %1 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %2, %2, %2 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %3, %3, %3 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
        "v_add_f32_dpp %0, %4, %4 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
        "v_add_f32_dpp %1, %5, %5 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
        "v_add_f32_dpp %2, %6, %6 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
        "v_add_f32_dpp %3, %7, %7 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
        "s_nop 0"  // with the wait state the compiler adds after the block: two before a lane-crossing read of %3
        : "+v"(p[0]), "+v"(p[1]), "+v"(p[2]), "+v"(p[3]), "+v"(p[4]), "+v"(p[5]), "+v"(p[6]), "+v"(p[7])
        : "v"(p[8]), "v"(p[9]), "v"(p[10]), "v"(p[11]), "v"(p[12]), "v"(p[13]), "v"(p[14]), "v"(p[15]));
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      // first result: row 0 of p[k] over row 0 of p[2+k]; second: row 1 of p[k] over row 1 of p[2+k]
      const auto sw = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, p[k]), __builtin_bit_cast(unsigned, p[2 + k]),
                                                       false, false);
      const unsigned first = sw[0], second = sw[1];  // element-wise copies first: a bit_cast straight from sw[1] reads sw[0]
      p[k] = __uint_as_float(first) + __uint_as_float(second);
    }
    {
      const bool hi = cl & 1;
      const float keep = hi ? p[1] : p[0];
      const float send = hi ? p[0] : p[1];
      p[0] = keep + dpp_move<0xB1>(send);
    }
    p[0] += dpp_move<0x4E>(p[0]);
    if constexpr (SW >= 64) p[0] += __shfl_xor(p[0], 32);
    return;
  }
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

// Which m a lane (position cl in its slot) holds after slot_reduce16.
template <int SW>
__device__ __forceinline__ int reduced_index16(int cl) {
  if constexpr (SW >= 32) return (cl & 12) | ((cl >> 3) & 2) | (cl & 1);  // lane bits 3, 2, 4, 0
  return ((cl & 1) << 3) | ((cl & 2) << 1) | ((cl & 4) >> 1) | ((cl & 8) >> 3);
}

// Writes the reduced gY values of edge j into the LDS tile sGY[m][kChunk].
template <int SW>
__device__ __forceinline__ void store_reduced16(const float (&p)[16], int cl, int j, float *sGY) {
  if constexpr (SW >= 32) {
    if ((cl & ~29) == 0) sGY[reduced_index16<SW>(cl) * kChunk + j] = p[0];  // one lane per m: lane bits 1 and 5 clear
  } else if constexpr (SW == 16) {
    sGY[reduced_index16<SW>(cl) * kChunk + j] = p[0];
  } else {
    const int m0 = (((cl & 1) << 2) | (cl & 2) | ((cl & 4) >> 2)) * 2;
    sGY[m0 * kChunk + j] = p[0];
    sGY[(m0 + 1) * kChunk + j] = p[1];
  }
}

// Length of an edge vector as the spline-fused kernels take it.  The edge pass decides by it which rows of the per-edge
// scratch it writes and the sender pass which rows it reads, so both must get the same bits: the operations are spelled
// out (no contraction left to the compiler).
__device__ __forceinline__ float edge_length(float v0, float v1, float v2) {
  return sqrtf(fmaf(v2, v2, fmaf(v1, v1, v0 * v0)));
}

// Parts a node's edge range is cut into where one wave per node would leave most of the device idle (a 216-atom cell is
// 216 waves for 1 024 SIMDs, each walking its ~90 edges one after the other): as many as fill about 2 048 wave slots
// and leave a part a dozen edges on average, at most 8.
inline int parts_for(int64_t nnodes, int64_t nedges) {
  if (nnodes <= 0) return 1;
  const int64_t by_slots = 2048 / nnodes, by_edges = nedges / (12 * nnodes);
  const int64_t parts = by_slots < by_edges ? by_slots : by_edges;
  return parts < 1 ? 1 : (parts > 8 ? 8 : static_cast<int>(parts));
}

// Sender pass of the backward, shared by both variants (defined in mp.hip).  With live_vec (edge vectors [E, 3]) or
// live_r (edge lengths [E]) given, only the rows of edges within r_max are read: the spline-fused edge pass writes no
// others.
int launch_sender_pass(int channels, const float *gXe, const int32_t *perm, const int32_t *offsets, int64_t nnodes,
                       int64_t nedges, float *gX, hipStream_t st, const float *live_vec = nullptr,
                       const float *live_r = nullptr, float r_max = 0.f);

// Forward from edge vectors with the radial table in LDS, one degree and one 32-channel slice per workgroup (defined in
// mp_sliced.hip): whether it takes a launch of this shape, and the launch.
bool sliced_forward_applies(int64_t nnodes, int channels, int nknots);
int launch_sliced_forward(const float *X, const float *vec, const float *knots, const float *coeffs, int nknots, float r_width,
                          float r_max, const int32_t *sender, const int32_t *first_occ, int64_t nnodes, int64_t nedges,
                          int channels, float *out, hipStream_t st);

// The spline-fused backward edge pass from edge vectors without gX, writing (this layer's vector gradient + addend[e])
// (defined in mp_spline.hip; operands as cm_mp_edge_backward, already checked by the caller).
int edge_backward_onto(const float *X, const float *vectors, const float *r_knots, const float *coeffs, int nknots, float r_width,
                       float r_max, const float *grad_out, const int32_t *sender, const int32_t *first_occ, int64_t nnodes,
                       int64_t nedges, int channels, float *grad_vectors, const float *addend, hipStream_t st);

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
