// Channel-mixing linear layers on the matrix cores, fp32 in and out.
//
//   OUT[n, m, :] = scale * X[n, m, :] . W[g(n)][l(m)]      (scale = 1/sqrt(K) in the model)
//
// for features with 16 components per node (l(m) = floor(sqrt(m)), four weight blocks per group) or with a
// single scalar component per node (one weight block per group).
//
// A workgroup of four wavefronts owns a tile of 128 nodes x one component m x all Nout columns, so
// every row of the tile uses the same K x Nout weight block W[g][l(m)].  K is walked in chunks of 32:
// the X rows of the tile (each chunk of a row is one 128-byte line) and the matching columns of the
// TRANSPOSED weights ([Nout, K], which the caller already keeps for the backward) are staged in LDS
// with coalesced 16-byte loads, and each wave feeds the matrix cores with 16-byte LDS reads.  Weights
// therefore cross L2 once per 128 rows instead of once per 32.  All (group, m, tile) combinations go out in
// a single launch; per-element weights are selected through a node permutation that lists the nodes group
// by group, without any host synchronisation.
//
// Arithmetic: every fp32 operand is split into three bf16 pieces when it is staged (a = hi + mid + lo, 24 mantissa bits
// in all), and the product is accumulated in fp32 from the six piece products that matter (hi.hi, hi.mid, mid.hi, hi.lo,
// lo.hi, mid.mid; the dropped ones are below 2^-24 of the product) on v_mfma_f32_32x32x16_bf16, whose rate is 16x that of
// the fp32 matrix instruction.  The result matches an fp32 GEMM to rounding (measured rms error 1.7e-7 against fp64 on
// unit-variance data, plain fp32 accumulation 2.0e-7), and the GEMM phase is a third of what v_mfma_f32_32x32x2_f32 on the
// fp32 values needs (measured 1.2-1.4x faster end to end at every width from 64 to 256), so the kernel runs at what
// its memory traffic allows.
#include <algorithm>
#include <cmath>
#include <type_traits>

#include "common.hpp"
#include "mfma_split.hpp"

namespace cm {
namespace {

constexpr int kWaves = 4;
constexpr int kTileNodes = 32 * kWaves;  // rows per workgroup (MFMA M = 32 per wave)
constexpr int kKC = 32;                  // K columns staged per step
constexpr int kLdH = kKC + 8;            // padded LDS row stride of a bf16 plane (elements; 80 bytes: conflict-free b128 reads)

// A wave's 32 x (32 NT) block of accumulators to memory, four bytes per lane and store (a store instruction covers two
// rows of 128 bytes): OUT = acc * scale (+ residual).  The residual may be OUT itself, so the compiler cannot move a
// load of it across a store: all of a lane's residual values are read before its first store (every element is read
// and written by the same lane), instead of one dependent load per store.  The product is rounded before the residual is
// added, as in the kernels that stage it in LDS.
template <int NT>
__device__ __forceinline__ void store_block(const v16f (&acc)[NT], const int *sNode, int wave, int half, int mrow, int ncomp, int m,
                                            int row_stride, int col0, float scale, const float *residual, float *OUT) {
  if (residual) {
    float res[16][NT];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int node = sNode[32 * wave + 8 * (r / 4) + 4 * half + (r % 4)];
      const float *rp = residual + (static_cast<int64_t>(node >= 0 ? node : 0) * ncomp + m) * row_stride + col0 + mrow;
#pragma unroll
      for (int t = 0; t < NT; ++t) res[r][t] = node >= 0 ? rp[32 * t] : 0.f;
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int node = sNode[32 * wave + 8 * (r / 4) + 4 * half + (r % 4)];
      if (node < 0) continue;
      float *op = OUT + (static_cast<int64_t>(node) * ncomp + m) * row_stride + col0 + mrow;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma clang fp contract(off)
        const float v = acc[t][r] * scale;
        op[32 * t] = v + res[r][t];
      }
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int node = sNode[32 * wave + 8 * (r / 4) + 4 * half + (r % 4)];
    if (node < 0) continue;
    float *op = OUT + (static_cast<int64_t>(node) * ncomp + m) * row_stride + col0 + mrow;
#pragma unroll
    for (int t = 0; t < NT; ++t) op[32 * t] = acc[t][r] * scale;
  }
}

// A workgroup computes 32 * NT output columns, starting at column blockIdx.y * 32 * NT of the nout_total columns of a row
// (one workgroup per tile for all columns where there are many tiles; few tiles are spread over more workgroups, 32
// columns each, which shortens the chain of staging and matrix instructions a tile waits for: every output element sums
// the same products in the same order either way).  SCALED: X is multiplied by row_scale on the way in
// At 160 and 192 columns two workgroups fit a compute unit by their LDS (70 / 77 KB) and, told so, the compiler keeps the
// kernel within the 256 registers that leaves each wave (measured 25-30 % faster on [N,16,C] features there).
template <int NT, bool SCALED>
__global__ __launch_bounds__(kWaves *kWave, ((NT == 5 || NT == 6) ? 2 : 1)) void linear_kernel(const float *__restrict__ X, const float *__restrict__ WT,
                                                               const int32_t *__restrict__ node_perm,
                                                               const int32_t *__restrict__ group_offsets, int nnodes,
                                                               int ngroups, int zero_last_group, int ncomp, int K,
                                                               float scale, const float *__restrict__ row_scale,
                                                               const float *residual, float *OUT, int nout_total) {
  constexpr int NOUT = 32 * NT;
  const int col0 = blockIdx.y * NOUT;
  // three bf16 planes per operand: plane p of X at sAp + p * kTileNodes * kLdH, of the weights at sBp + p * NOUT * kLdH
  // (77 KB at Nout = 192, 92 KB at 256: beyond 64 KB, within the 160 KB of a gfx950 compute unit)
  __shared__ __attribute__((aligned(16))) __bf16 sAp[3 * kTileNodes * kLdH];
  __shared__ __attribute__((aligned(16))) __bf16 sBp[3 * NOUT * kLdH];
  __shared__ int sNode[kTileNodes];

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  // the components of a tile are neighbours in the launch order: they share the tile's row_scale rows and touch
  // adjacent rows of X and OUT while those are hot
  const int m = blockIdx.x % ncomp;  // component 0..ncomp-1
  const int l = ncomp == 1 ? 0 : l_of_m(m);
  const int nblocks = ncomp == 1 ? 1 : 4;  // weight blocks per group

  // locate (group, first position in the grouped node order) of this tile
  int g, pos0, gend;
  if (!locate_group_tile(group_offsets, ngroups, nnodes, blockIdx.x / ncomp, kTileNodes, g, pos0, gend)) return;
  const int nrows = min(kTileNodes, gend - pos0);

  if (tid < kTileNodes) {
    int node = -1;
    if (tid < nrows) {
      node = node_perm ? node_perm[pos0 + tid] : pos0 + tid;
      if (static_cast<unsigned>(node) >= static_cast<unsigned>(nnodes)) node = -1;
    }
    sNode[tid] = node;
  }
  __syncthreads();

  if (zero_last_group && g == ngroups - 1) {
    // rows that belong to no weight group: the product is defined as zero (a residual still passes through)
    for (int i = tid; i < kTileNodes * NOUT; i += kWaves * kWave) {
      const int node = sNode[i / NOUT];
      if (node >= 0) {
        const int64_t at = (static_cast<int64_t>(node) * ncomp + m) * nout_total + col0 + i % NOUT;
        OUT[at] = residual ? residual[at] : 0.f;
      }
    }
    return;
  }
  const float *Wg = WT + ((static_cast<int64_t>(g) * nblocks + l) * nout_total + col0) * K;  // [NOUT, K] of [nout_total, K]

  v16f acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;

  // staging map: kKC / 4 threads x 16 bytes cover the staged columns of a row
  constexpr int kTPR = kKC / 4;                    // threads per row
  constexpr int kRPP = kWaves * kWave / kTPR;      // rows per pass
  const int srow = tid / kTPR;
  const int scol = (tid % kTPR) * 4;
  // MFMA operand map: row / column within the 32-wide block and which half of the 8-wide k step
  const int mrow = lane % 32;
  const int half = lane / 32;

  constexpr int A_PASSES = kTileNodes / kRPP;
  constexpr int B_PASSES = NOUT / kRPP;
  f4 pa[A_PASSES], pb[B_PASSES], ps[SCALED ? A_PASSES : 1];
  // global -> register prefetch of one K chunk; the next chunk is in flight while the current one is multiplied
  auto prefetch = [&](int kc) {
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      const int node = sNode[kRPP * i + srow];
      pa[i] = zero4();
      if (node >= 0) {
        pa[i] = ld4_stream(X + (static_cast<int64_t>(node) * ncomp + m) * K + kc + scol);
        // optional per-node, per-column factor shared by all components (the contraction's upstream gradient); it is
        // applied when the chunk moves to LDS, so that nothing waits for these loads here
        if constexpr (SCALED) ps[i] = ld4(row_scale + static_cast<int64_t>(node) * K + kc + scol);
      }
    }
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) pb[i] = ld4(Wg + static_cast<int64_t>(kRPP * i + srow) * K + kc + scol);
  };
  prefetch(0);
  for (int kc = 0; kc < K; kc += kKC) {
    __syncthreads();  // previous chunk fully consumed
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      f4 v = pa[i];
      if constexpr (SCALED) v *= ps[i];
      bf16x4 h, md, lw;
      split3(v, h, md, lw);
      const int at = (kRPP * i + srow) * kLdH + scol;
      *reinterpret_cast<bf16x4 *>(sAp + at) = h;
      *reinterpret_cast<bf16x4 *>(sAp + kTileNodes * kLdH + at) = md;
      *reinterpret_cast<bf16x4 *>(sAp + 2 * kTileNodes * kLdH + at) = lw;
    }
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) {
      bf16x4 h, md, lw;
      split3(pb[i], h, md, lw);
      const int at = (kRPP * i + srow) * kLdH + scol;
      *reinterpret_cast<bf16x4 *>(sBp + at) = h;
      *reinterpret_cast<bf16x4 *>(sBp + NOUT * kLdH + at) = md;
      *reinterpret_cast<bf16x4 *>(sBp + 2 * NOUT * kLdH + at) = lw;
    }
    __syncthreads();
    if (kc + kKC < K) prefetch(kc + kKC);

#pragma unroll
    for (int ks = 0; ks < kKC; ks += 16) {
      // a lane feeds 8 consecutive k of its row: k = ks + 8 * half .. + 7
      const int aoff = (32 * wave + mrow) * kLdH + ks + 8 * half;
      bf16x8 a[3], b[NT][3];
#pragma unroll
      for (int p = 0; p < 3; ++p) a[p] = *reinterpret_cast<const bf16x8 *>(sAp + p * kTileNodes * kLdH + aoff);
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int p = 0; p < 3; ++p)
          b[t][p] = *reinterpret_cast<const bf16x8 *>(sBp + p * NOUT * kLdH + (32 * t + mrow) * kLdH + ks + 8 * half);
      // piece products from small to large; consecutive MFMAs go to different accumulators
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[2], b[t][0], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[t][2], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[t][1], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[t][0], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[t][1], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[t][0], acc[t], 0, 0, 0);
    }
  }

  // accumulator r of a lane is row 8*(r/4) + 4*(lane/32) + r%4, column lane%32 of the wave's 32x32 block
  store_block<NT>(acc, sNode, wave, half, mrow, ncomp, m, nout_total, col0, scale, residual, OUT);
}

// -----------------------------------------------------------------------------------------------
// Few tiles (a system of a few hundred atoms): the launch is over in a few microseconds, most of which a workgroup of the
// kernel above spends waiting for one K chunk after the other, with next to nothing to multiply in between.  Here a
// workgroup (one tile, one component, 32 output columns) requests every K chunk of both operands, the row scales and
// the residual values at once and waits for memory once; K = 32 KCH.  Staging, operand split, piece products and their
// order, and the epilogue's roundings are those of the kernel above: the same bits.
template <int KCH, bool SCALED>
__global__ __launch_bounds__(kWaves *kWave) void linear_few_tiles_kernel(const float *__restrict__ X, const float *__restrict__ WT,
                                                                         const int32_t *__restrict__ node_perm,
                                                                         const int32_t *__restrict__ group_offsets, int nnodes,
                                                                         int ngroups, int zero_last_group, int ncomp, float scale,
                                                                         const float *__restrict__ row_scale, const float *residual,
                                                                         float *OUT, int nout_total) {
  constexpr int K = kKC * KCH;
  constexpr int NOUT = 32;
  const int col0 = blockIdx.y * NOUT;
  __shared__ __attribute__((aligned(16))) __bf16 sAp[3 * kTileNodes * kLdH];
  __shared__ __attribute__((aligned(16))) __bf16 sBp[3 * NOUT * kLdH];
  __shared__ int sNode[kTileNodes];

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int m = blockIdx.x % ncomp;
  const int l = ncomp == 1 ? 0 : l_of_m(m);
  const int nblocks = ncomp == 1 ? 1 : 4;

  int g, pos0, gend;
  if (!locate_group_tile(group_offsets, ngroups, nnodes, blockIdx.x / ncomp, kTileNodes, g, pos0, gend)) return;
  const int nrows = min(kTileNodes, gend - pos0);
  if (tid < kTileNodes) {
    int node = -1;
    if (tid < nrows) {
      node = node_perm ? node_perm[pos0 + tid] : pos0 + tid;
      if (static_cast<unsigned>(node) >= static_cast<unsigned>(nnodes)) node = -1;
    }
    sNode[tid] = node;
  }
  __syncthreads();

  if (zero_last_group && g == ngroups - 1) {
    for (int i = tid; i < kTileNodes * NOUT; i += kWaves * kWave) {
      const int node = sNode[i / NOUT];
      if (node >= 0) {
        const int64_t at = (static_cast<int64_t>(node) * ncomp + m) * nout_total + col0 + i % NOUT;
        OUT[at] = residual ? residual[at] : 0.f;
      }
    }
    return;
  }
  const float *Wg = WT + ((static_cast<int64_t>(g) * nblocks + l) * nout_total + col0) * K;  // [NOUT, K] of [nout_total, K]

  constexpr int kTPR = kKC / 4;
  constexpr int kRPP = kWaves * kWave / kTPR;
  static_assert(kRPP == NOUT, "one pass of the staging map covers the 32 weight rows");
  constexpr int A_PASSES = kTileNodes / kRPP;
  const int srow = tid / kTPR;
  const int scol = (tid % kTPR) * 4;
  const int mrow = lane % 32;
  const int half = lane / 32;

  // everything this workgroup reads, requested before anything is waited for
  f4 pa[KCH][A_PASSES], pb[KCH], ps[SCALED ? KCH : 1][A_PASSES];
#pragma unroll
  for (int i = 0; i < A_PASSES; ++i) {
    const int node = sNode[kRPP * i + srow];
    const float *xp = X + (static_cast<int64_t>(node >= 0 ? node : 0) * ncomp + m) * K + scol;
    const float *sp = SCALED ? row_scale + static_cast<int64_t>(node >= 0 ? node : 0) * K + scol : nullptr;
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      pa[c][i] = node >= 0 ? ld4_stream(xp + kKC * c) : zero4();
      if constexpr (SCALED) ps[c][i] = node >= 0 ? ld4(sp + kKC * c) : zero4();
    }
  }
#pragma unroll
  for (int c = 0; c < KCH; ++c) pb[c] = ld4(Wg + static_cast<int64_t>(srow) * K + kKC * c + scol);
  float res[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int node = sNode[32 * wave + 8 * (r / 4) + 4 * half + (r % 4)];
    res[r] = (residual && node >= 0) ? residual[(static_cast<int64_t>(node) * ncomp + m) * nout_total + col0 + mrow] : 0.f;
  }

  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
  for (int c = 0; c < KCH; ++c) {
    if (c > 0) __syncthreads();  // previous chunk fully consumed
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      f4 v = pa[c][i];
      if constexpr (SCALED) v *= ps[c][i];
      bf16x4 h, md, lw;
      split3(v, h, md, lw);
      const int at = (kRPP * i + srow) * kLdH + scol;
      *reinterpret_cast<bf16x4 *>(sAp + at) = h;
      *reinterpret_cast<bf16x4 *>(sAp + kTileNodes * kLdH + at) = md;
      *reinterpret_cast<bf16x4 *>(sAp + 2 * kTileNodes * kLdH + at) = lw;
    }
    {
      bf16x4 h, md, lw;
      split3(pb[c], h, md, lw);
      const int at = srow * kLdH + scol;
      *reinterpret_cast<bf16x4 *>(sBp + at) = h;
      *reinterpret_cast<bf16x4 *>(sBp + NOUT * kLdH + at) = md;
      *reinterpret_cast<bf16x4 *>(sBp + 2 * NOUT * kLdH + at) = lw;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < kKC; ks += 16) {
      const int aoff = (32 * wave + mrow) * kLdH + ks + 8 * half;
      bf16x8 a[3], b[3];
#pragma unroll
      for (int p = 0; p < 3; ++p) {
        a[p] = *reinterpret_cast<const bf16x8 *>(sAp + p * kTileNodes * kLdH + aoff);
        b[p] = *reinterpret_cast<const bf16x8 *>(sBp + p * NOUT * kLdH + mrow * kLdH + ks + 8 * half);
      }
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[2], b[0], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[2], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[1], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[0], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[1], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[0], acc, 0, 0, 0);
    }
  }

#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int node = sNode[32 * wave + 8 * (r / 4) + 4 * half + (r % 4)];
    if (node < 0) continue;
    float *op = OUT + (static_cast<int64_t>(node) * ncomp + m) * nout_total + col0 + mrow;
    {
#pragma clang fp contract(off)  // the product is rounded before the residual is added, as everywhere
      const float v = acc[r] * scale;
      *op = residual ? v + res[r] : v;
    }
  }
}

// -----------------------------------------------------------------------------------------------
// Variant with the feature rows on a ring of raw fp32 chunks in LDS, filled by direct global -> LDS loads.
//
// What bounds the kernel above is the amount of X that a workgroup has in flight: one 16 KB chunk, and only while it
// multiplies the previous one.  Here the X chunks never pass through registers: each wave fetches the 32 rows it
// multiplies itself, 16 bytes per lane, straight into a three-stage ring (global_load_lds_dwordx4), so one or two chunks
// are in flight at all times; it splits its rows into the bf16 pieces as it feeds the matrix cores (every row is split
// once, by its own wave, so this costs what the staging pass did, and the staged piece planes of X with their LDS
// writes and re-reads go away).  The weights take the old road (registers -> pieces -> LDS planes), one chunk ahead.
//
// Vector-memory operations retire in issue order and one counter covers them all.  The compiler would wait for "all
// of them" wherever it sees a load under a branch or a direct-to-LDS load that may alias a later LDS read, which
// would drain the ring at every chunk.  So every vector-memory operation of the main loop is issued from inline assembly,
// unseen by the compiler, in a fixed order, and waited for explicitly:
//     iteration c:   barrier | wait: all but the 4 loads of X chunk c+1 | weights c -> planes | issue weights c+1
//                    (and scales c+1), then X chunk c+2 | barrier | multiply chunk c
// The assembly statements that wait also carry the loaded registers as read-write operands, which keeps every use
// behind the wait.  M0 (the LDS address of a direct load) is written inside those statements; nothing else in this
// kernel uses it.
//
// LDS layout of a ring stage: row r of the tile at r * 128 bytes, its eight 16-byte pieces at positions
// piece ^ (r & 7), so that the 32 rows a wave reads at the same piece index fall on different banks (a direct load
// writes lane i at base + 16 i: the layout is chosen through which piece each lane fetches).
// -----------------------------------------------------------------------------------------------
constexpr int kStages = 3;
constexpr int kStageBytes = kTileNodes * kKC * 4;

// M0 is written here and named as clobbered; the compiler reserves that register and warns that it does not track it
// across the statement, which is the point of the remark in the comment above: nothing else in this kernel may rely on it.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma16(const float *src, unsigned lds_byte_address) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" : : "v"(src), "s"(lds_byte_address) : "memory", "m0");
}
#pragma clang diagnostic pop
__device__ __forceinline__ void ldg16(f4 &dst, const float *src) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(src) : "memory");
}
// Marks the point from which a register that a hand-issued load lands in holds the loaded value (the wait that covers the
// load precedes it): no use can move above it, and the build's scan of the generated code, which refuses any instruction
// that touches such a register between the load's issue and this mark, reads the comment it leaves in the assembly.
__device__ __forceinline__ void after_wait(f4 &v) { asm volatile("; landed %0" : "+v"(v)); }

// two workgroups per compute unit (two waves per SIMD) wherever LDS allows it: 256 registers per lane
template <int NT, bool SCALED>
__global__ __launch_bounds__(kWaves *kWave, (NT <= 4 ? 2 : 1)) void linear_ring_kernel(const float *__restrict__ X, const float *__restrict__ WT,
                                                                    const int32_t *__restrict__ node_perm,
                                                                    const int32_t *__restrict__ group_offsets, int nnodes,
                                                                    int ngroups, int zero_last_group, int ncomp, int K,
                                                                    float scale, const float *__restrict__ row_scale,
                                                                    const float *residual, float *OUT) {
  constexpr int NOUT = 32 * NT;
  __shared__ __attribute__((aligned(16))) float sRaw[kStages * kTileNodes * kKC];
  __shared__ __attribute__((aligned(16))) __bf16 sBp[3 * NOUT * kLdH];
  __shared__ int sNode[kTileNodes];

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int m = blockIdx.x % ncomp;
  const int l = ncomp == 1 ? 0 : l_of_m(m);
  const int nblocks = ncomp == 1 ? 1 : 4;

  int g, pos0, gend;
  if (!locate_group_tile(group_offsets, ngroups, nnodes, blockIdx.x / ncomp, kTileNodes, g, pos0, gend)) return;
  const int nrows = min(kTileNodes, gend - pos0);

  if (tid < kTileNodes) {
    int node = -1;
    if (tid < nrows) {
      node = node_perm ? node_perm[pos0 + tid] : pos0 + tid;
      if (static_cast<unsigned>(node) >= static_cast<unsigned>(nnodes)) node = -1;
    }
    sNode[tid] = node;
  }
  __syncthreads();

  if (zero_last_group && g == ngroups - 1) {
    for (int i = tid; i < kTileNodes * NOUT; i += kWaves * kWave) {
      const int node = sNode[i / NOUT];
      if (node >= 0) {
        const int64_t at = (static_cast<int64_t>(node) * ncomp + m) * NOUT + i % NOUT;
        OUT[at] = residual ? residual[at] : 0.f;
      }
    }
    return;
  }
  const float *Wg = WT + (static_cast<int64_t>(g) * nblocks + l) * NOUT * K;  // [NOUT, K]

  v16f acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;

  // weights: staging map as in the kernel above (8 threads x 16 bytes per row of the chunk, 32 rows per pass)
  constexpr int kTPR = kKC / 4;
  constexpr int kRPP = kWaves * kWave / kTPR;
  static_assert(kRPP == 32 && NOUT % kRPP == 0, "staging map");
  const int srow = tid / kTPR;
  const int scol = (tid % kTPR) * 4;
  const float *wsrc = Wg + static_cast<int64_t>(srow) * K + scol;  // + 32 i K for pass i, + kc
  // matrix-core operand map
  const int mrow = lane % 32;
  const int half = lane / 32;

  // X: one direct load covers 8 rows x 128 bytes; a wave issues four per chunk, for its own 32 rows.  Rows beyond the
  // tile fetch row 0 of X (their products are never stored).
  const int drow = lane / 8;
  const int dpiece = (lane & 7) ^ drow;
  const float *xsrc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int node = sNode[32 * wave + 8 * i + drow];
    xsrc[i] = X + (static_cast<int64_t>(node >= 0 ? node : 0) * ncomp + m) * K + 4 * dpiece;
  }
  const unsigned raw_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(sRaw)) + static_cast<unsigned>(wave) * (32 * kKC * 4);
  auto issue_x = [&](int kc, int stage) {
#pragma unroll
    for (int i = 0; i < 4; ++i) dma16(xsrc[i] + kc, raw_base + static_cast<unsigned>(stage) * kStageBytes + i * (8 * kKC * 4));
  };
  // the wave's own A fragments: 8 consecutive k of row 32 wave + mrow, i.e. pieces ks/4 + 2 half and the next one
  const float *araw = sRaw + (32 * wave + mrow) * kKC;
  const int swz = mrow & 7;

  f4 pb[NT];
  f4 sc[2][4];
  const float *ssrc = nullptr;
  if constexpr (SCALED) {
    const int node = sNode[32 * wave + mrow];
    ssrc = row_scale + static_cast<int64_t>(node >= 0 ? node : 0) * K + 8 * half;
  }
  auto issue_w = [&](int kc, auto par) {
    constexpr int P = decltype(par)::value;
#pragma unroll
    for (int i = 0; i < NT; ++i) ldg16(pb[i], wsrc + static_cast<int64_t>(kRPP * i) * K + kc);
    if constexpr (SCALED) {
#pragma unroll
      for (int q = 0; q < 4; ++q) ldg16(sc[P][q], ssrc + kc + 16 * (q / 2) + 4 * (q % 2));
    }
  };

  // What the next iteration consumes has landed when an iteration (or the prologue) ends: the wait sits at the end of
  // the code that issued the loads, so that every register a load was issued into passes through after_wait before
  // the loop's back edge (a copy the compiler makes there then copies the loaded value).
  auto landed = [&](auto par) {
    constexpr int P = decltype(par)::value;
#pragma unroll
    for (int i = 0; i < NT; ++i) after_wait(pb[i]);
    if constexpr (SCALED) {
#pragma unroll
      for (int q = 0; q < 4; ++q) after_wait(sc[P][q]);
    }
  };
  const int nch = K / kKC;
  issue_w(0, std::integral_constant<int, 0>{});
  issue_x(0, 0);
  if (nch > 1) {
    issue_x(kKC, 1);
    asm volatile("s_waitcnt vmcnt(4)" ::: "memory");  // all but the four loads of X chunk 1
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  landed(std::integral_constant<int, 0>{});

  auto iteration = [&](int c, int stage, auto par) {
    constexpr int P = decltype(par)::value;
    const int kc = c * kKC;
    // every wave has finished multiplying chunk c - 1: the weight planes and ring stage (c + 2) % 3 are free.  Weights
    // (and scales) of chunk c and X chunk c have landed (waited for where they were issued); the four loads of X chunk
    // c + 1 may still be out
    asm volatile("s_barrier" ::: "memory");
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      bf16x4 h, md, lw;
      split3(pb[i], h, md, lw);
      const int at = (kRPP * i + srow) * kLdH + scol;
      *reinterpret_cast<bf16x4 *>(sBp + at) = h;
      *reinterpret_cast<bf16x4 *>(sBp + NOUT * kLdH + at) = md;
      *reinterpret_cast<bf16x4 *>(sBp + 2 * NOUT * kLdH + at) = lw;
    }
    if (c + 1 < nch) issue_w(kc + kKC, std::integral_constant<int, 1 - P>{});
    if (c + 2 < nch) issue_x(kc + 2 * kKC, stage >= 1 ? stage - 1 : 2);  // (stage + 2) % 3
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // weight planes written

    const float *ast = araw + stage * (kTileNodes * kKC);
#pragma unroll
    for (int ks = 0; ks < kKC; ks += 16) {
      const int piece = ks / 4 + 2 * half;
      f4 r0 = *reinterpret_cast<const f4 *>(ast + 4 * (piece ^ swz));
      f4 r1 = *reinterpret_cast<const f4 *>(ast + 4 * ((piece + 1) ^ swz));
      if constexpr (SCALED) {
        r0 *= sc[P][2 * (ks / 16)];
        r1 *= sc[P][2 * (ks / 16) + 1];
      }
      bf16x4 h0, m0, l0, h1, m1, l1;
      split3(r0, h0, m0, l0);
      split3(r1, h1, m1, l1);
      bf16x8 a[3], b[NT][3];
      a[0] = __builtin_shufflevector(h0, h1, 0, 1, 2, 3, 4, 5, 6, 7);
      a[1] = __builtin_shufflevector(m0, m1, 0, 1, 2, 3, 4, 5, 6, 7);
      a[2] = __builtin_shufflevector(l0, l1, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int p = 0; p < 3; ++p)
          b[t][p] = *reinterpret_cast<const bf16x8 *>(sBp + p * NOUT * kLdH + (32 * t + mrow) * kLdH + ks + 8 * half);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[2], b[t][0], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[t][2], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[t][1], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[t][0], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[t][1], acc[t], 0, 0, 0);
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[t][0], acc[t], 0, 0, 0);
    }
    // the next chunk's weights, scales and X rows: everything but the four loads of the X chunk after it, if one was issued
    if (c + 1 < nch) {
      if (c + 2 < nch)
        asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
      else
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    landed(std::integral_constant<int, 1 - P>{});
  };
  int stage = 0;
  for (int c = 0; c < nch; c += 2) {
    iteration(c, stage, std::integral_constant<int, 0>{});
    stage = stage == 2 ? 0 : stage + 1;
    if (c + 1 >= nch) break;
    iteration(c + 1, stage, std::integral_constant<int, 1>{});
    stage = stage == 2 ? 0 : stage + 1;
  }
  // Nothing is in flight here (the last chunk waited for everything and issued nothing); said once more in a form that
  // the build's scan of the generated code, which does not know that the loop issues only while it goes on, can read.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  if constexpr (NT <= 4) {
    // Output through LDS, so that rows leave as 16-byte stores (a lane's accumulators are one column of 16 rows: stored
    // directly they are 64 four-byte stores per lane).  Every wave is past its last multiply after the barrier, so the
    // ring and the weight planes are free: each wave lays its 32 x Nout block out row-major in its own piece of them.
    asm volatile("s_barrier" ::: "memory");
    constexpr int TILE = 32 * NOUT;  // floats per wave
    static_assert(4 * TILE <= kStages * kTileNodes * kKC || (3 * TILE <= kStages * kTileNodes * kKC && TILE * 4 <= 3 * NOUT * kLdH * 2),
                  "output staging does not fit the ring and the weight planes");
    float *tile = (4 * TILE <= kStages * kTileNodes * kKC || wave < 3) ? sRaw + wave * TILE : reinterpret_cast<float *>(sBp);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = 8 * (r / 4) + 4 * half + (r % 4);
#pragma unroll
      for (int t = 0; t < NT; ++t) tile[row * NOUT + 32 * t + mrow] = acc[t][r] * scale;
    }
    constexpr int PPR = NOUT / 4;  // 16-byte pieces per row
#pragma unroll
    for (int i = 0; i < TILE / 4 / kWave; ++i) {
      const int q = i * kWave + lane;
      const int row = q / PPR, col = 4 * (q % PPR);
      const int node = sNode[32 * wave + row];
      if (node >= 0) {
        const int64_t at = (static_cast<int64_t>(node) * ncomp + m) * NOUT + col;
        f4 v = *reinterpret_cast<const f4 *>(tile + row * NOUT + col);
        if (residual) v += ld4(residual + at);  // may be OUT itself: every element is read and written by the same lane
        st4(OUT + at, v);
      }
    }
  } else {
    store_block<NT>(acc, sNode, wave, half, mrow, ncomp, m, NOUT, 0, scale, residual, OUT);
  }
}

// -----------------------------------------------------------------------------------------------
// Variant with the weights resident in LDS (16 components per node, K = Nout up to 128).
//
// The kernels above stage the K x Nout weight block again for every tile of 128 rows (as many bytes from L2 as the tile
// has from HBM) and walk K in barrier-separated phases.  Here a launch has one workgroup per compute unit, and a
// workgroup takes a contiguous piece of the list of all 32-row tiles, ordered by (weight group, l, node tile, m within
// l), so that it needs one or two weight blocks in its whole life: it splits a block once into three bf16 planes that
// cover all of K (102 KB at 128 x 128) and then its four waves run independently of each other, one 32-row tile at a
// time, with no barrier until the weight block changes.
//
// What a wave has in flight lives in registers, not in LDS: the loads of tile i + 1 (16 x 16 bytes per lane at 128
// columns, whole 128-byte lines of 8 rows per instruction) are issued before tile i is multiplied and land in
// accumulator-file registers; 64 KB per compute unit are on their way at any time.  When its turn comes a tile changes
// from that row-major layout to the operand layout of the matrix instruction (a lane holds 8 values of one row per
// 16-wide k step) through the wave's own corner of LDS, 64 columns at a time.  The order of k inside a step is free as
// long as both operands agree; it is chosen such that a lane reads two aligned 16-byte pieces.  The operands are swapped
// with respect to the kernels above (weights as the row operand, X rows as the column operand): a lane's accumulators
// are then 4 consecutive output columns of one row; a block of 32 columns goes back through the same corner of LDS and
// leaves as whole lines.  The piece products and their order are those of the kernels above.
//
// Contract of the hand-issued memory operations of the tile loop (the loads and the stores): a load names its landing
// registers at issue time although the data arrives by the explicit wait that precedes their first use, which is
// sound only while the compiler neither copies nor spills them in between; they are accumulator-file registers,
// which nothing else in the kernel wants, and the build refuses scratch memory in this kernel and any instruction other
// than a load that writes a register its loads land in.  A store is followed by the two idle issue slots that the hardware needs before the
// stored registers may be overwritten (the compiler inserts them for the stores it knows; without them the last lanes of
// the following block were stored instead).
//
// What was measured on the way (25 000 x 128, one box each): loads of 32 bytes per lane and row, which is what a lane
// feeds per k step, request every line four times, and the kernel then ran at the rate of the compute unit's queue of
// outstanding misses (118 us; whole lines: 99 us); stores under a branch make the compiler wait for everything in
// flight at the top of the loop (hence no conditional rows, see the row numbers below); weaving the operand split of
// the next k step between the matrix instructions took it to 87 us.  Without its matrix instructions the kernel takes
// 62 us and without its loads and stores 72 us: what remains is that one wave per SIMD does its memory waits, its LDS
// round trips and its matrix instructions one after the other.  Two waves per SIMD (eight waves, a tile landing in
// chunks of 32 columns, no weaving) came out equal at this size and 7 % slower at 100 000 nodes; two tiles ahead
// instead of one changes nothing (and 64 outstanding instructions per wave is where the counter ends).
// -----------------------------------------------------------------------------------------------
constexpr int kResWaves = 4;
constexpr int kResMaxGroups = 128;
constexpr int kResMinNodes = 2048;
constexpr int kOutLd = 36;            // floats per row of a wave's output staging block (32 columns + 16 bytes)
constexpr int kResSegNodeTiles = 64;  // node tiles whose row numbers a segment keeps in LDS

template <int K, int NT, bool SCALED>
__global__ __launch_bounds__(kResWaves *kWave, 1) void linear_resident_kernel(
    const float *__restrict__ X, const float *__restrict__ WT, const int32_t *__restrict__ node_perm,
    const int32_t *__restrict__ group_offsets, int nnodes, int ngroups, int zero_last_group, int ldo, float scale,
    const float *__restrict__ row_scale, float *__restrict__ OUT) {
  constexpr int NOUT = 32 * NT;  // columns of this workgroup: blockIdx.y * NOUT onwards of the ldo columns of OUT
  constexpr int LD = K + 8;      // row stride of a plane in elements: an odd number of 16-byte units
  constexpr int KS = K / 16;
  __shared__ __attribute__((aligned(16))) __bf16 sW[3 * NOUT * LD];
  __shared__ int sId[kResSegNodeTiles * 32];
  constexpr int kChunk = K <= 96 ? K : 64;  // columns of X per trip through LDS
  constexpr int kTLd = kChunk + 4;          // floats per row of the transposition block: an odd number of 16-byte units
  constexpr int kStageFloats = 32 * (kTLd > kOutLd ? kTLd : kOutLd);  // a wave's own corner of LDS
  __shared__ __attribute__((aligned(16))) float sStage[kResWaves * kStageFloats];
  __shared__ int sOff[kResMaxGroups + 1];
  __shared__ int sCum[kResMaxGroups + 1];

  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int mrow = lane % 32;
  const int half = lane / 32;
  const int c0 = blockIdx.y * NOUT;

  // groups that have weights, their row ranges in the grouped node order and their first tile in the tile list
  const int ngw = zero_last_group ? ngroups - 1 : ngroups;
  if (tid == 0) {
    int cum = 0;
    for (int g = 0; g < ngw; ++g) {
      const int lo = group_offsets ? group_offsets[g] : 0, hi = group_offsets ? group_offsets[g + 1] : nnodes;
      sOff[g] = lo;
      sCum[g] = cum;
      cum += 16 * ((max(hi - lo, 0) + 31) / 32);
    }
    sOff[ngw] = group_offsets ? group_offsets[ngw] : nnodes;
    sCum[ngw] = cum;
  }
  if (zero_last_group && blockIdx.y == 0) {
    // rows that belong to no weight group: the product is defined as zero (a residual still passes through)
    const int z0 = group_offsets[ngroups - 1], nz = group_offsets[ngroups] - z0;
    const int rowq = 16 * ldo / 4;
    const int64_t total = static_cast<int64_t>(nz) * rowq;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + tid; i < total; i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
      const int node = node_perm[z0 + static_cast<int>(i / rowq)];
      if (static_cast<unsigned>(node) < static_cast<unsigned>(nnodes)) st4(OUT + static_cast<int64_t>(node) * 16 * ldo + 4 * (i % rowq), zero4());
    }
  }
  __syncthreads();

  const int ntiles = sCum[ngw];
  const int i1 = static_cast<int>(static_cast<int64_t>(ntiles) * (blockIdx.x + 1) / gridDim.x);
  int i = static_cast<int>(static_cast<int64_t>(ntiles) * blockIdx.x / gridDim.x);
  int g = 0, staged_g = -1, staged_l = -1;

  while (i < i1) {
    while (sCum[g + 1] <= i) ++g;
    const int tg = (sCum[g + 1] - sCum[g]) / 16;  // node tiles of the group
    const int l = l_of_m((i - sCum[g]) / tg);
    const int nm = 2 * l + 1;
    const int blk0 = sCum[g] + tg * l * l;        // first tile of (g, l): tile blk0 + t * nm + (m - l * l)
    const int t_first = (i - blk0) / nm;
    const int seg_end = min(min(i1, blk0 + tg * nm), blk0 + (t_first + kResSegNodeTiles) * nm);
    const int t_count = (seg_end - 1 - blk0) / nm - t_first + 1;
    const int off0 = sOff[g], off1 = sOff[g + 1];

    __syncthreads();  // every wave is done with the previous segment
    // Row numbers of the segment's node tiles.  A row beyond the end of the group (or an index outside the node range)
    // stands in for the first row of its tile: it then computes that row's values once more and stores the same bits
    // to the same place, so that no load or store of the tile loop is conditional.
    for (int r = tid; r < 32 * t_count; r += kResWaves * kWave) {
      const int p0 = off0 + 32 * (t_first + r / 32);
      const int p = p0 + r % 32;
      int node = node_perm ? node_perm[p < off1 ? p : p0] : (p < off1 ? p : p0);
      if (static_cast<unsigned>(node) >= static_cast<unsigned>(nnodes)) node = node_perm ? node_perm[p0] : p0;
      if (static_cast<unsigned>(node) >= static_cast<unsigned>(nnodes)) node = 0;
      sId[r] = node;
    }
    if (g != staged_g || l != staged_l) {
      // W^T[c0 + j, :] of block (g, l) -> three planes; inside every 16 k the two middle groups of four trade places, so
      // that the 8 values a lane reads at 16 s + 8 half are k = 16 s + 4 half + {0..3, 8..11}
      const float *Wg = WT + ((static_cast<int64_t>(g) * 4 + l) * ldo + c0) * K;
      // all loads of a thread first (16 at 128 x 128), then the splits: one trip through L2 instead of one per piece
      constexpr int kPieces = NOUT * (K / 4) / (kResWaves * kWave);
      static_assert(NOUT * (K / 4) % (kResWaves * kWave) == 0, "weight staging map");
      f4 wv[kPieces];
#pragma unroll
      for (int it = 0; it < kPieces; ++it) {
        const int q = it * (kResWaves * kWave) + tid;
        wv[it] = ld4(Wg + static_cast<int64_t>(q / (K / 4)) * K + 4 * (q % (K / 4)));
      }
#pragma unroll
      for (int it = 0; it < kPieces; ++it) {
        const int q = it * (kResWaves * kWave) + tid;
        const int j = q / (K / 4), kq = q % (K / 4);
        bf16x4 h, md, lw;
        split3(wv[it], h, md, lw);
        const int sub = kq & 3;
        const int at = j * LD + 16 * (kq >> 2) + 4 * (sub == 1 ? 2 : (sub == 2 ? 1 : sub));
        *reinterpret_cast<bf16x4 *>(sW + at) = h;
        *reinterpret_cast<bf16x4 *>(sW + NOUT * LD + at) = md;
        *reinterpret_cast<bf16x4 *>(sW + 2 * NOUT * LD + at) = lw;
      }
      staged_g = g;
      staged_l = l;
    }
    __syncthreads();

    // this wave's contiguous share of the segment
    const int per = (seg_end - i + kResWaves - 1) / kResWaves;
    const int wb = i + wave * per, we = min(seg_end, wb + per);
    i = seg_end;
    if (wb >= we) continue;

    // Tile loop.  Every global access in it is issued from assembly in a fixed order and waited for by an explicit count
    // (the compiler would sink part of a prefetch down to its use and then wait for everything that is in flight, the
    // stores of the previous tile included):
    //     tile i:  wait: all but the stores of tile i - 1 | landing registers -> working registers (times row_scale)
    //              | issue the loads of tile i + 1 | multiply | output block by block through LDS, issue the stores
    // The landing registers are accumulator-file registers (a load may write them directly; nothing else competes for
    // them, so the compiler has no reason to move them while a load is in flight), the working set lives in ordinary
    // registers.
    // Loads are whole lines: one instruction fetches 128 bytes of each of 8 rows (lane = 16-byte piece opiece of row
    // 8 rg + orow; in 32-byte pieces, which is what a lane feeds per k step, every line would be requested four times and
    // the compute unit's queue of outstanding misses would hold a quarter of the bytes).  The landed values change to the
    // operand layout through the wave's own corner of LDS, kChunk columns at a time.
    constexpr int kLines = kChunk / 32;  // 128-byte lines of a row per chunk
    constexpr int kChunks = K / kChunk;
    static_assert(K % kChunk == 0 && kChunk % 32 == 0, "chunks of whole lines");
    f4 land[2 * KS];                           // index (chunk * 4 + rg) * kLines + line
    f4 sland[SCALED ? 2 * KS : 1];
    float *stg = sStage + wave * kStageFloats;
    const int orow = lane / 8, opiece = lane % 8;
    int t_scales = -1;  // node tile whose row_scale rows are in (or on their way into) sland
    auto issue = [&](int idx, int &m_of, int &tb_of) {
      const int j = idx - blk0;
      const int t = j / nm;
      m_of = l * l + (j - t * nm);
      tb_of = 32 * (t - t_first);
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int nd = sId[tb_of + 8 * rg + orow];
        const float *xp = X + (static_cast<int64_t>(nd) * 16 + m_of) * K + 4 * opiece;
#pragma unroll
        for (int c = 0; c < kChunks; ++c)
#pragma unroll
          for (int ln = 0; ln < kLines; ++ln)
            asm volatile("global_load_dwordx4 %0, %1, off offset:%2 nt" : "=a"(land[(c * 4 + rg) * kLines + ln]) : "v"(xp), "n"(4 * (c * kChunk + 32 * ln)) : "memory");
      }
      if constexpr (SCALED) {
        // the 2 l + 1 tiles of a node tile follow each other and share their row_scale rows: fetched once (these loads
        // are older than the stores the wait at the top of a tile lets stay out, whether they are issued or not)
        if (t != t_scales) {
          t_scales = t;
#pragma unroll
          for (int rg = 0; rg < 4; ++rg) {
            const float *sp = row_scale + static_cast<int64_t>(sId[tb_of + 8 * rg + orow]) * K + 4 * opiece;
#pragma unroll
            for (int c = 0; c < kChunks; ++c)
#pragma unroll
              for (int ln = 0; ln < kLines; ++ln)
                asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=a"(sland[(c * 4 + rg) * kLines + ln]) : "v"(sp), "n"(4 * (c * kChunk + 32 * ln)) : "memory");
          }
        }
      }
    };
    const __bf16 *wl = sW + mrow * LD + 8 * half;
    int m_next, tb_next;
    issue(wb, m_next, tb_next);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    for (int idx = wb; idx < we; ++idx) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * NT) : "memory");
      const int m_cur = m_next, tb_cur = tb_next;
      f4 cur[2 * KS];
#pragma unroll
      for (int c = 0; c < kChunks; ++c) {
        wave_lds_fence();
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)
#pragma unroll
          for (int ln = 0; ln < kLines; ++ln) {
            const int j = (c * 4 + rg) * kLines + ln;
            asm volatile("; landed %0" : "+a"(land[j]));
            f4 v = land[j];
            if constexpr (SCALED) {
              asm volatile("; landed %0" : "+a"(sland[j]));
              v *= sland[j];
            }
            *reinterpret_cast<f4 *>(stg + (8 * rg + orow) * kTLd + 32 * ln + 4 * opiece) = v;
          }
        wave_lds_fence();
        // k step s of the chunk: the lane's values are columns 16 s + 4 half + {0..3} and 16 s + 8 + 4 half + {0..3}
#pragma unroll
        for (int sc = 0; sc < kChunk / 16; ++sc) {
          const int s = c * (kChunk / 16) + sc;
          cur[2 * s] = *reinterpret_cast<const f4 *>(stg + mrow * kTLd + 16 * sc + 4 * half);
          cur[2 * s + 1] = *reinterpret_cast<const f4 *>(stg + mrow * kTLd + 16 * sc + 8 + 4 * half);
        }
      }
#pragma unroll
      for (int j = 0; j < 2 * KS; ++j) asm volatile("" : "+v"(cur[j]));
      if (idx + 1 < we) issue(idx + 1, m_next, tb_next);

      v16f acc[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
      // One wave per SIMD: nothing but this wave's own instruction stream can fill the issue slots between two matrix
      // instructions (32 cycles apart), so the k loop is pipelined in the source: the pieces of X and the weight fragments of
      // step s + 1 are prepared while the 6 NT matrix instructions of step s run, and the scheduler is told to weave them
      // (per matrix instruction: three vector instructions, and an LDS read for the first 3 NT of them).
      constexpr int kSplitOps = (64 + 6 * NT - 1) / (6 * NT);  // the split of a step is about 60 vector instructions
      bf16x8 xq[2][3], wq[2][NT][3];
      auto prepare = [&](int s, auto par) {
        constexpr int P = decltype(par)::value;
        bf16x4 h0, m0, l0, h1, m1, l1;
        split3(cur[2 * s], h0, m0, l0);
        split3(cur[2 * s + 1], h1, m1, l1);
        xq[P][0] = __builtin_shufflevector(h0, h1, 0, 1, 2, 3, 4, 5, 6, 7);
        xq[P][1] = __builtin_shufflevector(m0, m1, 0, 1, 2, 3, 4, 5, 6, 7);
        xq[P][2] = __builtin_shufflevector(l0, l1, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int p = 0; p < 3; ++p) wq[P][t][p] = *reinterpret_cast<const bf16x8 *>(wl + p * NOUT * LD + 32 * t * LD + 16 * s);
      };
      auto step = [&](int s, auto par) {
        constexpr int P = decltype(par)::value;
        if (s + 1 < KS) prepare(s + 1, std::integral_constant<int, 1 - P>{});
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wq[P][t][0], xq[P][2], acc[t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wq[P][t][2], xq[P][0], acc[t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wq[P][t][1], xq[P][1], acc[t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wq[P][t][0], xq[P][1], acc[t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wq[P][t][1], xq[P][0], acc[t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wq[P][t][0], xq[P][0], acc[t], 0, 0, 0);
        if (s + 1 < KS) {
#pragma unroll
          for (int i = 0; i < 6 * NT; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                  // one matrix instruction
            if (i < 3 * NT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
            __builtin_amdgcn_sched_group_barrier(0x002, kSplitOps, 0);          // a share of the split arithmetic
          }
        }
        // nothing else moves across k steps: fragment reads of later steps hoisted further would not fit the register file
        __builtin_amdgcn_sched_barrier(0);
      };
      prepare(0, std::integral_constant<int, 0>{});
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < KS; s += 2) {
        step(s, std::integral_constant<int, 0>{});
        if (s + 1 < KS) step(s + 1, std::integral_constant<int, 1>{});
      }
      // accumulator r of a lane: output column 32 t + 8 (r / 4) + 4 half + r % 4 of row mrow of the tile.  Stored from
      // here a row would leave in 32-byte pieces; a block of 32 columns goes through the wave's own corner of LDS instead
      // (rows padded to 9 x 16 bytes: conflict-free both ways) and leaves as whole 128-byte lines, 8 rows per store.
      float *orows[4];
#pragma unroll
      for (int r = 0; r < 4; ++r)
        orows[r] = OUT + (static_cast<int64_t>(sId[tb_cur + 8 * r + orow]) * 16 + m_cur) * ldo + c0 + 4 * opiece;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        wave_lds_fence();
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<f4 *>(stg + mrow * kOutLd + 8 * q + 4 * half) = f4{acc[t][4 * q], acc[t][4 * q + 1], acc[t][4 * q + 2], acc[t][4 * q + 3]} * scale;
        wave_lds_fence();
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const f4 v = *reinterpret_cast<const f4 *>(stg + (8 * r + orow) * kOutLd + 4 * opiece);
          // the two idle issue slots are what the compiler puts between a 16-byte store and an instruction that
          // overwrites the registers it stores from; it does not see this store
          asm volatile("global_store_dwordx4 %0, %1, off offset:%2\n\ts_nop 1" : : "v"(orows[r]), "v"(v), "n"(128 * t) : "memory");
        }
      }
    }
    // every landing register has been consumed: nothing this wave issued can still write a register
  }
}

template <int K, int NT>
int launch_resident(const float *X, const float *WT, const int32_t *perm, const int32_t *offs, int64_t nnodes, int ngroups,
                    int zero_last_group, int Nout, float scale, const float *row_scale, float *OUT, hipStream_t st) {
  // one workgroup per compute unit.  (The kernel can also split the columns over grid.y, 32 NT per workgroup: the
  // workgroups that share X rows are then a multiple of 8 apart in launch order, i.e. on one XCD and its L2.  Measured at
  // 192 = 2 x 96 and 256 = 4 x 64 columns it only equals the kernels above, because every column block splits the X rows
  // again, so those widths are not routed here.)
  const int ycount = Nout / (32 * NT);
  const dim3 grid(static_cast<unsigned>(std::max(8, device_compute_units() / ycount / 8 * 8)), static_cast<unsigned>(ycount)), block(kResWaves * kWave);
  if (row_scale)
    hipLaunchKernelGGL((linear_resident_kernel<K, NT, true>), grid, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes), ngroups,
                       zero_last_group, Nout, scale, row_scale, OUT);
  else
    hipLaunchKernelGGL((linear_resident_kernel<K, NT, false>), grid, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes), ngroups,
                       zero_last_group, Nout, scale, row_scale, OUT);
  return check_launch("cm_linear");
}

template <int NT>
int launch(const float *X, const float *WT, const int32_t *perm, const int32_t *offs, int64_t nnodes, int ngroups,
           int zero_last_group, int ncomp, int K, float scale, const float *row_scale, const float *residual, float *OUT,
           hipStream_t st) {
  const int64_t tiles = ceil_div(nnodes, kTileNodes) + (offs ? ngroups : 0);
  const dim3 grid(static_cast<unsigned>(tiles * ncomp)), block(kWaves * kWave);
  constexpr int NOUT = 32 * NT;
  // few tiles (less than half a workgroup per compute unit): 32 columns per workgroup
  if (NT > 1 && tiles * ncomp * 2 <= device_compute_units()) {
    const dim3 split(grid.x, NT);
    if (K <= 4 * kKC) {  // every chunk requested at once (registers for four of them)
#define CM_FEW(KCH_, SCALED_)                                                                                                       \
  hipLaunchKernelGGL((linear_few_tiles_kernel<KCH_, SCALED_>), split, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes), ngroups, \
                     zero_last_group, ncomp, scale, row_scale, residual, OUT, NOUT)
      switch (K / kKC) {
        case 1: if (row_scale) CM_FEW(1, true); else CM_FEW(1, false); break;
        case 2: if (row_scale) CM_FEW(2, true); else CM_FEW(2, false); break;
        case 3: if (row_scale) CM_FEW(3, true); else CM_FEW(3, false); break;
        default: if (row_scale) CM_FEW(4, true); else CM_FEW(4, false); break;
      }
#undef CM_FEW
      return check_launch("cm_linear");
    }
    if (row_scale)
      hipLaunchKernelGGL((linear_kernel<1, true>), split, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes), ngroups,
                         zero_last_group, ncomp, K, scale, row_scale, residual, OUT, NOUT);
    else
      hipLaunchKernelGGL((linear_kernel<1, false>), split, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes), ngroups,
                         zero_last_group, ncomp, K, scale, row_scale, residual, OUT, NOUT);
    return check_launch("cm_linear");
  }
  // The ring variant wherever it runs two workgroups per compute unit or the plain one does not either (Nout up to 128,
  // and 224 / 256), and K has more than one chunk to overlap; measured at 25 000 nodes: 108 vs 119-127 us at 128
  // columns, 76 vs 80-83 at 96, equal at 64, 224 and 256, slower at 32 (one chunk), 160 and 192 (one workgroup per CU).
  // The row_scale variant at 256 columns does not fit the register file and would spill, which the hand-issued loads
  // of the ring kernel do not tolerate (the build checks that no instantiated ring kernel uses scratch memory): it
  // runs on the plain kernel.
  constexpr bool kRing = NT == 2 || NT == 3 || NT == 4 || NT >= 7;
  constexpr bool kRingScaled = kRing && NT < 8;
  if constexpr (kRing) {
    if (K > kKC && (!row_scale || kRingScaled)) {
      if constexpr (kRingScaled) {
        if (row_scale) {
          hipLaunchKernelGGL((linear_ring_kernel<NT, true>), grid, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes),
                             ngroups, zero_last_group, ncomp, K, scale, row_scale, residual, OUT);
          return check_launch("cm_linear");
        }
      }
      hipLaunchKernelGGL((linear_ring_kernel<NT, false>), grid, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes), ngroups,
                         zero_last_group, ncomp, K, scale, row_scale, residual, OUT);
      return check_launch("cm_linear");
    }
  }
  if (row_scale)
    hipLaunchKernelGGL((linear_kernel<NT, true>), grid, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes), ngroups,
                       zero_last_group, ncomp, K, scale, row_scale, residual, OUT, NOUT);
  else
    hipLaunchKernelGGL((linear_kernel<NT, false>), grid, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes), ngroups,
                       zero_last_group, ncomp, K, scale, row_scale, residual, OUT, NOUT);
  return check_launch("cm_linear");
}

}  // namespace
}  // namespace cm

extern "C" int cm_linear(const float *X, const float *W_T, const int32_t *node_perm, const int32_t *group_offsets,
                         int64_t nnodes, int ngroups, int zero_last_group, int ncomp, int K, int Nout, float scale,
                         const float *row_scale, const float *residual, float *OUT, cm_stream_t stream) {
  CM_REQUIRE(ncomp == 1 || ncomp == 16, "cm_linear: ncomp=%d must be 1 or 16", ncomp);
  CM_REQUIRE(!zero_last_group || (group_offsets != nullptr && ngroups >= 2),
             "cm_linear: a zero group needs node_perm / group_offsets and at least one weight group before it");
  CM_REQUIRE(nnodes >= 0 && nnodes < INT32_MAX / 16, "cm_linear: nnodes out of range");
  CM_REQUIRE(K >= 32 && K <= 256 && K % 32 == 0, "cm_linear: K=%d must be a multiple of 32 in [32, 256]", K);
  CM_REQUIRE(Nout >= 32 && Nout <= 256 && Nout % 32 == 0, "cm_linear: Nout=%d must be a multiple of 32 in [32, 256]", Nout);
  CM_REQUIRE(ngroups >= 1, "cm_linear: ngroups must be at least 1");
  CM_REQUIRE((node_perm == nullptr) == (group_offsets == nullptr), "cm_linear: node_perm and group_offsets go together");
  CM_REQUIRE(group_offsets != nullptr || ngroups == 1, "cm_linear: ngroups > 1 needs node_perm / group_offsets");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(X && W_T && OUT, "cm_linear: NULL pointer");
  hipStream_t st = cm::as_stream(stream);
  // 16 components per node, square weights up to 128 and enough rows to give every compute unit a few tiles: the
  // kernel that keeps the weights in LDS (measured against the ring kernel at 25 000 nodes: 87 vs 102-112 us at 128
  // channels, 58 vs 67-71 at 96, 42 vs 47 at 64; 360 vs 430 us at 100 000 x 128; equal at 2 500 nodes)
  if (ncomp == 16 && K == Nout && !residual && ngroups <= cm::kResMaxGroups && nnodes >= cm::kResMinNodes) {
    switch (K) {
#define CM_CASE(K_, NT_) \
      case K_: return cm::launch_resident<K_, NT_>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, Nout, scale, row_scale, OUT, st);
      CM_CASE(64, 2) CM_CASE(96, 3) CM_CASE(128, 4)
#undef CM_CASE
    }
  }
  switch (Nout / 32) {
    case 1: return cm::launch<1>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, residual, OUT, st);
    case 2: return cm::launch<2>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, residual, OUT, st);
    case 3: return cm::launch<3>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, residual, OUT, st);
    case 4: return cm::launch<4>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, residual, OUT, st);
    case 5: return cm::launch<5>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, residual, OUT, st);
    case 6: return cm::launch<6>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, residual, OUT, st);
    case 7: return cm::launch<7>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, residual, OUT, st);
    case 8: return cm::launch<8>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, residual, OUT, st);
  }
  return CM_EINVAL;
}
