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

#include "common.hpp"

namespace cm {
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;
constexpr int kTileNodes = 32 * kWaves;  // rows per workgroup (MFMA M = 32 per wave)
constexpr int kKC = 32;                  // K columns staged per step
constexpr int kLdH = kKC + 8;            // padded LDS row stride of a bf16 plane (elements; 80 bytes: conflict-free b128 reads)

// a = hi + mid + lo with bf16 pieces (round to nearest at every step; the remainders are exact in fp32)
__device__ __forceinline__ void split3(f4 v, bf16x4 &hi, bf16x4 &mid, bf16x4 &lo) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const __bf16 h = static_cast<__bf16>(v[j]);
    const float r1 = v[j] - static_cast<float>(h);
    const __bf16 m = static_cast<__bf16>(r1);
    const float r2 = r1 - static_cast<float>(m);
    hi[j] = h;
    mid[j] = m;
    lo[j] = static_cast<__bf16>(r2);
  }
}

// Nout = 32 * NT; SCALED: X is multiplied by row_scale on the way in
template <int NT, bool SCALED>
__global__ __launch_bounds__(kWaves *kWave) void linear_kernel(const float *__restrict__ X, const float *__restrict__ WT,
                                                               const int32_t *__restrict__ node_perm,
                                                               const int32_t *__restrict__ group_offsets, int nnodes,
                                                               int ngroups, int zero_last_group, int ncomp, int K,
                                                               float scale, const float *__restrict__ row_scale,
                                                               float *__restrict__ OUT) {
  constexpr int NOUT = 32 * NT;
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
  int tile = blockIdx.x / ncomp;
  int g = 0, pos0 = 0, gend = nnodes;
  if (group_offsets) {
    bool found = false;
    for (g = 0; g < ngroups; ++g) {
      const int lo = group_offsets[g], hi = group_offsets[g + 1];
      const int tiles = (hi - lo + kTileNodes - 1) / kTileNodes;
      if (tile < tiles) {
        pos0 = lo + tile * kTileNodes;
        gend = hi;
        found = true;
        break;
      }
      tile -= tiles;
    }
    if (!found) return;
  } else {
    pos0 = tile * kTileNodes;
    if (pos0 >= nnodes) return;
  }
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
    // rows that belong to no weight group: defined as zero
    for (int i = tid; i < kTileNodes * NOUT; i += kWaves * kWave) {
      const int node = sNode[i / NOUT];
      if (node >= 0) OUT[(static_cast<int64_t>(node) * ncomp + m) * NOUT + i % NOUT] = 0.f;
    }
    return;
  }
  const float *Wg = WT + (static_cast<int64_t>(g) * nblocks + l) * NOUT * K;  // [NOUT, K]

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
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = 32 * wave + 8 * (r / 4) + 4 * half + (r % 4);
    const int node = sNode[row];
    if (node >= 0) {
      float *op = OUT + (static_cast<int64_t>(node) * ncomp + m) * NOUT + mrow;
#pragma unroll
      for (int t = 0; t < NT; ++t) op[32 * t] = acc[t][r] * scale;
    }
  }
}

template <int NT>
int launch(const float *X, const float *WT, const int32_t *perm, const int32_t *offs, int64_t nnodes, int ngroups,
           int zero_last_group, int ncomp, int K, float scale, const float *row_scale, float *OUT, hipStream_t st) {
  const int64_t tiles = ceil_div(nnodes, kTileNodes) + (offs ? ngroups : 0);
  const dim3 grid(static_cast<unsigned>(tiles * ncomp)), block(kWaves * kWave);
  if (row_scale)
    hipLaunchKernelGGL((linear_kernel<NT, true>), grid, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes), ngroups,
                       zero_last_group, ncomp, K, scale, row_scale, OUT);
  else
    hipLaunchKernelGGL((linear_kernel<NT, false>), grid, block, 0, st, X, WT, perm, offs, static_cast<int>(nnodes), ngroups,
                       zero_last_group, ncomp, K, scale, row_scale, OUT);
  return check_launch("cm_linear");
}

}  // namespace
}  // namespace cm

extern "C" int cm_linear(const float *X, const float *W_T, const int32_t *node_perm, const int32_t *group_offsets,
                         int64_t nnodes, int ngroups, int zero_last_group, int ncomp, int K, int Nout, float scale,
                         const float *row_scale, float *OUT, cm_stream_t stream) {
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
  switch (Nout / 32) {
    case 1: return cm::launch<1>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, OUT, st);
    case 2: return cm::launch<2>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, OUT, st);
    case 3: return cm::launch<3>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, OUT, st);
    case 4: return cm::launch<4>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, OUT, st);
    case 5: return cm::launch<5>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, OUT, st);
    case 6: return cm::launch<6>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, OUT, st);
    case 7: return cm::launch<7>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, OUT, st);
    case 8: return cm::launch<8>(X, W_T, node_perm, group_offsets, nnodes, ngroups, zero_last_group, ncomp, K, scale, row_scale, OUT, st);
  }
  return CM_EINVAL;
}
