// The chains of [N, C] x [C, C] products between the two interaction layers, one launch per direction.
//
// Between the first layer's contraction and the second layer's message passing the model applies three small linears to
// the same rows (reference: models/InvariantMACE.py:41-53 linear_matmul for the product's linear and linear_up, :56-74
// the per-element skip connection):
//
//   forward    h1 = B1 . Wprod1          sc = skip_e(h1)   (weights of the node's element)      X2 = h1 . Wup
//   backward   gh1 = gX2 . Wup^T + g1 + skip_e^T(g2)       gB1 = gh1 . Wprod1^T
//
// As separate launches of the linear kernel each of them keeps the device busy for a few microseconds and costs a
// launch; here a workgroup takes a tile of 128 nodes of one element through the whole chain.  The intermediate rows
// (h1, gh1) stay in LDS as fp32 and are the X operand of the next product.  Arithmetic, operand split and accumulation
// order are those of the linear kernels (three bf16 pieces per fp32 operand, six piece products on
// v_mfma_f32_32x32x16_bf16, K in chunks of 32), and every intermediate is rounded to fp32 where the separate launches
// store it, so the chain returns the bits of the separate launches.
//
// g1 and g2 are the gradients of minus the (weighted) sum of node energies with respect to the two layers' features:
// g1[n, c] = -weight[n] scale w1[c] is formed here from the linear readout's weights; g2 = -dE/dh2 arrives as dE/dh2 and
// its sign goes into the scale of the skip product.
#include "common.hpp"
#include "mfma_split.hpp"

// Products and the additions that follow them stay separate roundings, as they are where separate launches store the
// product before the next one adds to it.
#pragma clang fp contract(off)

namespace cm {
namespace {

constexpr int kGlWaves = 4;
constexpr int kGlTile = 32 * kGlWaves;  // nodes per workgroup
constexpr int kGlKC = 32;               // K columns staged per step
constexpr int kGlLdH = kGlKC + 8;       // padded row stride of a bf16 plane (elements)

template <int NT>
struct GlueShared {
  static constexpr int C = 32 * NT;
  static constexpr int kLdT = C + 4;  // padded row stride of the fp32 tile (floats): rows 16 bytes apart in bank space
  __bf16 a[3 * kGlTile * kGlLdH];
  __bf16 b[3 * C * kGlLdH];
  float tile[kGlTile * kLdT];
  int node[kGlTile];
};

// Tile of the grouped node order that a workgroup owns: false when the workgroup has none.
__device__ __forceinline__ bool locate_tile(const int32_t *__restrict__ group_offsets, int ngroups, int nnodes, int tile, int &g,
                                            int &pos0, int &gend) {
  g = 0, pos0 = 0, gend = nnodes;
  if (group_offsets) {
    for (g = 0; g < ngroups; ++g) {
      const int lo = group_offsets[g], hi = group_offsets[g + 1];
      const int tiles = (hi - lo + kGlTile - 1) / kGlTile;
      if (tile < tiles) {
        pos0 = lo + tile * kGlTile;
        gend = hi;
        return true;
      }
      tile -= tiles;
    }
    return false;
  }
  pos0 = tile * kGlTile;
  return pos0 < nnodes;
}

// acc = X . W over K = C, X rows given by `xrow(row, col)` (four consecutive columns of a tile row), W as its transpose
// Wg [C, C] (row = output column).  All threads of the workgroup take part; ends with every wave past its last LDS read
// of the planes only after the caller's next barrier.
template <int NT, class XRow>
__device__ __forceinline__ void product(GlueShared<NT> &s, XRow xrow, const float *__restrict__ Wg, v16f (&acc)[NT]) {
  constexpr int C = 32 * NT;
  const int tid = threadIdx.x;
  const int lane = tid % kWave, wave = tid / kWave;
  constexpr int kTPR = kGlKC / 4;                 // threads per staged row
  constexpr int kRPP = kGlWaves * kWave / kTPR;   // rows per pass
  constexpr int A_PASSES = kGlTile / kRPP, B_PASSES = C / kRPP;
  const int srow = tid / kTPR, scol = (tid % kTPR) * 4;
  const int mrow = lane % 32, half = lane / 32;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
  f4 pa[A_PASSES], pb[B_PASSES];
  auto prefetch = [&](int kc) {
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) pa[i] = xrow(kRPP * i + srow, kc + scol);
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) pb[i] = ld4(Wg + static_cast<int64_t>(kRPP * i + srow) * C + kc + scol);
  };
  prefetch(0);
  for (int kc = 0; kc < C; kc += kGlKC) {
    __syncthreads();  // previous chunk fully consumed
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) {
      bf16x4 h, md, lw;
      split3(pa[i], h, md, lw);
      const int at = (kRPP * i + srow) * kGlLdH + scol;
      *reinterpret_cast<bf16x4 *>(s.a + at) = h;
      *reinterpret_cast<bf16x4 *>(s.a + kGlTile * kGlLdH + at) = md;
      *reinterpret_cast<bf16x4 *>(s.a + 2 * kGlTile * kGlLdH + at) = lw;
    }
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) {
      bf16x4 h, md, lw;
      split3(pb[i], h, md, lw);
      const int at = (kRPP * i + srow) * kGlLdH + scol;
      *reinterpret_cast<bf16x4 *>(s.b + at) = h;
      *reinterpret_cast<bf16x4 *>(s.b + C * kGlLdH + at) = md;
      *reinterpret_cast<bf16x4 *>(s.b + 2 * C * kGlLdH + at) = lw;
    }
    __syncthreads();
    if (kc + kGlKC < C) prefetch(kc + kGlKC);
#pragma unroll
    for (int ks = 0; ks < kGlKC; ks += 16) {
      const int aoff = (32 * wave + mrow) * kGlLdH + ks + 8 * half;
      bf16x8 a[3], b[NT][3];
#pragma unroll
      for (int p = 0; p < 3; ++p) a[p] = *reinterpret_cast<const bf16x8 *>(s.a + p * kGlTile * kGlLdH + aoff);
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int p = 0; p < 3; ++p)
          b[t][p] = *reinterpret_cast<const bf16x8 *>(s.b + p * C * kGlLdH + (32 * t + mrow) * kGlLdH + ks + 8 * half);
      // piece products from small to large, as in the linear kernels
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
}

// Accumulator r of a lane is row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32 + 32 t of the wave's block.
template <int NT, class F>
__device__ __forceinline__ void for_each_output(const v16f (&acc)[NT], F f) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int mrow = lane % 32, half = lane / 32;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = 32 * wave + 8 * (r / 4) + 4 * half + (r % 4);
#pragma unroll
    for (int t = 0; t < NT; ++t) f(row, 32 * t + mrow, acc[t][r]);
  }
}

template <int NT>
__device__ __forceinline__ void stage_nodes(GlueShared<NT> &s, const int32_t *__restrict__ node_perm, int pos0, int gend, int nnodes) {
  const int tid = threadIdx.x;
  if (tid < kGlTile) {
    int node = -1;
    if (tid < min(kGlTile, gend - pos0)) {
      node = node_perm ? node_perm[pos0 + tid] : pos0 + tid;
      if (static_cast<unsigned>(node) >= static_cast<unsigned>(nnodes)) node = -1;
    }
    s.node[tid] = node;
  }
  __syncthreads();
}

// ---- forward: h1 = B1 . Wprod, sc = skip_scale h1 . Wskip[element], X2 = h1 . Wup ---------------------------------
template <int NT>
__global__ __launch_bounds__(kGlWaves *kWave) void node_glue_forward_kernel(
    const float *__restrict__ B1, const float *__restrict__ prod_WT, const float *__restrict__ skip_WT,
    const float *__restrict__ up_WT, const int32_t *__restrict__ node_perm, const int32_t *__restrict__ group_offsets, int nnodes,
    int ngroups, float skip_scale, float *__restrict__ h1, float *__restrict__ sc, float *__restrict__ X2) {
  constexpr int C = 32 * NT;
  using S = GlueShared<NT>;
  __shared__ __attribute__((aligned(16))) S s;
  int g, pos0, gend;
  if (!locate_tile(group_offsets, ngroups, nnodes, blockIdx.x, g, pos0, gend)) return;
  stage_nodes<NT>(s, node_perm, pos0, gend, nnodes);

  v16f acc[NT];
  product<NT>(s, [&](int row, int col) {
    const int node = s.node[row];
    return node >= 0 ? ld4(B1 + static_cast<int64_t>(node) * C + col) : zero4();
  }, prod_WT, acc);
  for_each_output<NT>(acc, [&](int row, int col, float v) {
    const float out = v * 1.0f;
    s.tile[row * S::kLdT + col] = out;
    const int node = s.node[row];
    if (node >= 0) h1[static_cast<int64_t>(node) * C + col] = out;
  });
  __syncthreads();  // the tile is complete before any wave stages from it
  auto tile_row = [&](int row, int col) { return *reinterpret_cast<const f4 *>(s.tile + row * S::kLdT + col); };

  if (g == ngroups - 1) {
    // nodes of no element: the skip connection is defined as zero there
    for_each_output<NT>(acc, [&](int row, int col, float) {
      const int node = s.node[row];
      if (node >= 0) sc[static_cast<int64_t>(node) * C + col] = 0.f;
    });
  } else {
    product<NT>(s, tile_row, skip_WT + static_cast<int64_t>(g) * C * C, acc);
    for_each_output<NT>(acc, [&](int row, int col, float v) {
      const int node = s.node[row];
      if (node >= 0) sc[static_cast<int64_t>(node) * C + col] = v * skip_scale;
    });
  }
  product<NT>(s, tile_row, up_WT, acc);
  for_each_output<NT>(acc, [&](int row, int col, float v) {
    const int node = s.node[row];
    if (node >= 0) X2[static_cast<int64_t>(node) * C + col] = v * 1.0f;
  });
}

// ---- backward: gh1 = gX2 . Wup^T + g1 - skip_scale dE/dh2 . Wskip[element]^T, gB1 = gh1 . Wprod^T ------------------
template <int NT>
__global__ __launch_bounds__(kGlWaves *kWave) void node_glue_backward_kernel(
    const float *__restrict__ gX2, const float *__restrict__ d_h2, const float *__restrict__ up_W, const float *__restrict__ skip_W,
    const float *__restrict__ prod_W, const double *__restrict__ w1, double scale, const double *__restrict__ node_weights,
    const int32_t *__restrict__ node_perm, const int32_t *__restrict__ group_offsets, int nnodes, int ngroups, float skip_scale,
    float *__restrict__ gB1) {
  constexpr int C = 32 * NT;
  using S = GlueShared<NT>;
  __shared__ __attribute__((aligned(16))) S s;
  int g, pos0, gend;
  if (!locate_tile(group_offsets, ngroups, nnodes, blockIdx.x, g, pos0, gend)) return;
  stage_nodes<NT>(s, node_perm, pos0, gend, nnodes);

  v16f acc[NT];
  auto rows_of = [&](const float *X) {
    return [X](int row, int col) {
      const int node = s.node[row];
      return node >= 0 ? ld4(X + static_cast<int64_t>(node) * C + col) : zero4();
    };
  };
  product<NT>(s, rows_of(gX2), up_W, acc);
  for_each_output<NT>(acc, [&](int row, int col, float v) {
    const int node = s.node[row];
    const double nw = (node_weights && node >= 0) ? node_weights[node] : 1.0;
    const float g1 = static_cast<float>(-1.0 * scale * w1[col] * nw);
    const float part = v * 1.0f;
    s.tile[row * S::kLdT + col] = part + g1;
  });
  if (g != ngroups - 1) {
    product<NT>(s, rows_of(d_h2), skip_W + static_cast<int64_t>(g) * C * C, acc);
    // each element of the tile is read and written by the lane that wrote it above
    for_each_output<NT>(acc, [&](int row, int col, float v) {
      const float part = v * -skip_scale;
      s.tile[row * S::kLdT + col] += part;
    });
  }
  __syncthreads();  // the tile is complete before any wave stages from it
  product<NT>(s, [&](int row, int col) { return *reinterpret_cast<const f4 *>(s.tile + row * S::kLdT + col); }, prod_W, acc);
  for_each_output<NT>(acc, [&](int row, int col, float v) {
    const int node = s.node[row];
    if (node >= 0) gB1[static_cast<int64_t>(node) * C + col] = v * 1.0f;
  });
}

template <int NT>
void launch_forward(const float *B1, const float *prod_WT, const float *skip_WT, const float *up_WT, const int32_t *perm,
                    const int32_t *offs, int64_t nnodes, int ngroups, float skip_scale, float *h1, float *sc, float *X2,
                    hipStream_t st) {
  const unsigned tiles = static_cast<unsigned>(ceil_div(nnodes, kGlTile) + ngroups);
  hipLaunchKernelGGL(node_glue_forward_kernel<NT>, dim3(tiles), dim3(kGlWaves * kWave), 0, st, B1, prod_WT, skip_WT, up_WT, perm,
                     offs, static_cast<int>(nnodes), ngroups, skip_scale, h1, sc, X2);
}

template <int NT>
void launch_backward(const float *gX2, const float *d_h2, const float *up_W, const float *skip_W, const float *prod_W,
                     const double *w1, double scale, const double *node_weights, const int32_t *perm, const int32_t *offs,
                     int64_t nnodes, int ngroups, float skip_scale, float *gB1, hipStream_t st) {
  const unsigned tiles = static_cast<unsigned>(ceil_div(nnodes, kGlTile) + ngroups);
  hipLaunchKernelGGL(node_glue_backward_kernel<NT>, dim3(tiles), dim3(kGlWaves * kWave), 0, st, gX2, d_h2, up_W, skip_W, prod_W,
                     w1, scale, node_weights, perm, offs, static_cast<int>(nnodes), ngroups, skip_scale, gB1);
}

}  // namespace
}  // namespace cm

extern "C" int cm_node_glue_supported(int channels) { return channels >= 32 && channels <= 128 && channels % 32 == 0; }

extern "C" int cm_node_glue_forward(const float *B1, const float *prod_WT, const float *skip_WT, const float *up_WT,
                                    const int32_t *node_perm, const int32_t *group_offsets, int64_t nnodes, int ngroups,
                                    int channels, float skip_scale, float *h1, float *sc, float *X2, cm_stream_t stream) {
  CM_REQUIRE(cm_node_glue_supported(channels), "cm_node_glue_forward: channels=%d must be 32, 64, 96 or 128", channels);
  CM_REQUIRE(nnodes >= 0 && nnodes < INT32_MAX / 256, "cm_node_glue_forward: nnodes out of range");
  CM_REQUIRE(ngroups >= 2, "cm_node_glue_forward: ngroups counts the elements plus the group of nodes without one");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(B1 && prod_WT && skip_WT && up_WT && node_perm && group_offsets && h1 && sc && X2, "cm_node_glue_forward: NULL pointer");
  hipStream_t st = cm::as_stream(stream);
  switch (channels / 32) {
    case 1: cm::launch_forward<1>(B1, prod_WT, skip_WT, up_WT, node_perm, group_offsets, nnodes, ngroups, skip_scale, h1, sc, X2, st); break;
    case 2: cm::launch_forward<2>(B1, prod_WT, skip_WT, up_WT, node_perm, group_offsets, nnodes, ngroups, skip_scale, h1, sc, X2, st); break;
    case 3: cm::launch_forward<3>(B1, prod_WT, skip_WT, up_WT, node_perm, group_offsets, nnodes, ngroups, skip_scale, h1, sc, X2, st); break;
    case 4: cm::launch_forward<4>(B1, prod_WT, skip_WT, up_WT, node_perm, group_offsets, nnodes, ngroups, skip_scale, h1, sc, X2, st); break;
  }
  return cm::check_launch("cm_node_glue_forward");
}

extern "C" int cm_node_glue_backward(const float *gX2, const float *d_h2, const float *up_W, const float *skip_W,
                                     const float *prod_W, const double *w1, double scale, const double *node_weights,
                                     const int32_t *node_perm, const int32_t *group_offsets, int64_t nnodes, int ngroups,
                                     int channels, float skip_scale, float *gB1, cm_stream_t stream) {
  CM_REQUIRE(cm_node_glue_supported(channels), "cm_node_glue_backward: channels=%d must be 32, 64, 96 or 128", channels);
  CM_REQUIRE(nnodes >= 0 && nnodes < INT32_MAX / 256, "cm_node_glue_backward: nnodes out of range");
  CM_REQUIRE(ngroups >= 2, "cm_node_glue_backward: ngroups counts the elements plus the group of nodes without one");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(gX2 && d_h2 && up_W && skip_W && prod_W && w1 && node_perm && group_offsets && gB1, "cm_node_glue_backward: NULL pointer");
  hipStream_t st = cm::as_stream(stream);
  switch (channels / 32) {
    case 1: cm::launch_backward<1>(gX2, d_h2, up_W, skip_W, prod_W, w1, scale, node_weights, node_perm, group_offsets, nnodes, ngroups, skip_scale, gB1, st); break;
    case 2: cm::launch_backward<2>(gX2, d_h2, up_W, skip_W, prod_W, w1, scale, node_weights, node_perm, group_offsets, nnodes, ngroups, skip_scale, gB1, st); break;
    case 3: cm::launch_backward<3>(gX2, d_h2, up_W, skip_W, prod_W, w1, scale, node_weights, node_perm, group_offsets, nnodes, ngroups, skip_scale, gB1, st); break;
    case 4: cm::launch_backward<4>(gX2, d_h2, up_W, skip_W, prod_W, w1, scale, node_weights, node_perm, group_offsets, nnodes, ngroups, skip_scale, gB1, st); break;
  }
  return cm::check_launch("cm_node_glue_backward");
}
