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
// launch; here a workgroup takes a tile of 128 nodes of one element (32 where the node count leaves most compute units
// without a tile of 128) through the whole chain.  The intermediate rows
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
#include "node_glue.hpp"

// Products and the additions that follow them stay separate roundings, as they are where separate launches store the
// product before the next one adds to it.
#pragma clang fp contract(off)

namespace cm {
namespace {

constexpr int kGlTile = 128;       // nodes per workgroup (ROWS below), or
constexpr int kGlSmallTile = 32;   // where 128-node tiles would occupy less than half of the compute units
constexpr int kGlKC = 32;          // K columns staged per step
constexpr int kGlLdH = kGlKC + 8;  // padded row stride of a bf16 plane (elements)
constexpr int kGlTPR = kGlKC / 4;  // threads that cover the 32 columns of a staged row, 16 bytes each

// A workgroup has (ROWS / 32) * NT waves (C = 32 NT): wave w owns the 32 x 32 block of the tile's output at rows
// 32 (w % (ROWS / 32)), columns 32 (w / (ROWS / 32)).  With one wave per block a product's matrix instructions, operand reads and staging
// are spread over four waves per SIMD, which hide each other's latencies; with four waves and NT blocks each, a chain of
// three products on one tile of 128 took twice as long (26 against 13 us at 128 channels).  A tile's three products keep
// the matrix cores of one compute unit busy for 8 us at 128 rows and 128 channels, however few tiles there are: a system
// of a few hundred atoms takes tiles of 32 rows, NT waves each, on four times as many compute units.
template <int NT, int ROWS>
struct GlueShared {
  static constexpr int C = 32 * NT;
  static constexpr int kRows = ROWS;
  static constexpr int kRowWaves = ROWS / 32;
  static constexpr int kThreads = kRowWaves * NT * kWave;
  static constexpr int kLdT = C + 4;  // padded row stride of the fp32 tile (floats): rows 16 bytes apart in bank space
  // pieces of 16 bytes per thread and K chunk: X (ROWS rows x 8 pieces over kThreads threads), weights (C rows x 8)
  static constexpr int kAPieces = (ROWS * kGlTPR + kThreads - 1) / kThreads;
  static constexpr int kBPieces = C * kGlTPR / kThreads;
  static_assert(C * kGlTPR % kThreads == 0, "the weight pieces divide evenly among the threads");
  __bf16 a[3 * ROWS * kGlLdH];
  __bf16 b[3 * C * kGlLdH];
  float tile[ROWS * kLdT];
  int node[ROWS];
};

// Operands of a product on their way from memory: a thread's 16-byte pieces of every K chunk, requested all at once
// and long before the product that consumes them.
template <class S>
struct WeightPieces {
  f4 v[S::C / kGlKC][S::kBPieces];  // [chunk][i]: row (tid + i kThreads) / 8 of the transposed block, columns 32 chunk + 4 (tid % 8) ..
};
template <class S>
struct RowPieces {
  f4 v[S::C / kGlKC][S::kAPieces];
};

template <class S>
__device__ __forceinline__ void fetch_weights(const float *__restrict__ Wg, WeightPieces<S> &w) {
#pragma unroll
  for (int i = 0; i < S::kBPieces; ++i) {
    const int piece = threadIdx.x + i * S::kThreads;
    const int srow = piece / kGlTPR, scol = (piece % kGlTPR) * 4;
#pragma unroll
    for (int k = 0; k < S::C / kGlKC; ++k) w.v[k][i] = ld4(Wg + static_cast<int64_t>(srow) * S::C + kGlKC * k + scol);
  }
}

// rows of X [*, C] named by the tile's node list (zeros for rows beyond the tile)
template <class S>
__device__ __forceinline__ void fetch_rows(const S &s, const float *__restrict__ X, RowPieces<S> &a) {
#pragma unroll
  for (int i = 0; i < S::kAPieces; ++i) {
    const int piece = threadIdx.x + i * S::kThreads;
    const int row = piece / kGlTPR, scol = (piece % kGlTPR) * 4;
    const int node = row < S::kRows ? s.node[row] : -1;
#pragma unroll
    for (int k = 0; k < S::C / kGlKC; ++k) a.v[k][i] = node >= 0 ? ld4(X + static_cast<int64_t>(node) * S::C + kGlKC * k + scol) : zero4();
  }
}

// acc = the wave's 32 x 32 block of X . W over K = C.  X: the pieces fetched by fetch_rows, or (FROM_TILE) the fp32 tile in
// LDS; W: the pieces fetched by fetch_weights from the transposed block [C out, C in].  All threads of the workgroup
// take part; on return the operand planes may still be read by slower waves: whatever overwrites them next sits behind
// a barrier.
template <class S, bool FROM_TILE>
__device__ __forceinline__ void product(S &s, const RowPieces<S> *rows, const WeightPieces<S> &w, v16f &acc) {
  constexpr int C = S::C, ROWS = S::kRows;
  const int tid = threadIdx.x;
  const int lane = tid % kWave, wave = tid / kWave;
  const int wr = wave % S::kRowWaves, wc = wave / S::kRowWaves;
  const int mrow = lane % 32, half = lane / 32;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
  for (int k = 0; k < C / kGlKC; ++k) {
    __syncthreads();  // previous chunk fully consumed (and, before the first, the tile complete)
#pragma unroll
    for (int i = 0; i < S::kAPieces; ++i) {
      const int piece = tid + i * S::kThreads;
      const int row = piece / kGlTPR, scol = (piece % kGlTPR) * 4;
      if (S::kAPieces * S::kThreads != ROWS * kGlTPR && row >= ROWS) continue;
      f4 x;
      if constexpr (FROM_TILE)
        x = *reinterpret_cast<const f4 *>(s.tile + row * S::kLdT + kGlKC * k + scol);
      else
        x = rows->v[k][i];
      bf16x4 h, md, lw;
      split3(x, h, md, lw);
      const int at = row * kGlLdH + scol;
      *reinterpret_cast<bf16x4 *>(s.a + at) = h;
      *reinterpret_cast<bf16x4 *>(s.a + ROWS * kGlLdH + at) = md;
      *reinterpret_cast<bf16x4 *>(s.a + 2 * ROWS * kGlLdH + at) = lw;
    }
#pragma unroll
    for (int i = 0; i < S::kBPieces; ++i) {
      const int piece = tid + i * S::kThreads;
      bf16x4 h, md, lw;
      split3(w.v[k][i], h, md, lw);
      const int at = (piece / kGlTPR) * kGlLdH + (piece % kGlTPR) * 4;
      *reinterpret_cast<bf16x4 *>(s.b + at) = h;
      *reinterpret_cast<bf16x4 *>(s.b + C * kGlLdH + at) = md;
      *reinterpret_cast<bf16x4 *>(s.b + 2 * C * kGlLdH + at) = lw;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < kGlKC; ks += 16) {
      bf16x8 a[3], b[3];
#pragma unroll
      for (int p = 0; p < 3; ++p) {
        a[p] = *reinterpret_cast<const bf16x8 *>(s.a + p * ROWS * kGlLdH + (32 * wr + mrow) * kGlLdH + ks + 8 * half);
        b[p] = *reinterpret_cast<const bf16x8 *>(s.b + p * C * kGlLdH + (32 * wc + mrow) * kGlLdH + ks + 8 * half);
      }
      // piece products from small to large, as in the linear kernels
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[2], b[0], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[2], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[1], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[0], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[1], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[0], acc, 0, 0, 0);
    }
  }
}

// Accumulator r of a lane is row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32 of the wave's block.
template <class S, class F>
__device__ __forceinline__ void for_each_output(const v16f &acc, F f) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int mrow = lane % 32, half = lane / 32;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    f(32 * (wave % S::kRowWaves) + 8 * (r / 4) + 4 * half + (r % 4), 32 * (wave / S::kRowWaves) + mrow, acc[r]);
}

template <class S>
__device__ __forceinline__ void stage_nodes(S &s, const int32_t *__restrict__ node_perm, int pos0, int gend, int nnodes) {
  const int tid = threadIdx.x;
  if (tid < S::kRows) {
    int node = -1;
    if (tid < min(S::kRows, gend - pos0)) {
      node = node_perm ? node_perm[pos0 + tid] : pos0 + tid;
      if (static_cast<unsigned>(node) >= static_cast<unsigned>(nnodes)) node = -1;
    }
    s.node[tid] = node;
  }
  __syncthreads();
}

// ---- forward: h1 = B1 . Wprod, sc = skip_scale h1 . Wskip[element], X2 = h1 . Wup ---------------------------------
template <int NT, int ROWS>
__global__ __launch_bounds__(ROWS / 32 * NT *kWave) void node_glue_forward_kernel(
    const float *__restrict__ B1, const float *__restrict__ prod_WT, const float *__restrict__ skip_WT,
    const float *__restrict__ up_WT, const int32_t *__restrict__ node_perm, const int32_t *__restrict__ group_offsets, int nnodes,
    int ngroups, float skip_scale, float *__restrict__ h1, float *__restrict__ sc, float *__restrict__ X2) {
  constexpr int C = 32 * NT;
  using S = GlueShared<NT, ROWS>;
  __shared__ __attribute__((aligned(16))) S s;
  int g, pos0, gend;
  if (!locate_group_tile(group_offsets, ngroups, nnodes, blockIdx.x, ROWS, g, pos0, gend)) return;
  stage_nodes(s, node_perm, pos0, gend, nnodes);

  const bool no_element = g == ngroups - 1;  // nodes of no element: the skip connection is defined as zero there
  WeightPieces<S> wa, wb;
  RowPieces<S> a0;
  fetch_weights<S>(prod_WT, wa);
  fetch_rows(s, B1, a0);
  if (!no_element) fetch_weights<S>(skip_WT + static_cast<int64_t>(g) * C * C, wb);  // in flight during the first product

  v16f acc;
  product<S, false>(s, &a0, wa, acc);
  fetch_weights<S>(up_WT, wa);
  for_each_output<S>(acc, [&](int row, int col, float v) {
    const float out = v * 1.0f;
    s.tile[row * S::kLdT + col] = out;
    const int node = s.node[row];
    if (node >= 0) h1[static_cast<int64_t>(node) * C + col] = out;
  });
  // (the tile is complete behind the barrier at the top of the next product)
  if (no_element) {
    for_each_output<S>(acc, [&](int row, int col, float) {
      const int node = s.node[row];
      if (node >= 0) sc[static_cast<int64_t>(node) * C + col] = 0.f;
    });
  } else {
    product<S, true>(s, nullptr, wb, acc);
    for_each_output<S>(acc, [&](int row, int col, float v) {
      const int node = s.node[row];
      if (node >= 0) sc[static_cast<int64_t>(node) * C + col] = v * skip_scale;
    });
  }
  product<S, true>(s, nullptr, wa, acc);
  for_each_output<S>(acc, [&](int row, int col, float v) {
    const int node = s.node[row];
    if (node >= 0) X2[static_cast<int64_t>(node) * C + col] = v * 1.0f;
  });
}

// Energies per graph, riding in the backward launch (its tiles do not depend on them): out[g] = sum over the graph's nodes
// of weight[n] * node_es[n], strided partial sums of the workgroup's threads (the largest power of two of them) and a tree
// over them: a fixed order.
struct EnergySums {
  const double *node_es, *node_weights;
  const int32_t *graph_ptr;
  double *out;
  int ngraphs;
  const double *graph_e0;  // a constant per graph added into `total` (NULL: zero)
  double *total;           // NULL: not asked for
};
template <int THREADS>  // a power of two, at most the workgroup's size
__device__ __forceinline__ void graph_energy(const EnergySums &q, int graph, double *part) {
  const int tid = threadIdx.x;
  if (tid < THREADS) {
    const int lo = q.graph_ptr[graph], hi = q.graph_ptr[graph + 1];
    auto term = [&](int i) { return q.node_weights ? q.node_weights[i] * q.node_es[i] : q.node_es[i]; };
    // four strided partial sums per thread, their loads requested together: one sum after the other waits for memory
    // once per node, and this workgroup would outlast the tiles of the launch
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
    int i = lo + tid;
    for (; i + 3 * THREADS < hi; i += 4 * THREADS) {
      const double t0 = term(i), t1 = term(i + THREADS), t2 = term(i + 2 * THREADS), t3 = term(i + 3 * THREADS);
      s0 += t0, s1 += t1, s2 += t2, s3 += t3;
    }
    for (; i < hi; i += THREADS) s0 += term(i);
    part[tid] = (s0 + s1) + (s2 + s3);
  }
  __syncthreads();
  for (int d = THREADS / 2; d > 0; d >>= 1) {
    if (tid < d) part[tid] += part[tid + d];
    __syncthreads();
  }
  if (tid == 0) {
    q.out[graph] = part[0];
    if (q.total) q.total[graph] = part[0] + (q.graph_e0 ? q.graph_e0[graph] : 0.0);
  }
}

// ---- backward: gh1 = gX2 . Wup^T + g1 - skip_scale dE/dh2 . Wskip[element]^T, gB1 = gh1 . Wprod^T ------------------
template <int NT, int ROWS>
__global__ __launch_bounds__(ROWS / 32 * NT *kWave) void node_glue_backward_kernel(
    const float *__restrict__ gX2, const float *__restrict__ d_h2, const float *__restrict__ up_W, const float *__restrict__ skip_W,
    const float *__restrict__ prod_W, const double *__restrict__ w1, double scale, const double *__restrict__ node_weights,
    const int32_t *__restrict__ node_perm, const int32_t *__restrict__ group_offsets, int nnodes, int ngroups, float skip_scale,
    float *__restrict__ gB1, EnergySums sums, int first_tile) {
  constexpr int C = 32 * NT;
  using S = GlueShared<NT, ROWS>;
  __shared__ __attribute__((aligned(16))) S s;
  if (static_cast<int>(blockIdx.x) < first_tile) {
    // workgroups ahead of the tiles: the energy of one graph each, from node energies an earlier launch wrote
    constexpr int kSum = S::kThreads >= 1024 ? 1024 : (S::kThreads >= 512 ? 512 : (S::kThreads >= 256 ? 256 : (S::kThreads >= 128 ? 128 : 64)));
    static_assert(sizeof(s.tile) >= kSum * sizeof(double), "the tile holds the partial sums");
    graph_energy<kSum>(sums, blockIdx.x, reinterpret_cast<double *>(s.tile));
    return;
  }
  int g, pos0, gend;
  if (!locate_group_tile(group_offsets, ngroups, nnodes, blockIdx.x - first_tile, ROWS, g, pos0, gend)) return;
  stage_nodes(s, node_perm, pos0, gend, nnodes);

  const bool no_element = g == ngroups - 1;
  WeightPieces<S> wa, wb;
  RowPieces<S> a0, a1;
  fetch_weights<S>(up_W, wa);
  fetch_rows(s, gX2, a0);
  if (!no_element) {  // in flight during the first product
    fetch_weights<S>(skip_W + static_cast<int64_t>(g) * C * C, wb);
    fetch_rows(s, d_h2, a1);
  }

  v16f acc;
  product<S, false>(s, &a0, wa, acc);
  fetch_weights<S>(prod_W, wa);
  for_each_output<S>(acc, [&](int row, int col, float v) {
    const int node = s.node[row];
    const double nw = (node_weights && node >= 0) ? node_weights[node] : 1.0;
    const float g1 = static_cast<float>(-1.0 * scale * w1[col] * nw);
    const float part = v * 1.0f;
    s.tile[row * S::kLdT + col] = part + g1;
  });
  if (!no_element) {
    product<S, false>(s, &a1, wb, acc);
    // each element of the tile is read and written by the lane that wrote it above
    for_each_output<S>(acc, [&](int row, int col, float v) {
      const float part = v * -skip_scale;
      s.tile[row * S::kLdT + col] += part;
    });
  }
  product<S, true>(s, nullptr, wa, acc);
  for_each_output<S>(acc, [&](int row, int col, float v) {
    const int node = s.node[row];
    if (node >= 0) gB1[static_cast<int64_t>(node) * C + col] = v * 1.0f;
  });
}

// 128-node tiles where they give at least half of the compute units one each, 32-node tiles below that
inline bool small_tiles(int64_t nnodes) { return ceil_div(nnodes, kGlTile) * 2 < device_compute_units(); }

template <int NT>
void launch_forward(const float *B1, const float *prod_WT, const float *skip_WT, const float *up_WT, const int32_t *perm,
                    const int32_t *offs, int64_t nnodes, int ngroups, float skip_scale, float *h1, float *sc, float *X2,
                    hipStream_t st) {
  if (small_tiles(nnodes)) {
    const unsigned tiles = static_cast<unsigned>(ceil_div(nnodes, kGlSmallTile) + ngroups);
    hipLaunchKernelGGL((node_glue_forward_kernel<NT, kGlSmallTile>), dim3(tiles), dim3(NT * kWave), 0, st, B1, prod_WT, skip_WT, up_WT,
                       perm, offs, static_cast<int>(nnodes), ngroups, skip_scale, h1, sc, X2);
    return;
  }
  const unsigned tiles = static_cast<unsigned>(ceil_div(nnodes, kGlTile) + ngroups);
  hipLaunchKernelGGL((node_glue_forward_kernel<NT, kGlTile>), dim3(tiles), dim3(4 * NT * kWave), 0, st, B1, prod_WT, skip_WT, up_WT, perm,
                     offs, static_cast<int>(nnodes), ngroups, skip_scale, h1, sc, X2);
}

template <int NT>
void launch_backward(const float *gX2, const float *d_h2, const float *up_W, const float *skip_W, const float *prod_W,
                     const double *w1, double scale, const double *node_weights, const int32_t *perm, const int32_t *offs,
                     int64_t nnodes, int ngroups, float skip_scale, float *gB1, const EnergySums &sums, hipStream_t st) {
  const unsigned extra = sums.out ? static_cast<unsigned>(sums.ngraphs) : 0u;
  if (small_tiles(nnodes)) {
    const unsigned tiles = static_cast<unsigned>(ceil_div(nnodes, kGlSmallTile) + ngroups);
    hipLaunchKernelGGL((node_glue_backward_kernel<NT, kGlSmallTile>), dim3(tiles + extra), dim3(NT * kWave), 0, st, gX2, d_h2, up_W,
                       skip_W, prod_W, w1, scale, node_weights, perm, offs, static_cast<int>(nnodes), ngroups, skip_scale, gB1, sums,
                       static_cast<int>(extra));
    return;
  }
  const unsigned tiles = static_cast<unsigned>(ceil_div(nnodes, kGlTile) + ngroups);
  hipLaunchKernelGGL((node_glue_backward_kernel<NT, kGlTile>), dim3(tiles + extra), dim3(4 * NT * kWave), 0, st, gX2, d_h2, up_W, skip_W,
                     prod_W, w1, scale, node_weights, perm, offs, static_cast<int>(nnodes), ngroups, skip_scale, gB1, sums,
                     static_cast<int>(extra));
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

namespace cm {

// cm_node_glue_backward whose launch also sums the node energies per graph (operands checked by the caller, cm_mace_step)
int node_glue_backward_with_energy_sums(const float *gX2, const float *d_h2, const float *up_W, const float *skip_W, const float *prod_W,
                                        const double *w1, double scale, const double *node_weights, const int32_t *node_perm,
                                        const int32_t *group_offsets, int64_t nnodes, int ngroups, int channels, float skip_scale,
                                        float *gB1, const double *node_es, const int32_t *graph_ptr, int ngraphs, double *energies,
                                        const double *graph_e0, double *total_energies, hipStream_t st) {
  const EnergySums sums{node_es, node_weights, graph_ptr, energies, ngraphs, graph_e0, total_energies};
  switch (channels / 32) {
    case 1: launch_backward<1>(gX2, d_h2, up_W, skip_W, prod_W, w1, scale, node_weights, node_perm, group_offsets, nnodes, ngroups, skip_scale, gB1, sums, st); break;
    case 2: launch_backward<2>(gX2, d_h2, up_W, skip_W, prod_W, w1, scale, node_weights, node_perm, group_offsets, nnodes, ngroups, skip_scale, gB1, sums, st); break;
    case 3: launch_backward<3>(gX2, d_h2, up_W, skip_W, prod_W, w1, scale, node_weights, node_perm, group_offsets, nnodes, ngroups, skip_scale, gB1, sums, st); break;
    case 4: launch_backward<4>(gX2, d_h2, up_W, skip_W, prod_W, w1, scale, node_weights, node_perm, group_offsets, nnodes, ngroups, skip_scale, gB1, sums, st); break;
    default: set_error("node glue: channels=%d not supported", channels); return CM_EINVAL;
  }
  return check_launch("cm_node_glue_backward");
}

}  // namespace cm

extern "C" int cm_node_glue_backward(const float *gX2, const float *d_h2, const float *up_W, const float *skip_W,
                                     const float *prod_W, const double *w1, double scale, const double *node_weights,
                                     const int32_t *node_perm, const int32_t *group_offsets, int64_t nnodes, int ngroups,
                                     int channels, float skip_scale, float *gB1, cm_stream_t stream) {
  CM_REQUIRE(cm_node_glue_supported(channels), "cm_node_glue_backward: channels=%d must be 32, 64, 96 or 128", channels);
  CM_REQUIRE(nnodes >= 0 && nnodes < INT32_MAX / 256, "cm_node_glue_backward: nnodes out of range");
  CM_REQUIRE(ngroups >= 2, "cm_node_glue_backward: ngroups counts the elements plus the group of nodes without one");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(gX2 && d_h2 && up_W && skip_W && prod_W && w1 && node_perm && group_offsets && gB1, "cm_node_glue_backward: NULL pointer");
  return cm::node_glue_backward_with_energy_sums(gX2, d_h2, up_W, skip_W, prod_W, w1, scale, node_weights, node_perm, group_offsets,
                                                 nnodes, ngroups, channels, skip_scale, gB1, nullptr, nullptr, 0, nullptr, nullptr,
                                                 nullptr, cm::as_stream(stream));
}
