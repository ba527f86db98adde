// Edge geometry: vectors and lengths from positions, and the scatter of their gradients back to
// the atoms (what makes forces out of per-edge gradients).
//
// Forward: vec[e] = pos[b[e]] - pos[a[e]] + shift[e] in fp64, rounded once to fp32 for the
// kernels downstream, plus its length.  Backward: the gradient of an atom is the signed sum of the
// edge-vector gradients over the edges that start (a) or end (b) at it; both sums run over
// contiguous index ranges (CSR of the sorted row a, sender-sorted view of row b), one wavefront per
// atom, accumulated in fp64 with a fixed reduction order -- no atomics, bit-reproducible.
//
// Optional row map: with `rows` given, atom n of the edge lists is row rows[n] of `pos` and of the position gradient.
// A caller that works on a relabelled copy of the graph then keeps positions and forces in its own order and needs no
// gather on the way in or out.
#include "common.hpp"

namespace cm {
namespace {

__device__ __forceinline__ int row_of(const int32_t *__restrict__ rows, int n) { return rows ? rows[n] : n; }

__global__ void edge_geometry_forward_kernel(const double *__restrict__ pos, const int32_t *__restrict__ a,
                                             const int32_t *__restrict__ b, const double *__restrict__ shifts,
                                             const int32_t *__restrict__ rows, int64_t nedges, int nnodes,
                                             float *__restrict__ vec, float *__restrict__ len) {
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (e >= nedges) return;
  double v[3];
  edge_vector_f64(pos, a, b, shifts, rows, e, nnodes, v);
  vec[3 * e + 0] = static_cast<float>(v[0]);
  vec[3 * e + 1] = static_cast<float>(v[1]);
  vec[3 * e + 2] = static_cast<float>(v[2]);
  len[e] = static_cast<float>(sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]));
}

// total gradient with respect to the edge vector: g_vec + g_len * vec / |vec| (vec recomputed in fp64).  Without a
// length gradient nothing but g_vec is touched.
template <bool HAS_GLEN>
__device__ __forceinline__ void edge_grad(const double *__restrict__ pos, const double *__restrict__ shifts,
                                          const int32_t *__restrict__ a, const int32_t *__restrict__ b,
                                          const int32_t *__restrict__ rows, const float *__restrict__ gvec,
                                          const float *__restrict__ glen, int64_t e, int nnodes, double (&g)[3]) {
  if constexpr (!HAS_GLEN) {
#pragma unroll
    for (int k = 0; k < 3; ++k) g[k] = gvec ? static_cast<double>(gvec[3 * e + k]) : 0.0;
    return;
  }
  const int ia = a[e], ib = b[e];
  g[0] = g[1] = g[2] = 0.0;
  if (static_cast<unsigned>(ia) >= static_cast<unsigned>(nnodes) || static_cast<unsigned>(ib) >= static_cast<unsigned>(nnodes)) return;
  double v[3];
  const int ra = row_of(rows, ia), rb = row_of(rows, ib);
#pragma unroll
  for (int k = 0; k < 3; ++k) v[k] = pos[3 * rb + k] - pos[3 * ra + k] + shifts[3 * e + k];
  const double r = sqrt(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]);
  const double s = r > 0.0 ? static_cast<double>(glen[e]) / r : 0.0;
#pragma unroll
  for (int k = 0; k < 3; ++k) g[k] = (gvec ? static_cast<double>(gvec[3 * e + k]) : 0.0) + s * v[k];
}

template <bool HAS_GLEN>
__global__ void edge_grad_kernel(const double *__restrict__ pos, const double *__restrict__ shifts,
                                 const int32_t *__restrict__ a, const int32_t *__restrict__ b,
                                 const int32_t *__restrict__ rows, const float *__restrict__ gvec,
                                 const float *__restrict__ glen, int64_t nedges, int nnodes, double *__restrict__ gshift) {
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (e >= nedges) return;
  double g[3];
  edge_grad<HAS_GLEN>(pos, shifts, a, b, rows, gvec, glen, e, nnodes, g);
  gshift[3 * e + 0] = g[0];
  gshift[3 * e + 1] = g[1];
  gshift[3 * e + 2] = g[2];
}

template <bool HAS_GLEN>
__global__ __launch_bounds__(256) void edge_geometry_backward_kernel(
    const double *__restrict__ pos, const double *__restrict__ shifts, const int32_t *__restrict__ a,
    const int32_t *__restrict__ b, const int32_t *__restrict__ rows, const int32_t *__restrict__ a_first_occ,
    const int32_t *__restrict__ b_perm, const int32_t *__restrict__ b_offsets, const float *__restrict__ gvec,
    const float *__restrict__ glen, int64_t nedges, int nnodes, double *__restrict__ gpos) {
  const int lane = threadIdx.x % kWave;
  const int node = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (node >= nnodes) return;
  double acc[3] = {0.0, 0.0, 0.0};
  double g[3];
  // edges that end at this atom (row b): + gradient
  for (int k = b_offsets[node] + lane; k < b_offsets[node + 1]; k += kWave) {
    const int e = b_perm[k];
    if (static_cast<unsigned>(e) >= static_cast<uint64_t>(nedges)) continue;
    edge_grad<HAS_GLEN>(pos, shifts, a, b, rows, gvec, glen, e, nnodes, g);
    acc[0] += g[0];
    acc[1] += g[1];
    acc[2] += g[2];
  }
  // edges that start at this atom (row a, contiguous): - gradient
  int ea0 = a_first_occ[node], ea1 = a_first_occ[nnodes + node];
  clamp_edge_range(ea0, ea1, nedges);
  for (int e = ea0 + lane; e < ea1; e += kWave) {
    edge_grad<HAS_GLEN>(pos, shifts, a, b, rows, gvec, glen, e, nnodes, g);
    acc[0] -= g[0];
    acc[1] -= g[1];
    acc[2] -= g[2];
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    acc[0] += __shfl_xor(acc[0], off);
    acc[1] += __shfl_xor(acc[1], off);
    acc[2] += __shfl_xor(acc[2], off);
  }
  if (lane == 0) {
    const int row = row_of(rows, node);
    gpos[3 * row + 0] = acc[0];
    gpos[3 * row + 1] = acc[1];
    gpos[3 * row + 2] = acc[2];
  }
}

}  // namespace
}  // namespace cm

extern "C" int cm_edge_geometry_forward(const double *positions, const int32_t *row_a, const int32_t *row_b,
                                        const double *shifts, const int32_t *node_rows, int64_t nnodes, int64_t nedges,
                                        float *vectors, float *lengths, cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0 && nnodes >= 0 && nnodes < INT32_MAX / 4, "cm_edge_geometry_forward: sizes out of range");
  if (nedges == 0) return CM_OK;
  CM_REQUIRE(positions && row_a && row_b && shifts && vectors && lengths, "cm_edge_geometry_forward: NULL pointer");
  const int block = 256;
  hipLaunchKernelGGL(cm::edge_geometry_forward_kernel, dim3(static_cast<unsigned>(cm::ceil_div(nedges, block))), dim3(block),
                     0, cm::as_stream(stream), positions, row_a, row_b, shifts, node_rows, nedges, static_cast<int>(nnodes), vectors,
                     lengths);
  return cm::check_launch("cm_edge_geometry_forward");
}

extern "C" int cm_edge_geometry_backward(const double *positions, const int32_t *row_a, const int32_t *row_b,
                                         const double *shifts, const int32_t *node_rows, const int32_t *a_first_occ,
                                         const int32_t *b_perm, const int32_t *b_offsets, const float *grad_vectors,
                                         const float *grad_lengths,
                                         int64_t nnodes, int64_t nedges, double *grad_positions, double *grad_shifts,
                                         cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0 && nnodes >= 0 && nnodes < INT32_MAX / 4, "cm_edge_geometry_backward: sizes out of range");
  if (nnodes == 0) return CM_OK;
  CM_REQUIRE(a_first_occ && b_offsets, "cm_edge_geometry_backward: NULL index structure");
  CM_REQUIRE(nedges == 0 || (positions && row_a && row_b && shifts && b_perm), "cm_edge_geometry_backward: NULL pointer");
  hipStream_t st = cm::as_stream(stream);
  if (grad_positions) {
    const int block = 256, per = block / cm::kWave;
    const dim3 grid(static_cast<unsigned>(cm::ceil_div(nnodes, per)));
    if (grad_lengths)
      hipLaunchKernelGGL(cm::edge_geometry_backward_kernel<true>, grid, dim3(block), 0, st, positions, shifts, row_a, row_b,
                         node_rows, a_first_occ, b_perm, b_offsets, grad_vectors, grad_lengths, nedges, static_cast<int>(nnodes), grad_positions);
    else
      hipLaunchKernelGGL(cm::edge_geometry_backward_kernel<false>, grid, dim3(block), 0, st, positions, shifts, row_a, row_b,
                         node_rows, a_first_occ, b_perm, b_offsets, grad_vectors, grad_lengths, nedges, static_cast<int>(nnodes), grad_positions);
  }
  if (grad_shifts && nedges > 0) {
    const int block = 256;
    const dim3 grid(static_cast<unsigned>(cm::ceil_div(nedges, block)));
    if (grad_lengths)
      hipLaunchKernelGGL(cm::edge_grad_kernel<true>, grid, dim3(block), 0, st, positions, shifts, row_a, row_b, node_rows,
                         grad_vectors, grad_lengths, nedges, static_cast<int>(nnodes), grad_shifts);
    else
      hipLaunchKernelGGL(cm::edge_grad_kernel<false>, grid, dim3(block), 0, st, positions, shifts, row_a, row_b, node_rows,
                         grad_vectors, grad_lengths, nedges, static_cast<int>(nnodes), grad_shifts);
  }
  return cm::check_launch("cm_edge_geometry_backward");
}
