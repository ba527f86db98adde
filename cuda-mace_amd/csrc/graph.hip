// Index structures of one neighbour list, derived on the device in one call and without a host synchronisation.
//
// The model works on a relabelled copy of the graph in which atoms that are close in space have close indices, so that
// the gathers of sender rows hit in cache, and on lists in which every receiver's pairs beyond the cutoff (the skin shell
// of a Verlet list) come last, nearest first, so that the message-passing kernels can stop at the last pair inside the
// cutoff.  The reference has no counterpart: it takes the list as upstream's host-side search returns it
// (tests/test_utils.py:62-105) and rebuilds its own index table inside every forward call
// (jit_wrappers/src/invariant_message_passing_wrapper.cpp:91-93).
//
//   atoms    sorted by (graph, bin of a 3-D grid, original index); grid of at most `bins` cells per axis, cells at least
//            half a cutoff wide, over the bounding box of the positions
//   edges    of the incoming list (sorted by row i) move with their atom i as whole segments; inside a segment the pairs
//            within the cutoff come first, by the new label of atom j (ties in the list's order), then the others by
//            length (ties in the list's order).  No global sort of the edges: a wave ranks the pairs of one atom.
//   derived  CSR offsets of the new row i, the view of the new list sorted by row j.
#include <cfloat>

#include "common.hpp"

// Products and sums as written (no fused multiply-adds): a host restatement then computes the same grid cells and orders
// pairs of equal length identically.
#pragma clang fp contract(off)

namespace cm {
namespace {

constexpr int kBoxThreads = 1024;
constexpr int kScanThreads = 1024;
constexpr int kScanStage = 32 * 1024;  // values staged in LDS at a time (128 KB)
constexpr int kSegLds = 1024;  // keys of a segment that a wave keeps in LDS

// box[0..2] = smallest coordinate per axis, box[3] = largest extent over the axes (one workgroup; a fixed order)
__global__ __launch_bounds__(kBoxThreads) void bounding_box_kernel(const double *__restrict__ pos, int64_t n, double *__restrict__ box) {
  __shared__ double lo[3][kBoxThreads], hi[3][kBoxThreads];
  const int t = threadIdx.x;
  double mn[3] = {DBL_MAX, DBL_MAX, DBL_MAX}, mx[3] = {-DBL_MAX, -DBL_MAX, -DBL_MAX};
  for (int64_t i = t; i < n; i += kBoxThreads) {
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const double v = pos[3 * i + k];
      mn[k] = v < mn[k] ? v : mn[k];
      mx[k] = v > mx[k] ? v : mx[k];
    }
  }
#pragma unroll
  for (int k = 0; k < 3; ++k) lo[k][t] = mn[k], hi[k][t] = mx[k];
  __syncthreads();
  for (int d = kBoxThreads / 2; d > 0; d >>= 1) {
    if (t < d) {
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        lo[k][t] = lo[k][t + d] < lo[k][t] ? lo[k][t + d] : lo[k][t];
        hi[k][t] = hi[k][t + d] > hi[k][t] ? hi[k][t + d] : hi[k][t];
      }
    }
    __syncthreads();
  }
  if (t == 0) {
    double extent = 0.0;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      box[k] = n > 0 ? lo[k][0] : 0.0;
      const double e = n > 0 ? hi[k][0] - lo[k][0] : 0.0;
      extent = e > extent ? e : extent;
    }
    box[3] = extent;
  }
}

// key = ((graph * bins + bx) * bins + by) * bins + bz
__global__ void atom_key_kernel(const double *__restrict__ pos, const int32_t *__restrict__ graph_of_node, int64_t n,
                                const double *__restrict__ box, double min_width, int bins, int ngraphs, int32_t *__restrict__ keys) {
  const int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (i >= n) return;
  double width = box[3] / bins * (1.0 + 1e-12);
  width = width > min_width ? width : min_width;
  int b[3];
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const double f = floor((pos[3 * i + k] - box[k]) / width);
    b[k] = f < 0.0 ? 0 : (f >= bins ? bins - 1 : static_cast<int>(f));  // NaN positions land in bin 0
  }
  int g = graph_of_node ? graph_of_node[i] : 0;
  g = g < 0 ? 0 : (g >= ngraphs ? ngraphs - 1 : g);
  keys[i] = ((g * bins + b[0]) * bins + b[1]) * bins + b[2];
}

// inverse[perm[a]] = a; degree of the new atom a = length of the segment of its old atom
__global__ void relabel_nodes_kernel(const int32_t *__restrict__ perm, const int32_t *__restrict__ old_first_occ, int nnodes,
                                     int64_t nedges, int32_t *__restrict__ inverse, int32_t *__restrict__ degree) {
  const int a = blockIdx.x * blockDim.x + threadIdx.x;
  if (a >= nnodes) return;
  const int o = perm[a];
  inverse[o] = a;
  int e0 = old_first_occ[o], e1 = old_first_occ[nnodes + o];
  clamp_edge_range(e0, e1, nedges);
  degree[a] = e1 - e0;
}

// One workgroup: first_occ[a] = exclusive scan of degree, first_occ[n + a] = inclusive scan (the CSR layout the
// message-passing kernels take: starts, then ends).
__global__ __launch_bounds__(kScanThreads) void degree_scan_kernel(const int32_t *__restrict__ degree, int n,
                                                                   int32_t *__restrict__ first_occ) {
  __shared__ int part[kScanThreads];
  __shared__ int stage[kScanStage];
  workgroup_exclusive_scan<kScanThreads, kScanStage, int>(
      n, stage, part, [&](int k) { return degree[k]; },
      [&](int k, int before, int value) {
        first_occ[k] = before;
        first_occ[n + k] = before + value;
      });
}

// Sort key of an edge inside its segment: pairs within the cutoff by the new label of atom j, the others behind them
// by length (the bit pattern of a non-negative double orders like its value).
__global__ void edge_key_kernel(const double *__restrict__ pos, const int32_t *__restrict__ row_i, const int32_t *__restrict__ row_j,
                                const double *__restrict__ shifts, const int32_t *__restrict__ inverse, int64_t nedges, int nnodes,
                                double r_max, unsigned long long *__restrict__ key) {
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (e >= nedges) return;
  const int i = row_i[e], j = row_j[e];
  unsigned long long k = 0x7fffffffull;  // a pair that names no atom: behind the pairs within the cutoff
  if (static_cast<unsigned>(i) < static_cast<unsigned>(nnodes) && static_cast<unsigned>(j) < static_cast<unsigned>(nnodes)) {
    double v[3];
#pragma unroll
    for (int c = 0; c < 3; ++c) v[c] = (pos[3 * static_cast<int64_t>(j) + c] - pos[3 * static_cast<int64_t>(i) + c]) + shifts[3 * e + c];
    const double len = sqrt((v[0] * v[0] + v[1] * v[1]) + v[2] * v[2]);
    k = len > r_max ? (1ull << 63) | static_cast<unsigned long long>(__double_as_longlong(len))
                    : static_cast<unsigned long long>(static_cast<unsigned>(inverse[j]));
  }
  key[e] = k;
}

// One wave per new atom: ranks the pairs of its segment by (key, position in the list) and writes them to their places.
__global__ __launch_bounds__(kWave) void place_edges_kernel(const int32_t *__restrict__ perm, const int32_t *__restrict__ inverse,
                                                            const int32_t *__restrict__ old_first_occ,
                                                            const int32_t *__restrict__ new_first_occ,
                                                            const int32_t *__restrict__ row_j, const double *__restrict__ shifts,
                                                            const unsigned long long *__restrict__ key, int nnodes, int64_t nedges,
                                                            int32_t *__restrict__ receiver, int32_t *__restrict__ sender,
                                                            int32_t *__restrict__ edge_perm, double *__restrict__ shifts_out) {
  __shared__ unsigned long long sk[kSegLds];
  const int a = blockIdx.x, lane = threadIdx.x;
  const int o = perm[a];
  int s0 = old_first_occ[o], s1 = old_first_occ[nnodes + o];
  clamp_edge_range(s0, s1, nedges);
  const int d = s1 - s0;
  const int base = new_first_occ[a];
  const bool in_lds = d <= kSegLds;
  if (in_lds) {
    for (int t = lane; t < d; t += kWave) sk[t] = key[s0 + t];
    __syncthreads();
  }
  for (int k = lane; k < d; k += kWave) {
    const unsigned long long mine = in_lds ? sk[k] : key[s0 + k];
    int rank = 0;
    for (int t = 0; t < d; ++t) {
      const unsigned long long other = in_lds ? sk[t] : key[s0 + t];
      rank += (other < mine || (other == mine && t < k)) ? 1 : 0;
    }
    const int64_t e = s0 + k, at = base + rank;
    const int j = row_j[e];
    receiver[at] = a;
    sender[at] = static_cast<unsigned>(j) < static_cast<unsigned>(nnodes) ? inverse[j] : j;
    edge_perm[at] = static_cast<int32_t>(e);
    shifts_out[3 * at + 0] = shifts[3 * e + 0];
    shifts_out[3 * at + 1] = shifts[3 * e + 1];
    shifts_out[3 * at + 2] = shifts[3 * e + 2];
  }
}

inline size_t align256(size_t n) { return (n + 255) & ~static_cast<size_t>(255); }

struct PrepareLayout {
  double *box;
  int32_t *atom_keys, *bin_offsets, *old_first_occ, *degree;
  unsigned long long *edge_key;
  void *sort_ws;
  size_t sort_bytes, bytes;
  PrepareLayout(void *base, int64_t N, int64_t E, int64_t nkeys) {
    size_t at = 0;
    auto take = [&](size_t n) {
      char *p = base ? static_cast<char *>(base) + at : nullptr;
      at += align256(n);
      return p;
    };
    box = reinterpret_cast<double *>(take(4 * sizeof(double)));
    atom_keys = reinterpret_cast<int32_t *>(take(static_cast<size_t>(N) * 4));
    bin_offsets = reinterpret_cast<int32_t *>(take(static_cast<size_t>(nkeys + 1) * 4));
    old_first_occ = reinterpret_cast<int32_t *>(take(static_cast<size_t>(2 * N) * 4));
    degree = reinterpret_cast<int32_t *>(take(static_cast<size_t>(N) * 4));
    edge_key = reinterpret_cast<unsigned long long *>(take(static_cast<size_t>(E) * 8));
    const size_t a = cm_stable_key_sort_workspace(N, nkeys), b = cm_stable_key_sort_workspace(E, N);
    sort_bytes = a > b ? a : b;
    sort_ws = take(sort_bytes);
    bytes = at;
  }
};

}  // namespace
}  // namespace cm

extern "C" size_t cm_graph_prepare_workspace(int64_t nnodes, int64_t nedges, int ngraphs, int bins) {
  if (nnodes < 0 || nedges < 0 || ngraphs < 1 || bins < 1) return 0;
  return cm::PrepareLayout(nullptr, nnodes, nedges, static_cast<int64_t>(ngraphs) * bins * bins * bins).bytes;
}

extern "C" int cm_graph_prepare(const double *positions, const int32_t *row_i, const int32_t *row_j, const double *shifts,
                                const int32_t *graph_of_node, int64_t nnodes, int64_t nedges, int ngraphs, double r_max, int bins,
                                int32_t *node_perm, int32_t *node_inverse, int32_t *receiver, int32_t *sender, int32_t *edge_perm,
                                double *shifts_out, int32_t *first_occ, int32_t *sender_perm, int32_t *sender_offsets,
                                void *workspace, size_t workspace_bytes, cm_stream_t stream) {
  CM_REQUIRE(nnodes >= 0 && nedges >= 0 && nnodes < INT32_MAX / 4 && nedges < INT32_MAX / 3, "cm_graph_prepare: sizes out of range");
  CM_REQUIRE(ngraphs >= 1 && bins >= 1 && bins <= 64, "cm_graph_prepare: need at least one graph and 1 to 64 bins per axis");
  const int64_t nkeys = static_cast<int64_t>(ngraphs) * bins * bins * bins;
  CM_REQUIRE(nkeys < (int64_t{1} << 24), "cm_graph_prepare: ngraphs * bins^3 = %lld keys, at most 2^24 - 1", static_cast<long long>(nkeys));
  CM_REQUIRE(r_max > 0.0, "cm_graph_prepare: r_max must be positive");
  CM_REQUIRE(sender_offsets && (nnodes == 0 || first_occ), "cm_graph_prepare: NULL output");
  CM_REQUIRE(nnodes == 0 || (positions && node_perm && node_inverse), "cm_graph_prepare: NULL node operand");
  CM_REQUIRE(nedges == 0 || (row_i && row_j && shifts && receiver && sender && edge_perm && shifts_out && sender_perm),
             "cm_graph_prepare: NULL edge operand");
  const cm::PrepareLayout L(workspace, nnodes, nedges, nkeys);
  if (workspace == nullptr || workspace_bytes < L.bytes) {
    cm::set_error("cm_graph_prepare: workspace of %zu bytes, need %zu", workspace_bytes, L.bytes);
    return CM_ENOSPC;
  }
  CM_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, "cm_graph_prepare: workspace must be 256-byte aligned");
  hipStream_t st = cm::as_stream(stream);
  const int N = static_cast<int>(nnodes);
  const unsigned gn = static_cast<unsigned>(cm::ceil_div(nnodes > 0 ? nnodes : 1, 256));
  const unsigned ge = static_cast<unsigned>(cm::ceil_div(nedges > 0 ? nedges : 1, 256));
  int rc;
  // atoms: bounding box -> grid keys -> stable counting sort
  hipLaunchKernelGGL(cm::bounding_box_kernel, dim3(1), dim3(cm::kBoxThreads), 0, st, positions, nnodes, L.box);
  if (nnodes > 0)
    hipLaunchKernelGGL(cm::atom_key_kernel, dim3(gn), dim3(256), 0, st, positions, graph_of_node, nnodes, L.box, 0.5 * r_max, bins,
                       ngraphs, L.atom_keys);
  if ((rc = cm::check_launch("cm_graph_prepare")) != CM_OK) return rc;
  if ((rc = cm_stable_key_sort(L.atom_keys, nnodes, nkeys, node_perm, L.bin_offsets, L.sort_ws, L.sort_bytes, stream)) != CM_OK) return rc;
  // old CSR, inverse, degrees in the new order, new CSR
  if ((rc = cm_first_occurences(row_i, nedges, nnodes, L.old_first_occ, stream)) != CM_OK) return rc;
  if (nnodes > 0)
    hipLaunchKernelGGL(cm::relabel_nodes_kernel, dim3(gn), dim3(256), 0, st, node_perm, L.old_first_occ, N, nedges, node_inverse, L.degree);
  hipLaunchKernelGGL(cm::degree_scan_kernel, dim3(1), dim3(cm::kScanThreads), 0, st, L.degree, N, first_occ);
  // edges: key inside the segment, then every segment ranked and written by one wave
  if (nedges > 0) {
    hipLaunchKernelGGL(cm::edge_key_kernel, dim3(ge), dim3(256), 0, st, positions, row_i, row_j, shifts, node_inverse, nedges, N, r_max,
                       L.edge_key);
    hipLaunchKernelGGL(cm::place_edges_kernel, dim3(static_cast<unsigned>(nnodes)), dim3(cm::kWave), 0, st, node_perm, node_inverse,
                       L.old_first_occ, first_occ, row_j, shifts, L.edge_key, N, nedges, receiver, sender, edge_perm, shifts_out);
  }
  if ((rc = cm::check_launch("cm_graph_prepare")) != CM_OK) return rc;
  // the new list sorted by row j
  return cm_stable_key_sort(sender, nedges, nnodes, sender_perm, sender_offsets, L.sort_ws, L.sort_bytes, stream);
}
