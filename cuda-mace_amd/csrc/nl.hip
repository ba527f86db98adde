// Neighbour list on the device: all ordered pairs (i, j, S) with |r_j - r_i + S . cell| < cutoff, sorted
// lexicographically by (i, j, Sx, Sy, Sz) -- the edge list the message-passing kernels consume (row i sorted).
//
// Cell list in fractional coordinates of the (possibly triclinic) cell: bins at least one cutoff wide along every
// axis (measured perpendicular to the other two cell vectors), atoms counting-sorted by bin, one wavefront per
// atom scanning the neighbouring bins with the lanes spread over a bin's atoms.  Two passes over the candidates
// (count, then fill after an exclusive scan) give every atom a contiguous segment without atomics; inside a
// segment the hits are placed at their rank under the (j, S) order, so the result is the unique sorted list and
// is reproducible bit for bit.
//
// The accept test uses the ORIGINAL fp64 positions and the integer image S only:
//     v = (r_j - r_i) + (Sx c0 + Sy c1 + Sz c2),   v0 v0 + v1 v1 + v2 v2 < cutoff^2,   (j, S) != (i, 0)
// evaluated left to right without fused multiply-adds, so that a host restatement of the same expression decides
// every borderline pair identically.  Bins only choose the candidates; they are 1e-9 wider than the cutoff so that
// rounding in the fractional coordinates cannot lose a pair.  Atoms may lie outside the cell (unwrapped
// trajectories): the wrap count of each atom enters S.
#include <algorithm>
#include <cmath>

#include "common.hpp"

namespace cm {
namespace {

constexpr int kGridThreads = 1024;
constexpr int kOffsetsStage = 16 * 1024;  // values staged in LDS at a time by the offsets scan (128 KB)
constexpr double kBinSlack = 1.0 + 1e-9;
constexpr int kMaxScan = 32;  // most images of the cell scanned on each side of an atom

struct Grid {
  double inv[9];    // inverse of the effective cell (row-vector convention: frac = r . inv)
  double cellv[9];  // the cell as given (used for S . cell)
  double fmin[3];   // lower bound of the binned range per axis (0 for periodic axes)
  double fscale[3]; // bins per unit of fractional coordinate
  int nb[3];        // bins per axis
  int nscan[3];     // bins to scan on each side
  int periodic[3];
  int status;       // 0 ok, 1 periodic axis with a singular cell, 2 cell thinner than cutoff / 32
};

struct Workspace {
  Grid *grid;
  int32_t *wrap;          // [N, 3]
  int32_t *keys;          // [N]
  int32_t *cell_perm;     // [N]
  int32_t *cell_offsets;  // [max_cells + 1]
  int32_t *degree;        // [N]
  void *sort_ws;
  size_t sort_ws_bytes;
  size_t total;
};

size_t align256(size_t b) { return (b + 255) & ~static_cast<size_t>(255); }

Workspace carve(void *base, int64_t n, int64_t max_cells) {
  Workspace w;
  char *p = static_cast<char *>(base);
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char *q = p ? p + off : nullptr;
    off += align256(bytes);
    return q;
  };
  w.grid = reinterpret_cast<Grid *>(take(sizeof(Grid)));
  w.wrap = reinterpret_cast<int32_t *>(take(sizeof(int32_t) * 3 * n));
  w.keys = reinterpret_cast<int32_t *>(take(sizeof(int32_t) * n));
  w.cell_perm = reinterpret_cast<int32_t *>(take(sizeof(int32_t) * n));
  w.cell_offsets = reinterpret_cast<int32_t *>(take(sizeof(int32_t) * (max_cells + 1)));
  w.degree = reinterpret_cast<int32_t *>(take(sizeof(int32_t) * n));
  w.sort_ws_bytes = cm_stable_key_sort_workspace(n, max_cells);
  w.sort_ws = take(w.sort_ws_bytes);
  w.total = off;
  return w;
}

__device__ __forceinline__ int floor_div(int a, int b) {
  int q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
  return q;
}

// One workgroup: effective cell and its inverse, extent of the atoms along non-periodic axes, bin counts.
__global__ __launch_bounds__(kGridThreads) void nl_grid_kernel(const double *__restrict__ pos, const double *__restrict__ cell,
                                                               int px, int py, int pz, double cutoff, int nnodes,
                                                               int max_cells, Grid *__restrict__ grid) {
  __shared__ double inv[9];
  __shared__ double lo[3][kGridThreads / kWave], hi[3][kGridThreads / kWave];
  __shared__ int singular;
  const int t = threadIdx.x;
  if (t == 0) {
    double c[9];
    for (int k = 0; k < 9; ++k) c[k] = cell ? cell[k] : 0.0;
    const double cx[3] = {c[4] * c[8] - c[5] * c[7], c[5] * c[6] - c[3] * c[8], c[3] * c[7] - c[4] * c[6]};  // c1 x c2
    const double det = c[0] * cx[0] + c[1] * cx[1] + c[2] * cx[2];
    const double n0 = sqrt(c[0] * c[0] + c[1] * c[1] + c[2] * c[2]), n1 = sqrt(c[3] * c[3] + c[4] * c[4] + c[5] * c[5]),
                 n2 = sqrt(c[6] * c[6] + c[7] * c[7] + c[8] * c[8]);
    const bool bad = !(fabs(det) > 1e-12 * n0 * n1 * n2) || !isfinite(det);
    singular = bad;
    if (bad) {
      for (int k = 0; k < 9; ++k) inv[k] = (k % 4 == 0) ? 1.0 : 0.0;
    } else {
      // inverse of the 3x3 matrix with rows c0, c1, c2: columns are the cross products / det
      const double r = 1.0 / det;
      inv[0] = cx[0] * r;
      inv[3] = cx[1] * r;
      inv[6] = cx[2] * r;
      inv[1] = (c[7] * c[2] - c[8] * c[1]) * r;  // (c2 x c0)
      inv[4] = (c[8] * c[0] - c[6] * c[2]) * r;
      inv[7] = (c[6] * c[1] - c[7] * c[0]) * r;
      inv[2] = (c[1] * c[5] - c[2] * c[4]) * r;  // (c0 x c1)
      inv[5] = (c[2] * c[3] - c[0] * c[5]) * r;
      inv[8] = (c[0] * c[4] - c[1] * c[3]) * r;
    }
  }
  __syncthreads();
  double mn[3] = {INFINITY, INFINITY, INFINITY}, mx[3] = {-INFINITY, -INFINITY, -INFINITY};
  for (int i = t; i < nnodes; i += kGridThreads) {
    const double x = pos[3 * i], y = pos[3 * i + 1], z = pos[3 * i + 2];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      const double f = x * inv[k] + y * inv[3 + k] + z * inv[6 + k];
      mn[k] = fmin(mn[k], f);
      mx[k] = fmax(mx[k], f);
    }
  }
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    for (int off = kWave / 2; off > 0; off >>= 1) {
      mn[k] = fmin(mn[k], __shfl_xor(mn[k], off));
      mx[k] = fmax(mx[k], __shfl_xor(mx[k], off));
    }
    if (t % kWave == 0) {
      lo[k][t / kWave] = mn[k];
      hi[k][t / kWave] = mx[k];
    }
  }
  __syncthreads();
  if (t == 0) {
    const int per[3] = {px, py, pz};
    Grid g;
    for (int k = 0; k < 9; ++k) {
      g.inv[k] = inv[k];
      g.cellv[k] = cell ? cell[k] : 0.0;
    }
    g.status = (singular && (px || py || pz)) ? 1 : 0;
    double width[3];  // distance covered by the binned range of axis k, perpendicular to the other two axes
    for (int k = 0; k < 3; ++k) {
      double a = INFINITY, b = -INFINITY;
      for (int w = 0; w < kGridThreads / kWave; ++w) {
        a = fmin(a, lo[k][w]);
        b = fmax(b, hi[k][w]);
      }
      const double height = 1.0 / sqrt(inv[k] * inv[k] + inv[3 + k] * inv[3 + k] + inv[6 + k] * inv[6 + k]);
      g.periodic[k] = per[k] ? 1 : 0;
      if (per[k]) {
        g.fmin[k] = 0.0;
        width[k] = height;
        const double bins = floor(height / (cutoff * kBinSlack));
        g.nb[k] = bins >= 1.0 ? static_cast<int>(fmin(bins, 1.0e6)) : 1;
      } else {
        const double ext = (nnodes > 0 && b > a) ? (b - a) : 0.0;
        g.fmin[k] = nnodes > 0 ? a : 0.0;
        width[k] = ext * height;
        const double bins = floor(width[k] / (cutoff * kBinSlack));
        g.nb[k] = bins >= 1.0 ? static_cast<int>(fmin(bins, 1.0e6)) : 1;
      }
    }
    // keep the number of bins within what the caller's workspace holds: halve the finest axis until it fits
    while (static_cast<int64_t>(g.nb[0]) * g.nb[1] * g.nb[2] > max_cells) {
      int k = 0;
      if (g.nb[1] > g.nb[k]) k = 1;
      if (g.nb[2] > g.nb[k]) k = 2;
      g.nb[k] = (g.nb[k] + 1) / 2;
    }
    for (int k = 0; k < 3; ++k) {
      if (g.periodic[k]) {
        g.fscale[k] = g.nb[k];
        const double binw = width[k] / g.nb[k];
        g.nscan[k] = static_cast<int>(ceil(cutoff * kBinSlack / binw));
      } else {
        const double ext = width[k] > 0.0 ? width[k] : 0.0;
        // fscale maps (f - fmin) to a bin number; a zero extent puts every atom in bin 0
        const double height = 1.0 / sqrt(inv[k] * inv[k] + inv[3 + k] * inv[3 + k] + inv[6 + k] * inv[6 + k]);
        g.fscale[k] = ext > 0.0 ? g.nb[k] * height / ext : 0.0;
        g.nscan[k] = g.nb[k] > 1 ? static_cast<int>(ceil(cutoff * kBinSlack / (ext / g.nb[k]))) : 0;
      }
      if (g.nscan[k] < 0) g.nscan[k] = 0;
      if (g.nscan[k] > kMaxScan) {  // a cell far thinner than the cutoff: refuse rather than scan thousands of images
        g.nscan[k] = 0;
        g.status = 2;
      }
    }
    *grid = g;
  }
}

__global__ void nl_bin_kernel(const double *__restrict__ pos, const Grid *__restrict__ grid, int nnodes,
                              int32_t *__restrict__ wrap, int32_t *__restrict__ keys) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nnodes) return;
  const double x = pos[3 * i], y = pos[3 * i + 1], z = pos[3 * i + 2];
  int b[3];
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    double f = x * grid->inv[k] + y * grid->inv[3 + k] + z * grid->inv[6 + k];
    int w = 0;
    if (grid->periodic[k]) {
      const double fl = floor(f);
      f -= fl;
      w = static_cast<int>(fl);
      if (f >= 1.0) {
        f -= 1.0;
        w += 1;
      }
    } else {
      f -= grid->fmin[k];
    }
    int bk = static_cast<int>(f * grid->fscale[k]);
    bk = bk < 0 ? 0 : (bk > grid->nb[k] - 1 ? grid->nb[k] - 1 : bk);
    b[k] = bk;
    wrap[3 * i + k] = w;
  }
  keys[i] = (b[0] * grid->nb[1] + b[1]) * grid->nb[2] + b[2];
}

// The accept test; see the head of this file.  No contraction into fused multiply-adds.
__device__ __forceinline__ bool within(const double *__restrict__ pi, const double *__restrict__ pj, const int (&S)[3],
                                       const double *__restrict__ c, double rc2) {
#pragma clang fp contract(off)
  double d2 = 0.0;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const double shift = (S[0] * c[k] + S[1] * c[3 + k]) + S[2] * c[6 + k];
    const double v = (pj[k] - pi[k]) + shift;
    d2 = k == 0 ? v * v : d2 + v * v;
  }
  return d2 < rc2;
}

// One wavefront per atom.  FILL = false: degree[i] = number of neighbours.  FILL = true: the neighbours (j, S) are
// written to scratch[offsets[i] ...] in scan order (j in scratch[0:E], S in scratch[E:4E]).
template <bool FILL>
__global__ __launch_bounds__(256) void nl_scan_kernel(const double *__restrict__ pos, const Grid *__restrict__ grid,
                                                      const int32_t *__restrict__ wrap, const int32_t *__restrict__ keys,
                                                      const int32_t *__restrict__ cell_perm,
                                                      const int32_t *__restrict__ cell_offsets, double cutoff, int nnodes,
                                                      const int32_t *__restrict__ offsets, int64_t nedges,
                                                      int32_t *__restrict__ degree, int32_t *__restrict__ scratch) {
  const int lane = threadIdx.x % kWave;
  const int i = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (i >= nnodes) return;
  const int nb0 = grid->nb[0], nb1 = grid->nb[1], nb2 = grid->nb[2];
  const int key = keys[i];
  const int bi[3] = {key / (nb1 * nb2), (key / nb2) % nb1, key % nb2};
  const int wi[3] = {wrap[3 * i], wrap[3 * i + 1], wrap[3 * i + 2]};
  const double pi[3] = {pos[3 * i], pos[3 * i + 1], pos[3 * i + 2]};
  const double rc2 = cutoff * cutoff;
  const double *c = grid->cellv;
  const int64_t seg = FILL ? offsets[i] : 0;
  int count = 0;
  if (grid->status == 0) {
    for (int d0 = -grid->nscan[0]; d0 <= grid->nscan[0]; ++d0) {
      int b0 = bi[0] + d0, B0 = 0;
      if (grid->periodic[0]) {
        B0 = floor_div(b0, nb0);
        b0 -= B0 * nb0;
      } else if (b0 < 0 || b0 >= nb0) {
        continue;
      }
      for (int d1 = -grid->nscan[1]; d1 <= grid->nscan[1]; ++d1) {
        int b1 = bi[1] + d1, B1 = 0;
        if (grid->periodic[1]) {
          B1 = floor_div(b1, nb1);
          b1 -= B1 * nb1;
        } else if (b1 < 0 || b1 >= nb1) {
          continue;
        }
        for (int d2 = -grid->nscan[2]; d2 <= grid->nscan[2]; ++d2) {
          int b2 = bi[2] + d2, B2 = 0;
          if (grid->periodic[2]) {
            B2 = floor_div(b2, nb2);
            b2 -= B2 * nb2;
          } else if (b2 < 0 || b2 >= nb2) {
            continue;
          }
          const int cellid = (b0 * nb1 + b1) * nb2 + b2;
          const int k0 = cell_offsets[cellid], k1 = cell_offsets[cellid + 1];
          for (int kb = k0; kb < k1; kb += kWave) {
            const int k = kb + lane;
            bool hit = false;
            int j = 0;
            int S[3] = {0, 0, 0};
            if (k < k1) {
              j = cell_perm[k];
              S[0] = B0 + wi[0] - wrap[3 * j];
              S[1] = B1 + wi[1] - wrap[3 * j + 1];
              S[2] = B2 + wi[2] - wrap[3 * j + 2];
              const double pj[3] = {pos[3 * j], pos[3 * j + 1], pos[3 * j + 2]};
              hit = within(pi, pj, S, c, rc2) && !(j == i && S[0] == 0 && S[1] == 0 && S[2] == 0);
            }
            const unsigned long long mask = __ballot(hit);
            if constexpr (FILL) {
              if (hit) {
                const int64_t at = seg + count + __popcll(mask & ((1ull << lane) - 1ull));
                if (at < nedges) {
                  scratch[at] = j;
                  scratch[nedges + 3 * at + 0] = S[0];
                  scratch[nedges + 3 * at + 1] = S[1];
                  scratch[nedges + 3 * at + 2] = S[2];
                }
              }
            }
            count += __popcll(mask);
          }
        }
      }
    }
  }
  if constexpr (!FILL) {
    if (lane == 0) degree[i] = count;
  }
}

// offsets[0 .. n] = exclusive scan of degree[0 .. n-1]; one workgroup, every thread a contiguous run.
__global__ __launch_bounds__(kGridThreads) void nl_offsets_kernel(const int32_t *__restrict__ degree, int n,
                                                                  int32_t *__restrict__ offsets) {
  __shared__ long long part[kGridThreads];
  __shared__ long long stage[kOffsetsStage];
  const long long total = workgroup_exclusive_scan<kGridThreads, kOffsetsStage, long long>(
      n, stage, part, [&](int k) { return degree[k]; },
      [&](int k, long long before, long long) { offsets[k] = static_cast<int32_t>(before > INT32_MAX ? INT32_MAX : before); });
  if (threadIdx.x == 0) offsets[n] = static_cast<int32_t>(total > INT32_MAX ? INT32_MAX : total);
}

__device__ __forceinline__ bool key_less(int ja, const int32_t *Sa, int jb, const int32_t *Sb) {
  if (ja != jb) return ja < jb;
  if (Sa[0] != Sb[0]) return Sa[0] < Sb[0];
  if (Sa[1] != Sb[1]) return Sa[1] < Sb[1];
  return Sa[2] < Sb[2];
}

// One wavefront per atom: every hit of its segment goes to its rank under the (j, S) order.
__global__ __launch_bounds__(256) void nl_rank_kernel(const int32_t *__restrict__ offsets, int nnodes, int64_t nedges,
                                                      const int32_t *__restrict__ scratch, int32_t *__restrict__ row_i,
                                                      int32_t *__restrict__ row_j, int32_t *__restrict__ unit_shifts) {
  const int lane = threadIdx.x % kWave;
  const int i = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (i >= nnodes) return;
  const int64_t e0 = offsets[i];
  const int64_t e1 = min(static_cast<int64_t>(offsets[i + 1]), nedges);
  const int32_t *sj = scratch;
  const int32_t *sS = scratch + nedges;
  for (int64_t e = e0 + lane; e < e1; e += kWave) {
    const int j = sj[e];
    const int32_t S[3] = {sS[3 * e], sS[3 * e + 1], sS[3 * e + 2]};
    int rank = 0;
    for (int64_t q = e0; q < e1; ++q) rank += key_less(sj[q], sS + 3 * q, j, S) ? 1 : 0;
    const int64_t at = e0 + rank;
    row_i[at] = i;
    row_j[at] = j;
    unit_shifts[3 * at + 0] = S[0];
    unit_shifts[3 * at + 1] = S[1];
    unit_shifts[3 * at + 2] = S[2];
  }
}

// ---- the test a Verlet list needs before it is reused: how far has any atom moved since the list was built ----
__global__ void clear_u64_kernel(unsigned long long *out) { *out = 0ull; }

// Non-negative doubles order like their bit patterns, so the maximum over the grid is an integer atomic.
__global__ __launch_bounds__(256) void max_displacement_kernel(const double *__restrict__ positions,
                                                               const double *__restrict__ reference, int64_t nnodes,
                                                               unsigned long long *__restrict__ out) {
#pragma clang fp contract(off)  // squares and sums as written, like the accept test of the list itself
  double worst = 0.0;
  for (int64_t n = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; n < nnodes;
       n += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const double d0 = positions[3 * n + 0] - reference[3 * n + 0];
    const double d1 = positions[3 * n + 1] - reference[3 * n + 1];
    const double d2 = positions[3 * n + 2] - reference[3 * n + 2];
    const double r2 = d0 * d0 + d1 * d1 + d2 * d2;
    worst = r2 > worst ? r2 : worst;  // a NaN coordinate is caught below
    if (!(r2 == r2)) worst = __builtin_inf();
  }
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const double other = __shfl_down(worst, off);
    worst = other > worst ? other : worst;
  }
  if (threadIdx.x % kWave == 0) atomicMax(out, static_cast<unsigned long long>(__double_as_longlong(worst)));
}

}  // namespace
}  // namespace cm

extern "C" int cm_max_displacement(const double *positions, const double *reference, int64_t nnodes, double *out_sq,
                                   cm_stream_t stream) {
  CM_REQUIRE(nnodes >= 0, "cm_max_displacement: negative size");
  CM_REQUIRE(out_sq && (nnodes == 0 || (positions && reference)), "cm_max_displacement: NULL pointer");
  hipStream_t st = cm::as_stream(stream);
  unsigned long long *out = reinterpret_cast<unsigned long long *>(out_sq);
  hipLaunchKernelGGL(cm::clear_u64_kernel, dim3(1), dim3(1), 0, st, out);
  if (nnodes > 0) {
    const unsigned blocks = static_cast<unsigned>(std::min<int64_t>(cm::ceil_div(nnodes, 256), 1024));
    hipLaunchKernelGGL(cm::max_displacement_kernel, dim3(blocks), dim3(256), 0, st, positions, reference, nnodes, out);
  }
  return cm::check_launch("cm_max_displacement");
}

extern "C" size_t cm_neighbour_list_workspace(int64_t nnodes, int64_t max_cells) {
  if (nnodes < 0 || max_cells < 1) return 0;
  return cm::carve(nullptr, nnodes, max_cells).total;
}

extern "C" int cm_neighbour_list_count(const double *positions, const double *cell, int pbc_x, int pbc_y, int pbc_z,
                                       double cutoff, int64_t nnodes, int64_t max_cells, void *workspace,
                                       size_t workspace_bytes, int32_t *offsets, int32_t *status, cm_stream_t stream) {
  CM_REQUIRE(nnodes >= 0 && nnodes < INT32_MAX / 4, "cm_neighbour_list_count: nnodes out of range");
  CM_REQUIRE(max_cells >= 1 && max_cells < INT32_MAX / 2, "cm_neighbour_list_count: max_cells out of range");
  CM_REQUIRE(cutoff > 0.0 && std::isfinite(cutoff), "cm_neighbour_list_count: cutoff must be positive and finite");
  CM_REQUIRE(offsets != nullptr && status != nullptr, "cm_neighbour_list_count: offsets / status is NULL");
  CM_REQUIRE(nnodes == 0 || positions != nullptr, "cm_neighbour_list_count: positions is NULL");
  CM_REQUIRE(cell != nullptr || !(pbc_x || pbc_y || pbc_z), "cm_neighbour_list_count: a periodic axis needs a cell");
  const cm::Workspace w = cm::carve(workspace, nnodes, max_cells);
  if (workspace == nullptr || workspace_bytes < w.total) {
    cm::set_error("cm_neighbour_list_count: workspace of %zu bytes, need %zu", workspace_bytes, w.total);
    return CM_ENOSPC;
  }
  hipStream_t st = cm::as_stream(stream);
  const int n = static_cast<int>(nnodes);
  hipLaunchKernelGGL(cm::nl_grid_kernel, dim3(1), dim3(cm::kGridThreads), 0, st, positions, cell, pbc_x, pbc_y, pbc_z, cutoff, n,
                     static_cast<int>(max_cells), w.grid);
  if (n > 0)
    hipLaunchKernelGGL(cm::nl_bin_kernel, dim3(static_cast<unsigned>(cm::ceil_div(n, 256))), dim3(256), 0, st, positions, w.grid,
                       n, w.wrap, w.keys);
  int rc = cm::check_launch("cm_neighbour_list_count (binning)");
  if (rc != CM_OK) return rc;
  rc = cm_stable_key_sort(w.keys, nnodes, max_cells, w.cell_perm, w.cell_offsets, w.sort_ws, w.sort_ws_bytes, stream);
  if (rc != CM_OK) return rc;
  if (n > 0)
    hipLaunchKernelGGL(cm::nl_scan_kernel<false>, dim3(static_cast<unsigned>(cm::ceil_div(n, 4))), dim3(256), 0, st, positions,
                       w.grid, w.wrap, w.keys, w.cell_perm, w.cell_offsets, cutoff, n, static_cast<const int32_t *>(nullptr),
                       int64_t{0}, w.degree, static_cast<int32_t *>(nullptr));
  hipLaunchKernelGGL(cm::nl_offsets_kernel, dim3(1), dim3(cm::kGridThreads), 0, st, w.degree, n, offsets);
  // the status word sits behind the grid header; copy it out with a kernel-free device-to-device copy
  if (hipMemcpyAsync(status, &w.grid->status, sizeof(int32_t), hipMemcpyDeviceToDevice, st) != hipSuccess) {
    cm::set_error("cm_neighbour_list_count: status copy failed");
    return CM_ELAUNCH;
  }
  return cm::check_launch("cm_neighbour_list_count");
}

extern "C" int cm_neighbour_list_fill(const double *positions, double cutoff, int64_t nnodes, int64_t max_cells,
                                      const void *workspace, const int32_t *offsets, int64_t nedges, int32_t *edge_scratch,
                                      int32_t *row_i, int32_t *row_j, int32_t *unit_shifts, cm_stream_t stream) {
  CM_REQUIRE(nnodes >= 0 && nnodes < INT32_MAX / 4, "cm_neighbour_list_fill: nnodes out of range");
  CM_REQUIRE(max_cells >= 1 && max_cells < INT32_MAX / 2, "cm_neighbour_list_fill: max_cells out of range");
  CM_REQUIRE(nedges >= 0 && nedges < INT32_MAX / 4, "cm_neighbour_list_fill: nedges out of range");
  CM_REQUIRE(cutoff > 0.0 && std::isfinite(cutoff), "cm_neighbour_list_fill: cutoff must be positive and finite");
  if (nnodes == 0 || nedges == 0) return CM_OK;
  CM_REQUIRE(positions && workspace && offsets && edge_scratch && row_i && row_j && unit_shifts,
             "cm_neighbour_list_fill: NULL pointer");
  const cm::Workspace w = cm::carve(const_cast<void *>(workspace), nnodes, max_cells);
  hipStream_t st = cm::as_stream(stream);
  const int n = static_cast<int>(nnodes);
  const dim3 grid(static_cast<unsigned>(cm::ceil_div(n, 4)));
  hipLaunchKernelGGL(cm::nl_scan_kernel<true>, grid, dim3(256), 0, st, positions, w.grid, w.wrap, w.keys, w.cell_perm,
                     w.cell_offsets, cutoff, n, offsets, nedges, static_cast<int32_t *>(nullptr), edge_scratch);
  hipLaunchKernelGGL(cm::nl_rank_kernel, grid, dim3(256), 0, st, offsets, n, nedges, edge_scratch, row_i, row_j, unit_shifts);
  return cm::check_launch("cm_neighbour_list_fill");
}
