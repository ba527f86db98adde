// Tabulated radial functions (natural cubic spline): evaluation and its derivative-weighted sum.
// The coefficient table ([nknots-1, 4, J], 2 MB at J = 512) stays in L2; the forward is a pure
// write stream of R[E, J], the backward a pure read stream of grad_R[E, J].
#include <algorithm>

#include "common.hpp"

namespace cm {
namespace {

__device__ __forceinline__ int knot_index(float r, float r_width, int nknots) {
  int idx = static_cast<int>(r / r_width);
  return idx < 0 ? 0 : (idx > nknots - 2 ? nknots - 2 : idx);
}

// One thread per four consecutive outputs of one edge.
template <bool DERIV>
__global__ void spline_forward_kernel(const float *__restrict__ r, const float *__restrict__ r_knots,
                                      const float *__restrict__ coeffs, int64_t nedges, int nknots, int J,
                                      float r_width, float r_max, float *__restrict__ R_out,
                                      float *__restrict__ R_deriv) {
  const int J4 = J / 4;
  const int64_t t = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (t >= nedges * J4) return;
  const int64_t e = t / J4;
  const int j = static_cast<int>(t - e * J4) * 4;
  const float re = r[e];
  f4 val = zero4(), der = zero4();
  if (re <= r_max) {
    const int idx = knot_index(re, r_width, nknots);
    const float x = re - r_knots[idx];
    const float *cp = coeffs + static_cast<int64_t>(idx) * 4 * J + j;
    const f4 a = ld4(cp), b = ld4(cp + J), c = ld4(cp + 2 * J), d = ld4(cp + 3 * J);
    val = a + x * (b + x * (c + x * d));
    if (DERIV) der = b + x * (2.f * c + (3.f * x) * d);
  }
  st4_stream(R_out + e * J + j, val);
  if (DERIV) st4_stream(R_deriv + e * J + j, der);
}

// ---- LDS-table variant of the forward for long edge lists --------------------------------------------------------
// The kernel above pulls the four coefficient vectors of every output through L1 (64 bytes read for 16 written); with
// the 2 MB table spread over all intervals nothing of it stays in a 32 KB L1, so the compute unit's L1 path carries four
// times the bytes of the HBM write stream and sets the pace.  Here a workgroup owns 32 consecutive outputs (one
// 128-byte line of every edge's row) and keeps their coefficients for EVERY interval in LDS ([interval][4][32]
// floats, 512 bytes per interval, a row of zeros behind the last one for edges beyond the cutoff; 139 KB at most); it
// then walks its share of the edges, eight lanes per edge (16 bytes each), eight edges per wave and trip, and each wave
// store writes eight whole lines (4.0 -> 5.2 TB/s at 1.3 million edges x 512 outputs; stores that scatter whole lines
// over rows do not reach what a contiguous stream does).  The workgroups of one
// output slice sit `nslices` apart in the grid, so at any time all slices, hence all parts of a row, are being written.
constexpr int kSpThreads = 512;
constexpr int kSpSlice = 32;            // outputs per workgroup
constexpr int kSpMaxIntervals = 272;    // rows of the slice, the row of zeros included: 272 * 4 * 32 * 4 B = 139 264 B of LDS
constexpr int64_t kSpMinEdges = 1 << 15;

__global__ __launch_bounds__(kSpThreads) void spline_forward_sliced_kernel(
    const float *__restrict__ r, const float *__restrict__ r_knots, const float *__restrict__ coeffs, int64_t nedges,
    int nknots, int J, float r_width, float r_max, float *__restrict__ R_out, int nslices, int share) {
  __shared__ __attribute__((aligned(16))) float sTab[kSpMaxIntervals * 4 * kSpSlice];
  __shared__ float sKnots[kSpMaxIntervals + 1];
  const int tid = threadIdx.x;
  const int slice = blockIdx.x % nslices;
  const int part = blockIdx.x / nslices;
  const int j0 = slice * kSpSlice;
  // 16-byte pieces: row = 4 * interval + coefficient, eight pieces per row (J is a multiple of 4: a piece is inside the
  // table or beyond it as a whole)
  for (int t = tid; t < (nknots - 1) * 4 * (kSpSlice / 4); t += kSpThreads) {
    const int row = t >> 3, q = t & 7;
    const int j = j0 + 4 * q;
    *reinterpret_cast<f4 *>(sTab + row * kSpSlice + 4 * q) = j < J ? ld4(coeffs + static_cast<int64_t>(row) * J + j) : zero4();
  }
  if (tid < 4 * (kSpSlice / 4)) *reinterpret_cast<f4 *>(sTab + (nknots - 1) * 4 * kSpSlice + 4 * tid) = zero4();  // row of zeros
  for (int t = tid; t < nknots; t += kSpThreads) sKnots[t] = r_knots[t];
  __syncthreads();

  const int lane = tid % kWave;
  const int q = lane & 7;   // 16-byte piece of the slice
  const int g = lane >> 3;  // edge of a trip
  const int j = j0 + 4 * q;
  const bool inside = j < J;  // false in the last slice of a row that is no multiple of 32 wide
  const char *tab = reinterpret_cast<const char *>(sTab) + 16 * q;
  const unsigned zero_row = static_cast<unsigned>(nknots - 1) * (4 * kSpSlice * 4);
  // A wave takes 64 consecutive edges per round: every lane prepares one of them (interval, offset inside it; an edge
  // beyond the cutoff points at the row of zeros), then eight trips of eight edges, each lane fetching its trip's edge
  // from the lane that prepared it.  The radii of the wave's next round are requested before the trips.
  const int64_t rounds = (nedges + kWave - 1) / kWave;
  const int64_t stride = static_cast<int64_t>(share) * (kSpThreads / kWave);
  int64_t round = static_cast<int64_t>(part) * (kSpThreads / kWave) + tid / kWave;
  if (round >= rounds) return;
  const int64_t last = nedges - 1;
  float re = r[min(round * kWave + lane, last)];
  for (; round < rounds; round += stride) {
    const int64_t nxt = round + stride < rounds ? round + stride : round;
    const float re_next = r[min(nxt * kWave + lane, last)];
    const bool live = re <= r_max;
    const int idx = knot_index(re, r_width, nknots);
    const unsigned off = live ? static_cast<unsigned>(idx) * (4 * kSpSlice * 4) : zero_row;
    const float x = live ? re - sKnots[idx] : 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int src = 8 * t + g;
      const char *row = tab + __shfl(off, src);
      const float xs = __shfl(x, src);
      const f4 a = *reinterpret_cast<const f4 *>(row), b = *reinterpret_cast<const f4 *>(row + 128),
               c = *reinterpret_cast<const f4 *>(row + 256), d = *reinterpret_cast<const f4 *>(row + 384);
      const int64_t e = round * kWave + src;
      if (inside && e <= last) st4_stream(R_out + e * J + j, a + xs * (b + xs * (c + xs * d)));
    }
    re = re_next;
  }
}

bool spline_sliced_applies(int64_t nedges, int nknots, int J) {
  return nedges >= kSpMinEdges && nknots - 1 < kSpMaxIntervals && ceil_div(J, kSpSlice) <= device_compute_units();
}

void launch_spline_forward_sliced(const float *r, const float *r_knots, const float *coeffs, int64_t nedges, int nknots, int J,
                                  float r_width, float r_max, float *R_out, hipStream_t st) {
  const int nslices = static_cast<int>(ceil_div(J, kSpSlice));
  const int share = device_compute_units() / nslices;
  hipLaunchKernelGGL(spline_forward_sliced_kernel, dim3(static_cast<unsigned>(nslices * share)), dim3(kSpThreads), 0, st, r,
                     r_knots, coeffs, nedges, nknots, J, r_width, r_max, R_out, nslices, share);
}

// One wavefront per edge: grad_r[e] = sum_j grad_R[e, j] * dR/dr[e, j].
__global__ __launch_bounds__(256) void spline_backward_kernel(
    const float *__restrict__ r, const float *__restrict__ r_knots, const float *__restrict__ coeffs,
    const float *__restrict__ gR, int64_t nedges, int nknots, int J, float r_width, float r_max,
    float *__restrict__ gr) {
  const int lane = threadIdx.x % kWave;
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x / kWave) + threadIdx.x / kWave;
  if (e >= nedges) return;
  const float re = r[e];
  float sum = 0.f;
  if (re <= r_max) {
    const int idx = knot_index(re, r_width, nknots);
    const float x = re - r_knots[idx];
    const float *cp = coeffs + static_cast<int64_t>(idx) * 4 * J;
    const float *gp = gR + e * J;
    f4 acc = zero4();
    for (int j = 4 * lane; j < J; j += 4 * kWave) {
      const f4 b = ld4(cp + J + j), c = ld4(cp + 2 * J + j), d = ld4(cp + 3 * J + j);
      acc += ld4_stream(gp + j) * (b + x * (2.f * c + (3.f * x) * d));
    }
    sum = hsum4(acc);
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  if (lane == 0) gr[e] = sum;
}

// ---- LDS-table variant of the backward for long edge lists -------------------------------------------------------
// As in the forward, the kernel above reads 48 bytes of coefficients through L1 for every 16 bytes of the gradient
// stream.  Here a workgroup owns a chunk of consecutive edges and sums them slice by slice: for each slice of 32
// outputs it loads the derivative's coefficients (b, 2c, 3d per interval: 384 bytes, 104 KB at most) into LDS, streams
// that slice of its edges' gradient rows (one 128-byte line per edge) and adds each edge's partial sum to the edge's
// cell in LDS; after the last slice the cells go to grad_r.  One lane group adds to a cell per slice, and the slices
// follow each other in a fixed order (workgroup b starts at slice b % nslices, so that at any time all parts of the
// rows are being read): the result is reproducible.  The table is re-read from L2 once per slice and chunk, a sixth of
// the bytes of the gradient stream at 5 000 edges per chunk.
constexpr int kSpBwdRow = 3 * kSpSlice;  // floats per interval
constexpr int kSpBwdChunk = 8192;        // edges per chunk at most (their sums: 32 KB of LDS)

__global__ __launch_bounds__(kSpThreads) void spline_backward_sliced_kernel(
    const float *__restrict__ r, const float *__restrict__ r_knots, const float *__restrict__ coeffs,
    const float *__restrict__ gR, int64_t nedges, int nknots, int J, float r_width, float r_max, float *__restrict__ gr,
    int nslices, int chunk) {
  __shared__ __attribute__((aligned(16))) float sTab[kSpMaxIntervals * kSpBwdRow];
  __shared__ float sKnots[kSpMaxIntervals + 1];
  __shared__ float sSum[kSpBwdChunk];
  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int q = lane & 7;   // 16-byte piece of the slice
  const int g = lane >> 3;  // edge of a trip
  const char *tab = reinterpret_cast<const char *>(sTab) + 16 * q;
  const unsigned zero_row = static_cast<unsigned>(nknots - 1) * (kSpBwdRow * 4);
  for (int t = tid; t < nknots; t += kSpThreads) sKnots[t] = r_knots[t];

  for (int64_t c0 = static_cast<int64_t>(blockIdx.x) * chunk; c0 < nedges; c0 += static_cast<int64_t>(gridDim.x) * chunk) {
    const int n = static_cast<int>(min(static_cast<int64_t>(chunk), nedges - c0));
    for (int t = tid; t < n; t += kSpThreads) sSum[t] = 0.f;
    for (int pass = 0; pass < nslices; ++pass) {
      const int slice = static_cast<int>((blockIdx.x + static_cast<unsigned>(pass)) % static_cast<unsigned>(nslices));
      const int j0 = slice * kSpSlice;
      __syncthreads();  // the table of the previous slice is no longer read (and the sums are cleared)
      for (int t = tid; t < (nknots - 1) * 3 * (kSpSlice / 4); t += kSpThreads) {
        const int row = t >> 3, piece = t & 7;
        const int idx = row / 3, k = row - 3 * idx;  // k = 0, 1, 2: b, 2 c, 3 d
        const int j = j0 + 4 * piece;
        const f4 v = j < J ? ld4(coeffs + (static_cast<int64_t>(idx) * 4 + k + 1) * J + j) : zero4();
        *reinterpret_cast<f4 *>(sTab + row * kSpSlice + 4 * piece) = static_cast<float>(k + 1) * v;
      }
      if (tid < 3 * (kSpSlice / 4)) *reinterpret_cast<f4 *>(sTab + (nknots - 1) * kSpBwdRow + 4 * tid) = zero4();  // row of zeros
      __syncthreads();
      const int j = j0 + 4 * q;
      const bool inside = j < J;
      const int jc = inside ? j : 0;  // lanes beyond the row read its first piece and drop it
      for (int base = wave * kWave; base < n; base += kSpThreads) {
        // every lane prepares one of the round's 64 edges
        const float re = r[c0 + min(base + lane, n - 1)];
        const bool live = re <= r_max;
        const int idx = knot_index(re, r_width, nknots);
        const unsigned off = live ? static_cast<unsigned>(idx) * (kSpBwdRow * 4) : zero_row;
        const float x = live ? re - sKnots[idx] : 0.f;
        f4 gv[8];
#pragma unroll
        for (int t = 0; t < 8; ++t)  // unconditional: an edge beyond the chunk reads the chunk's last edge and is dropped
          gv[t] = ld4_stream(gR + (c0 + min(base + 8 * t + g, n - 1)) * J + jc);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const int src = 8 * t + g;
          const unsigned o = __shfl(off, src);
          const float xs = __shfl(x, src);
          const char *row = tab + o;
          const f4 b = *reinterpret_cast<const f4 *>(row), c2 = *reinterpret_cast<const f4 *>(row + 128),
                   d3 = *reinterpret_cast<const f4 *>(row + 256);
          float part = hsum4(gv[t] * (b + xs * (c2 + xs * d3)));
          part = (inside && o != zero_row) ? part : 0.f;  // an edge beyond the cutoff contributes nothing, whatever its gradient
          part += __shfl_xor(part, 1);
          part += __shfl_xor(part, 2);
          part += __shfl_xor(part, 4);
          if (q == 0 && base + src < n) sSum[base + src] += part;  // this lane alone adds to the cell in this slice; slices are barriers apart
        }
      }
    }
    __syncthreads();
    for (int t = tid; t < n; t += kSpThreads) gr[c0 + t] = sSum[t];
    __syncthreads();
  }
}

void launch_spline_backward_sliced(const float *r, const float *r_knots, const float *coeffs, const float *gR, int64_t nedges,
                                   int nknots, int J, float r_width, float r_max, float *gr, hipStream_t st) {
  const int cus = device_compute_units();
  const int64_t per_group = ceil_div(ceil_div(nedges, cus), kSpBwdChunk);  // chunks per workgroup
  const int chunk = static_cast<int>(ceil_div(ceil_div(nedges, cus * per_group), kWave) * kWave);  // <= kSpBwdChunk, whole rounds
  const int groups = static_cast<int>(std::min<int64_t>(cus, ceil_div(nedges, chunk)));
  hipLaunchKernelGGL(spline_backward_sliced_kernel, dim3(static_cast<unsigned>(groups)), dim3(kSpThreads), 0, st, r, r_knots,
                     coeffs, gR, nedges, nknots, J, r_width, r_max, gr, static_cast<int>(ceil_div(J, kSpSlice)), chunk);
}

// fp64 variants (the reference dispatches the spline on float and double, jit_wrappers/src/cubic_spline_wrapper.cpp:50,
// :123): one thread per output, same knot lookup and Horner forms as above.
__device__ __forceinline__ int knot_index(double r, double r_width, int nknots) {
  int idx = static_cast<int>(r / r_width);
  return idx < 0 ? 0 : (idx > nknots - 2 ? nknots - 2 : idx);
}

template <bool DERIV>
__global__ void spline_forward_f64_kernel(const double *__restrict__ r, const double *__restrict__ r_knots,
                                          const double *__restrict__ coeffs, int64_t nedges, int nknots, int J,
                                          double r_width, double r_max, double *__restrict__ R_out,
                                          double *__restrict__ R_deriv) {
  const int64_t t = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (t >= nedges * J) return;
  const int64_t e = t / J;
  const int j = static_cast<int>(t - e * J);
  const double re = r[e];
  double val = 0.0, der = 0.0;
  if (re <= r_max) {
    const int idx = knot_index(re, r_width, nknots);
    const double x = re - r_knots[idx];
    const double *cp = coeffs + static_cast<int64_t>(idx) * 4 * J + j;
    const double a = cp[0], b = cp[J], c = cp[2 * J], d = cp[3 * J];
    val = a + x * (b + x * (c + x * d));
    if (DERIV) der = b + x * (2.0 * c + (3.0 * x) * d);
  }
  R_out[t] = val;
  if (DERIV) R_deriv[t] = der;
}

__global__ __launch_bounds__(256) void spline_backward_f64_kernel(
    const double *__restrict__ r, const double *__restrict__ r_knots, const double *__restrict__ coeffs,
    const double *__restrict__ gR, int64_t nedges, int nknots, int J, double r_width, double r_max,
    double *__restrict__ gr) {
  const int lane = threadIdx.x % kWave;
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x / kWave) + threadIdx.x / kWave;
  if (e >= nedges) return;
  const double re = r[e];
  double sum = 0.0;
  if (re <= r_max) {
    const int idx = knot_index(re, r_width, nknots);
    const double x = re - r_knots[idx];
    const double *cp = coeffs + static_cast<int64_t>(idx) * 4 * J;
    const double *gp = gR + e * J;
    for (int j = lane; j < J; j += kWave) sum += gp[j] * (cp[J + j] + x * (2.0 * cp[2 * J + j] + (3.0 * x) * cp[3 * J + j]));
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  if (lane == 0) gr[e] = sum;
}

}  // namespace
}  // namespace cm

extern "C" int cm_spline_forward(const float *r, const float *r_knots, const float *coeffs, int64_t nedges,
                                 int nknots, int noutputs, float r_width, float r_max, float *R_out,
                                 float *R_deriv, cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0, "cm_spline_forward: negative size");
  CM_REQUIRE(nknots >= 2, "cm_spline_forward: need at least two knots, got %d", nknots);
  CM_REQUIRE(noutputs > 0 && noutputs % 4 == 0, "cm_spline_forward: noutputs=%d must be a positive multiple of 4", noutputs);
  CM_REQUIRE(r_width > 0.f, "cm_spline_forward: r_width must be positive");
  if (nedges == 0) return CM_OK;
  CM_REQUIRE(r && r_knots && coeffs && R_out, "cm_spline_forward: NULL pointer");
  // With the derivative as a second output the direct kernel below writes two streams per set of coefficient loads and
  // reaches 6.3 TB/s at 1.3 million edges x 512 outputs; the LDS-table kernel's line-by-line stores stay at 5.2 TB/s.
  if (!R_deriv && cm::spline_sliced_applies(nedges, nknots, noutputs)) {
    cm::launch_spline_forward_sliced(r, r_knots, coeffs, nedges, nknots, noutputs, r_width, r_max, R_out, cm::as_stream(stream));
    return cm::check_launch("cm_spline_forward");
  }
  const int block = 256;
  const int64_t threads = nedges * (noutputs / 4);
  CM_REQUIRE(cm::ceil_div(threads, block) < INT32_MAX, "cm_spline_forward: problem too large for one launch");
  const dim3 grid(static_cast<unsigned>(cm::ceil_div(threads, block)));
  if (R_deriv)
    hipLaunchKernelGGL(cm::spline_forward_kernel<true>, grid, dim3(block), 0, cm::as_stream(stream), r, r_knots, coeffs,
                       nedges, nknots, noutputs, r_width, r_max, R_out, R_deriv);
  else
    hipLaunchKernelGGL(cm::spline_forward_kernel<false>, grid, dim3(block), 0, cm::as_stream(stream), r, r_knots, coeffs,
                       nedges, nknots, noutputs, r_width, r_max, R_out, R_deriv);
  return cm::check_launch("cm_spline_forward");
}

extern "C" int cm_spline_backward(const float *r, const float *r_knots, const float *coeffs, const float *grad_R,
                                  int64_t nedges, int nknots, int noutputs, float r_width, float r_max,
                                  float *grad_r, cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0, "cm_spline_backward: negative size");
  CM_REQUIRE(nknots >= 2, "cm_spline_backward: need at least two knots, got %d", nknots);
  CM_REQUIRE(noutputs > 0 && noutputs % 4 == 0, "cm_spline_backward: noutputs=%d must be a positive multiple of 4", noutputs);
  CM_REQUIRE(r_width > 0.f, "cm_spline_backward: r_width must be positive");
  if (nedges == 0) return CM_OK;
  CM_REQUIRE(r && r_knots && coeffs && grad_R && grad_r, "cm_spline_backward: NULL pointer");
  if (cm::spline_sliced_applies(nedges, nknots, noutputs)) {
    cm::launch_spline_backward_sliced(r, r_knots, coeffs, grad_R, nedges, nknots, noutputs, r_width, r_max, grad_r,
                                      cm::as_stream(stream));
    return cm::check_launch("cm_spline_backward");
  }
  const int block = 256;
  const int per = block / cm::kWave;
  hipLaunchKernelGGL(cm::spline_backward_kernel, dim3(static_cast<unsigned>(cm::ceil_div(nedges, per))), dim3(block), 0,
                     cm::as_stream(stream), r, r_knots, coeffs, grad_R, nedges, nknots, noutputs, r_width, r_max, grad_r);
  return cm::check_launch("cm_spline_backward");
}

extern "C" int cm_spline_forward_f64(const double *r, const double *r_knots, const double *coeffs, int64_t nedges,
                                     int nknots, int noutputs, double r_width, double r_max, double *R_out,
                                     double *R_deriv, cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0, "cm_spline_forward_f64: negative size");
  CM_REQUIRE(nknots >= 2, "cm_spline_forward_f64: need at least two knots, got %d", nknots);
  CM_REQUIRE(noutputs > 0, "cm_spline_forward_f64: noutputs=%d must be positive", noutputs);
  CM_REQUIRE(r_width > 0.0, "cm_spline_forward_f64: r_width must be positive");
  if (nedges == 0) return CM_OK;
  CM_REQUIRE(r && r_knots && coeffs && R_out, "cm_spline_forward_f64: NULL pointer");
  const int block = 256;
  const int64_t threads = nedges * noutputs;
  CM_REQUIRE(cm::ceil_div(threads, block) < INT32_MAX, "cm_spline_forward_f64: problem too large for one launch");
  const dim3 grid(static_cast<unsigned>(cm::ceil_div(threads, block)));
  if (R_deriv)
    hipLaunchKernelGGL(cm::spline_forward_f64_kernel<true>, grid, dim3(block), 0, cm::as_stream(stream), r, r_knots, coeffs,
                       nedges, nknots, noutputs, r_width, r_max, R_out, R_deriv);
  else
    hipLaunchKernelGGL(cm::spline_forward_f64_kernel<false>, grid, dim3(block), 0, cm::as_stream(stream), r, r_knots, coeffs,
                       nedges, nknots, noutputs, r_width, r_max, R_out, R_deriv);
  return cm::check_launch("cm_spline_forward_f64");
}

extern "C" int cm_spline_backward_f64(const double *r, const double *r_knots, const double *coeffs, const double *grad_R,
                                      int64_t nedges, int nknots, int noutputs, double r_width, double r_max,
                                      double *grad_r, cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0, "cm_spline_backward_f64: negative size");
  CM_REQUIRE(nknots >= 2, "cm_spline_backward_f64: need at least two knots, got %d", nknots);
  CM_REQUIRE(noutputs > 0, "cm_spline_backward_f64: noutputs=%d must be positive", noutputs);
  CM_REQUIRE(r_width > 0.0, "cm_spline_backward_f64: r_width must be positive");
  if (nedges == 0) return CM_OK;
  CM_REQUIRE(r && r_knots && coeffs && grad_R && grad_r, "cm_spline_backward_f64: NULL pointer");
  const int block = 256;
  const int per = block / cm::kWave;
  hipLaunchKernelGGL(cm::spline_backward_f64_kernel, dim3(static_cast<unsigned>(cm::ceil_div(nedges, per))), dim3(block), 0,
                     cm::as_stream(stream), r, r_knots, coeffs, grad_R, nedges, nknots, noutputs, r_width, r_max, grad_r);
  return cm::check_launch("cm_spline_backward_f64");
}
