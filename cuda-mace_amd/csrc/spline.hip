// Tabulated radial functions (natural cubic spline): evaluation and its derivative-weighted sum.
// The coefficient table ([nknots-1, 4, J], 2 MB at J = 512) stays in L2; the forward is a pure
// write stream of R[E, J], the backward a pure read stream of grad_R[E, J].
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
