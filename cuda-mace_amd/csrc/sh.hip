// Real spherical harmonics l <= 3 and their vector-Jacobian product, one thread per edge.
// Pure streaming kernels: consecutive lanes read consecutive edges (12-byte stride on the way in)
// and write 16 coalesced rows of Y[16, E].  The backward recomputes the derivatives from xyz, so no
// [16, 3, E] Jacobian ever goes to HBM.  Built for fp32 (the model's precision) and fp64 (the reference dispatches both,
// jit_wrappers/src/spherical_harmonics_wrapper.cpp:36, :105).
#include "sh_device.hpp"

namespace cm {
namespace {

template <typename T>
__global__ void sh_forward_kernel(const T *__restrict__ xyz, int64_t nedges, T *__restrict__ Y) {
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (e >= nedges) return;
  const sh::DirectionT<T> d = sh::direction(xyz[3 * e + 0], xyz[3 * e + 1], xyz[3 * e + 2]);
  T y[16];
  sh::eval(d, y);
#pragma unroll
  for (int m = 0; m < 16; ++m) Y[m * nedges + e] = y[m];
}

template <typename T>
__global__ void sh_backward_kernel(const T *__restrict__ xyz, const T *__restrict__ gY, int64_t nedges,
                                   T *__restrict__ gxyz) {
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (e >= nedges) return;
  const sh::DirectionT<T> d = sh::direction(xyz[3 * e + 0], xyz[3 * e + 1], xyz[3 * e + 2]);
  T g[16], gin[3];
  g[0] = T(0);
#pragma unroll
  for (int m = 1; m < 16; ++m) g[m] = gY[m * nedges + e];
  sh::vjp(d, g, gin);
  gxyz[3 * e + 0] = gin[0];
  gxyz[3 * e + 1] = gin[1];
  gxyz[3 * e + 2] = gin[2];
}

template <typename T>
int forward(const char *what, const T *xyz, int64_t nedges, T *Y, cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0, "%s: negative size", what);
  if (nedges == 0) return CM_OK;
  CM_REQUIRE(xyz && Y, "%s: NULL pointer", what);
  const int block = 256;
  hipLaunchKernelGGL(sh_forward_kernel<T>, dim3(static_cast<unsigned>(ceil_div(nedges, block))), dim3(block), 0,
                     as_stream(stream), xyz, nedges, Y);
  return check_launch(what);
}

template <typename T>
int backward(const char *what, const T *xyz, const T *grad_Y, int64_t nedges, T *grad_xyz, cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0, "%s: negative size", what);
  if (nedges == 0) return CM_OK;
  CM_REQUIRE(xyz && grad_Y && grad_xyz, "%s: NULL pointer", what);
  const int block = 256;
  hipLaunchKernelGGL(sh_backward_kernel<T>, dim3(static_cast<unsigned>(ceil_div(nedges, block))), dim3(block), 0,
                     as_stream(stream), xyz, grad_Y, nedges, grad_xyz);
  return check_launch(what);
}

}  // namespace
}  // namespace cm

extern "C" int cm_sh_forward(const float *xyz, int64_t nedges, float *Y, cm_stream_t stream) {
  return cm::forward("cm_sh_forward", xyz, nedges, Y, stream);
}

extern "C" int cm_sh_backward(const float *xyz, const float *grad_Y, int64_t nedges, float *grad_xyz,
                              cm_stream_t stream) {
  return cm::backward("cm_sh_backward", xyz, grad_Y, nedges, grad_xyz, stream);
}

extern "C" int cm_sh_forward_f64(const double *xyz, int64_t nedges, double *Y, cm_stream_t stream) {
  return cm::forward("cm_sh_forward_f64", xyz, nedges, Y, stream);
}

extern "C" int cm_sh_backward_f64(const double *xyz, const double *grad_Y, int64_t nedges, double *grad_xyz,
                                  cm_stream_t stream) {
  return cm::backward("cm_sh_backward_f64", xyz, grad_Y, nedges, grad_xyz, stream);
}
