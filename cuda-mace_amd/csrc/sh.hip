// Real spherical harmonics l <= 3 and their vector-Jacobian product, one thread per edge.
// Pure streaming kernels: consecutive lanes read consecutive edges (12-byte stride on the way in)
// and write 16 coalesced rows of Y[16, E].  The backward recomputes the derivatives from xyz, so no
// [16, 3, E] Jacobian ever goes to HBM.
#include "sh_device.hpp"

namespace cm {
namespace {

__global__ void sh_forward_kernel(const float *__restrict__ xyz, int64_t nedges, float *__restrict__ Y) {
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (e >= nedges) return;
  const sh::Direction d = sh::direction(xyz[3 * e + 0], xyz[3 * e + 1], xyz[3 * e + 2]);
  float y[16];
  sh::eval(d, y);
#pragma unroll
  for (int m = 0; m < 16; ++m) Y[m * nedges + e] = y[m];
}

__global__ void sh_backward_kernel(const float *__restrict__ xyz, const float *__restrict__ gY, int64_t nedges,
                                   float *__restrict__ gxyz) {
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (e >= nedges) return;
  const sh::Direction d = sh::direction(xyz[3 * e + 0], xyz[3 * e + 1], xyz[3 * e + 2]);
  float g[16], gin[3];
  g[0] = 0.f;
#pragma unroll
  for (int m = 1; m < 16; ++m) g[m] = gY[m * nedges + e];
  sh::vjp(d, g, gin);
  gxyz[3 * e + 0] = gin[0];
  gxyz[3 * e + 1] = gin[1];
  gxyz[3 * e + 2] = gin[2];
}

}  // namespace
}  // namespace cm

extern "C" int cm_sh_forward(const float *xyz, int64_t nedges, float *Y, cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0, "cm_sh_forward: negative size");
  if (nedges == 0) return CM_OK;
  CM_REQUIRE(xyz && Y, "cm_sh_forward: NULL pointer");
  const int block = 256;
  hipLaunchKernelGGL(cm::sh_forward_kernel, dim3(static_cast<unsigned>(cm::ceil_div(nedges, block))), dim3(block), 0,
                     cm::as_stream(stream), xyz, nedges, Y);
  return cm::check_launch("cm_sh_forward");
}

extern "C" int cm_sh_backward(const float *xyz, const float *grad_Y, int64_t nedges, float *grad_xyz,
                              cm_stream_t stream) {
  CM_REQUIRE(nedges >= 0, "cm_sh_backward: negative size");
  if (nedges == 0) return CM_OK;
  CM_REQUIRE(xyz && grad_Y && grad_xyz, "cm_sh_backward: NULL pointer");
  const int block = 256;
  hipLaunchKernelGGL(cm::sh_backward_kernel, dim3(static_cast<unsigned>(cm::ceil_div(nedges, block))), dim3(block), 0,
                     cm::as_stream(stream), xyz, grad_Y, nedges, grad_xyz);
  return cm::check_launch("cm_sh_backward");
}
