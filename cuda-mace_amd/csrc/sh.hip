// Real spherical harmonics l <= 3 and their vector-Jacobian product, one thread per edge.
// Pure streaming kernels: consecutive lanes read consecutive edges (12-byte stride on the way in)
// and write 16 coalesced rows of Y[16, E].  The backward recomputes the derivatives from xyz, so no
// [16, 3, E] Jacobian ever goes to HBM.
#include "common.hpp"

namespace cm {
namespace {

// sqrt(4 pi) is folded into the constants: Y_00 = 1 and sum_{m in l} Y_lm^2 = 2l + 1.
constexpr float kS3 = 1.7320508075688772f;    // sqrt(3)
constexpr float kS5 = 2.23606797749979f;      // sqrt(5)
constexpr float kS7 = 2.6457513110645907f;    // sqrt(7)
constexpr float kS15 = 3.872983346207417f;    // sqrt(15)
constexpr float kS105 = 10.246950765959598f;  // sqrt(105)
constexpr float kA = 2.091650066335189f;      // sqrt(35/8)
constexpr float kB = 1.6201851746019651f;     // sqrt(21/8)

__global__ void sh_forward_kernel(const float *__restrict__ xyz, int64_t nedges, float *__restrict__ Y) {
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (e >= nedges) return;
  // axis permutation of the inputs: (x, y, z) = (in[2], in[0], in[1])
  float y = xyz[3 * e + 0], z = xyz[3 * e + 1], x = xyz[3 * e + 2];
  const float ir = 1.0f / sqrtf(x * x + y * y + z * z);
  x *= ir;
  y *= ir;
  z *= ir;
  const float x2 = x * x, y2 = y * y, z2 = z * z;
  float *o = Y + e;
  o[0 * nedges] = 1.0f;
  o[1 * nedges] = kS3 * y;
  o[2 * nedges] = kS3 * z;
  o[3 * nedges] = kS3 * x;
  o[4 * nedges] = kS15 * x * y;
  o[5 * nedges] = kS15 * y * z;
  o[6 * nedges] = 0.5f * kS5 * (2.f * z2 - x2 - y2);
  o[7 * nedges] = kS15 * x * z;
  o[8 * nedges] = 0.5f * kS15 * (x2 - y2);
  o[9 * nedges] = kA * y * (3.f * x2 - y2);
  o[10 * nedges] = kS105 * x * y * z;
  o[11 * nedges] = kB * y * (4.f * z2 - x2 - y2);
  o[12 * nedges] = 0.5f * kS7 * z * (2.f * z2 - 3.f * x2 - 3.f * y2);
  o[13 * nedges] = kB * x * (4.f * z2 - x2 - y2);
  o[14 * nedges] = 0.5f * kS105 * z * (x2 - y2);
  o[15 * nedges] = kA * x * (x2 - 3.f * y2);
}

__global__ void sh_backward_kernel(const float *__restrict__ xyz, const float *__restrict__ gY, int64_t nedges,
                                   float *__restrict__ gxyz) {
  const int64_t e = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x;
  if (e >= nedges) return;
  float y = xyz[3 * e + 0], z = xyz[3 * e + 1], x = xyz[3 * e + 2];
  const float ir = 1.0f / sqrtf(x * x + y * y + z * z);
  x *= ir;
  y *= ir;
  z *= ir;
  const float x2 = x * x, y2 = y * y, z2 = z * z;
  float g[16];
#pragma unroll
  for (int m = 1; m < 16; ++m) g[m] = gY[m * nedges + e];

  // gradient of S = sum_m g_m Y_m with respect to the unit vector, components treated as free
  float sx = kS3 * g[3] + kS15 * (y * g[4] + z * g[7] + x * g[8]) - kS5 * x * g[6];
  float sy = kS3 * g[1] + kS15 * (x * g[4] + z * g[5] - y * g[8]) - kS5 * y * g[6];
  float sz = kS3 * g[2] + kS15 * (y * g[5] + x * g[7]) + 2.f * kS5 * z * g[6];

  sx += 6.f * kA * x * y * g[9] + kS105 * y * z * g[10] - 2.f * kB * x * y * g[11] - 3.f * kS7 * x * z * g[12] +
        kB * (4.f * z2 - 3.f * x2 - y2) * g[13] + kS105 * x * z * g[14] + 3.f * kA * (x2 - y2) * g[15];
  sy += 3.f * kA * (x2 - y2) * g[9] + kS105 * x * z * g[10] + kB * (4.f * z2 - x2 - 3.f * y2) * g[11] -
        3.f * kS7 * y * z * g[12] - 2.f * kB * x * y * g[13] - kS105 * y * z * g[14] - 6.f * kA * x * y * g[15];
  sz += kS105 * x * y * g[10] + 8.f * kB * y * z * g[11] + 1.5f * kS7 * (2.f * z2 - x2 - y2) * g[12] +
        8.f * kB * x * z * g[13] + 0.5f * kS105 * (x2 - y2) * g[14];

  // chain rule through the normalisation: (I - v v^T) / |r|
  const float dot = sx * x + sy * y + sz * z;
  gxyz[3 * e + 0] = (sy - y * dot) * ir;
  gxyz[3 * e + 1] = (sz - z * dot) * ir;
  gxyz[3 * e + 2] = (sx - x * dot) * ir;
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
