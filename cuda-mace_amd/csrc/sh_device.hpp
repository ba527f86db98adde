// Real spherical harmonics l <= 3 of a direction and their vector-Jacobian product, as device functions shared by the
// stand-alone harmonics kernels and the message-passing kernels that evaluate the harmonics per edge on the fly.
// Convention: input axes are permuted to (x, y, z) = (in[2], in[0], in[1]); "component" normalisation, i.e. sqrt(4 pi)
// is folded into the constants so that Y_00 = 1 and sum_{m in l} Y_lm^2 = 2l + 1; components ordered m = -l..l.
#pragma once

#include "common.hpp"

namespace cm {
namespace sh {

constexpr float kS3 = 1.7320508075688772f;    // sqrt(3)
constexpr float kS5 = 2.23606797749979f;      // sqrt(5)
constexpr float kS7 = 2.6457513110645907f;    // sqrt(7)
constexpr float kS15 = 3.872983346207417f;    // sqrt(15)
constexpr float kS105 = 10.246950765959598f;  // sqrt(105)
constexpr float kA = 2.091650066335189f;      // sqrt(35/8)
constexpr float kB = 1.6201851746019651f;     // sqrt(21/8)

// Unit vector (permuted axes) and inverse length of an input vector (in0, in1, in2).
struct Direction {
  float x, y, z, ir;
};

__device__ __forceinline__ Direction direction(float in0, float in1, float in2) {
  Direction d;
  d.ir = 1.0f / sqrtf(in0 * in0 + in1 * in1 + in2 * in2);
  d.x = in2 * d.ir;
  d.y = in0 * d.ir;
  d.z = in1 * d.ir;
  return d;
}

__device__ __forceinline__ void eval(const Direction &d, float (&Y)[16]) {
  const float x = d.x, y = d.y, z = d.z;
  const float x2 = x * x, y2 = y * y, z2 = z * z;
  Y[0] = 1.0f;
  Y[1] = kS3 * y;
  Y[2] = kS3 * z;
  Y[3] = kS3 * x;
  Y[4] = kS15 * x * y;
  Y[5] = kS15 * y * z;
  Y[6] = 0.5f * kS5 * (2.f * z2 - x2 - y2);
  Y[7] = kS15 * x * z;
  Y[8] = 0.5f * kS15 * (x2 - y2);
  Y[9] = kA * y * (3.f * x2 - y2);
  Y[10] = kS105 * x * y * z;
  Y[11] = kB * y * (4.f * z2 - x2 - y2);
  Y[12] = 0.5f * kS7 * z * (2.f * z2 - 3.f * x2 - 3.f * y2);
  Y[13] = kB * x * (4.f * z2 - x2 - y2);
  Y[14] = 0.5f * kS105 * z * (x2 - y2);
  Y[15] = kA * x * (x2 - 3.f * y2);
}

// Gradient of S = sum_m g[m] Y_m(direction(in)) with respect to the un-normalised input, in input axis order.
// g[0] does not matter (Y_0 is constant).
__device__ __forceinline__ void vjp(const Direction &d, const float (&g)[16], float (&gin)[3]) {
  const float x = d.x, y = d.y, z = d.z;
  const float x2 = x * x, y2 = y * y, z2 = z * z;
  // gradient with respect to the unit vector, its components treated as free
  float sx = kS3 * g[3] + kS15 * (y * g[4] + z * g[7] + x * g[8]) - kS5 * x * g[6];
  float sy = kS3 * g[1] + kS15 * (x * g[4] + z * g[5] - y * g[8]) - kS5 * y * g[6];
  float sz = kS3 * g[2] + kS15 * (y * g[5] + x * g[7]) + 2.f * kS5 * z * g[6];
  sx += 6.f * kA * x * y * g[9] + kS105 * y * z * g[10] - 2.f * kB * x * y * g[11] - 3.f * kS7 * x * z * g[12] +
        kB * (4.f * z2 - 3.f * x2 - y2) * g[13] + kS105 * x * z * g[14] + 3.f * kA * (x2 - y2) * g[15];
  sy += 3.f * kA * (x2 - y2) * g[9] + kS105 * x * z * g[10] + kB * (4.f * z2 - x2 - 3.f * y2) * g[11] -
        3.f * kS7 * y * z * g[12] - 2.f * kB * x * y * g[13] - kS105 * y * z * g[14] - 6.f * kA * x * y * g[15];
  sz += kS105 * x * y * g[10] + 8.f * kB * y * z * g[11] + 1.5f * kS7 * (2.f * z2 - x2 - y2) * g[12] +
        8.f * kB * x * z * g[13] + 0.5f * kS105 * (x2 - y2) * g[14];
  // chain rule through the normalisation: (I - v v^T) / |in|
  const float dot = sx * x + sy * y + sz * z;
  gin[0] = (sy - y * dot) * d.ir;
  gin[1] = (sz - z * dot) * d.ir;
  gin[2] = (sx - x * dot) * d.ir;
}

}  // namespace sh
}  // namespace cm
