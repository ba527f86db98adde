// Real spherical harmonics l <= 3 of a direction and their vector-Jacobian product, as device functions shared by the
// stand-alone harmonics kernels and the message-passing kernels that evaluate the harmonics per edge on the fly.
// Convention: input axes are permuted to (x, y, z) = (in[2], in[0], in[1]); "component" normalisation, i.e. sqrt(4 pi)
// is folded into the constants so that Y_00 = 1 and sum_{m in l} Y_lm^2 = 2l + 1; components ordered m = -l..l.
#pragma once

#include "common.hpp"

namespace cm {
namespace sh {

// Constants per scalar type; the fp32 values are written as float literals so that they round once.
template <typename T>
struct Const;
template <>
struct Const<float> {
  static constexpr float kS3 = 1.7320508075688772f;    // sqrt(3)
  static constexpr float kS5 = 2.23606797749979f;      // sqrt(5)
  static constexpr float kS7 = 2.6457513110645907f;    // sqrt(7)
  static constexpr float kS15 = 3.872983346207417f;    // sqrt(15)
  static constexpr float kS105 = 10.246950765959598f;  // sqrt(105)
  static constexpr float kA = 2.091650066335189f;      // sqrt(35/8)
  static constexpr float kB = 1.6201851746019651f;     // sqrt(21/8)
};
template <>
struct Const<double> {
  static constexpr double kS3 = 1.7320508075688772;
  static constexpr double kS5 = 2.23606797749979;
  static constexpr double kS7 = 2.6457513110645907;
  static constexpr double kS15 = 3.872983346207417;
  static constexpr double kS105 = 10.246950765959598;
  static constexpr double kA = 2.091650066335189;
  static constexpr double kB = 1.6201851746019651;
};

__device__ __forceinline__ float inv_sqrt(float v) { return 1.0f / sqrtf(v); }
__device__ __forceinline__ double inv_sqrt(double v) { return 1.0 / sqrt(v); }

// Unit vector (permuted axes) and inverse length of an input vector (in0, in1, in2).
template <typename T>
struct DirectionT {
  T x, y, z, ir;
};
using Direction = DirectionT<float>;

template <typename T>
__device__ __forceinline__ DirectionT<T> direction(T in0, T in1, T in2) {
  DirectionT<T> d;
  d.ir = inv_sqrt(in0 * in0 + in1 * in1 + in2 * in2);
  d.x = in2 * d.ir;
  d.y = in0 * d.ir;
  d.z = in1 * d.ir;
  return d;
}

template <typename T>
__device__ __forceinline__ void eval(const DirectionT<T> &d, T (&Y)[16]) {
  using K = Const<T>;
  constexpr T kS3 = K::kS3, kS5 = K::kS5, kS7 = K::kS7, kS15 = K::kS15, kS105 = K::kS105, kA = K::kA, kB = K::kB;
  const T x = d.x, y = d.y, z = d.z;
  const T x2 = x * x, y2 = y * y, z2 = z * z;
  Y[0] = T(1.0);
  Y[1] = kS3 * y;
  Y[2] = kS3 * z;
  Y[3] = kS3 * x;
  Y[4] = kS15 * x * y;
  Y[5] = kS15 * y * z;
  Y[6] = T(0.5) * kS5 * (T(2) * z2 - x2 - y2);
  Y[7] = kS15 * x * z;
  Y[8] = T(0.5) * kS15 * (x2 - y2);
  Y[9] = kA * y * (T(3) * x2 - y2);
  Y[10] = kS105 * x * y * z;
  Y[11] = kB * y * (T(4) * z2 - x2 - y2);
  Y[12] = T(0.5) * kS7 * z * (T(2) * z2 - T(3) * x2 - T(3) * y2);
  Y[13] = kB * x * (T(4) * z2 - x2 - y2);
  Y[14] = T(0.5) * kS105 * z * (x2 - y2);
  Y[15] = kA * x * (x2 - T(3) * y2);
}

// Gradient of S = sum_m g[m] Y_m(direction(in)) with respect to the un-normalised input, in input axis order.
// g[0] does not matter (Y_0 is constant).
template <typename T>
__device__ __forceinline__ void vjp(const DirectionT<T> &d, const T (&g)[16], T (&gin)[3]) {
  using K = Const<T>;
  constexpr T kS3 = K::kS3, kS5 = K::kS5, kS7 = K::kS7, kS15 = K::kS15, kS105 = K::kS105, kA = K::kA, kB = K::kB;
  const T x = d.x, y = d.y, z = d.z;
  const T x2 = x * x, y2 = y * y, z2 = z * z;
  // gradient with respect to the unit vector, its components treated as free
  T sx = kS3 * g[3] + kS15 * (y * g[4] + z * g[7] + x * g[8]) - kS5 * x * g[6];
  T sy = kS3 * g[1] + kS15 * (x * g[4] + z * g[5] - y * g[8]) - kS5 * y * g[6];
  T sz = kS3 * g[2] + kS15 * (y * g[5] + x * g[7]) + T(2) * kS5 * z * g[6];
  sx += T(6) * kA * x * y * g[9] + kS105 * y * z * g[10] - T(2) * kB * x * y * g[11] - T(3) * kS7 * x * z * g[12] +
        kB * (T(4) * z2 - T(3) * x2 - y2) * g[13] + kS105 * x * z * g[14] + T(3) * kA * (x2 - y2) * g[15];
  sy += T(3) * kA * (x2 - y2) * g[9] + kS105 * x * z * g[10] + kB * (T(4) * z2 - x2 - T(3) * y2) * g[11] -
        T(3) * kS7 * y * z * g[12] - T(2) * kB * x * y * g[13] - kS105 * y * z * g[14] - T(6) * kA * x * y * g[15];
  sz += kS105 * x * y * g[10] + T(8) * kB * y * z * g[11] + T(1.5) * kS7 * (T(2) * z2 - x2 - y2) * g[12] +
        T(8) * kB * x * z * g[13] + T(0.5) * kS105 * (x2 - y2) * g[14];
  // chain rule through the normalisation: (I - v v^T) / |in|
  const T dot = sx * x + sy * y + sz * z;
  gin[0] = (sy - y * dot) * d.ir;
  gin[1] = (sz - z * dot) * d.ir;
  gin[2] = (sx - x * dot) * d.ir;
}

}  // namespace sh
}  // namespace cm
