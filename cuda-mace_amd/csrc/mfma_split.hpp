// Operand types of v_mfma_f32_32x32x16_bf16 and the split of an fp32 value into three bf16 pieces, shared by the kernels
// that run fp32 products on the bf16 matrix instruction (linear.hip, node_glue.hip).
#pragma once

#include "common.hpp"

namespace cm {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

// a = hi + mid + lo with bf16 pieces (round to nearest at every step; the remainders are exact in fp32).  Two values at a
// time: the packed conversion rounds both and leaves the pieces in the order the matrix instruction takes them, and a
// piece widens back to fp32 by a shift or a mask (11 instructions per pair; element by element the compiler converts
// every value alone, widens it, and packs the pairs at the end with further conversions: 15).
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f2 __attribute__((ext_vector_type(2)));
typedef unsigned u2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void split3_pair(float v0, float v1, unsigned &hi, unsigned &mid, unsigned &lo) {
  hi = __builtin_bit_cast(unsigned, __builtin_convertvector(f2{v0, v1}, bf16x2));
  const float r0 = v0 - __builtin_bit_cast(float, hi << 16), r1 = v1 - __builtin_bit_cast(float, hi & 0xffff0000u);
  mid = __builtin_bit_cast(unsigned, __builtin_convertvector(f2{r0, r1}, bf16x2));
  const float q0 = r0 - __builtin_bit_cast(float, mid << 16), q1 = r1 - __builtin_bit_cast(float, mid & 0xffff0000u);
  lo = __builtin_bit_cast(unsigned, __builtin_convertvector(f2{q0, q1}, bf16x2));
}
__device__ __forceinline__ void split3(f4 v, bf16x4 &hi, bf16x4 &mid, bf16x4 &lo) {
  unsigned h0, m0, l0, h1, m1, l1;
  split3_pair(v.x, v.y, h0, m0, l0);
  split3_pair(v.z, v.w, h1, m1, l1);
  hi = __builtin_bit_cast(bf16x4, u2{h0, h1});
  mid = __builtin_bit_cast(bf16x4, u2{m0, m1});
  lo = __builtin_bit_cast(bf16x4, u2{l0, l1});
}

}  // namespace cm
