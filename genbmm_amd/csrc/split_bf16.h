// A float as three bfloat16 parts, and the matrix instruction that multiplies them.
//
// x = h + m + l exactly (h = x rounded to bfloat16, m = x - h rounded, l the rest rounded; exact
// while l stays a normal number, i.e. down to |x| of about 2^-100), so a product of two floats
// is the sum of nine products of parts, of which the six largest - hh, hm, mh, mm, hl, lh -
// leave out less than 2^-23 of it.  v_mfma_f32_32x32x16_bf16 multiplies the parts exactly and
// adds in fp32.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"

namespace GENBMM_NS {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

// (x0, x1) rounded to bf16, x0 in the low half: one v_cvt_pk_bf16_f32
__device__ __forceinline__ unsigned pk_bf16(float x0, float x1) {
  floatx2 v;
  v.x = x0; v.y = x1;
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ float bf_lo(unsigned pk) { return __builtin_bit_cast(float, pk << 16); }
__device__ __forceinline__ float bf_hi(unsigned pk) { return __builtin_bit_cast(float, pk & 0xffff0000u); }
// h + m + l = x exactly, for both values of a pair
__device__ __forceinline__ void split2(float x0, float x1, unsigned& h, unsigned& m, unsigned& l) {
  h = pk_bf16(x0, x1);
  const float r0 = x0 - bf_lo(h), r1 = x1 - bf_hi(h);
  m = pk_bf16(r0, r1);
  l = pk_bf16(r0 - bf_lo(m), r1 - bf_hi(m));
}

__device__ __forceinline__ floatx16 mfma_bf16(bf16x8 a, bf16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

}  // namespace GENBMM_NS
