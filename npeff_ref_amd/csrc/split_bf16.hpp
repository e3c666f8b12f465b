// fp32 numbers as sums of three bf16 numbers, for products on the bf16 matrix cores at fp32
// accuracy: x = h + m + l exactly (h = bf16(x), m = bf16(x - h), l = x - h - m; 3 x 8 significant
// bits cover the 24 of fp32).  Of the nine partial products of two such numbers the six largest
// (hh, hm, mh, hl, lh, mm) carry everything down to 2^-24 of the product.
#pragma once
#include <hip/hip_runtime.h>

namespace dn {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// The two bf16 numbers of a packed pair as floats: a shift and a mask.
__device__ inline f32x2 widen(const bf16x2& p) {
  const unsigned u = __builtin_bit_cast(unsigned, p);
  return f32x2{__uint_as_float(u << 16), __uint_as_float(u & 0xffff0000u)};
}
// One packed conversion per pair and part; the differences are exact.
__device__ inline void split3(const f32x2& x, bf16x2& h, bf16x2& m, bf16x2& l) {
  h = __builtin_convertvector(x, bf16x2);
  const f32x2 r1 = x - widen(h);
  m = __builtin_convertvector(r1, bf16x2);
  const f32x2 r2 = r1 - widen(m);
  l = __builtin_convertvector(r2, bf16x2);
}
__device__ inline void split3(const f32x4& x, bf16x4& h, bf16x4& m, bf16x4& l) {
  bf16x2 h0, m0, l0, h1, m1, l1;
  split3(f32x2{x[0], x[1]}, h0, m0, l0);
  split3(f32x2{x[2], x[3]}, h1, m1, l1);
  h = __builtin_shufflevector(h0, h1, 0, 1, 2, 3);
  m = __builtin_shufflevector(m0, m1, 0, 1, 2, 3);
  l = __builtin_shufflevector(l0, l1, 0, 1, 2, 3);
}
__device__ inline bf16x8 cat8(const bf16x4& a, const bf16x4& b) {
  return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}
__device__ inline float bf16_bits_to_float(unsigned short u) {
  return __uint_as_float((unsigned)u << 16);
}


#define DN_MFMA_B16(A, B, C) __builtin_amdgcn_mfma_f32_32x32x16_bf16(A, B, C, 0, 0, 0)

}  // namespace dn
