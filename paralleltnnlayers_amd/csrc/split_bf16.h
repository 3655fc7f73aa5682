// Exact fp32 products on the bf16 matrix cores, shared by the kernels that use
// them: every fp32 operand is split by truncation into three bf16 numbers
// h + m + l (24 significand bits = 3 x 8, so the split is exact) and a product is
// the six largest partial products on v_mfma_f32_32x32x16_bf16, accumulated in
// fp32.  The dropped terms are below 2^-24 of the product.
#ifndef CP4_SPLIT_BF16_H
#define CP4_SPLIT_BF16_H

#include <hip/hip_runtime.h>

namespace cp4 {
namespace split {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ f32x16 mfma16(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ unsigned pack_hi16(float a, float b) {
  return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}
__device__ __forceinline__ float trunc_bf16(float v) {
  return __uint_as_float(__float_as_uint(v) & 0xffff0000u);
}
// Exact split of 8 floats into bf16 parts h, m, l (x = h + m + l bit-exactly).
__device__ __forceinline__ void split8(const float (&v)[8], u32x4& h, u32x4& m, u32x4& l) {
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const float a = v[2 * d], b = v[2 * d + 1];
    h[d] = pack_hi16(a, b);
    const float ra = a - trunc_bf16(a), rb = b - trunc_bf16(b);
    m[d] = pack_hi16(ra, rb);
    const float sa = ra - trunc_bf16(ra), sb = rb - trunc_bf16(rb);
    l[d] = pack_hi16(sa, sb);
  }
}
__device__ __forceinline__ f32x16 mfma_split(u32x4 ah, u32x4 am, u32x4 al, u32x4 bh, u32x4 bm,
                                             u32x4 bl, f32x16 acc) {
  acc = mfma16(al, bh, acc);
  acc = mfma16(am, bm, acc);
  acc = mfma16(ah, bl, acc);
  acc = mfma16(am, bh, acc);
  acc = mfma16(ah, bm, acc);
  acc = mfma16(ah, bh, acc);
  return acc;
}

}  // namespace split
}  // namespace cp4
#endif  // CP4_SPLIT_BF16_H
