// MFMA operand fragments shared by the weight-only kernels: int8 / packed int4 weights -> 8 elements
// of x's dtype (bf16 or f16), the 16x16x32 MFMA on such fragments, and a fragment of ones.
#pragma once
#include "qmm_common.h"

namespace qmm_frag {

__device__ __forceinline__ uint32_t pack_hi16(float lo, float hi) {
  // {bf16(lo), bf16(hi)} by truncation: exact for integers of magnitude <= 256.
  return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  h2 v = __builtin_bit_cast(h2, __builtin_amdgcn_cvt_pkrtz(lo, hi));  // exact for small integers
  return __builtin_bit_cast(uint32_t, v);
}

// 8 int8 weights (two dwords) -> 8 elements of the x dtype.
template <int XT>
__device__ __forceinline__ i32x4 cvt_w8(uint32_t d0, uint32_t d1) {
  float f[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[i] = (float)(int8_t)(d0 >> (8 * i));
    f[4 + i] = (float)(int8_t)(d1 >> (8 * i));
  }
  i32x4 o;
  if constexpr (XT == XLA_AMD_DT_BF16) {
    o[0] = pack_hi16(f[0], f[1]); o[1] = pack_hi16(f[2], f[3]);
    o[2] = pack_hi16(f[4], f[5]); o[3] = pack_hi16(f[6], f[7]);
  } else {
    o[0] = pack_f16(f[0], f[1]); o[1] = pack_f16(f[2], f[3]);
    o[2] = pack_f16(f[4], f[5]); o[3] = pack_f16(f[6], f[7]);
  }
  return o;
}

// Two int8 weights (the low or the high half of a dword) -> two elements of the x dtype: a quarter of cvt_w8.
template <int XT, class HiC>
__device__ __forceinline__ uint32_t cvt_w2(uint32_t d, HiC) {
  constexpr int sh = HiC::value ? 16 : 0;
  const float lo = (float)(int8_t)(d >> sh), hi = (float)(int8_t)(d >> (sh + 8));
  if constexpr (XT == XLA_AMD_DT_BF16) return pack_hi16(lo, hi);
  else return pack_f16(lo, hi);
}

// 8 packed int4 weights (one dword, nibble j = column P[j], biased by 8) -> 8
// elements (1 + u/16) of the x dtype, u = w + 8 in 0..15.  The caller undoes
// the affine map with the exact x sum: sum w*x = 16*(sum a*x - 1.5*sum x).
template <int XT>
__device__ __forceinline__ i32x4 cvt_w4(uint32_t d) {
  i32x4 o;
  if constexpr (XT == XLA_AMD_DT_BF16) {
    const uint32_t mask = 0x00780078u, one = 0x3F803F80u;  // mantissa bits 3..6 of bf16
    o[0] = ((d << 3) & mask) | one;
    o[1] = ((d >> 1) & mask) | one;
    o[2] = ((d >> 5) & mask) | one;
    o[3] = ((d >> 9) & mask) | one;
  } else {
    const uint32_t mask = 0x03C003C0u, one = 0x3C003C00u;  // mantissa bits 6..9 of f16
    o[0] = ((d << 6) & mask) | one;
    o[1] = ((d << 2) & mask) | one;
    o[2] = ((d >> 2) & mask) | one;
    o[3] = ((d >> 6) & mask) | one;
  }
  return o;
}

template <int XT>
__device__ __forceinline__ f32x4 mfma16(i32x4 a, i32x4 b, f32x4 c) {
  if constexpr (XT == XLA_AMD_DT_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

template <int XT> __device__ __forceinline__ i32x4 ones_frag() {
  uint32_t one2 = XT == XLA_AMD_DT_BF16 ? 0x3F803F80u : 0x3C003C00u;
  i32x4 o = {(int)one2, (int)one2, (int)one2, (int)one2};
  return o;
}

}  // namespace qmm_frag
