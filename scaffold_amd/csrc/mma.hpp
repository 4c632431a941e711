// v_mfma_f32_32x32x16 wrappers for the 16-bit element types.
//   A operand (rows):    lane l holds row i = l % 32, k = 8 * (l / 32) .. + 7
//   B operand (columns): lane l holds column j = l % 32, k = 8 * (l / 32) .. + 7
//   result register r of lane l: column j = l % 32, row i = 8 * (r / 4) + 4 * (l / 32) + r % 4
#pragma once
#include "common.hpp"

namespace sfh {

typedef __bf16 mma_bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 mma_f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

template <typename T> struct Mma32;
template <> struct Mma32<bf16_t> {
  static __device__ __forceinline__ f32x16_t run(const uint4& a, const uint4& b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(mma_bf16x8_t, a), __builtin_bit_cast(mma_bf16x8_t, b), c, 0, 0,
                                                   0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
};
template <> struct Mma32<fp16_t> {
  static __device__ __forceinline__ f32x16_t run(const uint4& a, const uint4& b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(mma_f16x8_t, a), __builtin_bit_cast(mma_f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_fp16x2(lo, hi); }
};

}  // namespace sfh
