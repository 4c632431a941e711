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

template <typename T>
__device__ __forceinline__ uint4 load16(const T* p) { return *reinterpret_cast<const uint4*>(p); }

// Stores result block `acc` (32 produced channels x 32 voxels): this lane's voxel row starts at `row`
// (element pointer at channel 0 of the block); adds bias[c0 + channel] when given. The two lanes of a voxel trade
// channel runs first, so each stores two 16-byte pieces. All 64 lanes must call it; `valid` masks the stores.
template <typename T>
__device__ __forceinline__ void store_block(const f32x16_t& acc, T* row, const T* bias, int c0, int kg, bool valid) {
  uint32_t run[4][2];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int c = 8 * g + 4 * kg;
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = acc[4 * g + i] + (bias != nullptr ? to_float(bias[c0 + c + i]) : 0.f);
    run[g][0] = Mma32<T>::pack2(v[0], v[1]);
    run[g][1] = Mma32<T>::pack2(v[2], v[3]);
  }
  uint4 piece[2];
  trade_channel_runs(run, piece);
  if (valid) {
    *reinterpret_cast<uint4*>(row + 8 * kg) = piece[0];
    *reinterpret_cast<uint4*>(row + 16 + 8 * kg) = piece[1];
  }
}

}  // namespace sfh
