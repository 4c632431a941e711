// v_mfma_f32_32x32x16 wrappers for the 16-bit element types.
//   A operand (rows):    lane l holds row i = l % 32, k = 8 * (l / 32) .. + 7
//   B operand (columns): lane l holds column j = l % 32, k = 8 * (l / 32) .. + 7
//   result register r of lane l: column j = l % 32, row i = 8 * (r / 4) + 4 * (l / 32) + r % 4
#pragma once
#include "common.hpp"
#include "gn_stats.hpp"

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

// The same MFMA as inline asm: the accumulator pinned to accumulation registers and, in the first form, the row
// operand read from accumulation registers too (the compiler would otherwise copy such a fragment into a vector
// register before every use). The compiler does not know the result latency of an asm MFMA: an accumulator block
// must not be read (by anything but another MFMA, a few instructions later) without a wait.
typedef int mma_frag_t __attribute__((ext_vector_type(4)));  // one operand fragment of a lane (8 x 16 bit)
template <typename T> struct Mma32Pinned;
template <> struct Mma32Pinned<bf16_t> {
  static __device__ __forceinline__ void run_row_in_acc(const mma_frag_t& a, const uint4& b, f32x16_t& c) {
    const mma_frag_t bv = __builtin_bit_cast(mma_frag_t, b);
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "a"(a), "v"(bv));
  }
  static __device__ __forceinline__ void run(const mma_frag_t& a, const mma_frag_t& b, f32x16_t& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <> struct Mma32Pinned<fp16_t> {
  static __device__ __forceinline__ void run_row_in_acc(const mma_frag_t& a, const uint4& b, f32x16_t& c) {
    const mma_frag_t bv = __builtin_bit_cast(mma_frag_t, b);
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "a"(a), "v"(bv));
  }
  static __device__ __forceinline__ void run(const mma_frag_t& a, const mma_frag_t& b, f32x16_t& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};

template <typename T>
__device__ __forceinline__ uint4 load16(const T* p) { return *reinterpret_cast<const uint4*>(p); }

// Stores result block `acc` (32 produced channels x 32 voxels) plus `add` (same register layout: register r of
// this lane is channel 8 * (r / 4) + 4 * kg + r % 4): this lane's voxel row starts at `row` (element pointer at
// channel 0 of the block). The two lanes of a voxel trade channel runs first, so each stores two 16-byte pieces.
// All 64 lanes must call it; `valid` masks the stores.
// With `want`, the block's rounded values are also added to the lane's GroupNorm sums (valid voxels only); `first`: it
// is the first block added to `sums`.
template <typename T>
__device__ __forceinline__ void store_block_plus(const f32x16_t& acc, T* row, const float (&add)[16], int kg, bool valid,
                                                 RunSums& sums, bool want, bool first) {
  uint32_t run[4][2];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    run[g][0] = Mma32<T>::pack2(acc[4 * g] + add[4 * g], acc[4 * g + 1] + add[4 * g + 1]);
    run[g][1] = Mma32<T>::pack2(acc[4 * g + 2] + add[4 * g + 2], acc[4 * g + 3] + add[4 * g + 3]);
  }
  if (want) sums.template add<T>(run, valid, first);
  uint4 piece[2];
  trade_channel_runs(run, piece);
  if (valid) {
    *reinterpret_cast<uint4*>(row + 8 * kg) = piece[0];
    *reinterpret_cast<uint4*>(row + 16 + 8 * kg) = piece[1];
  }
}

template <typename T>
__device__ __forceinline__ void store_block_plus(const f32x16_t& acc, T* row, const float (&add)[16], int kg, bool valid) {
  RunSums unused;
  store_block_plus<T>(acc, row, add, kg, valid, unused, false, false);
}

// This lane's 16 bias values of the channel block from c0 (zeros without a bias), in result-register order.
template <typename T>
__device__ __forceinline__ void load_block_bias(const T* bias, int c0, int kg, float (&add)[16]) {
#pragma unroll
  for (int r = 0; r < 16; ++r) add[r] = 0.f;
  if (bias != nullptr) {
    T b[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) b[r] = bias[c0 + 8 * (r / 4) + 4 * kg + r % 4];
#pragma unroll
    for (int r = 0; r < 16; ++r) add[r] = to_float(b[r]);
  }
}

// As store_block_plus with bias[c0 + channel] (when given) as the addend.
template <typename T>
__device__ __forceinline__ void store_block(const f32x16_t& acc, T* row, const T* bias, int c0, int kg, bool valid, RunSums& sums,
                                            bool want, bool first) {
  float add[16];
  load_block_bias<T>(bias, c0, kg, add);
  store_block_plus<T>(acc, row, add, kg, valid, sums, want, first);
}
template <typename T>
__device__ __forceinline__ void store_block(const f32x16_t& acc, T* row, const T* bias, int c0, int kg, bool valid) {
  RunSums unused;
  store_block<T>(acc, row, bias, c0, kg, valid, unused, false, false);
}

}  // namespace sfh
