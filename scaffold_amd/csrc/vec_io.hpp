// 16-byte vector loads / stores of activation elements, widened to float.
#pragma once
#include "common.hpp"

namespace sfh {

template <typename T, int V> struct Ld;
template <int V> struct Ld<bf16_t, V> {
  static __device__ __forceinline__ void run(const bf16_t* p, float (&f)[V]) {
    if constexpr (V == 8) {
      const uint4 v = *reinterpret_cast<const uint4*>(p);
      f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x); f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
      f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z); f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
    } else {
      const uint2 v = *reinterpret_cast<const uint2*>(p);
      f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x); f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
    }
  }
};
template <int V> struct Ld<fp16_t, V> {
  static __device__ __forceinline__ void run(const fp16_t* p, float (&f)[V]) {
    if constexpr (V == 8) {
      const uint4 v = *reinterpret_cast<const uint4*>(p);
      f[0] = fp16_lo(v.x); f[1] = fp16_hi(v.x); f[2] = fp16_lo(v.y); f[3] = fp16_hi(v.y);
      f[4] = fp16_lo(v.z); f[5] = fp16_hi(v.z); f[6] = fp16_lo(v.w); f[7] = fp16_hi(v.w);
    } else {
      const uint2 v = *reinterpret_cast<const uint2*>(p);
      f[0] = fp16_lo(v.x); f[1] = fp16_hi(v.x); f[2] = fp16_lo(v.y); f[3] = fp16_hi(v.y);
    }
  }
};
template <int V> struct Ld<float, V> {
  static __device__ __forceinline__ void run(const float* p, float (&f)[V]) {
#pragma unroll
    for (int i = 0; i < V / 4; ++i) {
      const float4 v = *reinterpret_cast<const float4*>(p + 4 * i);
      f[4 * i] = v.x; f[4 * i + 1] = v.y; f[4 * i + 2] = v.z; f[4 * i + 3] = v.w;
    }
  }
};

template <typename T, int V> struct St;
template <int V> struct St<bf16_t, V> {
  static __device__ __forceinline__ void run(bf16_t* p, const float (&f)[V]) {
    uint32_t u[V / 2];
#pragma unroll
    for (int i = 0; i < V / 2; ++i) u[i] = pack_bf16x2(f[2 * i], f[2 * i + 1]);
    if constexpr (V == 8) *reinterpret_cast<uint4*>(p) = make_uint4(u[0], u[1], u[2], u[3]);
    else *reinterpret_cast<uint2*>(p) = make_uint2(u[0], u[1]);
  }
};
template <int V> struct St<fp16_t, V> {
  static __device__ __forceinline__ void run(fp16_t* p, const float (&f)[V]) {
    uint32_t u[V / 2];
#pragma unroll
    for (int i = 0; i < V / 2; ++i) u[i] = pack_fp16x2(f[2 * i], f[2 * i + 1]);
    if constexpr (V == 8) *reinterpret_cast<uint4*>(p) = make_uint4(u[0], u[1], u[2], u[3]);
    else *reinterpret_cast<uint2*>(p) = make_uint2(u[0], u[1]);
  }
};
template <int V> struct St<float, V> {
  static __device__ __forceinline__ void run(float* p, const float (&f)[V]) {
#pragma unroll
    for (int i = 0; i < V / 4; ++i)
      *reinterpret_cast<float4*>(p + 4 * i) = make_float4(f[4 * i], f[4 * i + 1], f[4 * i + 2], f[4 * i + 3]);
  }
};

template <typename T> struct VecOf { static constexpr int N = 8; };
template <> struct VecOf<float> { static constexpr int N = 4; };


}  // namespace sfh
