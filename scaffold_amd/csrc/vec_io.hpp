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


// V elements of T as they lie in memory (16 or 32 bytes): loaded now, widened to float when they are needed. Lets a loop
// keep the next rows' loads in flight in a quarter of the registers the widened values would take.
template <typename T, int V> struct Piece;
template <> struct Piece<bf16_t, 8> {
  uint4 q;
  __device__ __forceinline__ void load(const bf16_t* p) { q = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ void unpack(float (&f)[8]) const {
    f[0] = bf16_lo(q.x); f[1] = bf16_hi(q.x); f[2] = bf16_lo(q.y); f[3] = bf16_hi(q.y);
    f[4] = bf16_lo(q.z); f[5] = bf16_hi(q.z); f[6] = bf16_lo(q.w); f[7] = bf16_hi(q.w);
  }
};
template <> struct Piece<fp16_t, 8> {
  uint4 q;
  __device__ __forceinline__ void load(const fp16_t* p) { q = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ void unpack(float (&f)[8]) const {
    f[0] = fp16_lo(q.x); f[1] = fp16_hi(q.x); f[2] = fp16_lo(q.y); f[3] = fp16_hi(q.y);
    f[4] = fp16_lo(q.z); f[5] = fp16_hi(q.z); f[6] = fp16_lo(q.w); f[7] = fp16_hi(q.w);
  }
};
template <int V> struct Piece<float, V> {
  float4 q[V / 4];
  __device__ __forceinline__ void load(const float* p) {
#pragma unroll
    for (int i = 0; i < V / 4; ++i) q[i] = *reinterpret_cast<const float4*>(p + 4 * i);
  }
  __device__ __forceinline__ void unpack(float (&f)[V]) const {
#pragma unroll
    for (int i = 0; i < V / 4; ++i) { f[4 * i] = q[i].x; f[4 * i + 1] = q[i].y; f[4 * i + 2] = q[i].z; f[4 * i + 3] = q[i].w; }
  }
};

// U rows of one thread (row0, row0 + step, ...): rows at or past `end`, and every row of an idle thread, are read from
// `safe` (a row that exists) and not used.
template <typename T, int V, int U>
__device__ __forceinline__ void fetch_rows(Piece<T, V> (&b)[U], const T* xs, int64_t row0, int64_t step, int64_t end, int64_t safe,
                                           int C, bool active) {
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t rr = row0 + u * step;
    b[u].load(xs + ((active && rr < end) ? rr : safe) * C);
  }
}

}  // namespace sfh
