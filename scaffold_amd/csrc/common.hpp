// Shared device/host helpers for libscaffold_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/scaffold_hip.h"

namespace sfh {

// ---- error plumbing -----------------------------------------------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
// Checks the launch status of the kernel that was just enqueued.
int check_launch(const char* what);

// ---- element types ------------------------------------------------------------------
// Storage types are raw bit patterns; arithmetic is always done in float.
struct bf16_t { uint16_t bits; };
struct fp16_t { _Float16 v; };

__device__ __forceinline__ float to_float(bf16_t x) { return __uint_as_float(((uint32_t)x.bits) << 16); }
__device__ __forceinline__ float to_float(fp16_t x) { return (float)x.v; }
__device__ __forceinline__ float to_float(float x) { return x; }

// Round-to-nearest-even fp32 -> bf16 (NaN stays NaN): gfx950's v_cvt_pk_bf16_f32, no branches.
typedef __bf16 sfh_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float sfh_f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint16_t bf16_bits_rne(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

template <typename T> struct elem;
template <> struct elem<bf16_t> {
  static __device__ __forceinline__ bf16_t from_float(float f) { bf16_t r; r.bits = bf16_bits_rne(f); return r; }
};
template <> struct elem<fp16_t> {
  static __device__ __forceinline__ fp16_t from_float(float f) { fp16_t r; r.v = (_Float16)f; return r; }
};
template <> struct elem<float> {
  static __device__ __forceinline__ float from_float(float f) { return f; }
};

// Two bf16 packed in a dword -> two floats, and back.
__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const sfh_f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, sfh_bf16x2_t));
}
__device__ __forceinline__ uint32_t pack_fp16x2(float lo, float hi) {
  union { _Float16 h[2]; uint32_t u; } r;
  r.h[0] = (_Float16)lo; r.h[1] = (_Float16)hi;
  return r.u;
}
__device__ __forceinline__ float fp16_lo(uint32_t u) { union { uint32_t u; _Float16 h[2]; } r; r.u = u; return (float)r.h[0]; }
__device__ __forceinline__ float fp16_hi(uint32_t u) { union { uint32_t u; _Float16 h[2]; } r; r.u = u; return (float)r.h[1]; }

// Four packed runs of four 16-bit channels each, as an MFMA 32x32 result leaves them in the two lanes of a voxel
// (lane kg holds channels 8g + 4kg .. + 3 as run g): the lanes l and l + 32 trade runs so that lane kg ends up with
// the 16-byte pieces of channels 8kg .. 8kg + 7 (out[0]) and 16 + 8kg .. 16 + 8kg + 7 (out[1]). All 64 lanes must
// call it.
__device__ __forceinline__ void trade_channel_runs(const uint32_t (&run)[4][2], uint4 (&out)[2]) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const auto lo = __builtin_amdgcn_permlane32_swap(run[2 * h][0], run[2 * h + 1][0], false, false);
    const auto hi = __builtin_amdgcn_permlane32_swap(run[2 * h][1], run[2 * h + 1][1], false, false);
    out[h] = make_uint4(lo[0], hi[0], lo[1], hi[1]);
  }
}

inline size_t dtype_size(int dtype) { return dtype == SFH_FP32 ? 4 : 2; }
inline bool dtype_ok(int dtype) { return dtype == SFH_BF16 || dtype == SFH_FP16 || dtype == SFH_FP32; }

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Number of compute units the launch heuristics are written for (MI355X).
constexpr int kComputeUnits = 256;
constexpr int kXcds = 8;

// Maps the hardware workgroup id (dispatched round-robin over the 8 XCDs) to a logical
// tile id such that every XCD, and so every L2, works on one contiguous range of tiles.
__device__ __forceinline__ uint32_t xcd_remap(uint32_t pid, uint32_t total) {
  const uint32_t per = total / kXcds, rem = total % kXcds;
  const uint32_t xcd = pid % kXcds, slot = pid / kXcds;
  // XCDs [0, rem) own per+1 tiles, the rest own per tiles.
  const uint32_t start = xcd * per + (xcd < rem ? xcd : rem);
  return start + slot;
}

// A channels-last tensor handed over as two tensors over the same voxels whose channels follow each other: the first
// `first` channels (a multiple of 32) lie in the tensor passed in the usual place, the rest in `second`. It stands for
// the concatenation along the channels without anyone writing it: the reduction channels of a forward (its input), the
// produced channels of a data gradient (its output), the input channels of a weight gradient.
struct ChannelPair {
  void* second;
  int first;
};

}  // namespace sfh
