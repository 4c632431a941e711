// GroupNorm statistics emitted by the kernel that produces the tensor: unshifted sums of the ROUNDED outputs (the bits
// the normalisation will read back) and of their squares, per group, one record per producer workgroup:
//   part[sample][record][2][G]      (the layout the GroupNorm kernels fold: quantity 0 = sum, 1 = sum of squares)
// No atomics: every (record, group) slot is written by exactly one workgroup, the sums inside a workgroup are added in
// a fixed order, and the GroupNorm kernels add the records in a fixed order, so the statistics are reproducible.
// Offered for 16-bit outputs only: fp32 sums of 16-bit values keep more than the 8 (bf16) / 11 (fp16) bits of the data
// for any mean a tensor of such values can have relative to its spread, so the shift the stand-alone statistics pass
// uses (for fp32 tensors at mean >> std) is not needed here.
#pragma once
#include "common.hpp"

namespace sfh {

// Where a producer writes, or nothing (part == nullptr). `records` per sample; `cg` channels per group.
struct GnPartialOut {
  float* part;
  int groups, cg, records;
};

// acc + lo(a) * lo(b) + hi(a) * hi(b) of two packed 16-bit pairs, products and sum in fp32 (v_dot2_f32_bf16 /
// v_dot2_f32_f16: one instruction where unpacking and two multiply-adds take four), and the pair (1, 1).
typedef __bf16 gn_bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 gn_f16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dot2_acc(bf16_t, uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(gn_bf16x2_t, a), __builtin_bit_cast(gn_bf16x2_t, b), acc, false);
}
__device__ __forceinline__ float dot2_acc(fp16_t, uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(gn_f16x2_t, a), __builtin_bit_cast(gn_f16x2_t, b), acc, false);
}
__device__ __forceinline__ constexpr uint32_t ones2(bf16_t) { return 0x3f803f80u; }
__device__ __forceinline__ constexpr uint32_t ones2(fp16_t) { return 0x3c003c00u; }

// Sums of the four channel runs a lane holds of a 32-channel result block (run g = channels 8g + 4kg .. + 3, packed
// as two rounded pairs), over the voxels the lane has added so far.
struct RunSums {
  float s1[4], s2[4];
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int g = 0; g < 4; ++g) s1[g] = s2[g] = 0.f;
  }
  template <typename T>
  __device__ __forceinline__ void add(const uint32_t (&run)[4][2], bool inside) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t v = inside ? run[g][h] : 0u;  // a voxel past the ragged edge counts as zeros
        s1[g] = dot2_acc(T{}, v, ones2(T{}), s1[g]);
        s2[g] = dot2_acc(T{}, v, v, s2[g]);
      }
    }
  }
};

// Sum over the 32 lanes of each half-wave (the lanes that share a k-half kg hold the same channel runs of different
// voxels): afterwards every lane holds its half's total. Fixed butterfly order.
__device__ __forceinline__ float half_wave_sum(float v) {
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Workgroup of NW wavefronts, each lane with NSUB RunSums (result blocks ns = 0 .. NSUB-1 of the workgroup's channel
// span, which starts at global channel c0): folds them per group and writes the workgroup's slots of record `rec` of
// sample n. `lds` needs NW * NSUB * 16 floats and must be free for writing (the caller has synchronised). A group wider
// than the span (cg > 32 * NSUB) is completed by the other workgroups of the same tile, each in a record of its own.
template <int NW, int NSUB>
__device__ __forceinline__ void write_group_partials(const RunSums (&rs)[NSUB], float* lds, const GnPartialOut& o, int n, int rec, int c0,
                                                     int tid) {
  const int lane = tid & 63, wave = tid >> 6, kg = lane >> 5;
  // lds[wave][ns][run r = 2g + kg][q]
#pragma unroll
  for (int ns = 0; ns < NSUB; ++ns)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float t1 = half_wave_sum(rs[ns].s1[g]), t2 = half_wave_sum(rs[ns].s2[g]);
      if ((lane & 31) == 0) {
        float* dst = lds + ((wave * NSUB + ns) * 8 + 2 * g + kg) * 2;
        dst[0] = t1;
        dst[1] = t2;
      }
    }
  __syncthreads();
  const int span = 32 * NSUB;
  const int runs_per_group = (o.cg < span ? o.cg : span) / 4;
  const int ngroups = span / (runs_per_group * 4);
  if (tid < 2 * ngroups) {
    const int q = tid & 1, gl = tid >> 1;
    float t = 0.f;
    for (int w = 0; w < NW; ++w)
      for (int r = 0; r < runs_per_group; ++r) t += lds[((w * (NSUB * 8)) + gl * runs_per_group + r) * 2 + q];
    const int group = (c0 + gl * runs_per_group * 4) / o.cg;
    o.part[(((int64_t)n * o.records + rec) * 2 + q) * o.groups + group] = t;
  }
}

// Host side: whether a producer whose workgroups span `span` consecutive channels can serve groups of cg channels.
inline bool gn_partials_fit(int cout, int groups, int span) {
  if (groups < 1 || cout % groups != 0) return false;
  const int cg = cout / groups;
  if (cg % 4 != 0) return false;
  return cg <= span ? span % cg == 0 : cg % span == 0;
}

}  // namespace sfh
