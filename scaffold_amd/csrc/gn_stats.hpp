// GroupNorm statistics emitted by the kernel that produces the tensor: sums of the ROUNDED outputs (the bits the
// normalisation will read back) minus a shift K, and of the squares of those differences, per group, one record per
// producer workgroup:
//   part[sample][record][2][G]      (the layout the GroupNorm kernels fold: quantity 0 = sum, 1 = sum of squares)
// K[sample][group] comes from the caller -- any value near the group's mean, e.g. the mean the same layer had at its
// previous call; a null pointer stands for zeros. With K within a few standard deviations of the mean the variance
// S2/m - (S1/m)^2 does not cancel, however large the mean is against the spread (the job of the Welford merge in the
// reference, triton_group_norm.py:148-165); with K = 0 the fp32 sums still carry a relative variance error of about
// 3e-7 (mean/std)^2, below a bf16 output's own rounding up to |mean| = 100 std.
// No atomics: every (record, group) slot is written by exactly one workgroup, the sums inside a workgroup are added in
// a fixed order, and the GroupNorm kernels add the records in a fixed order, so the statistics are reproducible.
#pragma once
#include "common.hpp"

namespace sfh {

// Where a producer writes, or nothing (part == nullptr). `records` per sample; `cg` channels per group; `shift` is
// K[sample][group] or null.
struct GnPartialOut {
  float* part;
  int groups, cg, records;
  const float* shift;
};

__device__ __forceinline__ void unpack2(bf16_t, uint32_t u, float& lo, float& hi) {
  lo = bf16_lo(u);
  hi = bf16_hi(u);
}
__device__ __forceinline__ void unpack2(fp16_t, uint32_t u, float& lo, float& hi) {
  lo = fp16_lo(u);
  hi = fp16_hi(u);
}

// Sums of the four channel runs a lane holds of a 32-channel result block (run g = channels 8g + 4kg .. + 3, packed
// as two rounded pairs), over the voxels the lane has added so far; k[g] is the shift of run g's group.
struct RunSums {
  float s1[4], s2[4], k[4];
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int g = 0; g < 4; ++g) s1[g] = s2[g] = k[g] = 0.f;
  }
  // The shifts of the block whose first channel is c0 (a multiple of 32), for the lane's k-half kg and sample n.
  __device__ __forceinline__ void load_shift(const float* shift, int n, int groups, int cg, int c0, int kg) {
    if (shift == nullptr) return;
#pragma unroll
    for (int g = 0; g < 4; ++g) k[g] = shift[n * groups + (c0 + 8 * g + 4 * kg) / cg];
  }
  template <typename T>
  __device__ __forceinline__ void add(const uint32_t (&run)[4][2], bool inside) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float a, b, c, d;
      unpack2(T{}, run[g][0], a, b);
      unpack2(T{}, run[g][1], c, d);
      a -= k[g]; b -= k[g]; c -= k[g]; d -= k[g];
      const float t1 = (a + b) + (c + d);
      const float t2 = fmaf(a, a, b * b) + fmaf(c, c, d * d);
      s1[g] += inside ? t1 : 0.f;  // a voxel past the ragged edge counts as nothing
      s2[g] += inside ? t2 : 0.f;
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
