// GroupNorm statistics emitted by the kernel that produces the tensor, as Welford records: for every group a producer
// workgroup leaves (count, mean, M2) of the ROUNDED outputs it stored (the bits the normalisation will read back),
//   part[sample][record][group][4] = { count, mean, M2 = sum (v - mean)^2, 0 }
// and the GroupNorm kernels merge the records with the pairwise rule of Chan et al. in its k-way form (the merge of
// the reference's tile statistics, ScaFFold/unet/triton_group_norm.py:148-165,594-607). Nothing is carried from one
// call to the next and nothing comes from the caller: a record is a function of the values it covers alone.
//
// How a record stays accurate when the mean is large against the spread: sums are taken about a value of their own
// data. Every wavefront sums v - K and (v - K)^2 with K = the first output it stored inside the tensor (per 4-channel
// run), which is within a few standard deviations of the mean, so S2 - S1^2/n does not cancel; the wavefronts' sums
// become (n, mean, M2) and are merged pairwise (mean and M2 of two pieces from their counts, means and M2s), where the
// correction terms are small again.
// No atomics: every (record, group) slot is written by exactly one workgroup and every sum has a fixed order, so the
// statistics are the same bits on every run.
#pragma once
#include "common.hpp"

namespace sfh {

constexpr int kGnRecordFloats = 4;  // floats per (record, group)

// Where a producer writes, or nothing (part == nullptr). `records` per sample; `cg` channels per group.
struct GnPartialOut {
  float* part;
  int groups, cg, records;
};

// (count, mean, M2) being merged from pieces in a fixed order. The first non-empty piece's mean is the reference point
// c; a piece (n, mean, M2) adds n, n d and M2 + n d^2 with d = mean - c (sums about c of the piece's data, exactly what
// the pairwise merge accumulates), and the total is mean = c + A / N, M2 = Q - A^2 / N.
struct WelfordMerge {
  float n, c, a, q;
  __device__ __forceinline__ void clear() { n = c = a = q = 0.f; }
  __device__ __forceinline__ void add(float pn, float pmean, float pm2) {
    if (pn <= 0.f) return;
    if (n == 0.f) c = pmean;
    const float d = pmean - c;
    n += pn;
    a = fmaf(pn, d, a);
    q += fmaf(pn * d, d, pm2);
  }
  // a piece given as sums about K: s1 = sum (v - K), s2 = sum (v - K)^2 over pn values
  __device__ __forceinline__ void add_sums(float pn, float s1, float s2, float k) {
    if (pn <= 0.f) return;
    const float dm = s1 / pn;
    const float m2 = fmaf(-s1, dm, s2);
    add(pn, k + dm, m2 < 0.f ? 0.f : m2);
  }
  __device__ __forceinline__ float mean() const { return n > 0.f ? c + a / n : 0.f; }
  __device__ __forceinline__ float m2() const {
    const float v = n > 0.f ? fmaf(-a, a / n, q) : 0.f;
    return v < 0.f ? 0.f : v;
  }
};

__device__ __forceinline__ void unpack2(bf16_t, uint32_t u, float& lo, float& hi) {
  lo = bf16_lo(u);
  hi = bf16_hi(u);
}
__device__ __forceinline__ void unpack2(fp16_t, uint32_t u, float& lo, float& hi) {
  lo = fp16_lo(u);
  hi = fp16_hi(u);
}

__device__ __forceinline__ int lane_index() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

// Sums of the four channel runs a lane holds of a 32-channel result block (run g = channels 8g + 4kg .. + 3, packed
// as two rounded pairs), over the voxels the lane has added so far, about k[g]: the first channel of run g at the
// wavefront's first voxel (the same value in all 32 lanes that hold the run). In every kernel that uses this, a
// wavefront's first voxel -- lane 0 of its first 32-voxel piece -- has the smallest coordinates of all its voxels, so it
// lies inside the tensor whenever any of them does: the shift is then one of the values summed. (A wavefront wholly past
// a ragged edge counts nothing, whatever its shift.)
struct RunSums {
  float s1[4], s2[4], k[4];
  float cnt;  // voxels of this lane counted so far
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int g = 0; g < 4; ++g) s1[g] = s2[g] = k[g] = 0.f;
    cnt = 0.f;
  }
  // Takes the shift from the wavefront's first voxel: `run` is the first piece the wavefront adds. All 64 lanes must
  // call it.
  template <typename T>
  __device__ __forceinline__ void pick_shift(const uint32_t (&run)[4][2]) {
    const bool upper = (lane_index() & 32) != 0;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      // lane 0 holds the run for k-half 0, lane 32 for k-half 1
      const uint32_t v0 = (uint32_t)__builtin_amdgcn_readlane((int)run[g][0], 0);
      const uint32_t v1 = (uint32_t)__builtin_amdgcn_readlane((int)run[g][0], 32);
      float lo, hi;
      unpack2(T{}, upper ? v1 : v0, lo, hi);
      k[g] = lo;
    }
  }
  // `inside`: the lane's voxel lies inside the tensor; `first`: nothing has been added yet (then the shift is picked).
  template <typename T>
  __device__ __forceinline__ void add(const uint32_t (&run)[4][2], bool inside, bool first) {
    if (first) pick_shift<T>(run);
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
    cnt += inside ? 1.f : 0.f;
  }
};

// Sum over the 32 lanes of each half-wave (the lanes that share a k-half kg hold the same channel runs of different
// voxels): afterwards every lane holds its half's total. Fixed butterfly order.
__device__ __forceinline__ float half_wave_sum(float v) {
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Floats of LDS write_group_partials needs.
constexpr int gn_partials_lds_floats(int nw, int nsub) { return nw * nsub * 8 * 4; }

// Workgroup of NW wavefronts, each lane with NSUB RunSums (result blocks ns = 0 .. NSUB-1 of the workgroup's channel
// span, which starts at global channel c0): merges them per group and writes the workgroup's slots of record `rec` of
// sample n. `lds` needs gn_partials_lds_floats(NW, NSUB) floats and must be free for writing (the caller has
// synchronised). A group wider than the span (cg > 32 * NSUB) is completed by the other workgroups of the same tile,
// each in a record of its own.
template <int NW, int NSUB>
__device__ __forceinline__ void write_group_partials(const RunSums (&rs)[NSUB], float* lds, const GnPartialOut& o, int n, int rec, int c0,
                                                     int tid) {
  const int lane = tid & 63, wave = tid >> 6, kg = lane >> 5;
  // lds[wave][ns][run r = 2g + kg] = { values, sum, sum of squares, shift }
#pragma unroll
  for (int ns = 0; ns < NSUB; ++ns) {
    const float voxels = half_wave_sum(rs[ns].cnt);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float t1 = half_wave_sum(rs[ns].s1[g]), t2 = half_wave_sum(rs[ns].s2[g]);
      if ((lane & 31) == 0)
        *reinterpret_cast<float4*>(lds + ((wave * NSUB + ns) * 8 + 2 * g + kg) * 4) = make_float4(4.f * voxels, t1, t2, rs[ns].k[g]);
    }
  }
  __syncthreads();
  const int span = 32 * NSUB;
  const int runs_per_group = (o.cg < span ? o.cg : span) / 4;  // a power of two (gn_partials_fit)
  constexpr int RUNS = NSUB * 8, ENTRIES = NW * RUNS;
  if constexpr (ENTRIES <= 64 && (NW & (NW - 1)) == 0) {
    // One lane of the first wavefront per (wavefront, run) entry: each turns its sums into (n, mean, M2), then the
    // entries of a group -- runs_per_group neighbouring runs of every wavefront -- are merged pairwise (Chan et al.) in a
    // fixed butterfly: both partners of a step merge (lower lane, upper lane) in that order and get the same bits.
    if (tid < 64) {
      float pn = 0.f, mean = 0.f, m2 = 0.f;
      if (tid < ENTRIES) {
        const float4 e = *reinterpret_cast<const float4*>(lds + tid * 4);
        if (e.x > 0.f) {
          const float dm = e.y / e.x;
          pn = e.x;
          mean = e.w + dm;
          m2 = fmaf(-e.y, dm, e.z);
          m2 = m2 < 0.f ? 0.f : m2;
        }
      }
      auto merge_with = [&](int off) {
        const float qn = __shfl_xor(pn, off, 64), qmean = __shfl_xor(mean, off, 64), qm2 = __shfl_xor(m2, off, 64);
        const bool upper = (tid & off) != 0;
        const float n1 = upper ? qn : pn, n2 = upper ? pn : qn;
        const float mean1 = upper ? qmean : mean, mean2 = upper ? mean : qmean;
        const float ma = upper ? qm2 : m2, mb = upper ? m2 : qm2;
        const float nn = n1 + n2;
        const float w2 = nn > 0.f ? n2 / nn : 0.f;
        const float d = mean2 - mean1;
        pn = nn;
        mean = n1 > 0.f ? fmaf(d, w2, mean1) : mean2;
        m2 = (ma + mb) + (n1 > 0.f && n2 > 0.f ? d * d * n1 * w2 : 0.f);
      };
      for (int off = 1; off < runs_per_group; off <<= 1) merge_with(off);
#pragma unroll
      for (int off = RUNS; off < ENTRIES; off <<= 1) merge_with(off);
      if (tid < RUNS && (tid & (runs_per_group - 1)) == 0) {
        const int group = (c0 + tid * 4) / o.cg;
        *reinterpret_cast<float4*>(o.part + (((int64_t)n * o.records + rec) * o.groups + group) * kGnRecordFloats) =
            make_float4(pn, mean, m2, 0.f);
      }
    }
  } else {
    const int ngroups = span / (runs_per_group * 4);
    if (tid < ngroups) {
      WelfordMerge m;
      m.clear();
      for (int w = 0; w < NW; ++w)
        for (int r = 0; r < runs_per_group; ++r) {
          const float4 e = *reinterpret_cast<const float4*>(lds + (w * RUNS + tid * runs_per_group + r) * 4);
          m.add_sums(e.x, e.y, e.z, e.w);
        }
      const int group = (c0 + tid * runs_per_group * 4) / o.cg;
      *reinterpret_cast<float4*>(o.part + (((int64_t)n * o.records + rec) * o.groups + group) * kGnRecordFloats) =
          make_float4(m.n, m.mean(), m.m2(), 0.f);
    }
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
