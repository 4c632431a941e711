// Channels-last GroupNorm forward / backward for a dense (N, S, C) tensor.
//
// Statistics are fp32 and computed in one streaming pass with SHIFTED sums: every workgroup
// first derives, for each group, the same shift K (the mean of the group's channels over the
// first voxels of the sample) and then accumulates sum(x-K) and sum((x-K)^2). Because the shift
// is within a fraction of a standard deviation of the true mean, var = S2/m - (S1/m)^2 does not
// cancel the way E[x^2]-E[x]^2 does at mean >> std, and because every workgroup of a sample
// uses the identical shift the partial sums add without a pairwise (Chan) correction. This is
// the role the corrected two-pass tile statistics + Welford merge play in the reference
// (ScaFFold/unet/triton_group_norm.py:148-165,594-694).
//
// Launch chain (no atomics, partials at fixed scratch slots, fixed-order sums):
//   forward : gn_stats_partial -> [gn_stats_finalize] -> gn_normalize        (3*B bytes streamed)
//   backward: gn_bwd_partial   -> [gn_bwd_finalize]   -> gn_dx               (5*B bytes streamed)
// The finalize launches run only when a sample has more than 16 Ki floats of group-level partials; below that the
// consumer kernel folds the partials itself (every workgroup the same way, 64 KiB from L2 at most), which is
// cheaper than a launch of its own.
// The fused ReLU is spelled `y <= 0 ? 0 : y` and the backward gate `pre <= 0 ? 0 : dy` so that
// NaN propagates exactly as F.relu / threshold_backward do (triton_group_norm.py:176-198), and
// the gate is evaluated on the pre-activation recomputed with the forward's own expression.
//
// Two code paths, chosen by shape only: the vector path (16-byte loads, a thread owns a fixed
// set of channels) when C is a multiple of the vector width and the channels of a thread fall
// into whole groups; the scalar path (one workgroup per (sample, group)) otherwise.
#include <mutex>

#include "common.hpp"
#include "gn_stats.hpp"
#include "vec_io.hpp"

// No implicit mul+add contraction in this file: every FMA is written as fmaf(). The forward and the
// backward then round the pre-activation identically, and dy*gamma minus its own group mean cancels
// to an exact zero for one-element groups.
#pragma clang fp contract(off)

namespace sfh {

namespace {

constexpr int kBlock = 256;
constexpr int kShiftRows = 32;   // voxels that define the shift K
constexpr int kMaxSplit = 2048;  // workgroups per sample
constexpr int kFillWorkgroups = 256;   // workgroups a launch aims for when the sample is small: one per compute unit

struct GnPlan {
  bool vector;
  int vec;    // elements per thread and row
  int tpr;    // threads per voxel row = C / vec
  int rpp;    // voxel rows per pass of a workgroup
  int slots;  // group slots per thread: max(1, vec / (C/G))
  int nsplit; // workgroups per sample (reduction and elementwise passes alike)
  int64_t rows_per_split;
};

GnPlan make_plan(const sfh_groupnorm_desc& p, int x_dtype, bool aligned) {
  GnPlan pl{};
  pl.vec = x_dtype == SFH_FP32 ? 4 : 8;
  const int cg = p.c / p.groups;
  pl.vector = aligned && p.c % pl.vec == 0 && p.c / pl.vec <= kBlock && (cg % pl.vec == 0 || pl.vec % cg == 0);
  if (!pl.vector) {
    pl.nsplit = 1;
    pl.rows_per_split = p.spatial;
    return pl;
  }
  pl.tpr = p.c / pl.vec;
  pl.rpp = kBlock / pl.tpr;
  pl.slots = cg >= pl.vec ? 1 : pl.vec / cg;
  // 16 passes of 4 KiB per workgroup on large samples. On small ones a launch aims at one workgroup per compute unit
  // (every workgroup pays for folding the sample's partial records, and all of them run at once), at two when that
  // would take more than 8 passes: a 16 MiB sample is quickest as 512 x 8 passes, a 4 MiB one as 256 x 4.
  int64_t want = cdiv((int64_t)kFillWorkgroups, std::max(1, p.n));
  int64_t passes = p.spatial / ((int64_t)pl.rpp * want);
  if (passes > 8) {
    want = cdiv((int64_t)2 * kFillWorkgroups, std::max(1, p.n));
    passes = p.spatial / ((int64_t)pl.rpp * want);
  }
  passes = std::min<int64_t>(16, std::max<int64_t>(1, passes));
  int64_t rows = (int64_t)pl.rpp * passes;
  if (cdiv(p.spatial, rows) > kMaxSplit) rows = cdiv(cdiv(p.spatial, kMaxSplit), pl.rpp) * pl.rpp;
  pl.rows_per_split = rows;
  pl.nsplit = (int)cdiv(p.spatial, rows);
  return pl;
}

__device__ __forceinline__ float load_param(const void* p, int dtype, int i, float dflt) {
  if (p == nullptr) return dflt;
  if (dtype == SFH_FP32) return static_cast<const float*>(p)[i];
  if (dtype == SFH_BF16) return to_float(static_cast<const bf16_t*>(p)[i]);
  return to_float(static_cast<const fp16_t*>(p)[i]);
}

// V consecutive parameters from element c0 (a multiple of V) as one or two vector loads behind ONE branch on the
// dtype: a thread's eight gammas and eight betas fetched one scalar at a time, each behind its own dtype test, were
// sixteen trips to memory one after the other (1.8 us of a 6 us launch on a small tensor).
template <int V>
__device__ __forceinline__ void load_params(const void* p, int dtype, int c0, float dflt, float (&out)[V]) {
  static_assert(V == 4 || V == 8, "a thread's channel vector");
  if (p == nullptr) {
#pragma unroll
    for (int e = 0; e < V; ++e) out[e] = dflt;
  } else if (dtype == SFH_FP32) {
    const float* f = static_cast<const float*>(p) + c0;
    if ((reinterpret_cast<uintptr_t>(f) & 15) == 0) {
      Ld<float, V>::run(f, out);
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) out[e] = f[e];
    }
  } else if (dtype == SFH_BF16) {
    const bf16_t* h = static_cast<const bf16_t*>(p) + c0;
    if ((reinterpret_cast<uintptr_t>(h) & (2 * V - 1)) == 0) {
      Ld<bf16_t, V>::run(h, out);
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) out[e] = to_float(h[e]);
    }
  } else {
    const fp16_t* h = static_cast<const fp16_t*>(p) + c0;
    if ((reinterpret_cast<uintptr_t>(h) & (2 * V - 1)) == 0) {
      Ld<fp16_t, V>::run(h, out);
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) out[e] = to_float(h[e]);
    }
  }
}

__device__ __forceinline__ float relu_keep_nan(float y) { return y <= 0.f ? 0.f : y; }

// Fixed-order sum over a 64-lane wavefront; lane 0 holds the result.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

// Sums NVAL per-thread values over the voxel rows of the workgroup (threads sharing a channel
// vector cv) in a fixed order. Afterwards buf[v * kBlock + cv], cv < tpr, holds the totals. buf needs
// NVAL * kBlock floats.
// Where tpr divides the wavefront (a power of two up to 64, every thread active): a butterfly over the lanes of a
// wavefront that share cv, then the four wavefronts' totals through LDS in wavefront order -- three barriers whatever
// the row count. (A binary tree over the rows through LDS, one barrier per level, took 1.9 us of a 4.8 us launch at 8
// rows per workgroup and 3.1 us at 32.) Otherwise that tree.
template <int NVAL>
__device__ __forceinline__ void block_row_reduce(const float (&val)[NVAL], float* buf, int tpr, int rpp, bool active) {
  const int tid = threadIdx.x;
  if (tpr <= 64 && (tpr & (tpr - 1)) == 0) {  // uniform over the workgroup
    const int lane = tid & 63, wave = tid >> 6;
    float part[NVAL];
#pragma unroll
    for (int v = 0; v < NVAL; ++v) part[v] = val[v];
    for (int off = tpr; off < 64; off <<= 1) {
#pragma unroll
      for (int v = 0; v < NVAL; ++v) part[v] += __shfl_xor(part[v], off, 64);
    }
    __syncthreads();  // buf is free
    if (lane < tpr) {
#pragma unroll
      for (int v = 0; v < NVAL; ++v) buf[(v * 4 + wave) * 64 + lane] = part[v];
    }
    __syncthreads();
    // thread -> (value v, channel vector cv): the four wavefront totals in order
    constexpr int PER = (NVAL * 64 + kBlock - 1) / kBlock;  // outputs per thread at most (tpr = 64)
    float tot[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int idx = tid + k * kBlock, v = idx / tpr, cv = idx - v * tpr;
      tot[k] = 0.f;
      if (v < NVAL) tot[k] = (buf[(v * 4) * 64 + cv] + buf[(v * 4 + 1) * 64 + cv]) + (buf[(v * 4 + 2) * 64 + cv] + buf[(v * 4 + 3) * 64 + cv]);
    }
    __syncthreads();  // every total is in a register: the staging area becomes the result
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int idx = tid + k * kBlock, v = idx / tpr, cv = idx - v * tpr;
      if (v < NVAL) buf[v * kBlock + cv] = tot[k];
    }
    __syncthreads();
    return;
  }
  const int r = tid / tpr;
  __syncthreads();
  if (active) {
#pragma unroll
    for (int v = 0; v < NVAL; ++v) buf[v * kBlock + tid] = val[v];
  }
  __syncthreads();
  int top = 1;
  while (top < rpp) top <<= 1;
  for (int stride = top >> 1; stride > 0; stride >>= 1) {
    if (active && r < stride && r + stride < rpp) {
#pragma unroll
      for (int v = 0; v < NVAL; ++v) buf[v * kBlock + tid] += buf[v * kBlock + tid + stride * tpr];
    }
    __syncthreads();
  }
}

// Folds the per-channel-vector totals of NQ quantities (SLOTS slots each, value index
// q * SLOTS + s) into per-group totals out[q * G + g].
template <int SLOTS, int NQ>
__device__ __forceinline__ void fold_groups(const float* buf, float* out, int G, int cg, int vec) {
  for (int g = threadIdx.x; g < G; g += kBlock) {
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      float s = 0.f;
      if (SLOTS > 1) {
        s = buf[(q * SLOTS + (g % SLOTS)) * kBlock + g / SLOTS];
      } else {
        const int per = cg / vec;
        for (int k = 0; k < per; ++k) s += buf[q * kBlock + g * per + k];
      }
      out[q * G + g] = s;
    }
  }
  __syncthreads();
}

// ---- forward: partial statistics (vector path) --------------------------------------------
// scratch (floats): shift[N][G] | part[N][nsplit][2][G]
template <typename T, int SLOTS>
__global__ void __launch_bounds__(kBlock) gn_stats_partial(const T* __restrict__ x, float* __restrict__ shift,
                                                           float* __restrict__ part, int64_t S, int C, int G, int tpr, int rpp,
                                                           int nsplit, int64_t rows_per_split) {
  constexpr int V = VecOf<T>::N;
  extern __shared__ float smem[];
  float* buf = smem;                        // 2 * SLOTS * kBlock
  float* out = smem + 2 * SLOTS * kBlock;   // 2 * G
  const int tid = threadIdx.x;
  const int n = blockIdx.y, split = blockIdx.x;
  const int cg = C / G;
  const int r = tid / tpr, cv = tid - r * tpr;
  const bool active = r < rpp;
  const T* xs = x + (int64_t)n * S * C + cv * V;
  const int64_t begin = (int64_t)split * rows_per_split;
  int64_t end = begin + rows_per_split;
  if (end > S) end = S;
  const int64_t step = rpp;
  int64_t row = begin + r;
  constexpr int U = 4;  // rows per batch: the next batch's loads are in flight while the current one is summed

  // Shift K: mean of every group over the first voxels of the sample, bit-identical in every
  // workgroup of the sample because it is computed from the same rows in the same order.
  const int64_t krows = S < kShiftRows ? S : kShiftRows;
  float kv[SLOTS];
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) kv[s] = 0.f;
  if (active) {
    for (int64_t krow = r; krow < krows; krow += rpp) {
      float f[V];
      Ld<T, V>::run(xs + krow * C, f);
#pragma unroll
      for (int e = 0; e < V; ++e) kv[e * SLOTS / V] += f[e];
    }
  }
  // the workgroup's first rows are requested before the shift is known: the reductions below wait for nothing of theirs
  Piece<T, V> cur[U];
  fetch_rows<T, V, U>(cur, xs, row, step, end, begin, C, active);
  block_row_reduce<SLOTS>(kv, buf, tpr, rpp, active);
  fold_groups<SLOTS, 1>(buf, out, G, cg, V);
  const float kinv = 1.f / ((float)krows * (float)cg);
  float K[SLOTS];
#pragma unroll
  for (int s = 0; s < SLOTS; ++s) {
    const int g = (SLOTS > 1) ? cv * SLOTS + s : (cv * V) / cg;
    K[s] = active ? out[g] * kinv : 0.f;
  }
  if (split == 0)
    for (int g = tid; g < G; g += kBlock) shift[n * G + g] = out[g] * kinv;

  float acc[2 * SLOTS];
#pragma unroll
  for (int s = 0; s < 2 * SLOTS; ++s) acc[s] = 0.f;
  if (active) {
    while (row < end) {
      const int64_t next = row + U * step;
      Piece<T, V> nxt[U];
      if (next < end) fetch_rows<T, V, U>(nxt, xs, next, step, end, begin, C, true);
      if (row + (U - 1) * step < end) {  // a whole batch
        float f0[V], f1[V], f2[V], f3[V];
        cur[0].unpack(f0);
        cur[1].unpack(f1);
        cur[2].unpack(f2);
        cur[3].unpack(f3);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const int s = e * SLOTS / V;
          const float d0 = f0[e] - K[s], d1 = f1[e] - K[s], d2 = f2[e] - K[s], d3 = f3[e] - K[s];
          acc[s] += (d0 + d1) + (d2 + d3);
          float q = acc[SLOTS + s];
          q = fmaf(d0, d0, q); q = fmaf(d1, d1, q); q = fmaf(d2, d2, q); q = fmaf(d3, d3, q);
          acc[SLOTS + s] = q;
        }
      } else {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (row + u * step < end) {
            float f0[V];
            cur[u].unpack(f0);
#pragma unroll
            for (int e = 0; e < V; ++e) {
              const int s = e * SLOTS / V;
              const float d0 = f0[e] - K[s];
              acc[s] += d0;
              acc[SLOTS + s] = fmaf(d0, d0, acc[SLOTS + s]);
            }
          }
        }
      }
      if (next < end) {
#pragma unroll
        for (int u = 0; u < U; ++u) cur[u] = nxt[u];
      }
      row = next;
    }
  }
  block_row_reduce<2 * SLOTS>(acc, buf, tpr, rpp, active);
  fold_groups<SLOTS, 2>(buf, out, G, cg, V);
  float* dst = part + ((int64_t)n * nsplit + split) * 2 * G;
  for (int i = tid; i < 2 * G; i += kBlock) dst[i] = out[i];
}

// One workgroup per (group, sample): fixed-order sum of the split partials, then
// mean = K + S1/m, var = S2/m - (S1/m)^2, rstd = 1/sqrt(var + eps).
__global__ void __launch_bounds__(kBlock) gn_stats_finalize(const float* __restrict__ shift, const float* __restrict__ part,
                                                            float* __restrict__ mean, float* __restrict__ rstd, int G, int nsplit,
                                                            float m, float eps) {
  __shared__ float wsum[kBlock / 64][2];
  const int g = blockIdx.x, n = blockIdx.y, tid = threadIdx.x;
  const float* base = part + (int64_t)n * nsplit * 2 * G + g;
  float s1 = 0.f, s2 = 0.f;
  // thread t owns records t, t + 256, ...: eight at a time, their loads all in flight before the first add
  int i = tid;
  for (; i + 7 * kBlock < nsplit; i += 8 * kBlock) {
    float a[8], b[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float* p = base + (int64_t)(i + u * kBlock) * 2 * G;
      a[u] = p[0];
      b[u] = p[G];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) { s1 += a[u]; s2 += b[u]; }
  }
  for (; i < nsplit; i += kBlock) {
    const float* p = base + (int64_t)i * 2 * G;
    s1 += p[0];
    s2 += p[G];
  }
  s1 = wave_sum(s1);
  s2 = wave_sum(s2);
  if ((tid & 63) == 0) { wsum[tid >> 6][0] = s1; wsum[tid >> 6][1] = s2; }
  __syncthreads();
  if (tid == 0) {
    s1 = s2 = 0.f;
#pragma unroll
    for (int w = 0; w < kBlock / 64; ++w) { s1 += wsum[w][0]; s2 += wsum[w][1]; }
    const float d = s1 / m;
    float var = s2 / m - d * d;
    var = var < 0.f ? 0.f : var;
    const float mu = shift[n * G + g] + d, rs = 1.f / sqrtf(var + eps);
    mean[n * G + g] = mu;
    rstd[n * G + g] = rs;
  }
}

// The same for Welford records a producer of x left, rec[sample][record][group] = { count, mean, M2, - } (gn_stats.hpp):
// merged about the first record's mean c. A record adds n, n d and M2 + n d^2 with d = mean - c, which are the sums
// about c of the values it covers; then mean = c + A/m, var = (Q - A^2/m)/m. Fixed order: thread t owns the records
// t, t + 256, ..., the threads are added by wavefront, the wavefronts in order.
__global__ void __launch_bounds__(kBlock) gn_welford_finalize(const float* __restrict__ rec, float* __restrict__ mean,
                                                              float* __restrict__ rstd, int G, int nrec, float m, float eps) {
  __shared__ float wsum[kBlock / 64][2];
  const int g = blockIdx.x, n = blockIdx.y, tid = threadIdx.x;
  const float4* base = reinterpret_cast<const float4*>(rec) + (int64_t)n * nrec * G + g;
  const float c = base[0].y;
  float a = 0.f, q = 0.f;
  int i = tid;
  for (; i + 7 * kBlock < nrec; i += 8 * kBlock) {
    float4 e[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) e[u] = base[(int64_t)(i + u * kBlock) * G];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float d = e[u].y - c;
      a = fmaf(e[u].x, d, a);
      q += fmaf(e[u].x * d, d, e[u].z);
    }
  }
  for (; i < nrec; i += kBlock) {
    const float4 e = base[(int64_t)i * G];
    const float d = e.y - c;
    a = fmaf(e.x, d, a);
    q += fmaf(e.x * d, d, e.z);
  }
  a = wave_sum(a);
  q = wave_sum(q);
  if ((tid & 63) == 0) { wsum[tid >> 6][0] = a; wsum[tid >> 6][1] = q; }
  __syncthreads();
  if (tid == 0) {
    a = q = 0.f;
#pragma unroll
    for (int w = 0; w < kBlock / 64; ++w) { a += wsum[w][0]; q += wsum[w][1]; }
    const float d = a / m;
    float var = fmaf(-a, d, q) / m;
    var = var < 0.f ? 0.f : var;
    mean[n * G + g] = c + d;
    rstd[n * G + g] = 1.f / sqrtf(var + eps);
  }
}

// Sums the split partials of one sample inside a consumer kernel, the same way in every workgroup that calls it (so
// all of them get the same bits). `rows` points at the sample's slots [split][quantity][group], 2 * G floats per
// split, nsplit * 2 * G <= kFoldFloats in total and 2 * G a power of two <= 64. Thread t reads the 16-byte pieces
// t, t + 256, ... (all loads in flight at once) and keeps one running sum per float of its piece's column; the
// threads that share a column are then added by a fixed butterfly inside each wavefront and the four wavefronts in
// order through LDS. Thread c < 2 * G ends up holding the total of column c (quantity c / G, group c % G) and passes
// it to emit(c, total).
constexpr int kFoldFloats = 16384;

__host__ __device__ __forceinline__ bool fold_in_consumer(int G, int nsplit, int per_group = 2) {
  const int cols = per_group * G;
  return cols >= 4 && cols <= 64 && (cols & (cols - 1)) == 0 && (int64_t)nsplit * cols <= kFoldFloats;
}
inline bool fold_in_consumer_host(int G, int nsplit, int per_group = 2) { return fold_in_consumer(G, nsplit, per_group); }

template <typename Emit>
__device__ __forceinline__ void fold_split_partials(const float* __restrict__ rows, int G, int nsplit, float* lds /* 4 * kBlock */,
                                                    Emit emit) {
  const int tid = threadIdx.x;
  const int cols = 2 * G, total = nsplit * cols;
  constexpr int NB = kFoldFloats / (4 * kBlock);  // pieces per thread at most
  float4 v[NB];
#pragma unroll
  for (int k = 0; k < NB; ++k) {
    const int i = (tid + k * kBlock) * 4;
    v[k] = i < total ? *reinterpret_cast<const float4*>(rows + i) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  // kBlock * 4 is a multiple of cols, so every piece of a thread lies in the same four columns
  float4 s = v[0];
#pragma unroll
  for (int k = 1; k < NB; ++k) { s.x += v[k].x; s.y += v[k].y; s.z += v[k].z; s.w += v[k].w; }
  // threads tid % (cols / 4) alike hold the same four columns: a butterfly over them inside the wavefront, then the four
  // wavefronts in order through LDS
  const int per = cols / 4;
  for (int off = 32; off >= per; off >>= 1) {
    s.x += __shfl_xor(s.x, off, 64);
    s.y += __shfl_xor(s.y, off, 64);
    s.z += __shfl_xor(s.z, off, 64);
    s.w += __shfl_xor(s.w, off, 64);
  }
  const int lane = tid & 63, wave = tid >> 6;
  if (lane < per) *reinterpret_cast<float4*>(lds + wave * cols + lane * 4) = s;
  __syncthreads();
  if (tid < cols) emit(tid, (lds[tid] + lds[cols + tid]) + (lds[2 * cols + tid] + lds[3 * cols + tid]));
}

// The same inside a consumer for a producer's Welford records rec[record][group] = { count, mean, M2, - } of one sample
// (G a power of two, nrec * 4 G <= kFoldFloats): a thread's pieces t, t + 256, ... all belong to group t % G; it
// merges them about the first record's mean c (see gn_welford_finalize), the threads of a group are added by a fixed
// butterfly inside each wavefront and the four wavefronts in order. Thread g < G passes its group's (c, A, Q) to emit.
template <typename Emit>
__device__ __forceinline__ void fold_welford_records(const float* __restrict__ rec, int G, int nrec, float* lds /* 4 * kBlock */,
                                                     Emit emit) {
  const int tid = threadIdx.x;
  const int total = nrec * G;
  constexpr int NB = kFoldFloats / (4 * kBlock);
  const float c = rec[(tid & (G - 1)) * kGnRecordFloats + 1];
  float4 v[NB];
#pragma unroll
  for (int k = 0; k < NB; ++k) {
    const int i = tid + k * kBlock;
    v[k] = i < total ? *reinterpret_cast<const float4*>(rec + (int64_t)i * kGnRecordFloats) : make_float4(0.f, c, 0.f, 0.f);
  }
  float a = 0.f, q = 0.f;
#pragma unroll
  for (int k = 0; k < NB; ++k) {
    const float d = v[k].y - c;
    a = fmaf(v[k].x, d, a);
    q += fmaf(v[k].x * d, d, v[k].z);
  }
  // threads tid % G alike hold the same group: a butterfly over them inside the wavefront, then the four wavefronts in
  // order through LDS
  for (int off = 32; off >= G; off >>= 1) {
    a += __shfl_xor(a, off, 64);
    q += __shfl_xor(q, off, 64);
  }
  const int lane = tid & 63, wave = tid >> 6;
  if (lane < G) {
    lds[(wave * G + lane) * 2] = a;
    lds[(wave * G + lane) * 2 + 1] = q;
  }
  __syncthreads();
  if (tid < G) {
    const float ta = (lds[2 * tid] + lds[2 * (G + tid)]) + (lds[2 * (2 * G + tid)] + lds[2 * (3 * G + tid)]);
    const float tq = (lds[2 * tid + 1] + lds[2 * (G + tid) + 1]) + (lds[2 * (2 * G + tid) + 1] + lds[2 * (3 * G + tid) + 1]);
    emit(tid, c, ta, tq);
  }
}

// ---- forward: normalise + affine (+ReLU) (vector path) ------------------------------------
// When the sample's split partials are few (fold_in_consumer), every workgroup derives mean and rstd from them itself
// (mean = K + S1/m, var = S2/m - (S1/m)^2, rstd = 1/sqrt(var + eps)): 32 KiB from L2 cost less than a launch of their
// own, and the first workgroup of a sample writes them out for the backward pass. Otherwise gn_stats_finalize has run.
template <typename T, typename TO>
__global__ void __launch_bounds__(kBlock) gn_normalize(const T* __restrict__ x, TO* __restrict__ y, const float* __restrict__ shift,
                                                       const float* __restrict__ part, float* __restrict__ mean,
                                                       float* __restrict__ rstd, const void* __restrict__ gamma,
                                                       const void* __restrict__ beta, int param_dtype, int64_t S, int C, int G,
                                                       int tpr, int rpp, int nsplit, int64_t rows_per_split, float m, float eps,
                                                       int relu, int64_t y_halo, int npart, int welford) {
  constexpr int V = VecOf<T>::N;
  extern __shared__ float gstat[];  // sums[2 G] | mean[G] | rstd[G] | fold scratch (4 * kBlock)
  const int tid = threadIdx.x;
  const int n = blockIdx.y;
  const int cg = C / G;
  const int r = tid / tpr, cv = tid - r * tpr;
  float* g_mean = gstat + 2 * G;
  float* g_rstd = gstat + 3 * G;
  // the workgroup's first rows are requested before anything else: the fold of the statistics below reads other memory
  constexpr int U = 4;  // rows per batch: the next batch's loads are in flight while the current one is normalised
  const T* xs = x + (int64_t)n * S * C + cv * V;
  const int64_t begin = (int64_t)blockIdx.x * rows_per_split;
  int64_t end = begin + rows_per_split;
  if (end > S) end = S;
  const int64_t step = rpp;
  int64_t row = begin + r;
  Piece<T, V> cur[U];
  fetch_rows<T, V, U>(cur, xs, row, step, end, begin, C, r < rpp);
  // `npart` partial records per sample: the statistics pass's own (one per workgroup of this grid, sums about the
  // common shift), or (`welford`) the records the producer of x left
  if (welford && fold_in_consumer(G, npart, kGnRecordFloats)) {
    fold_welford_records(part + (int64_t)n * npart * G * kGnRecordFloats, G, npart, gstat + 4 * G, [&](int g, float c, float a, float q) {
      const float d = a / m;
      float var = fmaf(-a, d, q) / m;
      var = var < 0.f ? 0.f : var;
      const float mu_g = c + d, rs_g = 1.f / sqrtf(var + eps);
      g_mean[g] = mu_g;
      g_rstd[g] = rs_g;
      if (blockIdx.x == 0) {  // for the backward pass
        mean[n * G + g] = mu_g;
        rstd[n * G + g] = rs_g;
      }
    });
  } else if (!welford && fold_in_consumer(G, npart)) {
    fold_split_partials(part + (int64_t)n * npart * 2 * G, G, npart, gstat + 4 * G, [&](int c, float t) { gstat[c] = t; });
    __syncthreads();
    if (tid < G) {
      const float d = gstat[tid] / m;
      float var = gstat[G + tid] / m - d * d;
      var = var < 0.f ? 0.f : var;
      const float mu_g = shift[n * G + tid] + d, rs_g = 1.f / sqrtf(var + eps);
      g_mean[tid] = mu_g;
      g_rstd[tid] = rs_g;
      if (blockIdx.x == 0) {  // for the backward pass
        mean[n * G + tid] = mu_g;
        rstd[n * G + tid] = rs_g;
      }
    }
  } else {
    for (int g = tid; g < G; g += kBlock) {  // a finalize launch has filled mean / rstd
      g_mean[g] = mean[n * G + g];
      g_rstd[g] = rstd[n * G + g];
    }
  }
  __syncthreads();
  // y is a slab of y_halo + S + y_halo rows per sample: the sample's workgroups zero the two faces between them
  const int64_t y_sample = (int64_t)n * (S + 2 * y_halo) * C;
  if (y_halo > 0) {
    const int64_t face_pieces = y_halo * C * (int64_t)sizeof(TO) / 16;
    uint4* lo = reinterpret_cast<uint4*>(y + y_sample);
    uint4* hi = reinterpret_cast<uint4*>(y + y_sample + (y_halo + S) * C);
    for (int64_t u = (int64_t)blockIdx.x * kBlock + tid; u < face_pieces; u += (int64_t)gridDim.x * kBlock) {
      lo[u] = make_uint4(0, 0, 0, 0);
      hi[u] = make_uint4(0, 0, 0, 0);
    }
  }
  if (r >= rpp) return;
  float mu[V], rs[V], ga[V], be[V];
  load_params<V>(gamma, param_dtype, cv * V, 1.f, ga);
  load_params<V>(beta, param_dtype, cv * V, 0.f, be);
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const int c = cv * V + e;
    mu[e] = g_mean[c / cg];
    rs[e] = g_rstd[c / cg];
  }
  TO* ys = y + y_sample + y_halo * C + cv * V;
  while (row < end) {
    const int64_t next = row + U * step;
    Piece<T, V> nxt[U];
    if (next < end) fetch_rows<T, V, U>(nxt, xs, next, step, end, begin, C, true);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (row + u * step < end) {
        float f[V], o[V];
        cur[u].unpack(f);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const float xh = (f[e] - mu[e]) * rs[e];
          const float v = fmaf(xh, ga[e], be[e]);
          o[e] = relu ? relu_keep_nan(v) : v;
        }
        St<TO, V>::run(ys + (row + u * step) * C, o);
      }
    }
    if (next < end) {
#pragma unroll
      for (int u = 0; u < U; ++u) cur[u] = nxt[u];
    }
    row = next;
  }
}

// ---- backward: per-channel partial sums (vector path) --------------------------------------
// part (floats): [N][nsplit][2][C]  with q = 0: sum dy'*xhat, q = 1: sum dy'
template <typename T, typename TG>
__global__ void __launch_bounds__(kBlock) gn_bwd_partial(const T* __restrict__ x, const TG* __restrict__ dy,
                                                         const float* __restrict__ mean, const float* __restrict__ rstd,
                                                         const void* __restrict__ gamma, const void* __restrict__ beta,
                                                         int param_dtype, float* __restrict__ part, float* __restrict__ gpart,
                                                         int64_t S, int C, int G, int tpr, int rpp, int nsplit,
                                                         int64_t rows_per_split, int relu) {
  constexpr int V = VecOf<T>::N;
  extern __shared__ float smem[];  // 2 * V * kBlock | gamma[C]
  float* gam = smem + 2 * V * kBlock;
  const int tid = threadIdx.x;
  const int n = blockIdx.y, split = blockIdx.x;
  const int cg = C / G;
  const int r = tid / tpr, cv = tid - r * tpr;
  const bool active = r < rpp;
  // the workgroup's first rows are requested before the statistics and parameters they will be combined with
  constexpr int U = 2;  // rows per batch: the next batch's loads are in flight while the current one is summed
  const int64_t base = (int64_t)n * S * C + cv * V;
  const T* xs = x + base;
  const TG* gs = dy + base;
  const int64_t begin = (int64_t)split * rows_per_split;
  int64_t end = begin + rows_per_split;
  if (end > S) end = S;
  const int64_t step = rpp;
  int64_t row = begin + r;
  Piece<T, V> cx[U];
  Piece<TG, V> cg_[U];
  fetch_rows<T, V, U>(cx, xs, row, step, end, begin, C, active);
  fetch_rows<TG, V, U>(cg_, gs, row, step, end, begin, C, active);
  float mu[V], rs[V], ga[V], be[V];
  load_params<V>(gamma, param_dtype, active ? cv * V : 0, 1.f, ga);
  load_params<V>(beta, param_dtype, active ? cv * V : 0, 0.f, be);
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const int c = active ? cv * V + e : 0;
    mu[e] = mean[n * G + c / cg];
    rs[e] = rstd[n * G + c / cg];
  }
  float acc[2 * V];
#pragma unroll
  for (int e = 0; e < 2 * V; ++e) acc[e] = 0.f;
  if (active) {
    while (row < end) {
      const int64_t next = row + U * step;
      Piece<T, V> nx[U];
      Piece<TG, V> ng[U];
      if (next < end) {
        fetch_rows<T, V, U>(nx, xs, next, step, end, begin, C, true);
        fetch_rows<TG, V, U>(ng, gs, next, step, end, begin, C, true);
      }
      if (row + step < end) {  // a whole batch
        float f0[V], g0[V], f1[V], g1[V];
        cx[0].unpack(f0);
        cg_[0].unpack(g0);
        cx[1].unpack(f1);
        cg_[1].unpack(g1);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const float xh0 = (f0[e] - mu[e]) * rs[e], xh1 = (f1[e] - mu[e]) * rs[e];
          float d0 = g0[e], d1 = g1[e];
          if (relu) {
            d0 = fmaf(xh0, ga[e], be[e]) <= 0.f ? 0.f : d0;
            d1 = fmaf(xh1, ga[e], be[e]) <= 0.f ? 0.f : d1;
          }
          acc[e] = fmaf(d0, xh0, acc[e]);
          acc[e] = fmaf(d1, xh1, acc[e]);
          acc[V + e] += d0 + d1;
        }
      } else {
        float f0[V], g0[V];
        cx[0].unpack(f0);
        cg_[0].unpack(g0);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const float xh0 = (f0[e] - mu[e]) * rs[e];
          float d0 = g0[e];
          if (relu) d0 = fmaf(xh0, ga[e], be[e]) <= 0.f ? 0.f : d0;
          acc[e] = fmaf(d0, xh0, acc[e]);
          acc[V + e] += d0;
        }
      }
      if (next < end) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          cx[u] = nx[u];
          cg_[u] = ng[u];
        }
      }
      row = next;
    }
  }
  if (tid < tpr) {  // the first row's threads hold every channel's gamma: the per-group fold below reads it from LDS
#pragma unroll
    for (int e = 0; e < V; ++e) gam[cv * V + e] = ga[e];
  }
  block_row_reduce<2 * V>(acc, smem, tpr, rpp, active);
  float* dst = part + ((int64_t)n * nsplit + split) * 2 * C;
  for (int i = tid; i < 2 * C; i += kBlock) {
    const int q = i / C, c = i - q * C;
    dst[i] = smem[(q * V + c % V) * kBlock + c / V];
  }
  // The same sums folded per group with the gamma weights (what dx needs): gpart[n][split][q][g]. Sixteen lanes share
  // a (quantity, group) pair, lane s takes channels s, s + 16, ... of the group, then a fixed tree over the 16 lanes.
  float* gdst = gpart + ((int64_t)n * nsplit + split) * 2 * G;
  for (int pair = tid >> 4; pair < 2 * G; pair += kBlock >> 4) {
    const int q = pair / G, g = pair - q * G;
    float t = 0.f;
    for (int cc = tid & 15; cc < cg; cc += 16) {
      const int c = g * cg + cc;
      t = fmaf(gam[c], smem[(q * V + c % V) * kBlock + c / V], t);
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) t += __shfl_down(t, off, 16);
    if ((tid & 15) == 0) gdst[pair] = t;
  }
}

// Fixed-order sum over a 256-thread workgroup (wavefront trees, then the four wave totals in order).
__device__ __forceinline__ float block_sum256(float v, float* red4) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red4[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red4[0] + red4[1]) + (red4[2] + red4[3]);
}

// Two sums at once (the same trees, one pair of barriers).
__device__ __forceinline__ void block_sum256_pair(float& a, float& b, float* red8) {
  a = wave_sum(a);
  b = wave_sum(b);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) {
    red8[threadIdx.x >> 6] = a;
    red8[4 + (threadIdx.x >> 6)] = b;
  }
  __syncthreads();
  a = (red8[0] + red8[1]) + (red8[2] + red8[3]);
  b = (red8[4] + red8[5]) + (red8[6] + red8[7]);
}

// Workgroups [0, N*G): coef[n][g] = (A, B) with A = mean(dy'*gamma), B = mean(dy'*gamma*xhat)
// over the group. Workgroups [N*G, N*G + C): dgamma[c], dbeta[c] summed over samples and splits.
__global__ void __launch_bounds__(kBlock) gn_bwd_finalize(const float* __restrict__ part, const void* __restrict__ gamma,
                                                          int param_dtype, float* __restrict__ coef, float* __restrict__ dgamma,
                                                          float* __restrict__ dbeta, int N, int C, int G, int nsplit, float m) {
  __shared__ float red4[4];
  const int b = blockIdx.x;
  const int cg = C / G;
  if (b < N * G) {
    const int n = b / G, g = b - n * G;
    // One flat index over (split, channel of the group): neighbouring threads read neighbouring channels and every
    // thread's loads are independent of one another.
    float s1 = 0.f, s2 = 0.f;
    const float* base = part + (int64_t)n * nsplit * 2 * C + g * cg;
    const int total = nsplit * cg;
    constexpr int U = 8;  // loads in flight per thread
    for (int i0 = threadIdx.x; i0 < total; i0 += U * kBlock) {
      float a1[U], a2[U], w[U];
#pragma unroll
      for (int k = 0; k < U; ++k) {
        const int i = i0 + k * kBlock;
        const int ic = i < total ? i : total - 1;
        const int sp = ic / cg, cc = ic - sp * cg;
        const float* p = base + (int64_t)sp * 2 * C + cc;
        a1[k] = p[0];
        a2[k] = p[C];
        w[k] = i < total ? load_param(gamma, param_dtype, g * cg + cc, 1.f) : 0.f;
      }
#pragma unroll
      for (int k = 0; k < U; ++k) {
        s1 = fmaf(w[k], a1[k], s1);
        s2 = fmaf(w[k], a2[k], s2);
      }
    }
    s1 = block_sum256(s1, red4);
    s2 = block_sum256(s2, red4);
    if (threadIdx.x == 0) {
      coef[(n * G + g) * 2] = s2 / m;
      coef[(n * G + g) * 2 + 1] = s1 / m;
    }
  } else {
    const int c = b - N * G;
    float s1 = 0.f, s2 = 0.f;
    const int total = N * nsplit;
    for (int i = threadIdx.x; i < total; i += kBlock) {
      const float* p = part + (int64_t)i * 2 * C;
      s1 += p[c];
      s2 += p[C + c];
    }
    s1 = block_sum256(s1, red4);
    s2 = block_sum256(s2, red4);
    if (threadIdx.x == 0) {
      if (dgamma != nullptr) dgamma[c] = s1;
      if (dbeta != nullptr) dbeta[c] = s2;
    }
  }
}

// dx = rstd * (dy'*gamma - A - xhat*B)   (ScaFFold/unet/triton_group_norm.py:908-1043)
// When the sample's group-level partials are few (fold_in_consumer) every workgroup derives the group coefficients
// A = mean(dy'*gamma), B = mean(dy'*gamma*xhat) from them itself, and workgroups of sample 0 finish by summing the
// per-channel partials of one channel each into dgamma / dbeta (samples and splits in index order): no finalize
// launch. Otherwise gn_bwd_finalize has filled `coef` and the parameter gradients.
template <typename T, typename TG>
__global__ void __launch_bounds__(kBlock) gn_dx(const T* __restrict__ x, const TG* __restrict__ dy, T* __restrict__ dx,
                                                const float* __restrict__ mean, const float* __restrict__ rstd,
                                                const void* __restrict__ gamma, const void* __restrict__ beta, int param_dtype,
                                                const float* __restrict__ coef, const float* __restrict__ part,
                                                const float* __restrict__ gpart, float* __restrict__ dgamma,
                                                float* __restrict__ dbeta, int N, int64_t S, int C, int G, int tpr, int rpp,
                                                int nsplit, int64_t rows_per_split, float m, int relu) {
  constexpr int V = VecOf<T>::N;
  extern __shared__ float gco[];  // sums[2 G] | fold scratch (4 * kBlock)
  __shared__ float red8[8];
  const int tid = threadIdx.x;
  const int n = blockIdx.y;
  const int cg = C / G;
  const int r = tid / tpr, cv = tid - r * tpr;
  // the workgroup's first rows are requested before anything else: the fold of the partials below reads other memory
  constexpr int U = 2;  // rows per batch: the next batch's loads are in flight while the current one is worked on
  const int64_t base = (int64_t)n * S * C + cv * V;
  const T* xs = x + base;
  const TG* gs = dy + base;
  const int64_t begin = (int64_t)blockIdx.x * rows_per_split;
  int64_t end = begin + rows_per_split;
  if (end > S) end = S;
  const int64_t step = rpp;
  int64_t row = begin + r;
  Piece<T, V> cx[U];
  Piece<TG, V> cg_[U];
  fetch_rows<T, V, U>(cx, xs, row, step, end, begin, C, r < rpp);
  fetch_rows<TG, V, U>(cg_, gs, row, step, end, begin, C, r < rpp);
  const bool fused = fold_in_consumer(G, nsplit);
  // The workgroup's share of the parameter gradients (the tail of this kernel) reads the per-channel partials of the
  // launch before: its first loads go out now, so that the tail does not start with a trip to memory of its own.
  const bool param_sums = fused && n == 0 && (dgamma != nullptr || dbeta != nullptr);
  const int total = N * nsplit;
  const int grp = tid >> 5, li = tid & 31;
  const bool one_channel = C <= (int)gridDim.x;  // at most one channel per workgroup: all 256 threads on it
  float pre1 = 0.f, pre2 = 0.f;
  if (param_sums) {
    const int c = one_channel ? (int)blockIdx.x : (int)blockIdx.x + grp * (int)gridDim.x;
    const int i = one_channel ? tid : li;
    if (c < C && i < total) {
      const float* p = part + (int64_t)i * 2 * C;
      pre1 = p[c];
      pre2 = p[C + c];
    }
  }
  if (fused) {
    // gpart quantity 0 = sum dy'*gamma*xhat (-> B), quantity 1 = sum dy'*gamma (-> A)
    fold_split_partials(gpart + (int64_t)n * nsplit * 2 * G, G, nsplit, gco + 2 * G, [&](int c, float t) { gco[c] = t / m; });
  } else {
    for (int i = tid; i < 2 * G; i += kBlock) {
      const int q = i / G, g = i - q * G;
      gco[i] = coef[(n * G + g) * 2 + (1 - q)];  // coef holds (A, B) per group
    }
  }
  __syncthreads();
  if (r < rpp) {
  float mu[V], rs[V], ga[V], be[V], ca[V], cb[V];
  load_params<V>(gamma, param_dtype, cv * V, 1.f, ga);
  load_params<V>(beta, param_dtype, cv * V, 0.f, be);
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const int c = cv * V + e;
    const int g = c / cg;
    mu[e] = mean[n * G + g];
    rs[e] = rstd[n * G + g];
    ca[e] = gco[G + g];
    cb[e] = gco[g];
  }
  T* ds = dx + base;
  while (row < end) {
    const int64_t next = row + U * step;
    Piece<T, V> nx[U];
    Piece<TG, V> ng[U];
    if (next < end) {
      fetch_rows<T, V, U>(nx, xs, next, step, end, begin, C, true);
      fetch_rows<TG, V, U>(ng, gs, next, step, end, begin, C, true);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (row + u * step < end) {
        float f[V], g[V], o[V];
        cx[u].unpack(f);
        cg_[u].unpack(g);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const float xh = (f[e] - mu[e]) * rs[e];
          float d = g[e];
          if (relu) d = fmaf(xh, ga[e], be[e]) <= 0.f ? 0.f : d;
          o[e] = rs[e] * ((d * ga[e] - ca[e]) - xh * cb[e]);
        }
        St<T, V>::run(ds + (row + u * step) * C, o);
      }
    }
    if (next < end) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        cx[u] = nx[u];
        cg_[u] = ng[u];
      }
    }
    row = next;
  }
  }
  if (param_sums) {
    // More channels than workgroups (the deepest levels): eight at a time, one per group of 32 lanes (workgroup b takes
    // channels b, b + gridDim.x, ...): each lane
    // adds every 32nd split partial of its channel, the 32 lanes meet in a butterfly; no LDS and no barrier. (One channel
    // at a time over all 256 threads cost the deepest level, 512 channels over 64 workgroups, 6 us of serial rounds.)
    // The first partial of every thread's first channel is in pre1 / pre2 already.
    if (one_channel) {
      for (int c = blockIdx.x; c < C; c += gridDim.x) {
        const bool first = c == (int)blockIdx.x;
        float s1 = first ? pre1 : 0.f, s2 = first ? pre2 : 0.f;
        for (int i = first ? tid + kBlock : tid; i < total; i += kBlock) {
          const float* p = part + (int64_t)i * 2 * C;
          s1 += p[c];
          s2 += p[C + c];
        }
        block_sum256_pair(s1, s2, red8);
        if (tid == 0) {
          if (dgamma != nullptr) dgamma[c] = s1;
          if (dbeta != nullptr) dbeta[c] = s2;
        }
      }
    } else
    for (int c0 = blockIdx.x; c0 < C; c0 += 8 * gridDim.x) {  // c0: the channel of group 0, uniform over the workgroup
      const int c = c0 + grp * gridDim.x;
      const bool first = c0 == (int)blockIdx.x;
      float s1 = first ? pre1 : 0.f, s2 = first ? pre2 : 0.f;
      if (c < C) {
        for (int i = first ? li + 32 : li; i < total; i += 32) {
          const float* p = part + (int64_t)i * 2 * C;
          s1 += p[c];
          s2 += p[C + c];
        }
      }
#pragma unroll
      for (int off = 16; off >= 1; off >>= 1) {
        s1 += __shfl_xor(s1, off, 32);
        s2 += __shfl_xor(s2, off, 32);
      }
      if (li == 0 && c < C) {
        if (dgamma != nullptr) dgamma[c] = s1;
        if (dbeta != nullptr) dbeta[c] = s2;
      }
    }
  }
}

// ---- scalar path: one workgroup per (group, sample) ---------------------------------------
__device__ __forceinline__ float block_sum(float v, float* red) {
  __syncthreads();
  red[threadIdx.x] = v;
  __syncthreads();
  for (int s = kBlock / 2; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
    __syncthreads();
  }
  return red[0];
}

template <typename T>
__global__ void __launch_bounds__(kBlock) gn_scalar_stats(const T* __restrict__ x, float* __restrict__ mean,
                                                          float* __restrict__ rstd, int64_t S, int C, int G, float eps) {
  __shared__ float red[kBlock];
  const int g = blockIdx.x, n = blockIdx.y;
  const int cg = C / G;
  const T* xs = x + (int64_t)n * S * C + g * cg;
  const int64_t m = S * cg;
  // shift: mean over the first voxels
  const int64_t km = (S < kShiftRows ? S : kShiftRows) * cg;
  float k = 0.f;
  for (int64_t i = threadIdx.x; i < km; i += kBlock) k += to_float(xs[(i / cg) * C + i % cg]);
  const float K = block_sum(k, red) / (float)km;
  float s1 = 0.f, s2 = 0.f;
  for (int64_t i = threadIdx.x; i < m; i += kBlock) {
    const float d = to_float(xs[(i / cg) * C + i % cg]) - K;
    s1 += d;
    s2 = fmaf(d, d, s2);
  }
  s1 = block_sum(s1, red);
  s2 = block_sum(s2, red);
  if (threadIdx.x == 0) {
    const float d = s1 / (float)m;
    float var = s2 / (float)m - d * d;
    var = var < 0.f ? 0.f : var;
    mean[n * G + g] = K + d;
    rstd[n * G + g] = 1.f / sqrtf(var + eps);
  }
}

template <typename T, typename TO>
__global__ void __launch_bounds__(kBlock) gn_scalar_normalize(const T* __restrict__ x, TO* __restrict__ y,
                                                              const float* __restrict__ mean, const float* __restrict__ rstd,
                                                              const void* __restrict__ gamma, const void* __restrict__ beta,
                                                              int param_dtype, int64_t S, int C, int G, int64_t total, int relu) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= total) return;
  const int c = (int)(i % C);
  const int n = (int)(i / ((int64_t)S * C));
  const int g = c / (C / G);
  const float xh = (to_float(x[i]) - mean[n * G + g]) * rstd[n * G + g];
  const float v = fmaf(xh, load_param(gamma, param_dtype, c, 1.f), load_param(beta, param_dtype, c, 0.f));
  y[i] = elem<TO>::from_float(relu ? relu_keep_nan(v) : v);
}

// Per (group, sample): per-channel sums into chan[n][2][C], then coef[n][g].
template <typename T, typename TG>
__global__ void __launch_bounds__(kBlock) gn_scalar_bwd_sums(const T* __restrict__ x, const TG* __restrict__ dy,
                                                             const float* __restrict__ mean, const float* __restrict__ rstd,
                                                             const void* __restrict__ gamma, const void* __restrict__ beta,
                                                             int param_dtype, float* __restrict__ chan, float* __restrict__ coef,
                                                             int64_t S, int C, int G, int relu) {
  __shared__ float red[kBlock];
  const int g = blockIdx.x, n = blockIdx.y;
  const int cg = C / G;
  const float mu = mean[n * G + g], rs = rstd[n * G + g];
  float a1 = 0.f, a2 = 0.f;
  for (int cc = 0; cc < cg; ++cc) {
    const int c = g * cg + cc;
    const float w = load_param(gamma, param_dtype, c, 1.f), b = load_param(beta, param_dtype, c, 0.f);
    const T* xs = x + (int64_t)n * S * C + c;
    const TG* gs = dy + (int64_t)n * S * C + c;
    float s1 = 0.f, s2 = 0.f;
    for (int64_t s = threadIdx.x; s < S; s += kBlock) {
      const float xh = (to_float(xs[s * C]) - mu) * rs;
      float d = to_float(gs[s * C]);
      if (relu) d = fmaf(xh, w, b) <= 0.f ? 0.f : d;
      s1 = fmaf(d, xh, s1);
      s2 += d;
    }
    s1 = block_sum(s1, red);
    s2 = block_sum(s2, red);
    if (threadIdx.x == 0) {
      chan[((int64_t)n * 2) * C + c] = s1;
      chan[((int64_t)n * 2 + 1) * C + c] = s2;
    }
    a1 = fmaf(w, s1, a1);
    a2 = fmaf(w, s2, a2);
  }
  if (threadIdx.x == 0) {
    const float m = (float)S * (float)cg;
    coef[(n * G + g) * 2] = a2 / m;
    coef[(n * G + g) * 2 + 1] = a1 / m;
  }
}

__global__ void __launch_bounds__(kBlock) gn_scalar_dparam(const float* __restrict__ chan, float* __restrict__ dgamma,
                                                           float* __restrict__ dbeta, int N, int C) {
  const int c = blockIdx.x * kBlock + threadIdx.x;
  if (c >= C) return;
  float s1 = 0.f, s2 = 0.f;
  for (int n = 0; n < N; ++n) {
    s1 += chan[((int64_t)n * 2) * C + c];
    s2 += chan[((int64_t)n * 2 + 1) * C + c];
  }
  if (dgamma != nullptr) dgamma[c] = s1;
  if (dbeta != nullptr) dbeta[c] = s2;
}

template <typename T, typename TG>
__global__ void __launch_bounds__(kBlock) gn_scalar_dx(const T* __restrict__ x, const TG* __restrict__ dy, T* __restrict__ dx,
                                                       const float* __restrict__ mean, const float* __restrict__ rstd,
                                                       const void* __restrict__ gamma, const void* __restrict__ beta,
                                                       int param_dtype, const float* __restrict__ coef, int64_t S, int C, int G,
                                                       int64_t total, int relu) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= total) return;
  const int c = (int)(i % C);
  const int n = (int)(i / ((int64_t)S * C));
  const int g = c / (C / G);
  const float rs = rstd[n * G + g];
  const float w = load_param(gamma, param_dtype, c, 1.f), b = load_param(beta, param_dtype, c, 0.f);
  const float xh = (to_float(x[i]) - mean[n * G + g]) * rs;
  float d = to_float(dy[i]);
  if (relu) d = fmaf(xh, w, b) <= 0.f ? 0.f : d;
  dx[i] = elem<T>::from_float(rs * ((d * w - coef[(n * G + g) * 2]) - xh * coef[(n * G + g) * 2 + 1]));
}

// ---- host-side dispatch --------------------------------------------------------------------
int check_desc(const sfh_groupnorm_desc* p, int x_dtype) {
  if (p == nullptr) return fail(SFH_ERR_INVALID, "groupnorm: null descriptor");
  if (!dtype_ok(x_dtype)) return fail(SFH_ERR_INVALID, "groupnorm: bad dtype %d", x_dtype);
  if (p->n < 1 || p->c < 1 || p->spatial < 1 || p->groups < 1 || p->c % p->groups != 0)
    return fail(SFH_ERR_INVALID, "groupnorm: need N,C,S >= 1 and C %% groups == 0 (N=%d C=%d S=%lld G=%d)", p->n, p->c,
                (long long)p->spatial, p->groups);
  if (p->n > 65535) return fail(SFH_ERR_UNSUPPORTED, "groupnorm: N=%d exceeds the grid limit", p->n);
  return SFH_OK;
}

bool aligned16(const void* a) { return (reinterpret_cast<uintptr_t>(a) & 15u) == 0; }

size_t fwd_ws_floats(const sfh_groupnorm_desc& p, const GnPlan& pl) {
  // shift[N][G] (padded to 16 bytes so the slots can be read as float4) | part[N][nsplit][2][G]
  return align_up((size_t)p.n * p.groups, 4) + (size_t)p.n * pl.nsplit * 2 * p.groups;
}
size_t bwd_ws_floats(const sfh_groupnorm_desc& p, const GnPlan& pl) {
  // coef[N][G][2] | part[N][nsplit][2][C] | gpart[N][nsplit][2][G]; every section starts on 16 bytes
  // (scalar path: chan[N][2][C] in the part slot)
  return align_up((size_t)p.n * p.groups * 2, 4) + align_up((size_t)p.n * pl.nsplit * 2 * p.c, 4) +
         (size_t)p.n * pl.nsplit * 2 * p.groups;
}

template <typename T, typename TO>
int fwd_typed(const sfh_groupnorm_desc& p, const GnPlan& pl, int param_dtype, const void* x, const void* gamma, const void* beta,
              void* y, int64_t y_halo, float* mean, float* rstd, float* ws, hipStream_t st, const float* given_records = nullptr,
              int given_nrec = 0) {
  const int G = p.groups, C = p.c;
  const int64_t S = p.spatial;
  if (y_halo > 0 && (!pl.vector || sizeof(T) != sizeof(TO) || (y_halo * C * sizeof(TO)) % 16 != 0))
    return fail(SFH_ERR_UNSUPPORTED, "groupnorm: the slab output needs the vector path and an output of the input's width");
  if (!pl.vector) {
    if (given_records != nullptr) return fail(SFH_ERR_UNSUPPORTED, "groupnorm: statistics from given records need the vector path");
    hipLaunchKernelGGL(gn_scalar_stats<T>, dim3(G, p.n), dim3(kBlock), 0, st, (const T*)x, mean, rstd, S, C, G, p.eps);
    if (int rc = check_launch("gn_scalar_stats")) return rc;
    const int64_t total = (int64_t)p.n * S * C;
    if (cdiv(total, kBlock) > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "groupnorm: tensor too large for the scalar path");
    hipLaunchKernelGGL((gn_scalar_normalize<T, TO>), dim3((unsigned)cdiv(total, kBlock)), dim3(kBlock), 0, st, (const T*)x,
                       (TO*)y, mean, rstd, gamma, beta, param_dtype, S, C, G, total, p.relu);
    return check_launch("gn_scalar_normalize");
  }
  const dim3 grid(pl.nsplit, p.n);
  const float* shift = nullptr;
  const float* part = given_records;  // Welford records of x's producer, or this call's own shifted sums
  int npart = given_nrec;
  const int welford = given_records != nullptr ? 1 : 0;
  if (given_records == nullptr) {
    float* my_shift = ws;
    float* my_part = ws + align_up((size_t)p.n * G, 4);
    const size_t lds = (size_t)(2 * pl.slots * kBlock + 2 * G) * sizeof(float);
#define SFH_GN_STATS(SL)                                                                                                      \
  hipLaunchKernelGGL((gn_stats_partial<T, SL>), grid, dim3(kBlock), lds, st, (const T*)x, my_shift, my_part, S, C, G, pl.tpr, \
                     pl.rpp, pl.nsplit, pl.rows_per_split)
    switch (pl.slots) {
      case 1: SFH_GN_STATS(1); break;
      case 2: SFH_GN_STATS(2); break;
      case 4: SFH_GN_STATS(4); break;
      default: SFH_GN_STATS(8); break;
    }
#undef SFH_GN_STATS
    if (int rc = check_launch("gn_stats_partial")) return rc;
    shift = my_shift; part = my_part; npart = pl.nsplit;
  }
  const float m = (float)S * (float)(C / G);
  if (welford) {
    if (!fold_in_consumer_host(G, npart, kGnRecordFloats)) {
      hipLaunchKernelGGL(gn_welford_finalize, dim3(G, p.n), dim3(kBlock), 0, st, part, mean, rstd, G, npart, m, p.eps);
      if (int rc = check_launch("gn_welford_finalize")) return rc;
    }
  } else if (!fold_in_consumer_host(G, npart)) {
    hipLaunchKernelGGL(gn_stats_finalize, dim3(G, p.n), dim3(kBlock), 0, st, shift, part, mean, rstd, G, npart, m, p.eps);
    if (int rc = check_launch("gn_stats_finalize")) return rc;
  }
  hipLaunchKernelGGL((gn_normalize<T, TO>), grid, dim3(kBlock), (size_t)(4 * G + 4 * kBlock) * sizeof(float), st, (const T*)x, (TO*)y, shift, part,
                     mean, rstd, gamma, beta, param_dtype, S, C, G, pl.tpr, pl.rpp, pl.nsplit, pl.rows_per_split, m, p.eps, p.relu, y_halo,
                     npart, welford);
  return check_launch("gn_normalize");
}

template <typename T, typename TG>
int bwd_typed(const sfh_groupnorm_desc& p, const GnPlan& pl, int param_dtype, const void* dy, const void* x, const void* gamma,
              const void* beta, const float* mean, const float* rstd, void* dx, float* dgamma, float* dbeta, float* ws,
              hipStream_t st) {
  const int G = p.groups, C = p.c;
  const int64_t S = p.spatial;
  float* coef = ws;
  float* part = ws + align_up((size_t)p.n * G * 2, 4);
  float* gpart = part + align_up((size_t)p.n * pl.nsplit * 2 * C, 4);
  if (!pl.vector) {
    hipLaunchKernelGGL((gn_scalar_bwd_sums<T, TG>), dim3(G, p.n), dim3(kBlock), 0, st, (const T*)x, (const TG*)dy, mean, rstd,
                       gamma, beta, param_dtype, part, coef, S, C, G, p.relu);
    if (int rc = check_launch("gn_scalar_bwd_sums")) return rc;
    if (dgamma != nullptr || dbeta != nullptr) {
      hipLaunchKernelGGL(gn_scalar_dparam, dim3((unsigned)cdiv(C, kBlock)), dim3(kBlock), 0, st, part, dgamma, dbeta, p.n, C);
      if (int rc = check_launch("gn_scalar_dparam")) return rc;
    }
    const int64_t total = (int64_t)p.n * S * C;
    if (cdiv(total, kBlock) > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "groupnorm: tensor too large for the scalar path");
    hipLaunchKernelGGL((gn_scalar_dx<T, TG>), dim3((unsigned)cdiv(total, kBlock)), dim3(kBlock), 0, st, (const T*)x,
                       (const TG*)dy, (T*)dx, mean, rstd, gamma, beta, param_dtype, coef, S, C, G, total, p.relu);
    return check_launch("gn_scalar_dx");
  }
  constexpr int V = VecOf<T>::N;
  const dim3 grid(pl.nsplit, p.n);
  hipLaunchKernelGGL((gn_bwd_partial<T, TG>), grid, dim3(kBlock), ((size_t)2 * V * kBlock + C) * sizeof(float), st, (const T*)x,
                     (const TG*)dy, mean, rstd, gamma, beta, param_dtype, part, gpart, S, C, G, pl.tpr, pl.rpp, pl.nsplit,
                     pl.rows_per_split, p.relu);
  if (int rc = check_launch("gn_bwd_partial")) return rc;
  const float m = (float)S * (float)(C / G);
  if (!fold_in_consumer_host(G, pl.nsplit)) {
    hipLaunchKernelGGL(gn_bwd_finalize, dim3(p.n * G + C), dim3(kBlock), 0, st, part, gamma, param_dtype, coef, dgamma, dbeta, p.n,
                       C, G, pl.nsplit, m);
    if (int rc = check_launch("gn_bwd_finalize")) return rc;
  }
  hipLaunchKernelGGL((gn_dx<T, TG>), grid, dim3(kBlock), (size_t)(2 * G + 4 * kBlock) * sizeof(float), st, (const T*)x,
                     (const TG*)dy, (T*)dx, mean, rstd, gamma, beta, param_dtype, coef, part, gpart, dgamma, dbeta, p.n, S, C, G,
                     pl.tpr, pl.rpp, pl.nsplit, pl.rows_per_split, m, p.relu);
  return check_launch("gn_dx");
}

}  // namespace
}  // namespace sfh

using namespace sfh;

extern "C" size_t sfh_groupnorm_fwd_workspace_bytes(const sfh_groupnorm_desc* p, int x_dtype) {
  if (check_desc(p, x_dtype) != SFH_OK) return 0;
  // Sized for the vector path whatever the pointer alignment turns out to be.
  const GnPlan pl = make_plan(*p, x_dtype, true);
  return align_up(fwd_ws_floats(*p, pl) * sizeof(float), 256);
}

static int groupnorm_fwd_any(const sfh_groupnorm_desc* p, int x_dtype, int y_dtype, int param_dtype, const void* x, const void* gamma,
                             const void* beta, void* y, int64_t y_halo, float* mean, float* rstd, void* workspace,
                             size_t workspace_bytes, void* stream, const float* given_records = nullptr, int given_nrec = 0) {
  if (int rc = check_desc(p, x_dtype)) return rc;
  if (!dtype_ok(y_dtype) || !dtype_ok(param_dtype)) return fail(SFH_ERR_INVALID, "groupnorm: bad output/param dtype");
  if (x == nullptr || y == nullptr || mean == nullptr || rstd == nullptr) return fail(SFH_ERR_INVALID, "groupnorm: null tensor");
  if (y_halo < 0) return fail(SFH_ERR_INVALID, "groupnorm: negative halo");
  const GnPlan pl = make_plan(*p, x_dtype, aligned16(x) && aligned16(y));
  if (pl.vector && given_records == nullptr) {
    const size_t need = fwd_ws_floats(*p, pl) * sizeof(float);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(SFH_ERR_WORKSPACE, "groupnorm fwd: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
  }
  hipStream_t st = (hipStream_t)stream;
  float* ws = (float*)workspace;
#define SFH_GN_FWD(TX, TY) \
  return fwd_typed<TX, TY>(*p, pl, param_dtype, x, gamma, beta, y, y_halo, mean, rstd, ws, st, given_records, given_nrec)
  if (x_dtype == SFH_BF16 && y_dtype == SFH_BF16) SFH_GN_FWD(bf16_t, bf16_t);
  if (x_dtype == SFH_BF16 && y_dtype == SFH_FP32) SFH_GN_FWD(bf16_t, float);
  if (x_dtype == SFH_BF16 && y_dtype == SFH_FP16) SFH_GN_FWD(bf16_t, fp16_t);
  if (x_dtype == SFH_FP16 && y_dtype == SFH_FP16) SFH_GN_FWD(fp16_t, fp16_t);
  if (x_dtype == SFH_FP16 && y_dtype == SFH_FP32) SFH_GN_FWD(fp16_t, float);
  if (x_dtype == SFH_FP16 && y_dtype == SFH_BF16) SFH_GN_FWD(fp16_t, bf16_t);
  if (x_dtype == SFH_FP32 && y_dtype == SFH_FP32) SFH_GN_FWD(float, float);
  if (x_dtype == SFH_FP32 && y_dtype == SFH_BF16) SFH_GN_FWD(float, bf16_t);
  SFH_GN_FWD(float, fp16_t);
#undef SFH_GN_FWD
}

extern "C" int sfh_groupnorm_fwd(const sfh_groupnorm_desc* p, int x_dtype, int y_dtype, int param_dtype, const void* x,
                                 const void* gamma, const void* beta, void* y, float* mean, float* rstd, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  return groupnorm_fwd_any(p, x_dtype, y_dtype, param_dtype, x, gamma, beta, y, 0, mean, rstd, workspace, workspace_bytes, stream);
}

extern "C" int sfh_groupnorm_fwd_slab(const sfh_groupnorm_desc* p, int x_dtype, int y_dtype, int param_dtype, const void* x,
                                      const void* gamma, const void* beta, void* y_slab, int64_t halo_rows, float* mean, float* rstd,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  return groupnorm_fwd_any(p, x_dtype, y_dtype, param_dtype, x, gamma, beta, y_slab, halo_rows, mean, rstd, workspace,
                           workspace_bytes, stream);
}

extern "C" int sfh_groupnorm_fwd_from_partials(const sfh_groupnorm_desc* p, int x_dtype, int y_dtype, int param_dtype, const void* x,
                                               const void* gamma, const void* beta, void* y_slab, int64_t halo_rows, float* mean,
                                               float* rstd, const float* partials, size_t partials_bytes, int32_t records,
                                               void* stream) {
  if (int rc = check_desc(p, x_dtype)) return rc;
  if (partials == nullptr || records < 1) return fail(SFH_ERR_INVALID, "groupnorm from partials: no records given");
  if (!aligned16(partials)) return fail(SFH_ERR_INVALID, "groupnorm from partials: the records must be 16-byte aligned");
  const size_t need = (size_t)p->n * records * p->groups * kGnRecordFloats * sizeof(float);
  if (partials_bytes < need)
    return fail(SFH_ERR_WORKSPACE, "groupnorm from partials: %d records per sample are %zu bytes, got %zu", records, need, partials_bytes);
  return groupnorm_fwd_any(p, x_dtype, y_dtype, param_dtype, x, gamma, beta, y_slab, halo_rows, mean, rstd, nullptr, 0, stream, partials,
                           records);
}

// ---- the forward for callers that may not allocate ------------------------------------------------------------------
// Same kernels, same launch plan, same results as sfh_groupnorm_fwd; the partial-statistics scratch is this file-scope
// device array instead of a caller's workspace. Every GPU the library runs on holds its own copy of the array (256 KiB,
// until the process ends) at its own address, looked up once per device with that device current. Calls on one GPU
// share the array: two that overlap in time (different streams) race. Nothing has to be cleared between calls: the
// statistics kernel writes every slot the later kernels read.
constexpr size_t kNoAllocScratchFloats = 64 * 1024;
static __device__ __align__(256) float g_gn_noalloc_scratch[kNoAllocScratchFloats];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_noalloc_mutex;
float* g_noalloc_ptr[kMaxDevices];  // device address of the array on each device (null: not looked up yet)

// Device address of the scratch array on the CURRENT device. The array's name is a host-side handle, not an address a
// kernel could use: the address comes from hipGetSymbolAddress, per device. The first lookup on a device may load the
// code object, so it must not happen while `st` is capturing: such a call is refused (prepare first).
int noalloc_scratch(float** out, hipStream_t st, bool may_look_up) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) return fail(SFH_ERR_LAUNCH, "groupnorm (no-alloc): no current device");
  if (dev >= kMaxDevices)
    return fail(SFH_ERR_UNSUPPORTED, "groupnorm (no-alloc): device %d is beyond the %d devices the scratch table holds", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_noalloc_mutex);
  if (g_noalloc_ptr[dev] == nullptr) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (!may_look_up || hipStreamIsCapturing(st, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone)
      return fail(SFH_ERR_INVALID, "groupnorm (no-alloc): the first call on device %d arrived on a capturing stream; call "
                  "sfh_groupnorm_fwd_noalloc_prepare() on the device before the capture", dev);
    void* ptr = nullptr;
    const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_gn_noalloc_scratch));
    if (err != hipSuccess || ptr == nullptr)
      return fail(SFH_ERR_LAUNCH, "groupnorm: hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(err));
    g_noalloc_ptr[dev] = static_cast<float*>(ptr);
  }
  *out = g_noalloc_ptr[dev];
  return SFH_OK;
}
}  // namespace

extern "C" int sfh_groupnorm_fwd_noalloc_prepare(void) {
  float* unused = nullptr;
  return noalloc_scratch(&unused, nullptr, true);
}

extern "C" size_t sfh_groupnorm_fwd_noalloc_max_bytes(void) { return kNoAllocScratchFloats * sizeof(float); }

extern "C" int sfh_groupnorm_fwd_noalloc(const sfh_groupnorm_desc* p, int x_dtype, int y_dtype, int param_dtype, const void* x,
                                         const void* gamma, const void* beta, void* y, float* mean, float* rstd, void* stream) {
  if (int rc = check_desc(p, x_dtype)) return rc;
  const GnPlan pl = make_plan(*p, x_dtype, aligned16(x) && aligned16(y));
  const size_t need = pl.vector ? fwd_ws_floats(*p, pl) * sizeof(float) : 0;
  if (need > kNoAllocScratchFloats * sizeof(float))
    return fail(SFH_ERR_WORKSPACE, "groupnorm fwd (no-alloc): this problem needs %zu bytes of scratch, the built-in buffer holds %zu; "
                "use sfh_groupnorm_fwd with a workspace", need, kNoAllocScratchFloats * sizeof(float));
  float* scratch = nullptr;
  if (int rc = noalloc_scratch(&scratch, (hipStream_t)stream, true)) return rc;
  return groupnorm_fwd_any(p, x_dtype, y_dtype, param_dtype, x, gamma, beta, y, 0, mean, rstd, scratch,
                           kNoAllocScratchFloats * sizeof(float), stream);
}

extern "C" size_t sfh_groupnorm_bwd_workspace_bytes(const sfh_groupnorm_desc* p, int x_dtype) {
  if (check_desc(p, x_dtype) != SFH_OK) return 0;
  const GnPlan pl = make_plan(*p, x_dtype, true);
  return align_up(bwd_ws_floats(*p, pl) * sizeof(float), 256);
}

extern "C" int sfh_groupnorm_bwd(const sfh_groupnorm_desc* p, int x_dtype, int dy_dtype, int param_dtype, const void* dy,
                                 const void* x, const void* gamma, const void* beta, const float* mean, const float* rstd,
                                 void* dx, float* dgamma, float* dbeta, void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_desc(p, x_dtype)) return rc;
  if (!dtype_ok(dy_dtype) || !dtype_ok(param_dtype)) return fail(SFH_ERR_INVALID, "groupnorm: bad gradient/param dtype");
  if (dy_dtype != x_dtype && dy_dtype != SFH_FP32)
    return fail(SFH_ERR_UNSUPPORTED, "groupnorm bwd: the gradient must have the input's dtype or fp32");
  if (dy == nullptr || x == nullptr || dx == nullptr || mean == nullptr || rstd == nullptr)
    return fail(SFH_ERR_INVALID, "groupnorm: null tensor");
  const GnPlan pl = make_plan(*p, x_dtype, aligned16(x) && aligned16(dy) && aligned16(dx));
  const size_t need = bwd_ws_floats(*p, pl) * sizeof(float);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(SFH_ERR_WORKSPACE, "groupnorm bwd: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
  hipStream_t st = (hipStream_t)stream;
  float* ws = (float*)workspace;
#define SFH_GN_BWD(TX, TG) \
  return bwd_typed<TX, TG>(*p, pl, param_dtype, dy, x, gamma, beta, mean, rstd, dx, dgamma, dbeta, ws, st)
  if (x_dtype == SFH_BF16 && dy_dtype == SFH_BF16) SFH_GN_BWD(bf16_t, bf16_t);
  if (x_dtype == SFH_BF16) SFH_GN_BWD(bf16_t, float);
  if (x_dtype == SFH_FP16 && dy_dtype == SFH_FP16) SFH_GN_BWD(fp16_t, fp16_t);
  if (x_dtype == SFH_FP16) SFH_GN_BWD(fp16_t, float);
  SFH_GN_BWD(float, float);
#undef SFH_GN_BWD
}
