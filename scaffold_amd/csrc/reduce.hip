// Deterministic fp32 reductions: the sum over split-K partial slices, and per-channel sums of a
// channels-last tensor (the bias gradient, ScaFFold/unet/conv3d.py:1231,1786). No atomics: every
// partial has a fixed slot and every sum a fixed order, so a call gives the same bits every time.
#include "reduce.hpp"
#include "gn_stats.hpp"
#include "vec_io.hpp"

namespace sfh {
namespace {

constexpr int kBlock = 256;

template <typename T>
__device__ __forceinline__ void sum_slices_flat_body(unsigned block, const float* __restrict__ part, T* __restrict__ out, int64_t nelem,
                                                          int splits) {
  const int64_t e = (int64_t)block * kBlock + threadIdx.x;
  if (e >= nelem) return;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  int sp = 0;
  for (; sp + 3 < splits; sp += 4) {
    s0 += part[(int64_t)sp * nelem + e];
    s1 += part[(int64_t)(sp + 1) * nelem + e];
    s2 += part[(int64_t)(sp + 2) * nelem + e];
    s3 += part[(int64_t)(sp + 3) * nelem + e];
  }
  for (; sp < splits; ++sp) s0 += part[(int64_t)sp * nelem + e];
  out[e] = elem<T>::from_float((s0 + s1) + (s2 + s3));
}

// Many slices, few elements: 16 elements x 16 slice lanes per workgroup; lane l sums slices l, l+16, ...
// and the 16 lane totals are added in lane order.
template <typename T>
__device__ __forceinline__ void sum_slices_grouped_body(unsigned block, const float* __restrict__ part, T* __restrict__ out, int64_t nelem,
                                                             int splits) {
  __shared__ float buf[16][17];
  const int el = threadIdx.x & 15, sl = threadIdx.x >> 4;
  const int64_t e = (int64_t)block * 16 + el;
  float s = 0.f;
  if (e < nelem) {
    // eight loads in flight per thread; the additions keep the slice order
    int sp = sl;
    for (; sp + 7 * 16 < splits; sp += 8 * 16) {
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = part[(int64_t)(sp + 16 * k) * nelem + e];
#pragma unroll
      for (int k = 0; k < 8; ++k) s += v[k];
    }
    for (; sp < splits; sp += 16) s += part[(int64_t)sp * nelem + e];
  }
  buf[sl][el] = s;
  __syncthreads();
  if (sl == 0 && e < nelem) {
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) t += buf[i][el];
    out[e] = elem<T>::from_float(t);
  }
}

// The same with four consecutive elements per thread: a workgroup reads 256 contiguous bytes of each slice (whole
// cache lines) with 16-byte loads. 64 elements x 16 slice lanes per workgroup.
template <typename T>
__device__ __forceinline__ void sum_slices_grouped4_body(unsigned block, const float* __restrict__ part, T* __restrict__ out, int64_t nelem,
                                                              int splits) {
  __shared__ float4 buf[16][17];
  const int el = threadIdx.x & 15, sl = threadIdx.x >> 4;
  const int64_t e = ((int64_t)block * 16 + el) * 4;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  if (e < nelem) {
    int sp = sl;
    for (; sp + 7 * 16 < splits; sp += 8 * 16) {
      float4 v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = *reinterpret_cast<const float4*>(part + (int64_t)(sp + 16 * k) * nelem + e);
#pragma unroll
      for (int k = 0; k < 8; ++k) { s.x += v[k].x; s.y += v[k].y; s.z += v[k].z; s.w += v[k].w; }
    }
    for (; sp < splits; sp += 16) {
      const float4 v = *reinterpret_cast<const float4*>(part + (int64_t)sp * nelem + e);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
  }
  buf[sl][el] = s;
  __syncthreads();
  if (sl == 0 && e < nelem) {
    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < 16; ++i) { t.x += buf[i][el].x; t.y += buf[i][el].y; t.z += buf[i][el].z; t.w += buf[i][el].w; }
    out[e] = elem<T>::from_float(t.x);
    out[e + 1] = elem<T>::from_float(t.y);
    out[e + 2] = elem<T>::from_float(t.z);
    out[e + 3] = elem<T>::from_float(t.w);
  }
}

// A handful of elements under thousands of slices (the bias gradient an up-convolution's weight-gradient kernel leaves:
// 32 channels x 32 Ki slices): one workgroup per element, thread t sums slices t, t + 256, ... with eight loads in
// flight, then a fixed tree over the 256 thread totals. (With 16 slice lanes per element a lane walked 2048 slices:
// 12.7 us for 4 MB.)
template <typename T>
__device__ __forceinline__ void sum_slices_tall_body(unsigned block, const float* __restrict__ part, T* __restrict__ out, int64_t nelem, int splits) {
  __shared__ float buf[kBlock];
  const int tid = threadIdx.x;
  const int64_t e = block;
  float s = 0.f;
  int sp = tid;
  for (; sp + 7 * kBlock < splits; sp += 8 * kBlock) {
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = part[(int64_t)(sp + kBlock * k) * nelem + e];
#pragma unroll
    for (int k = 0; k < 8; ++k) s += v[k];
  }
  for (; sp < splits; sp += kBlock) s += part[(int64_t)sp * nelem + e];
  buf[tid] = s;
  __syncthreads();
  for (int stride = kBlock / 2; stride > 0; stride >>= 1) {
    if (tid < stride) buf[tid] += buf[tid + stride];
    __syncthreads();
  }
  if (tid == 0) out[e] = elem<T>::from_float(buf[0]);
}

// What launch_sum picks for a job: the kernel body and its number of workgroups.
enum SumKind { kSumNone = 0, kSumTall, kSumGrouped4, kSumGrouped, kSumFlat };
struct SumJob {
  const float* part;
  void* out;
  int64_t nelem;
  int splits, kind;
  unsigned blocks;
};

inline SumJob sum_job(const float* part, void* out, int64_t nelem, int splits) {
  SumJob j{part, out, nelem, splits, kSumNone, 0u};
  if (nelem <= 0) return j;
  if (nelem <= 64 && splits >= 2048) { j.kind = kSumTall; j.blocks = (unsigned)nelem; }
  else if (splits >= 32 && nelem <= (1 << 22) && nelem % 4 == 0 && nelem >= 64 * 128 && (reinterpret_cast<uintptr_t>(part) & 15) == 0) {
    j.kind = kSumGrouped4; j.blocks = (unsigned)cdiv(nelem, 64);
  } else if (splits >= 32 && nelem <= (1 << 22)) { j.kind = kSumGrouped; j.blocks = (unsigned)cdiv(nelem, 16); }
  else { j.kind = kSumFlat; j.blocks = (unsigned)cdiv(nelem, kBlock); }
  return j;
}

template <typename T>
__device__ __forceinline__ void sum_job_body(const SumJob& j, unsigned block) {
  switch (j.kind) {
    case kSumTall: sum_slices_tall_body<T>(block, j.part, (T*)j.out, j.nelem, j.splits); break;
    case kSumGrouped4: sum_slices_grouped4_body<T>(block, j.part, (T*)j.out, j.nelem, j.splits); break;
    case kSumGrouped: sum_slices_grouped_body<T>(block, j.part, (T*)j.out, j.nelem, j.splits); break;
    default: sum_slices_flat_body<T>(block, j.part, (T*)j.out, j.nelem, j.splits); break;
  }
}

template <typename T>
__global__ void __launch_bounds__(kBlock) sum_slices_flat(const float* __restrict__ part, T* __restrict__ out, int64_t nelem, int splits) {
  sum_slices_flat_body<T>(blockIdx.x, part, out, nelem, splits);
}
template <typename T>
__global__ void __launch_bounds__(kBlock) sum_slices_grouped(const float* __restrict__ part, T* __restrict__ out, int64_t nelem, int splits) {
  sum_slices_grouped_body<T>(blockIdx.x, part, out, nelem, splits);
}
template <typename T>
__global__ void __launch_bounds__(kBlock) sum_slices_grouped4(const float* __restrict__ part, T* __restrict__ out, int64_t nelem, int splits) {
  sum_slices_grouped4_body<T>(blockIdx.x, part, out, nelem, splits);
}
template <typename T>
__global__ void __launch_bounds__(kBlock) sum_slices_tall(const float* __restrict__ part, T* __restrict__ out, int64_t nelem, int splits) {
  sum_slices_tall_body<T>(blockIdx.x, part, out, nelem, splits);
}
// Two sums in one launch (a weight gradient's slices and its bias gradient's): the first a.blocks workgroups run job a,
// the rest job b, each exactly as a launch of its own would.
template <typename T>
__global__ void __launch_bounds__(kBlock) sum_slices_two(SumJob a, SumJob b) {
  if (blockIdx.x < a.blocks) sum_job_body<T>(a, blockIdx.x);
  else sum_job_body<T>(b, blockIdx.x - a.blocks);
}

template <typename T>
int launch_sum(const float* part, void* out, int64_t nelem, int splits, hipStream_t st) {
  if (nelem <= 0) return SFH_OK;
  if (nelem <= 64 && splits >= 2048) {
    hipLaunchKernelGGL(sum_slices_tall<T>, dim3((unsigned)nelem), dim3(kBlock), 0, st, part, (T*)out, nelem, splits);
    return check_launch("sum_slices_tall");
  }
  if (splits >= 32 && nelem <= (1 << 22) && nelem % 4 == 0 && nelem >= 64 * 128 && (reinterpret_cast<uintptr_t>(part) & 15) == 0) {
    hipLaunchKernelGGL(sum_slices_grouped4<T>, dim3((unsigned)cdiv(nelem, 64)), dim3(kBlock), 0, st, part, (T*)out, nelem, splits);
    return check_launch("sum_slices_grouped4");
  }
  if (splits >= 32 && nelem <= (1 << 22)) {
    hipLaunchKernelGGL(sum_slices_grouped<T>, dim3((unsigned)cdiv(nelem, 16)), dim3(kBlock), 0, st, part, (T*)out, nelem, splits);
    return check_launch("sum_slices_grouped");
  }
  hipLaunchKernelGGL(sum_slices_flat<T>, dim3((unsigned)cdiv(nelem, kBlock)), dim3(kBlock), 0, st, part, (T*)out, nelem, splits);
  return check_launch("sum_slices_flat");
}

// Four consecutive elements per thread (16-byte loads of every slice), bias added before the one rounding.
// A non-null out1 splits the result along the channels: the first c_first of every row of `channels` go to `out`, the
// rest to out1 (both dense; c_first a multiple of 4, so a thread's four channels stay together).
template <typename T>
__global__ void __launch_bounds__(kBlock) sum_slices_bias_kernel(const float* __restrict__ part, const T* __restrict__ bias,
                                                                 T* __restrict__ out, int64_t nelem, int channels, int splits,
                                                                 T* __restrict__ out1, int c_first) {
  const int64_t e = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * 4;
  if (e >= nelem) return;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  // the slices in their order, eight, four or two loads in flight (one slice per trip to memory made the sum of eight
  // slices eight trips long)
  int sp = 0;
  for (; sp + 7 < splits; sp += 8) {
    float4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = *reinterpret_cast<const float4*>(part + (int64_t)(sp + k) * nelem + e);
#pragma unroll
    for (int k = 0; k < 8; ++k) { s.x += v[k].x; s.y += v[k].y; s.z += v[k].z; s.w += v[k].w; }
  }
  for (; sp + 3 < splits; sp += 4) {
    float4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = *reinterpret_cast<const float4*>(part + (int64_t)(sp + k) * nelem + e);
#pragma unroll
    for (int k = 0; k < 4; ++k) { s.x += v[k].x; s.y += v[k].y; s.z += v[k].z; s.w += v[k].w; }
  }
  for (; sp + 1 < splits; sp += 2) {
    const float4 v0 = *reinterpret_cast<const float4*>(part + (int64_t)sp * nelem + e);
    const float4 v1 = *reinterpret_cast<const float4*>(part + (int64_t)(sp + 1) * nelem + e);
    s.x += v0.x; s.y += v0.y; s.z += v0.z; s.w += v0.w;
    s.x += v1.x; s.y += v1.y; s.z += v1.z; s.w += v1.w;
  }
  for (; sp < splits; ++sp) {
    const float4 v = *reinterpret_cast<const float4*>(part + (int64_t)sp * nelem + e);
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  if (bias != nullptr) {
    const int c = (int)(e % channels);
    s.x += to_float(bias[c]); s.y += to_float(bias[c + 1]); s.z += to_float(bias[c + 2]); s.w += to_float(bias[c + 3]);
  }
  T* o = out + e;
  if (out1 != nullptr) {
    const int64_t row = e / channels;
    const int c = (int)(e - row * channels);
    o = c >= c_first ? out1 + row * (channels - c_first) + (c - c_first) : out + row * c_first + c;
  }
  o[0] = elem<T>::from_float(s.x);
  o[1] = elem<T>::from_float(s.y);
  o[2] = elem<T>::from_float(s.z);
  o[3] = elem<T>::from_float(s.w);
}

// Four consecutive 16-bit elements (8-byte aligned) as one store.
template <typename T>
__device__ __forceinline__ void store4(T* p, T a, T b, T c, T d) {
  static_assert(sizeof(T) == 2, "16-bit elements");
  const uint32_t lo = (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
  const uint32_t hi = (uint32_t)__builtin_bit_cast(uint16_t, c) | ((uint32_t)__builtin_bit_cast(uint16_t, d) << 16);
  *reinterpret_cast<uint2*>(p) = make_uint2(lo, hi);
}

// sum_slices_bias that also leaves GroupNorm records of the rounded result (16-bit outputs, layout and merge rule in
// gn_stats.hpp): a workgroup owns `chunks` consecutive pieces of 1024 elements of one sample; 1024 is a multiple of the
// channel count, so a thread's four consecutive channels are the same in every piece and belong to one group. A thread
// sums about its own first rounded value; the threads of a group are merged in thread order. One record per workgroup.
constexpr int kStatsPiece = 4 * kBlock;

template <typename T>
__global__ void __launch_bounds__(kBlock) sum_slices_bias_stats_kernel(const float* __restrict__ part, const T* __restrict__ bias,
                                                                       T* __restrict__ out, int64_t sample_elems, int64_t nelem,
                                                                       int channels, int splits, int chunks, GnPartialOut gn,
                                                                       int whole_store) {
  __shared__ float4 sums[kBlock];  // { values, sum, sum of squares, shift } of every thread
  const int tid = threadIdx.x, n = blockIdx.y;
  const int c = (tid * 4) % channels;
  float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
  if (bias != nullptr) { b0 = to_float(bias[c]); b1 = to_float(bias[c + 1]); b2 = to_float(bias[c + 2]); b3 = to_float(bias[c + 3]); }
  float shift = 0.f, s1 = 0.f, s2 = 0.f, cnt = 0.f;
  for (int k = 0; k < chunks; ++k) {
    const int64_t local = ((int64_t)blockIdx.x * chunks + k) * kStatsPiece + tid * 4;
    if (local >= sample_elems) break;
    const int64_t e = (int64_t)n * sample_elems + local;
    // the first eight slices' loads are in flight together (the reduction channels are cut into at most eight); the
    // sum keeps the slice order
    constexpr int kInFlight = 8;
    float4 v[kInFlight];
#pragma unroll
    for (int sp = 0; sp < kInFlight; ++sp)
      v[sp] = sp < splits ? *reinterpret_cast<const float4*>(part + (int64_t)sp * nelem + e) : make_float4(0.f, 0.f, 0.f, 0.f);
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int sp = 0; sp < kInFlight; ++sp) {
      if (sp < splits) { s.x += v[sp].x; s.y += v[sp].y; s.z += v[sp].z; s.w += v[sp].w; }
    }
    for (int sp = kInFlight; sp < splits; ++sp) {
      const float4 w = *reinterpret_cast<const float4*>(part + (int64_t)sp * nelem + e);
      s.x += w.x; s.y += w.y; s.z += w.z; s.w += w.w;
    }
    const T o0 = elem<T>::from_float(s.x + b0), o1 = elem<T>::from_float(s.y + b1), o2 = elem<T>::from_float(s.z + b2),
            o3 = elem<T>::from_float(s.w + b3);
    if (whole_store) store4(out + e, o0, o1, o2, o3);
    else { out[e] = o0; out[e + 1] = o1; out[e + 2] = o2; out[e + 3] = o3; }
    if (k == 0) shift = to_float(o0);
    const float r0 = to_float(o0) - shift, r1 = to_float(o1) - shift, r2 = to_float(o2) - shift, r3 = to_float(o3) - shift;
    s1 += (r0 + r1) + (r2 + r3);
    s2 += fmaf(r0, r0, r1 * r1) + fmaf(r2, r2, r3 * r3);
    cnt += 4.f;
  }
  // Every thread turns its sums into (count, mean, M2); then the 256 / groups threads' pieces of each group (kStatsPiece is
  // a multiple of the channel count and a group a multiple of four channels, so that many there are) are merged about the
  // mean of the group's first piece -- count, sum of n d and sum of M2 + n d^2 are plain sums, taken by a fixed tree over
  // LDS. (One thread per group walking its 32 pieces in turn, a division each, took 4 of this kernel's 9 us.)
  float pm = 0.f, pm2 = 0.f;
  if (cnt > 0.f) {
    const float dm = s1 / cnt;
    pm = shift + dm;
    pm2 = fmaf(-s1, dm, s2);
    pm2 = pm2 < 0.f ? 0.f : pm2;
  }
  sums[tid] = make_float4(cnt, pm, pm2, 0.f);
  __syncthreads();
  const int per_row = channels / 4, per_group = gn.cg / 4;
  const int epg = kBlock / gn.groups;  // pieces per group
  const int g = tid / epg, l = tid - g * epg;
  const int v = l / per_group, r = l - v * per_group;
  const float4 e = sums[v * per_row + g * per_group + r];
  // the group's first piece belongs to the lowest thread of the group: when it is empty (past the end of the sample) all are
  const float about = sums[g * per_group].y;
  const float d = e.y - about;
  __syncthreads();
  sums[tid] = make_float4(e.x, e.x * d, fmaf(e.x * d, d, e.z), 0.f);
  __syncthreads();
  for (int stride = epg >> 1; stride > 0; stride >>= 1) {
    if (l < stride) {
      const float4 a = sums[tid], b = sums[tid + stride];
      sums[tid] = make_float4(a.x + b.x, a.y + b.y, a.z + b.z, 0.f);
    }
    __syncthreads();
  }
  if (l == 0) {
    const float4 t = sums[tid];
    float mean = 0.f, m2 = 0.f;
    if (t.x > 0.f) {
      mean = about + t.y / t.x;
      m2 = fmaf(-t.y, t.y / t.x, t.z);
      m2 = m2 < 0.f ? 0.f : m2;
    }
    *reinterpret_cast<float4*>(gn.part + (((int64_t)n * gn.records + blockIdx.x) * gn.groups + g) * kGnRecordFloats) =
        make_float4(t.x, mean, m2, 0.f);
  }
}

// Per-channel partial sums: thread = (row slot, channel); a workgroup walks its row range with rpp rows per
// pass (consecutive threads read consecutive elements), folds the row slots through LDS and writes
// part[block][channel chunk]. Channel chunks of at most 256 lie along grid.y.
template <typename T>
__global__ void __launch_bounds__(kBlock) channel_partial(const T* __restrict__ g, float* __restrict__ part, int64_t rows, int C,
                                                          int64_t rows_per_block) {
  __shared__ float buf[kBlock];
  const int c0 = blockIdx.y * kBlock;
  const int cw = (C - c0) < kBlock ? (C - c0) : kBlock;
  const int rpp = kBlock / cw;
  const int tid = threadIdx.x;
  const int r = tid / cw, c = tid - r * cw;
  const int64_t begin = (int64_t)blockIdx.x * rows_per_block;
  int64_t end = begin + rows_per_block;
  if (end > rows) end = rows;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (r < rpp) {
    const T* p = g + c0 + c;
    int64_t row = begin + r;
    for (; row + 3 * (int64_t)rpp < end; row += 4 * (int64_t)rpp) {
      s0 += to_float(p[row * C]);
      s1 += to_float(p[(row + rpp) * C]);
      s2 += to_float(p[(row + 2 * rpp) * C]);
      s3 += to_float(p[(row + 3 * rpp) * C]);
    }
    for (; row < end; row += rpp) s0 += to_float(p[row * C]);
  }
  buf[tid] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (tid < cw) {
    float t = 0.f;
    for (int i = 0; i < rpp; ++i) t += buf[i * cw + tid];
    part[(int64_t)blockIdx.x * C + c0 + tid] = t;
  }
}

// The same sums with 16-byte loads: thread = (row slot, vector of V channels), C a multiple of V, C / V <= 256.
template <typename T>
__global__ void __launch_bounds__(kBlock) channel_partial_vec(const T* __restrict__ g, float* __restrict__ part, int64_t rows, int C,
                                                              int64_t rows_per_block) {
  constexpr int V = VecOf<T>::N;
  extern __shared__ float vbuf[];  // V * kBlock
  const int tpr = C / V;
  const int rpp = kBlock / tpr;
  const int tid = threadIdx.x;
  const int r = tid / tpr, cv = tid - r * tpr;
  const int64_t begin = (int64_t)blockIdx.x * rows_per_block;
  int64_t end = begin + rows_per_block;
  if (end > rows) end = rows;
  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = 0.f;
  if (r < rpp) {
    const T* p = g + cv * V;
    int64_t row = begin + r;
    for (; row + 3 * (int64_t)rpp < end; row += 4 * (int64_t)rpp) {
      float f0[V], f1[V], f2[V], f3[V];
      Ld<T, V>::run(p + row * C, f0);
      Ld<T, V>::run(p + (row + rpp) * C, f1);
      Ld<T, V>::run(p + (row + 2 * rpp) * C, f2);
      Ld<T, V>::run(p + (row + 3 * rpp) * C, f3);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += (f0[e] + f1[e]) + (f2[e] + f3[e]);
    }
    for (; row < end; row += rpp) {
      float f0[V];
      Ld<T, V>::run(p + row * C, f0);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += f0[e];
    }
  }
#pragma unroll
  for (int e = 0; e < V; ++e) vbuf[e * kBlock + tid] = r < rpp ? acc[e] : 0.f;
  __syncthreads();
  for (int c = tid; c < C; c += kBlock) {
    const int v = c / V, e = c - v * V;
    float t = 0.f;
    for (int i = 0; i < rpp; ++i) t += vbuf[e * kBlock + i * tpr + v];
    part[(int64_t)blockIdx.x * C + c] = t;
  }
}

template <typename T>
bool bias_vector_form(const void* g, int C) {
  constexpr int V = VecOf<T>::N;
  return C % V == 0 && C / V <= kBlock && (reinterpret_cast<uintptr_t>(g) & 15) == 0;
}

// Workgroups of the partial pass: at most 1024, each at least one pass of rows (a pass is 4 KiB in the vector form).
int bias_blocks(int64_t rows, int C) {
  int64_t per = cdiv(rows, 1024);
  const int64_t pass = C >= 8 && C <= 2048 ? (2048 / C < 1 ? 1 : 2048 / C) : 1;
  if (per < pass) per = pass;
  const int64_t n = cdiv(rows, per);
  return (int)(n < 1 ? 1 : n);
}

template <typename T>
int launch_bias(const void* g, int64_t rows, int C, float* ws, hipStream_t st) {
  const int nblk = bias_blocks(rows, C);
  const int64_t per = cdiv(rows, nblk);
  if (bias_vector_form<T>(g, C)) {
    hipLaunchKernelGGL(channel_partial_vec<T>, dim3((unsigned)nblk), dim3(kBlock), VecOf<T>::N * kBlock * sizeof(float), st,
                       (const T*)g, ws, rows, C, per);
    return check_launch("channel_partial_vec");
  }
  hipLaunchKernelGGL(channel_partial<T>, dim3((unsigned)nblk, (unsigned)cdiv(C, kBlock)), dim3(kBlock), 0, st, (const T*)g, ws, rows, C,
                     per);
  return check_launch("channel_partial");
}

}  // namespace

int sum_slices(int dtype, const float* part, void* out, int64_t nelem, int splits, hipStream_t st);

template <typename T>
int launch_sum_two(const SumJob& a, const SumJob& b, hipStream_t st) {
  hipLaunchKernelGGL(sum_slices_two<T>, dim3(a.blocks + b.blocks), dim3(kBlock), 0, st, a, b);
  return check_launch("sum_slices_two");
}

int sum_slices_two(int dtype, const float* part_a, void* out_a, int64_t nelem_a, int splits_a, const float* part_b, void* out_b,
                   int64_t nelem_b, int splits_b, hipStream_t st) {
  const SumJob a = sum_job(part_a, out_a, nelem_a, splits_a), b = sum_job(part_b, out_b, nelem_b, splits_b);
  if (a.kind == kSumNone || b.kind == kSumNone || (uint64_t)a.blocks + b.blocks > 0x7fffffffu) {
    if (int rc = sum_slices(dtype, part_a, out_a, nelem_a, splits_a, st)) return rc;
    return sum_slices(dtype, part_b, out_b, nelem_b, splits_b, st);
  }
  switch (dtype) {
    case SFH_BF16: return launch_sum_two<bf16_t>(a, b, st);
    case SFH_FP16: return launch_sum_two<fp16_t>(a, b, st);
    default: return launch_sum_two<float>(a, b, st);
  }
}

int sum_slices(int dtype, const float* part, void* out, int64_t nelem, int splits, hipStream_t st) {
  switch (dtype) {
    case SFH_BF16: return launch_sum<bf16_t>(part, out, nelem, splits, st);
    case SFH_FP16: return launch_sum<fp16_t>(part, out, nelem, splits, st);
    default: return launch_sum<float>(part, out, nelem, splits, st);
  }
}

int sum_slices_bias(int dtype, const float* part, const void* bias, void* out, int64_t nelem, int channels, int splits,
                    hipStream_t st, const ChannelPair* out2) {
  void* out1 = out2 != nullptr ? out2->second : nullptr;
  const int c_first = out2 != nullptr ? out2->first : 0;
  if (nelem <= 0) return SFH_OK;
  const dim3 grid((unsigned)cdiv(nelem / 4, kBlock));
  if (dtype == SFH_BF16)
    hipLaunchKernelGGL(sum_slices_bias_kernel<bf16_t>, grid, dim3(kBlock), 0, st, part, (const bf16_t*)bias, (bf16_t*)out, nelem,
                       channels, splits, (bf16_t*)out1, c_first);
  else if (dtype == SFH_FP16)
    hipLaunchKernelGGL(sum_slices_bias_kernel<fp16_t>, grid, dim3(kBlock), 0, st, part, (const fp16_t*)bias, (fp16_t*)out, nelem,
                       channels, splits, (fp16_t*)out1, c_first);
  else
    hipLaunchKernelGGL(sum_slices_bias_kernel<float>, grid, dim3(kBlock), 0, st, part, (const float*)bias, (float*)out, nelem,
                       channels, splits, (float*)out1, c_first);
  return check_launch("sum_slices_bias_kernel");
}

int sum_slices_bias_stats_records(int64_t sample_elems, int channels, int groups) {
  if (channels < 4 || kStatsPiece % channels != 0 || sample_elems % 4 != 0 || groups < 1 || channels % groups != 0 ||
      (channels / groups) % 4 != 0)
    return 0;
  const int64_t pieces = cdiv(sample_elems, kStatsPiece);
  const int64_t chunks = cdiv(pieces, 512);
  return (int)cdiv(pieces, chunks);
}

int sum_slices_bias_stats(int dtype, const float* part, const void* bias, void* out, int n, int64_t sample_elems, int channels,
                          int splits, const GnPartialOut& gn, hipStream_t st) {
  if (n <= 0 || sample_elems <= 0) return SFH_OK;
  const int records = sum_slices_bias_stats_records(sample_elems, channels, gn.groups);
  if (records == 0 || records != gn.records || (dtype != SFH_BF16 && dtype != SFH_FP16))
    return fail(SFH_ERR_UNSUPPORTED, "sum of slices with GroupNorm partials: not offered for this shape");
  const int chunks = (int)cdiv(cdiv(sample_elems, kStatsPiece), records);
  const dim3 grid((unsigned)records, (unsigned)n);
  const int whole_store = (reinterpret_cast<uintptr_t>(out) & 7u) == 0 ? 1 : 0;  // a thread's four outputs as one 8-byte store
  if (dtype == SFH_BF16)
    hipLaunchKernelGGL(sum_slices_bias_stats_kernel<bf16_t>, grid, dim3(kBlock), 0, st, part, (const bf16_t*)bias, (bf16_t*)out,
                       sample_elems, (int64_t)n * sample_elems, channels, splits, chunks, gn, whole_store);
  else
    hipLaunchKernelGGL(sum_slices_bias_stats_kernel<fp16_t>, grid, dim3(kBlock), 0, st, part, (const fp16_t*)bias, (fp16_t*)out,
                       sample_elems, (int64_t)n * sample_elems, channels, splits, chunks, gn, whole_store);
  return check_launch("sum_slices_bias_stats_kernel");
}

size_t bias_grad_workspace_bytes(int64_t rows, int channels) {
  return (size_t)bias_blocks(rows, channels) * channels * sizeof(float);
}

int bias_grad(int dtype, int out_dtype, const void* g, int64_t rows, int channels, void* gb, void* ws, hipStream_t st) {
  int rc;
  switch (dtype) {
    case SFH_BF16: rc = launch_bias<bf16_t>(g, rows, channels, (float*)ws, st); break;
    case SFH_FP16: rc = launch_bias<fp16_t>(g, rows, channels, (float*)ws, st); break;
    default: rc = launch_bias<float>(g, rows, channels, (float*)ws, st); break;
  }
  if (rc != SFH_OK) return rc;
  return sum_slices(out_dtype, (const float*)ws, gb, channels, bias_blocks(rows, channels), st);
}

}  // namespace sfh
