// Convolutions with a THIN side: one of the two channel counts is too small for MFMA tiles
// (the U-Net's Cin=1 3x3x3 stem and its 1x1x1 head to 11 classes). They are HBM-bound: every
// kernel streams the wide tensor once with 16-byte accesses and keeps the thin side in
// registers / LDS; arithmetic is fp32 FMA on the vector ALU.
//
// One formulation serves all of them. Over the voxels v of an iterated volume,
//   s_j(v), j < J : the thin values of the voxel -- either the K^3 taps of a one-channel tensor
//                   sampled at v*stride + tap*dilation - padding (zero outside), or the J channels
//                   of a thin tensor at v itself (1x1x1, stride 1, no padding);
//   wide-out  : out[v][c] = bias[c] + sum_j s_j(v) * W[j][c]           (stem forward, head dgrad)
//   thin-out  : out[v][j] = bias[j] + sum_c wide[v][c] * W[j][c]        (head forward)
//   reduce    : G[j][c]   = sum_v s_j(v) * wide[v][c]                   (stem wgrad, head wgrad)
// The reference serves these shapes with the same implicit-GEMM kernels at small tile sizes
// (triton_conv3d/gather_gemm.py:493-560, reduce_gemm.py:655-700).
#include "conv_thin.hpp"
#include <type_traits>
#include "mma.hpp"
#include "reduce.hpp"
#include "vec_io.hpp"

namespace sfh {

namespace {

constexpr int kBlock = 256;

// Thin sample j of iterated voxel (nn, d, h, w). K > 0: tap j of a one-channel tensor; K == 0: channel j.
template <typename T, int K>
__device__ __forceinline__ float thin_sample(const ThinArgs& a, const T* __restrict__ thin, int j, int nn, int d, int h, int w,
                                             int64_t v) {
  if constexpr (K == 0) {
    return j < a.J ? to_float(thin[v * a.ct + j]) : 0.f;
  } else {
    const int kd = j / (K * K), kh = (j / K) % K, kw = j % K;
    const int iz = d * a.sd - a.pd + kd * a.dd;
    const int iy = h * a.sh - a.ph + kh * a.dh;
    const int ix = w * a.sw - a.pw + kw * a.dw;
    const bool ok = (unsigned)iz < (unsigned)a.td && (unsigned)iy < (unsigned)a.th && (unsigned)ix < (unsigned)a.tw;
    const int64_t off = (((int64_t)nn * a.td + iz) * a.th + iy) * a.tw + ix;
    return ok ? to_float(thin[off]) : 0.f;
  }
}

// Voxel coordinates of a linear index; only the tap form needs them. 32-bit arithmetic when it fits.
template <int K>
__device__ __forceinline__ void decode_voxel(const ThinArgs& a, int64_t v, int& nn, int& d, int& h, int& w) {
  nn = d = h = w = 0;
  if constexpr (K != 0) {
    if (v <= 0x7fffffffLL) {
      uint32_t t = (uint32_t)v;
      w = (int)(t % (uint32_t)a.ow); t /= (uint32_t)a.ow;
      h = (int)(t % (uint32_t)a.oh); t /= (uint32_t)a.oh;
      d = (int)(t % (uint32_t)a.od);
      nn = (int)(t / (uint32_t)a.od);
    } else {
      w = (int)(v % a.ow);
      int64_t t = v / a.ow;
      h = (int)(t % a.oh);
      t /= a.oh;
      d = (int)(t % a.od);
      nn = (int)(t / a.od);
    }
  }
}

// ---- wide-out ------------------------------------------------------------------------------
// Thread = (voxel, V consecutive wide channels). W[j][c] sits in LDS as fp32.
template <typename T, int K, int J>
__global__ void __launch_bounds__(kBlock) thin_wide_out_kernel(ThinArgs a, const T* __restrict__ thin, const T* __restrict__ wt,
                                                               const T* __restrict__ bias, T* __restrict__ out, int64_t total) {
  constexpr int V = VecOf<T>::N;
  extern __shared__ float wl[];  // [J][cw]
  const int tid = threadIdx.x;
  for (int i = tid; i < J * a.cw; i += kBlock) {
    const int j = i / a.cw, c = i - j * a.cw;
    float val = 0.f;
    if (j < a.J) {
      int64_t off = (int64_t)c * a.ws_wide;
      if constexpr (K == 0) off += (int64_t)j * a.ws_thin;
      else off += (j / (K * K)) * a.ws_kd + ((j / K) % K) * a.ws_kh + (j % K) * a.ws_kw;
      val = to_float(wt[off]);
    }
    wl[i] = val;
  }
  __syncthreads();
  const int wq = a.cw / V, rpp = kBlock / wq;
  const int r = tid / wq, q = tid - r * wq;
  if (r >= rpp) return;
  float b[V];
#pragma unroll
  for (int e = 0; e < V; ++e) b[e] = bias != nullptr ? to_float(bias[q * V + e]) : 0.f;
  for (int64_t v = (int64_t)blockIdx.x * rpp + r; v < total; v += (int64_t)gridDim.x * rpp) {
    int nn, d, h, w;
    decode_voxel<K>(a, v, nn, d, h, w);
    float s[J];
#pragma unroll
    for (int j = 0; j < J; ++j) s[j] = thin_sample<T, K>(a, thin, j, nn, d, h, w, v);
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = b[e];
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const float* wr = wl + j * a.cw + q * V;
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = fmaf(s[j], wr[e], acc[e]);
    }
    St<T, V>::run(out + v * a.cw + q * V, acc);
  }
}

// ---- thin-out ------------------------------------------------------------------------------
// Thread = voxel: reads its cw wide channels in 16-byte pieces, produces the J thin outputs.
template <typename T, int J>
__global__ void __launch_bounds__(kBlock) thin_out_kernel(ThinArgs a, const T* __restrict__ wide, const T* __restrict__ wt,
                                                          const T* __restrict__ bias, T* __restrict__ out, int64_t total) {
  constexpr int V = VecOf<T>::N;
  extern __shared__ float wl[];  // [J][cw]
  const int tid = threadIdx.x;
  for (int i = tid; i < J * a.cw; i += kBlock) {
    const int j = i / a.cw, c = i - j * a.cw;
    wl[i] = j < a.J ? to_float(wt[(int64_t)c * a.ws_wide + (int64_t)j * a.ws_thin]) : 0.f;
  }
  __syncthreads();
  for (int64_t v = (int64_t)blockIdx.x * kBlock + tid; v < total; v += (int64_t)gridDim.x * kBlock) {
    float acc[J];
#pragma unroll
    for (int j = 0; j < J; ++j) acc[j] = (bias != nullptr && j < a.J) ? to_float(bias[j]) : 0.f;
    const T* xs = wide + v * a.cw;
    for (int c0 = 0; c0 < a.cw; c0 += V) {
      float f[V];
      Ld<T, V>::run(xs + c0, f);
#pragma unroll
      for (int j = 0; j < J; ++j) {
        const float* wr = wl + j * a.cw + c0;
#pragma unroll
        for (int e = 0; e < V; ++e) acc[j] = fmaf(f[e], wr[e], acc[j]);
      }
    }
    T* o = out + v * a.J;
#pragma unroll
    for (int j = 0; j < J; ++j)
      if (j < a.J) o[j] = elem<T>::from_float(acc[j]);
  }
}

// ---- pointwise head on the matrix cores -----------------------------------------------------------
// 16-bit types, K == 0 and a wide side of 32, 64 or 128 channels. A workgroup owns 128 consecutive voxels per
// round, a wavefront 32 of them; the thin side (at most 32 channels, e.g. the 11 classes) is zero-padded to one
// MFMA tile. The thin rows of a round are one contiguous byte range of the thin tensor, which moves between
// global memory and LDS in 16-byte pieces whatever the channel count.
constexpr int kHeadVoxels = 128;
constexpr int kHeadThinMax = 32;

// 8 consecutive wide channels from c0 of thin channel j (zero at and beyond J) as a packed MFMA operand piece.
template <typename T>
__device__ __forceinline__ uint4 head_weight_wide_run(const ThinArgs& a, const T* __restrict__ wt, int j, int c0) {
  uint16_t h[8];
#pragma unroll
  for (int e = 0; e < 8; ++e)
    h[e] = reinterpret_cast<const uint16_t*>(wt)[(int64_t)(c0 + e) * a.ws_wide + (int64_t)(j < a.J ? j : 0) * a.ws_thin];
  if (j >= a.J)
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = 0;
  return make_uint4(h[0] | (uint32_t)h[1] << 16, h[2] | (uint32_t)h[3] << 16, h[4] | (uint32_t)h[5] << 16, h[6] | (uint32_t)h[7] << 16);
}
// 8 consecutive thin channels from j0 of wide channel c.
template <typename T>
__device__ __forceinline__ uint4 head_weight_thin_run(const ThinArgs& a, const T* __restrict__ wt, int c, int j0) {
  uint16_t h[8];
#pragma unroll
  for (int e = 0; e < 8; ++e)
  {
    const int j = j0 + e < a.J ? j0 + e : 0;
    const uint16_t bits = reinterpret_cast<const uint16_t*>(wt)[(int64_t)c * a.ws_wide + (int64_t)j * a.ws_thin];
    h[e] = j0 + e < a.J ? bits : (uint16_t)0;
  }
  return make_uint4(h[0] | (uint32_t)h[1] << 16, h[2] | (uint32_t)h[3] << 16, h[4] | (uint32_t)h[5] << 16, h[6] | (uint32_t)h[7] << 16);
}

// thin-out: out[v][j] = bias[j] + sum_c wide[v][c] * W[j][c]. Result tile: rows = thin channels, columns = voxels.
template <typename T, int NC>
__global__ void __launch_bounds__(kBlock) head_thin_out_kernel(ThinArgs a, const T* __restrict__ wide, const T* __restrict__ wt,
                                                               const T* __restrict__ bias, T* __restrict__ out, int64_t total) {
  __shared__ __align__(16) T rows[kHeadVoxels * kHeadThinMax];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, kg = lane >> 5;
  const int J = a.J;
  uint4 wf[NC][2];
#pragma unroll
  for (int cc = 0; cc < NC; ++cc)
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) wf[cc][ks] = head_weight_wide_run<T>(a, wt, col, cc * 32 + ks * 16 + kg * 8);
  float bv[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int j = 8 * (r / 4) + 4 * kg + r % 4;
    const float b = bias != nullptr ? to_float(bias[j < J ? j : 0]) : 0.f;
    bv[r] = j < J ? b : 0.f;
  }
  for (int64_t base = (int64_t)blockIdx.x * kHeadVoxels; base < total; base += (int64_t)gridDim.x * kHeadVoxels) {
    const int64_t v = base + wave * 32 + col;
    const T* src = wide + (v < total ? v : total - 1) * a.cw + kg * 8;
    uint4 xf[NC][2];
#pragma unroll
    for (int cc = 0; cc < NC; ++cc)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) xf[cc][ks] = load16(src + cc * 32 + ks * 16);
    f32x16_t acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int cc = 0; cc < NC; ++cc)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) acc = Mma32<T>::run(wf[cc][ks], xf[cc][ks], acc);
    T* mine = rows + (wave * 32 + col) * J;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = 8 * (r / 4) + 4 * kg + r % 4;
      if (j < J) mine[j] = elem<T>::from_float(acc[r] + bv[r]);
    }
    __syncthreads();
    const int64_t left = total - base;
    const int nv = left < kHeadVoxels ? (int)left : kHeadVoxels;
    const int nelem = nv * J, npiece = nelem / 8;
    T* dst = out + base * J;
    for (int i = tid; i < npiece; i += kBlock) reinterpret_cast<uint4*>(dst)[i] = reinterpret_cast<const uint4*>(rows)[i];
    for (int i = npiece * 8 + tid; i < nelem; i += kBlock) dst[i] = rows[i];
    __syncthreads();
  }
}

// wide-out: out[v][c] = bias[c] + sum_j thin[v][j] * W[j][c]. Result tile: rows = wide channels, columns = voxels.
// NK = MFMA steps of 16 thin channels.
template <typename T, int NC, int NK>
__global__ void __launch_bounds__(kBlock) head_wide_out_kernel(ThinArgs a, const T* __restrict__ thin, const T* __restrict__ wt,
                                                               const T* __restrict__ bias, T* __restrict__ out, int64_t total) {
  // one row of slack: the operand read of the last voxel runs up to 16 * NK channels
  __shared__ __align__(16) uint16_t rows[(kHeadVoxels + 1) * kHeadThinMax];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, kg = lane >> 5;
  const int J = a.J;
  uint4 wf[NC][NK];
#pragma unroll
  for (int cc = 0; cc < NC; ++cc)
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) wf[cc][ks] = head_weight_thin_run<T>(a, wt, cc * 32 + col, ks * 16 + kg * 8);
  float bv[NC][16];
#pragma unroll
  for (int cc = 0; cc < NC; ++cc) load_block_bias<T>(bias, cc * 32, kg, bv[cc]);
  for (int64_t base = (int64_t)blockIdx.x * kHeadVoxels; base < total; base += (int64_t)gridDim.x * kHeadVoxels) {
    const int64_t left = total - base;
    const int nv = left < kHeadVoxels ? (int)left : kHeadVoxels;
    const int nelem = nv * J, npiece = nelem / 8;
    const uint16_t* src = reinterpret_cast<const uint16_t*>(thin) + base * J;
    for (int i = tid; i < npiece; i += kBlock) reinterpret_cast<uint4*>(rows)[i] = reinterpret_cast<const uint4*>(src)[i];
    for (int i = npiece * 8 + tid; i < nelem; i += kBlock) rows[i] = src[i];
    __syncthreads();
    const int lv = wave * 32 + col;
    const bool valid = lv < nv;
    const uint16_t* mine = rows + (valid ? lv : 0) * J;
    uint4 xf[NK];
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      uint32_t h[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = ks * 16 + kg * 8 + e;
        const uint32_t bits = mine[j];
        h[e] = j < J ? bits : 0u;
      }
      xf[ks] = make_uint4(h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16);
    }
    T* dst = out + (base + (valid ? lv : 0)) * a.cw;
#pragma unroll
    for (int cc = 0; cc < NC; ++cc) {
      f32x16_t acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) acc = Mma32<T>::run(wf[cc][ks], xf[ks], acc);
      store_block_plus<T>(acc, dst + cc * 32, bv[cc], kg, valid);
    }
    __syncthreads();
  }
}

// reduce: G[j][c] = sum_v thin[v][j] * wide[v][c]. The contraction runs over voxels, so both operands are read from
// LDS against their storage order (8 voxels of one channel per lane). A workgroup owns a contiguous voxel range in
// rounds of 128, its four wavefronts a quarter of each round; their tiles are folded in wave order into one fp32
// partial slice, already in the layout of the weight gradient. Tile rows at and beyond J carry garbage that is
// never written out; voxels beyond the range are zero on both sides.
template <typename T, int NC>
__global__ void __launch_bounds__(kBlock) head_reduce_kernel(ThinArgs a, const T* __restrict__ thin, const T* __restrict__ wide,
                                                             float* __restrict__ part, int64_t total, int64_t per_split,
                                                             float* __restrict__ bias_part) {
  // bias_part (optional): also the sums of the thin tensor over the voxels, [split][J] -- the bias gradient when the
  // thin tensor is the output gradient -- as one more MFMA against a column block of ones.
  constexpr int CW = NC * 32;
  __shared__ __align__(16) uint16_t trows[(kHeadVoxels + 1) * kHeadThinMax];
  constexpr int kFoldHalves = 4 * 32 * 33 * 2;  // the fold at the end reuses the wide rows
  __shared__ __align__(16) uint16_t wrows[kHeadVoxels * CW > kFoldHalves ? kHeadVoxels * CW : kFoldHalves];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, kg = lane >> 5;
  const int J = a.J;
  f32x16_t acc[NC];
#pragma unroll
  for (int cc = 0; cc < NC; ++cc)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[cc][r] = 0.f;
  f32x16_t bacc;
#pragma unroll
  for (int r = 0; r < 16; ++r) bacc[r] = 0.f;
  const uint32_t one2 = std::is_same<T, bf16_t>::value ? 0x3f803f80u : 0x3c003c00u;  // two ones of T
  const uint4 ones = make_uint4(one2, one2, one2, one2);
  const int64_t begin = (int64_t)blockIdx.x * per_split;
  int64_t end = begin + per_split;
  if (end > total) end = total;
  for (int64_t base = begin; base < end; base += kHeadVoxels) {
    const int64_t left = end - base;
    const int nv = left < kHeadVoxels ? (int)left : kHeadVoxels;
    {
      const int nelem = nv * J, npiece = nelem / 8;
      const uint16_t* src = reinterpret_cast<const uint16_t*>(thin) + base * J;
      for (int i = tid; i < npiece; i += kBlock) reinterpret_cast<uint4*>(trows)[i] = reinterpret_cast<const uint4*>(src)[i];
      for (int i = npiece * 8 + tid; i < nelem; i += kBlock) trows[i] = src[i];
      if (nv < kHeadVoxels)
        for (int i = nelem + tid; i < kHeadVoxels * J; i += kBlock) trows[i] = 0;
      const uint4* wsrc = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(wide) + base * CW);
      for (int i = tid; i < kHeadVoxels * CW / 8; i += kBlock)
        reinterpret_cast<uint4*>(wrows)[i] = i < nv * CW / 8 ? wsrc[i] : make_uint4(0, 0, 0, 0);
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const int v0 = wave * 32 + ks * 16 + kg * 8;
      uint32_t h[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) h[e] = trows[(v0 + e) * J + col];
      const uint4 tf = make_uint4(h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16);
      if (bias_part != nullptr) bacc = Mma32<T>::run(tf, ones, bacc);  // every column is the row sum
#pragma unroll
      for (int cc = 0; cc < NC; ++cc) {
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = wrows[(v0 + e) * CW + cc * 32 + col];
        const uint4 xf = make_uint4(h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16);
        acc[cc] = Mma32<T>::run(tf, xf, acc[cc]);
      }
    }
    __syncthreads();
  }
  // Fold the four wavefronts: tile element (j, c) of wave w sits at fold[w][j][c] (rows padded to 33 floats).
  float* fold = reinterpret_cast<float*>(wrows);
  float* dst = part + (int64_t)blockIdx.x * J * CW;
#pragma unroll
  for (int cc = 0; cc < NC; ++cc) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = 8 * (r / 4) + 4 * kg + r % 4;
      fold[(wave * 32 + j) * 33 + col] = acc[cc][r];
    }
    __syncthreads();
    for (int i = tid; i < J * 32; i += kBlock) {
      const int j = i >> 5, c = i & 31;
      float sum = fold[j * 33 + c];
#pragma unroll
      for (int w = 1; w < 4; ++w) sum += fold[(w * 32 + j) * 33 + c];
      dst[(int64_t)(cc * 32 + c) * a.so_wide + (int64_t)j * a.so_thin] = sum;
    }
    __syncthreads();
  }
  if (bias_part != nullptr) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = 8 * (r / 4) + 4 * kg + r % 4;
      fold[(wave * 32 + j) * 33 + col] = bacc[r];
    }
    __syncthreads();
    if (tid < J)
      bias_part[(int64_t)blockIdx.x * J + tid] = (fold[tid * 33] + fold[(32 + tid) * 33]) + (fold[(64 + tid) * 33] + fold[(96 + tid) * 33]);
  }
}

// ---- reduce (weight gradient) ----------------------------------------------------------------
// Thread = (voxel row, V wide channels) with J x V fp32 accumulators; a workgroup owns a contiguous
// voxel range and leaves one fp32 partial slice, already in the layout of the weight gradient; the
// slices are then summed in a fixed order.
template <typename T, int K, int J>
__global__ void __launch_bounds__(kBlock) thin_reduce_kernel(ThinArgs a, const T* __restrict__ thin, const T* __restrict__ wide,
                                                             float* __restrict__ part, int64_t total, int64_t per_split) {
  constexpr int V = VecOf<T>::N;
  constexpr int JC = 4;  // thin values folded per LDS round
  __shared__ float buf[JC * kBlock * V];
  const int tid = threadIdx.x;
  const int wq = a.cw / V, rpp = kBlock / wq;
  const int r = tid / wq, q = tid - r * wq;
  const bool active = r < rpp;
  float acc[J][V];
#pragma unroll
  for (int j = 0; j < J; ++j)
#pragma unroll
    for (int e = 0; e < V; ++e) acc[j][e] = 0.f;
  const int64_t begin = (int64_t)blockIdx.x * per_split;
  int64_t end = begin + per_split;
  if (end > total) end = total;
  if (active) {
    for (int64_t v = begin + r; v < end; v += rpp) {
      int nn, d, h, w;
      decode_voxel<K>(a, v, nn, d, h, w);
      float f[V];
      Ld<T, V>::run(wide + v * a.cw + q * V, f);
#pragma unroll
      for (int j = 0; j < J; ++j) {
        const float s = thin_sample<T, K>(a, thin, j, nn, d, h, w, v);
#pragma unroll
        for (int e = 0; e < V; ++e) acc[j][e] = fmaf(s, f[e], acc[j][e]);
      }
    }
  }
  // Fold the voxel rows: JC thin values at a time through LDS, columns summed in row order.
  float* dst = part + (int64_t)blockIdx.x * a.J * a.cw;
#pragma unroll
  for (int j0 = 0; j0 < J; j0 += JC) {
    __syncthreads();
    if (active) {
#pragma unroll
      for (int jj = 0; jj < JC; ++jj)
#pragma unroll
        for (int e = 0; e < V; ++e) buf[(jj * rpp + r) * a.cw + q * V + e] = (j0 + jj < J) ? acc[(j0 + jj) % J][e] : 0.f;
    }
    __syncthreads();
    for (int i = tid; i < JC * a.cw; i += kBlock) {
      const int jj = i / a.cw, c = i - jj * a.cw;
      if (j0 + jj < a.J) {
        float sum = 0.f;
        for (int rr = 0; rr < rpp; ++rr) sum += buf[(jj * rpp + rr) * a.cw + c];
        dst[(int64_t)c * a.so_wide + (int64_t)(j0 + jj) * a.so_thin] = sum;
      }
    }
  }
}

// ---- the one-channel 3x3x3, stride-1 stem through an LDS brick ----------------------------------
// The generic kernels above fetch the 27 taps of every voxel from global memory one scalar at a time, which
// makes them instruction-bound. At stride 1 neighbouring voxels share their taps: a workgroup stages the
// one-channel input brick of a 2 x 4 x 64 voxel tile (with its halo, zero outside the tensor) in LDS as fp32
// once and every tap becomes an LDS read at an immediate offset.
constexpr int kSTD = 2, kSTH = 4, kSTW = 64;                       // tile of output voxels
constexpr int kSBD = kSTD + 2, kSBH = kSTH + 2, kSBW = kSTW + 2;   // brick with halo
constexpr int kSBV = kSBD * kSBH * kSBW;

struct StemTile { int n, d0, h0, w0; };

__device__ __forceinline__ StemTile stem_tile(const ThinArgs& a, int tile, int tiles_h, int tiles_w, int tiles_d) {
  StemTile t;
  t.w0 = (tile % tiles_w) * kSTW; tile /= tiles_w;
  t.h0 = (tile % tiles_h) * kSTH; tile /= tiles_h;
  t.d0 = (tile % tiles_d) * kSTD;
  t.n = tile / tiles_d;
  return t;
}

template <typename T>
__device__ __forceinline__ void stem_stage(const ThinArgs& a, const T* __restrict__ x, const StemTile& t, float* brick) {
  const int id0 = t.d0 - a.pd, ih0 = t.h0 - a.ph, iw0 = t.w0 - a.pw;
  for (int i = threadIdx.x; i < kSBV; i += kBlock) {
    const int bw = i % kSBW, bh = (i / kSBW) % kSBH, bd = i / (kSBW * kSBH);
    const int id = id0 + bd, ih = ih0 + bh, iw = iw0 + bw;
    float v = 0.f;
    if ((unsigned)id < (unsigned)a.td && (unsigned)ih < (unsigned)a.th && (unsigned)iw < (unsigned)a.tw)
      v = to_float(x[(((int64_t)t.n * a.td + id) * a.th + ih) * a.tw + iw]);
    brick[i] = v;
  }
}

// out[v][c] = bias[c] + sum_tap x[v (+) tap] * w[c][tap]. Thread = (voxel slot, V output channels), its V x 27 weights
// in registers for the whole launch.
template <typename T>
__global__ void __launch_bounds__(kBlock) stem_fwd_kernel(ThinArgs a, const T* __restrict__ x, const T* __restrict__ wt,
                                                          const T* __restrict__ bias, T* __restrict__ out, int tiles_d, int tiles_h,
                                                          int tiles_w) {
  constexpr int V = VecOf<T>::N;
  __shared__ float brick[kSBV];
  const int tid = threadIdx.x;
  const int wq = a.cw / V, rpp = kBlock / wq;
  const int r = tid / wq, q = tid - r * wq;
  const bool active = r < rpp;
  float w[27][V], b[V];
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const int c = active ? q * V + e : 0;
    b[e] = bias != nullptr ? to_float(bias[c]) : 0.f;
#pragma unroll
    for (int j = 0; j < 27; ++j)
      w[j][e] = to_float(wt[(int64_t)c * a.ws_wide + (j / 9) * a.ws_kd + ((j / 3) % 3) * a.ws_kh + (j % 3) * a.ws_kw]);
  }
  const StemTile t = stem_tile(a, blockIdx.x, tiles_h, tiles_w, tiles_d);
  stem_stage<T>(a, x, t, brick);
  __syncthreads();
  if (!active) return;
  for (int vi = r; vi < kSTD * kSTH * kSTW; vi += rpp) {
    const int tw = vi % kSTW, th = (vi / kSTW) % kSTH, td = vi / (kSTW * kSTH);
    const int od = t.d0 + td, oh = t.h0 + th, ow = t.w0 + tw;
    if (od >= a.od || oh >= a.oh || ow >= a.ow) continue;
    const float* src = brick + (td * kSBH + th) * kSBW + tw;
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = b[e];
#pragma unroll
    for (int j = 0; j < 27; ++j) {
      const float s = src[((j / 9) * kSBH + (j / 3) % 3) * kSBW + j % 3];
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = fmaf(s, w[j][e], acc[e]);
    }
    St<T, V>::run(out + ((((int64_t)t.n * a.od + od) * a.oh + oh) * a.ow + ow) * a.cw + q * V, acc);
  }
}

// G[c][tap] = sum_v gy[v][c] * x[v (+) tap]: thread = (voxel slot, V channels) with 27 x V accumulators over the
// workgroup's range of tiles, folded through LDS into one fp32 slice per workgroup (layout of the weight gradient).
template <typename T>
__global__ void __launch_bounds__(kBlock) stem_wgrad_kernel(ThinArgs a, const T* __restrict__ x, const T* __restrict__ gy,
                                                            float* __restrict__ part, int tiles_d, int tiles_h, int tiles_w,
                                                            int ntiles, int tiles_per_wg) {
  constexpr int V = VecOf<T>::N;
  constexpr int JC = 4;
  __shared__ float brick[kSBV];
  __shared__ float buf[JC * kBlock * V];
  const int tid = threadIdx.x;
  const int wq = a.cw / V, rpp = kBlock / wq;
  const int r = tid / wq, q = tid - r * wq;
  const bool active = r < rpp;
  float acc[27][V];
#pragma unroll
  for (int j = 0; j < 27; ++j)
#pragma unroll
    for (int e = 0; e < V; ++e) acc[j][e] = 0.f;
  const int t_begin = blockIdx.x * tiles_per_wg;
  int t_end = t_begin + tiles_per_wg;
  if (t_end > ntiles) t_end = ntiles;
  for (int tile = t_begin; tile < t_end; ++tile) {
    const StemTile t = stem_tile(a, tile, tiles_h, tiles_w, tiles_d);
    __syncthreads();  // the previous tile's brick is consumed
    stem_stage<T>(a, x, t, brick);
    __syncthreads();
    if (active) {
      for (int vi = r; vi < kSTD * kSTH * kSTW; vi += rpp) {
        const int tw = vi % kSTW, th = (vi / kSTW) % kSTH, td = vi / (kSTW * kSTH);
        const int od = t.d0 + td, oh = t.h0 + th, ow = t.w0 + tw;
        if (od >= a.od || oh >= a.oh || ow >= a.ow) continue;
        float f[V];
        Ld<T, V>::run(gy + ((((int64_t)t.n * a.od + od) * a.oh + oh) * a.ow + ow) * a.cw + q * V, f);
        const float* src = brick + (td * kSBH + th) * kSBW + tw;
#pragma unroll
        for (int j = 0; j < 27; ++j) {
          const float s = src[((j / 9) * kSBH + (j / 3) % 3) * kSBW + j % 3];
#pragma unroll
          for (int e = 0; e < V; ++e) acc[j][e] = fmaf(s, f[e], acc[j][e]);
        }
      }
    }
  }
  float* dst = part + (int64_t)blockIdx.x * 27 * a.cw;
#pragma unroll
  for (int j0 = 0; j0 < 27; j0 += JC) {
    __syncthreads();
    if (active) {
#pragma unroll
      for (int jj = 0; jj < JC; ++jj)
#pragma unroll
        for (int e = 0; e < V; ++e) buf[(jj * rpp + r) * a.cw + q * V + e] = (j0 + jj < 27) ? acc[(j0 + jj) % 27][e] : 0.f;
    }
    __syncthreads();
    for (int i = tid; i < JC * a.cw; i += kBlock) {
      const int jj = i / a.cw, c = i - jj * a.cw;
      if (j0 + jj < 27) {
        float sum = 0.f;
        for (int rr = 0; rr < rpp; ++rr) sum += buf[(jj * rpp + rr) * a.cw + c];
        dst[(int64_t)c * a.so_wide + (int64_t)(j0 + jj) * a.so_thin] = sum;
      }
    }
  }
}

// ---- the same stem on the matrix cores (16-bit types, 32 or 64 output channels) ---------------------------------
// The 27 taps are the contraction (padded to 32 with zeros), the brick sits in LDS in the storage type, and a
// wavefront owns 32 voxels along w at a time: 4 of the tile's 16 such runs.
template <typename T>
__device__ __forceinline__ void stem_stage_bits(const ThinArgs& a, const T* __restrict__ x, const StemTile& t, uint16_t* brick) {
  const int id0 = t.d0 - a.pd, ih0 = t.h0 - a.ph, iw0 = t.w0 - a.pw;
  const uint16_t* xb = reinterpret_cast<const uint16_t*>(x);
  constexpr int kRounds = (kSBV + kBlock - 1) / kBlock;
  // all loads of a thread are issued before the first LDS write, so their latencies overlap
  uint16_t v[kRounds];
#pragma unroll
  for (int k = 0; k < kRounds; ++k) {
    const int i = threadIdx.x + k * kBlock;
    const int bw = i % kSBW, bh = (i / kSBW) % kSBH, bd = i / (kSBW * kSBH);
    const int id = id0 + bd, ih = ih0 + bh, iw = iw0 + bw;
    // unconditional loads from a clamped address: a load under a branch would wait for the one before it
    const bool in = i < kSBV && (unsigned)id < (unsigned)a.td && (unsigned)ih < (unsigned)a.th && (unsigned)iw < (unsigned)a.tw;
    const uint16_t bits = xb[in ? (((int64_t)t.n * a.td + id) * a.th + ih) * a.tw + iw : 0];
    v[k] = in ? bits : (uint16_t)0;
  }
#pragma unroll
  for (int k = 0; k < kRounds; ++k) {
    const int i = threadIdx.x + k * kBlock;
    if (i < kSBV) brick[i] = v[k];
  }
}

__device__ __forceinline__ uint4 pack_halves(const uint32_t (&h)[8]) {
  return make_uint4(h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16);
}

// brick offset of tap j relative to the voxel's own brick position
__device__ __forceinline__ int stem_tap_offset(int j) { return ((j / 9) * kSBH + (j / 3) % 3) * kSBW + j % 3; }

template <typename T, int NC>
__global__ void __launch_bounds__(kBlock) stem_fwd_mfma_kernel(ThinArgs a, const T* __restrict__ x, const T* __restrict__ wt,
                                                               const T* __restrict__ bias, T* __restrict__ out, int tiles_d,
                                                               int tiles_h, int tiles_w, GnPartialOut gn) {
  __shared__ __attribute__((aligned(16))) uint16_t brick[kSBV];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, kg = lane >> 5;
  // result tile: rows = output channels (weights), columns = voxels (taps of the voxel)
  uint4 wf[NC][2];
  int off[2][8];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = ks * 16 + kg * 8 + e;
      off[ks][e] = j < 27 ? stem_tap_offset(j) : -1;
    }
#pragma unroll
    for (int cc = 0; cc < NC; ++cc) {
      uint32_t h[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = ks * 16 + kg * 8 + e;
        const int jc = j < 27 ? j : 0;
        const int64_t at = (int64_t)(cc * 32 + col) * a.ws_wide + (jc / 9) * a.ws_kd + ((jc / 3) % 3) * a.ws_kh + (jc % 3) * a.ws_kw;
        const uint32_t bits = reinterpret_cast<const uint16_t*>(wt)[at];
        h[e] = j < 27 ? bits : 0u;
      }
      wf[cc][ks] = pack_halves(h);
    }
  }
  float bv[NC][16];
#pragma unroll
  for (int cc = 0; cc < NC; ++cc) load_block_bias<T>(bias, cc * 32, kg, bv[cc]);
  const StemTile t = stem_tile(a, blockIdx.x, tiles_h, tiles_w, tiles_d);
  stem_stage_bits<T>(a, x, t, brick);
  __syncthreads();
  RunSums gn_sums[NC];  // GroupNorm statistics of the rounded output, when the caller wants them
#pragma unroll
  for (int cc = 0; cc < NC; ++cc) {
    gn_sums[cc].clear();
  }
#pragma unroll 1
  for (int i = 0; i < 4; ++i) {
    const int run = wave * 4 + i, row = run >> 1;
    const int td = row / kSTH, th = row % kSTH, tw = (run & 1) * 32 + col;
    const uint16_t* src = brick + (td * kSBH + th) * kSBW + tw;
    uint4 xf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      uint32_t h[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int o = off[ks][e];
        const uint32_t bits = src[o < 0 ? 0 : o];
        h[e] = o < 0 ? 0u : bits;
      }
      xf[ks] = pack_halves(h);
    }
    const int od = t.d0 + td, oh = t.h0 + th, ow = t.w0 + tw;
    const bool valid = od < a.od && oh < a.oh && ow < a.ow;
    T* dst = out + (valid ? ((((int64_t)t.n * a.od + od) * a.oh + oh) * a.ow + ow) * a.cw : 0);
#pragma unroll
    for (int cc = 0; cc < NC; ++cc) {
      f32x16_t acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) acc = Mma32<T>::run(wf[cc][ks], xf[ks], acc);
      store_block_plus<T>(acc, dst + cc * 32, bv[cc], kg, valid, gn_sums[cc], gn.part != nullptr, i == 0);
    }
  }
  if (gn.part != nullptr) {
    __syncthreads();  // every wave is done reading the brick: the LDS is free
    static_assert(sizeof(brick) >= gn_partials_lds_floats(kBlock / 64, NC) * sizeof(float), "room for the wavefronts' sums");
    write_group_partials<kBlock / 64, NC>(gn_sums, reinterpret_cast<float*>(brick), gn, t.n,
                                          (int)(blockIdx.x % (unsigned)(tiles_d * tiles_h * tiles_w)), 0, tid);
  }
}

// G[c][tap] = sum_v gy[v][c] * x[v (+) tap] with the voxels as the contraction: result rows = channels (gy read
// against its storage order from an LDS copy of the tile's rows), columns = taps (8 consecutive brick cells per lane).
template <typename T, int NC>
__global__ void __launch_bounds__(kBlock) stem_wgrad_mfma_kernel(ThinArgs a, const T* __restrict__ x, const T* __restrict__ gy,
                                                                 float* __restrict__ part, int tiles_d, int tiles_h, int tiles_w,
                                                                 int ntiles, int tiles_per_wg) {
  constexpr int CW = NC * 32;
  constexpr int kTileVoxels = kSTD * kSTH * kSTW;
  constexpr int kRowPieces = kSTW * CW / 8;  // 16-byte pieces of one w-row of the tile
  __shared__ uint16_t brick[kSBV];
  __shared__ __align__(16) uint16_t grows[kTileVoxels * CW];
  static_assert(sizeof(grows) >= 4 * 32 * 33 * sizeof(float), "the fold at the end reuses the gradient rows");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, kg = lane >> 5;
  const int tap = stem_tap_offset(col < 27 ? col : 26);
  f32x16_t acc[NC];
#pragma unroll
  for (int cc = 0; cc < NC; ++cc)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[cc][r] = 0.f;
  const int t_begin = blockIdx.x * tiles_per_wg;
  int t_end = t_begin + tiles_per_wg;
  if (t_end > ntiles) t_end = ntiles;
  for (int tile = t_begin; tile < t_end; ++tile) {
    const StemTile t = stem_tile(a, tile, tiles_h, tiles_w, tiles_d);
    __syncthreads();  // the previous tile is consumed
    stem_stage_bits<T>(a, x, t, brick);
    constexpr int kPieceRounds = kSTD * kSTH * kRowPieces / kBlock;
    static_assert(kSTD * kSTH * kRowPieces % (8 * kBlock) == 0, "piece rounds come in groups of 8");
#pragma unroll 1
    for (int k0 = 0; k0 < kPieceRounds; k0 += 8) {
      uint4 v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int i = tid + (k0 + k) * kBlock;
        const int row = i / kRowPieces, p = i - row * kRowPieces;
        const int od = t.d0 + row / kSTH, oh = t.h0 + row % kSTH, ow = t.w0 + p / (CW / 8);
        const bool in = od < a.od && oh < a.oh && ow < a.ow;
        const uint4 u = *reinterpret_cast<const uint4*>(
            gy + (in ? ((((int64_t)t.n * a.od + od) * a.oh + oh) * a.ow + ow) * CW + (p % (CW / 8)) * 8 : 0));
        v[k] = in ? u : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) reinterpret_cast<uint4*>(grows)[tid + (k0 + k) * kBlock] = v[k];
    }
    __syncthreads();
#pragma unroll 1
    for (int i = 0; i < 4; ++i) {
      const int run = wave * 4 + i, row = run >> 1;
      const int td = row / kSTH, th = row % kSTH;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const int tw = (run & 1) * 32 + ks * 16 + kg * 8;
        const uint16_t* xs = brick + (td * kSBH + th) * kSBW + tw + tap;
        uint32_t h[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = xs[e];
        const uint4 xf = pack_halves(h);
        const uint16_t* gs = grows + (row * kSTW + tw) * CW + col;
#pragma unroll
        for (int cc = 0; cc < NC; ++cc) {
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = gs[e * CW + cc * 32];
          acc[cc] = Mma32<T>::run(pack_halves(h), xf, acc[cc]);
        }
      }
    }
  }
  __syncthreads();
  float* fold = reinterpret_cast<float*>(grows);
  float* dst = part + (int64_t)blockIdx.x * 27 * CW;
#pragma unroll
  for (int cc = 0; cc < NC; ++cc) {
    // result register r of this lane: channel 8 * (r / 4) + 4 * kg + r % 4, tap col
#pragma unroll
    for (int r = 0; r < 16; ++r) fold[(wave * 32 + 8 * (r / 4) + 4 * kg + r % 4) * 33 + col] = acc[cc][r];
    __syncthreads();
    for (int i = tid; i < 32 * 27; i += kBlock) {
      const int c = i / 27, j = i - c * 27;
      float sum = fold[c * 33 + j];
#pragma unroll
      for (int w = 1; w < 4; ++w) sum += fold[(w * 32 + c) * 33 + j];
      dst[(int64_t)(cc * 32 + c) * a.so_wide + (int64_t)j * a.so_thin] = sum;
    }
    __syncthreads();
  }
}

bool stem_brick_ok(const ThinArgs& a) {
  return a.K == 3 && a.sd == 1 && a.sh == 1 && a.sw == 1 && a.dd == 1 && a.dh == 1 && a.dw == 1 && a.pd <= 2 && a.ph <= 2 &&
         a.pw <= 2;
}

int64_t stem_tiles(const ThinArgs& a) {
  return (int64_t)a.n * cdiv(a.od, kSTD) * cdiv(a.oh, kSTH) * cdiv(a.ow, kSTW);
}

// the one-channel 3x3x3 stem on the matrix cores (16-bit types): 32 or 64 output channels
bool stem_matrix_ok(const ThinArgs& a) {
  return stem_brick_ok(a) && stem_tiles(a) <= 0x7fffffffLL && (a.cw == 32 || a.cw == 64);
}

int wide_channels_ok(const ThinArgs& a, int dtype) {
  const int v = dtype == SFH_FP32 ? 4 : 8;
  return a.cw % v == 0 && a.cw / v <= kBlock && a.cw >= v;
}

int grid_for(int64_t units, int per_block) {
  const int64_t want = cdiv(units, per_block);
  const int64_t cap = (int64_t)kComputeUnits * 8;
  return (int)(want < cap ? (want < 1 ? 1 : want) : cap);
}

template <typename T, int K, int J>
int launch_wide_out(const ThinArgs& a, const void* thin, const void* wt, const void* bias, void* out, hipStream_t st) {
  constexpr int V = VecOf<T>::N;
  const int64_t total = (int64_t)a.n * a.od * a.oh * a.ow;
  const int rpp = kBlock / (a.cw / V);
  hipLaunchKernelGGL((thin_wide_out_kernel<T, K, J>), dim3(grid_for(total, rpp)), dim3(kBlock), (size_t)J * a.cw * 4, st, a,
                     (const T*)thin, (const T*)wt, (const T*)bias, (T*)out, total);
  return check_launch("thin_wide_out_kernel");
}

template <typename T, int J>
int launch_thin_out(const ThinArgs& a, const void* wide, const void* wt, const void* bias, void* out, hipStream_t st) {
  const int64_t total = (int64_t)a.n * a.od * a.oh * a.ow;
  hipLaunchKernelGGL((thin_out_kernel<T, J>), dim3(grid_for(total, kBlock)), dim3(kBlock), (size_t)J * a.cw * 4, st, a,
                     (const T*)wide, (const T*)wt, (const T*)bias, (T*)out, total);
  return check_launch("thin_out_kernel");
}

template <typename T, int K, int J>
int launch_reduce(const ThinArgs& a, const void* thin, const void* wide, void* gw, int gw_dtype, void* ws, hipStream_t st) {
  const int64_t total = (int64_t)a.n * a.od * a.oh * a.ow;
  const int nsplit = thin_reduce_splits(a);
  const int64_t per = cdiv(total, nsplit);
  hipLaunchKernelGGL((thin_reduce_kernel<T, K, J>), dim3(nsplit), dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wide,
                     (float*)ws, total, per);
  if (int rc = check_launch("thin_reduce_kernel")) return rc;
  return sum_slices(gw_dtype, (const float*)ws, gw, (int64_t)a.J * a.cw, nsplit, st);
}

template <typename T, int NK>
int launch_head_wide_out_nk(const ThinArgs& a, const void* thin, const void* wt, const void* bias, void* out, hipStream_t st) {
  const int64_t total = (int64_t)a.n * a.od * a.oh * a.ow;
  const dim3 grid(grid_for(total, kHeadVoxels));
  if (a.cw == 32) hipLaunchKernelGGL((head_wide_out_kernel<T, 1, NK>), grid, dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wt, (const T*)bias, (T*)out, total);
  else if (a.cw == 64) hipLaunchKernelGGL((head_wide_out_kernel<T, 2, NK>), grid, dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wt, (const T*)bias, (T*)out, total);
  else hipLaunchKernelGGL((head_wide_out_kernel<T, 4, NK>), grid, dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wt, (const T*)bias, (T*)out, total);
  return check_launch("head_wide_out_kernel");
}
template <typename T>
int launch_head_wide_out(const ThinArgs& a, const void* thin, const void* wt, const void* bias, void* out, hipStream_t st) {
  return a.J <= 16 ? launch_head_wide_out_nk<T, 1>(a, thin, wt, bias, out, st) : launch_head_wide_out_nk<T, 2>(a, thin, wt, bias, out, st);
}

// J is padded to the next instantiated size; K in {0 (channels), 2, 3}.
template <typename T>
int dispatch_wide_out(const ThinArgs& a, const void* thin, const void* wt, const void* bias, void* out, hipStream_t st,
                      const GnPartialOut& gn) {
  if constexpr (sizeof(T) == 2) {
    if (stem_matrix_ok(a) && (uintptr_t)out % 16 == 0) {
      const dim3 grid((unsigned)stem_tiles(a));
      const int td = (int)cdiv(a.od, kSTD), th = (int)cdiv(a.oh, kSTH), tw = (int)cdiv(a.ow, kSTW);
      if (a.cw == 32) hipLaunchKernelGGL((stem_fwd_mfma_kernel<T, 1>), grid, dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wt, (const T*)bias, (T*)out, td, th, tw, gn);
      else hipLaunchKernelGGL((stem_fwd_mfma_kernel<T, 2>), grid, dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wt, (const T*)bias, (T*)out, td, th, tw, gn);
      return check_launch("stem_fwd_mfma_kernel");
    }
  }
  if (gn.part != nullptr) return fail(SFH_ERR_UNSUPPORTED, "thin-channel conv: GroupNorm partials need the matrix-core stem kernel and a 16-byte aligned output");
  if (stem_brick_ok(a) && stem_tiles(a) <= 0x7fffffffLL) {
    hipLaunchKernelGGL(stem_fwd_kernel<T>, dim3((unsigned)stem_tiles(a)), dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wt,
                       (const T*)bias, (T*)out, (int)cdiv(a.od, kSTD), (int)cdiv(a.oh, kSTH), (int)cdiv(a.ow, kSTW));
    return check_launch("stem_fwd_kernel");
  }
  if constexpr (sizeof(T) == 2) {
    if (a.K == 0 && (a.cw == 32 || a.cw == 64 || a.cw == 128) && ((uintptr_t)thin | (uintptr_t)out) % 16 == 0) return launch_head_wide_out<T>(a, thin, wt, bias, out, st);
  }
  if (a.K == 3) return launch_wide_out<T, 3, 27>(a, thin, wt, bias, out, st);
  if (a.K == 2) return launch_wide_out<T, 2, 8>(a, thin, wt, bias, out, st);
  if (a.J <= 4) return launch_wide_out<T, 0, 4>(a, thin, wt, bias, out, st);
  if (a.J <= 16) return launch_wide_out<T, 0, 16>(a, thin, wt, bias, out, st);
  return launch_wide_out<T, 0, 32>(a, thin, wt, bias, out, st);
}
template <typename T>
int dispatch_thin_out(const ThinArgs& a, const void* wide, const void* wt, const void* bias, void* out, hipStream_t st) {
  if constexpr (sizeof(T) == 2) {
    const int64_t total = (int64_t)a.n * a.od * a.oh * a.ow;
    const dim3 grid(grid_for(total, kHeadVoxels));
    if ((a.cw == 32 || a.cw == 64 || a.cw == 128) && ((uintptr_t)wide | (uintptr_t)out) % 16 == 0) {
      if (a.cw == 32) hipLaunchKernelGGL((head_thin_out_kernel<T, 1>), grid, dim3(kBlock), 0, st, a, (const T*)wide, (const T*)wt, (const T*)bias, (T*)out, total);
      else if (a.cw == 64) hipLaunchKernelGGL((head_thin_out_kernel<T, 2>), grid, dim3(kBlock), 0, st, a, (const T*)wide, (const T*)wt, (const T*)bias, (T*)out, total);
      else hipLaunchKernelGGL((head_thin_out_kernel<T, 4>), grid, dim3(kBlock), 0, st, a, (const T*)wide, (const T*)wt, (const T*)bias, (T*)out, total);
      return check_launch("head_thin_out_kernel");
    }
  }
  if (a.J <= 4) return launch_thin_out<T, 4>(a, wide, wt, bias, out, st);
  if (a.J <= 16) return launch_thin_out<T, 16>(a, wide, wt, bias, out, st);
  return launch_thin_out<T, 32>(a, wide, wt, bias, out, st);
}
// The kernel that leaves the thin tensor's sums beside the weight gradient: the 1x1x1 head with 32 / 64 / 128 wide channels.
bool head_reduce_applies(const ThinArgs& a) {
  return !stem_brick_ok(a) && a.K == 0 && (a.cw == 32 || a.cw == 64 || a.cw == 128);
}

template <typename T>
int dispatch_reduce(const ThinArgs& a, const void* thin, const void* wide, void* gw, int gw_dtype, void* ws, hipStream_t st, void* gb) {
  if (gb != nullptr && !(sizeof(T) == 2 && head_reduce_applies(a) && ((uintptr_t)thin | (uintptr_t)wide) % 16 == 0))
    return fail(SFH_ERR_UNSUPPORTED, "thin-channel weight gradient: the sums of the thin tensor are not offered for this problem");
  if constexpr (sizeof(T) == 2) {
    if (stem_brick_ok(a) && stem_tiles(a) <= 0x7fffffffLL && (a.cw == 32 || a.cw == 64) && (uintptr_t)wide % 16 == 0) {
      const int nsplit = thin_reduce_splits(a);
      const int ntiles = (int)stem_tiles(a);
      const int per = (int)cdiv(ntiles, nsplit);
      const int td = (int)cdiv(a.od, kSTD), th = (int)cdiv(a.oh, kSTH), tw = (int)cdiv(a.ow, kSTW);
      if (a.cw == 32) hipLaunchKernelGGL((stem_wgrad_mfma_kernel<T, 1>), dim3(nsplit), dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wide, (float*)ws, td, th, tw, ntiles, per);
      else hipLaunchKernelGGL((stem_wgrad_mfma_kernel<T, 2>), dim3(nsplit), dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wide, (float*)ws, td, th, tw, ntiles, per);
      if (int rc = check_launch("stem_wgrad_mfma_kernel")) return rc;
      return sum_slices(gw_dtype, (const float*)ws, gw, (int64_t)a.J * a.cw, nsplit, st);
    }
  }
  if (stem_brick_ok(a) && stem_tiles(a) <= 0x7fffffffLL) {
    const int nsplit = thin_reduce_splits(a);
    const int ntiles = (int)stem_tiles(a);
    const int per = (int)cdiv(ntiles, nsplit);
    hipLaunchKernelGGL(stem_wgrad_kernel<T>, dim3(nsplit), dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wide, (float*)ws,
                       (int)cdiv(a.od, kSTD), (int)cdiv(a.oh, kSTH), (int)cdiv(a.ow, kSTW), ntiles, per);
    if (int rc = check_launch("stem_wgrad_kernel")) return rc;
    return sum_slices(gw_dtype, (const float*)ws, gw, (int64_t)a.J * a.cw, nsplit, st);
  }
  if constexpr (sizeof(T) == 2) {
    if (a.K == 0 && (a.cw == 32 || a.cw == 64 || a.cw == 128) && ((uintptr_t)thin | (uintptr_t)wide) % 16 == 0) {
      const int64_t total = (int64_t)a.n * a.od * a.oh * a.ow;
      const int nsplit = thin_reduce_splits(a);
      const int64_t per = cdiv(cdiv(total, nsplit), kHeadVoxels) * kHeadVoxels;  // keeps every range 16-byte aligned
      const dim3 grid(nsplit);
      float* bias_part = gb != nullptr ? (float*)ws + (int64_t)nsplit * a.J * a.cw : nullptr;  // behind the weight slices
      if (a.cw == 32) hipLaunchKernelGGL((head_reduce_kernel<T, 1>), grid, dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wide, (float*)ws, total, per, bias_part);
      else if (a.cw == 64) hipLaunchKernelGGL((head_reduce_kernel<T, 2>), grid, dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wide, (float*)ws, total, per, bias_part);
      else hipLaunchKernelGGL((head_reduce_kernel<T, 4>), grid, dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wide, (float*)ws, total, per, bias_part);
      if (int rc = check_launch("head_reduce_kernel")) return rc;
      if (gb == nullptr) return sum_slices(gw_dtype, (const float*)ws, gw, (int64_t)a.J * a.cw, nsplit, st);
      return sum_slices_two(gw_dtype, (const float*)ws, gw, (int64_t)a.J * a.cw, nsplit, bias_part, gb, a.J, nsplit, st);
    }
  }
  if (a.K == 3) return launch_reduce<T, 3, 27>(a, thin, wide, gw, gw_dtype, ws, st);
  if (a.K == 2) return launch_reduce<T, 2, 8>(a, thin, wide, gw, gw_dtype, ws, st);
  if (a.J <= 4) return launch_reduce<T, 0, 4>(a, thin, wide, gw, gw_dtype, ws, st);
  if (a.J <= 16) return launch_reduce<T, 0, 16>(a, thin, wide, gw, gw_dtype, ws, st);
  return launch_reduce<T, 0, 32>(a, thin, wide, gw, gw_dtype, ws, st);
}

}  // namespace

bool thin_supported(const ThinArgs& a, int dtype) {
  if (!wide_channels_ok(a, dtype)) return false;
  if (a.K == 0) return a.J >= 1 && a.J <= 32 && a.ct == a.J;
  return (a.K == 2 || a.K == 3) && a.ct == 1 && a.J == a.K * a.K * a.K;
}

int thin_reduce_splits(const ThinArgs& a) {
  const int64_t total = (int64_t)a.n * a.od * a.oh * a.ow;
  // at least 2048 voxels per workgroup so that the fold at the end stays a small share
  int64_t n = cdiv(total, 2048);
  if (n > kComputeUnits * 2) n = kComputeUnits * 2;
  return (int)(n < 1 ? 1 : n);
}

size_t thin_reduce_workspace_bytes(const ThinArgs& a, bool with_thin_sums) {
  return (size_t)thin_reduce_splits(a) * a.J * (a.cw + (with_thin_sums ? 1 : 0)) * sizeof(float);
}

bool thin_reduce_offers_thin_sums(const ThinArgs& a, int dtype) {
  return (dtype == SFH_BF16 || dtype == SFH_FP16) && head_reduce_applies(a);
}

#define SFH_THIN_BY_DTYPE(fn, ...)                         \
  switch (dtype) {                                         \
    case SFH_BF16: return fn<bf16_t>(__VA_ARGS__);          \
    case SFH_FP16: return fn<fp16_t>(__VA_ARGS__);          \
    default: return fn<float>(__VA_ARGS__);                \
  }

int thin_wide_out_gn_records(const ThinArgs& a, int dtype, int groups) {
  if ((dtype != SFH_BF16 && dtype != SFH_FP16) || !stem_matrix_ok(a) || !gn_partials_fit(a.cw, groups, a.cw)) return 0;
  return (int)(stem_tiles(a) / a.n);
}

int thin_wide_out(const ThinArgs& a, int dtype, const void* thin, const void* wt, const void* bias, void* out, hipStream_t st,
                  const GnPartialOut* gn) {
  GnPartialOut o{nullptr, 0, 0, 0};
  if (gn != nullptr && gn->part != nullptr) {
    if (gn->records == 0 || gn->records != thin_wide_out_gn_records(a, dtype, gn->groups))
      return fail(SFH_ERR_INVALID, "thin-channel conv: GroupNorm partials asked for %d records, this launch leaves %d", gn->records,
                  thin_wide_out_gn_records(a, dtype, gn->groups));
    o = *gn;
    o.cg = a.cw / gn->groups;
  }
  SFH_THIN_BY_DTYPE(dispatch_wide_out, a, thin, wt, bias, out, st, o)
}
int thin_out(const ThinArgs& a, int dtype, const void* wide, const void* wt, const void* bias, void* out, hipStream_t st) {
  SFH_THIN_BY_DTYPE(dispatch_thin_out, a, wide, wt, bias, out, st)
}
int thin_reduce(const ThinArgs& a, int dtype, const void* thin, const void* wide, void* gw, int gw_dtype, void* ws, hipStream_t st,
                void* thin_sums) {
  SFH_THIN_BY_DTYPE(dispatch_reduce, a, thin, wide, gw, gw_dtype, ws, st, thin_sums)
}

}  // namespace sfh
