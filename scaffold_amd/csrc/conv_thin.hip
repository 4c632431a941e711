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

bool stem_brick_ok(const ThinArgs& a) {
  return a.K == 3 && a.sd == 1 && a.sh == 1 && a.sw == 1 && a.dd == 1 && a.dh == 1 && a.dw == 1 && a.pd <= 2 && a.ph <= 2 &&
         a.pw <= 2;
}

int64_t stem_tiles(const ThinArgs& a) {
  return (int64_t)a.n * cdiv(a.od, kSTD) * cdiv(a.oh, kSTH) * cdiv(a.ow, kSTW);
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

// J is padded to the next instantiated size; K in {0 (channels), 2, 3}.
template <typename T>
int dispatch_wide_out(const ThinArgs& a, const void* thin, const void* wt, const void* bias, void* out, hipStream_t st) {
  if (stem_brick_ok(a) && stem_tiles(a) <= 0x7fffffffLL) {
    hipLaunchKernelGGL(stem_fwd_kernel<T>, dim3((unsigned)stem_tiles(a)), dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wt,
                       (const T*)bias, (T*)out, (int)cdiv(a.od, kSTD), (int)cdiv(a.oh, kSTH), (int)cdiv(a.ow, kSTW));
    return check_launch("stem_fwd_kernel");
  }
  if (a.K == 3) return launch_wide_out<T, 3, 27>(a, thin, wt, bias, out, st);
  if (a.K == 2) return launch_wide_out<T, 2, 8>(a, thin, wt, bias, out, st);
  if (a.J <= 4) return launch_wide_out<T, 0, 4>(a, thin, wt, bias, out, st);
  if (a.J <= 16) return launch_wide_out<T, 0, 16>(a, thin, wt, bias, out, st);
  return launch_wide_out<T, 0, 32>(a, thin, wt, bias, out, st);
}
template <typename T>
int dispatch_thin_out(const ThinArgs& a, const void* wide, const void* wt, const void* bias, void* out, hipStream_t st) {
  if (a.J <= 4) return launch_thin_out<T, 4>(a, wide, wt, bias, out, st);
  if (a.J <= 16) return launch_thin_out<T, 16>(a, wide, wt, bias, out, st);
  return launch_thin_out<T, 32>(a, wide, wt, bias, out, st);
}
template <typename T>
int dispatch_reduce(const ThinArgs& a, const void* thin, const void* wide, void* gw, int gw_dtype, void* ws, hipStream_t st) {
  if (stem_brick_ok(a) && stem_tiles(a) <= 0x7fffffffLL) {
    const int nsplit = thin_reduce_splits(a);
    const int ntiles = (int)stem_tiles(a);
    const int per = (int)cdiv(ntiles, nsplit);
    hipLaunchKernelGGL(stem_wgrad_kernel<T>, dim3(nsplit), dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wide, (float*)ws,
                       (int)cdiv(a.od, kSTD), (int)cdiv(a.oh, kSTH), (int)cdiv(a.ow, kSTW), ntiles, per);
    if (int rc = check_launch("stem_wgrad_kernel")) return rc;
    return sum_slices(gw_dtype, (const float*)ws, gw, (int64_t)a.J * a.cw, nsplit, st);
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

size_t thin_reduce_workspace_bytes(const ThinArgs& a) {
  return (size_t)thin_reduce_splits(a) * a.J * a.cw * sizeof(float);
}

#define SFH_THIN_BY_DTYPE(fn, ...)                         \
  switch (dtype) {                                         \
    case SFH_BF16: return fn<bf16_t>(__VA_ARGS__);          \
    case SFH_FP16: return fn<fp16_t>(__VA_ARGS__);          \
    default: return fn<float>(__VA_ARGS__);                \
  }

int thin_wide_out(const ThinArgs& a, int dtype, const void* thin, const void* wt, const void* bias, void* out, hipStream_t st) {
  SFH_THIN_BY_DTYPE(dispatch_wide_out, a, thin, wt, bias, out, st)
}
int thin_out(const ThinArgs& a, int dtype, const void* wide, const void* wt, const void* bias, void* out, hipStream_t st) {
  SFH_THIN_BY_DTYPE(dispatch_thin_out, a, wide, wt, bias, out, st)
}
int thin_reduce(const ThinArgs& a, int dtype, const void* thin, const void* wide, void* gw, int gw_dtype, void* ws, hipStream_t st) {
  SFH_THIN_BY_DTYPE(dispatch_reduce, a, thin, wide, gw, gw_dtype, ws, st)
}

}  // namespace sfh
