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
int launch_reduce(const ThinArgs& a, const void* thin, const void* wide, void* gw, void* ws, hipStream_t st) {
  const int64_t total = (int64_t)a.n * a.od * a.oh * a.ow;
  const int nsplit = thin_reduce_splits(a);
  const int64_t per = cdiv(total, nsplit);
  hipLaunchKernelGGL((thin_reduce_kernel<T, K, J>), dim3(nsplit), dim3(kBlock), 0, st, a, (const T*)thin, (const T*)wide,
                     (float*)ws, total, per);
  if (int rc = check_launch("thin_reduce_kernel")) return rc;
  const int dtype = sizeof(T) == 4 ? SFH_FP32 : (__is_same(T, bf16_t) ? SFH_BF16 : SFH_FP16);
  return sum_slices(dtype, (const float*)ws, gw, (int64_t)a.J * a.cw, nsplit, st);
}

// J is padded to the next instantiated size; K in {0 (channels), 2, 3}.
template <typename T>
int dispatch_wide_out(const ThinArgs& a, const void* thin, const void* wt, const void* bias, void* out, hipStream_t st) {
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
int dispatch_reduce(const ThinArgs& a, const void* thin, const void* wide, void* gw, void* ws, hipStream_t st) {
  if (a.K == 3) return launch_reduce<T, 3, 27>(a, thin, wide, gw, ws, st);
  if (a.K == 2) return launch_reduce<T, 2, 8>(a, thin, wide, gw, ws, st);
  if (a.J <= 4) return launch_reduce<T, 0, 4>(a, thin, wide, gw, ws, st);
  if (a.J <= 16) return launch_reduce<T, 0, 16>(a, thin, wide, gw, ws, st);
  return launch_reduce<T, 0, 32>(a, thin, wide, gw, ws, st);
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
int thin_reduce(const ThinArgs& a, int dtype, const void* thin, const void* wide, void* gw, void* ws, hipStream_t st) {
  SFH_THIN_BY_DTYPE(dispatch_reduce, a, thin, wide, gw, ws, st)
}

}  // namespace sfh
