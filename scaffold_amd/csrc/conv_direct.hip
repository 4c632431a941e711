// Direct (non-MFMA) convolution kernels: every stride / dilation / padding / channel count
// and all three dtypes, fp32 FMA accumulation. They serve the shapes the MFMA kernels do not
// tile (odd channel counts, dilation, fp32 operands) and are the in-library cross-check for
// the fast paths. Index order follows the reference forward kernel: output row m unravels as
// (n, od, oh, ow) with ow fastest and the fused tap index is (kd*KH + kh)*KW + kw
// (triton_conv3d/gather_gemm.py:194-226,302).
#include "common.hpp"
#include "conv_direct.hpp"

namespace sfh {

// One thread per output element (m, co), co fastest so that stores are coalesced and the
// activation row of a voxel is broadcast across the lanes that share it.
template <typename T>
__global__ void __launch_bounds__(256) conv3d_direct_gather(DirectConvArgs a, const T* __restrict__ x,
                                                            const T* __restrict__ w, const T* __restrict__ bias,
                                                            T* __restrict__ y) {
  const int64_t total = (int64_t)a.n * a.od * a.oh * a.ow * a.cout;
  int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int co = (int)(idx % a.cout);
  int64_t m = idx / a.cout;
  const int ow = (int)(m % a.ow); m /= a.ow;
  const int oh = (int)(m % a.oh); m /= a.oh;
  const int od = (int)(m % a.od);
  const int nb = (int)(m / a.od);
  float acc = 0.f;
  const int taps = a.kd * a.kh * a.kw;
  for (int kd = 0; kd < a.kd; ++kd) {
    const int id = od * a.sd + kd * a.dd - a.pd;
    if (id < 0 || id >= a.id) continue;
    for (int kh = 0; kh < a.kh; ++kh) {
      const int ih = oh * a.sh + kh * a.dh - a.ph;
      if (ih < 0 || ih >= a.ih) continue;
      for (int kw = 0; kw < a.kw; ++kw) {
        const int iw = ow * a.sw + kw * a.dw - a.pw;
        if (iw < 0 || iw >= a.iw) continue;
        int tap = (kd * a.kh + kh) * a.kw + kw;
        int wkd = kd, wkh = kh, wkw = kw;
        if (a.flip) { wkd = a.kd - 1 - kd; wkh = a.kh - 1 - kh; wkw = a.kw - 1 - kw; tap = taps - 1 - tap; }
        const T* xp = x + ((((int64_t)nb * a.id + id) * a.ih + ih) * a.iw + iw) * a.cin;
        const T* wp = w + (int64_t)co * a.ws_co + (int64_t)wkd * a.ws_kd + (int64_t)wkh * a.ws_kh + (int64_t)wkw * a.ws_kw;
        for (int ci = 0; ci < a.cin; ++ci) acc = fmaf(to_float(xp[ci]), to_float(wp[(int64_t)ci * a.ws_ci]), acc);
      }
    }
  }
  if (bias != nullptr) acc += to_float(bias[co]);
  y[idx] = elem<T>::from_float(acc);
}

// Weight gradient: one workgroup per (co, tap); thread t owns input channel (t % CB) of the
// current channel block and voxel slice (t / CB); slices are summed through LDS in index
// order, so the result does not depend on scheduling.
template <typename T>
__global__ void __launch_bounds__(256) conv3d_direct_wgrad(DirectConvArgs a, int cb, const T* __restrict__ x,
                                                           const T* __restrict__ gy, T* __restrict__ gw) {
  __shared__ float red[256];
  const int taps = a.kd * a.kh * a.kw;
  const int co = blockIdx.x / taps;
  const int tap = blockIdx.x % taps;
  const int kw = tap % a.kw, kh = (tap / a.kw) % a.kh, kd = tap / (a.kw * a.kh);
  const int cl = threadIdx.x % cb, vs = threadIdx.x / cb, nvs = 256 / cb;
  const int64_t mtot = (int64_t)a.n * a.od * a.oh * a.ow;
  for (int c0 = 0; c0 < a.cin; c0 += cb) {
    const int ci = c0 + cl;
    float acc = 0.f;
    if (ci < a.cin) {
      for (int64_t m = vs; m < mtot; m += nvs) {
        int64_t r = m;
        const int ow = (int)(r % a.ow); r /= a.ow;
        const int oh = (int)(r % a.oh); r /= a.oh;
        const int od = (int)(r % a.od);
        const int nb = (int)(r / a.od);
        const int id = od * a.sd + kd * a.dd - a.pd;
        const int ih = oh * a.sh + kh * a.dh - a.ph;
        const int iw = ow * a.sw + kw * a.dw - a.pw;
        if (id < 0 || id >= a.id || ih < 0 || ih >= a.ih || iw < 0 || iw >= a.iw) continue;
        const float g = to_float(gy[m * a.cout + co]);
        const float v = to_float(x[((((int64_t)nb * a.id + id) * a.ih + ih) * a.iw + iw) * a.cin + ci]);
        acc = fmaf(g, v, acc);
      }
    }
    __syncthreads();
    red[threadIdx.x] = acc;
    __syncthreads();
    if (vs == 0 && ci < a.cin) {
      float s = 0.f;
      for (int k = 0; k < nvs; ++k) s += red[k * cb + cl];
      gw[((int64_t)co * taps + tap) * a.cin + ci] = elem<T>::from_float(s);
    }
  }
}

// kernel == stride transposed convolution: one thread per output element, which has exactly
// one contributing input voxel and tap (triton_conv3d/transposed.py:205-319).
template <typename T>
__global__ void __launch_bounds__(256) convT3d_direct(int n, int cin, int id, int ih, int iw, int cout, int kd, int kh, int kw,
                                                      int64_t ws_ci, int64_t ws_co, int64_t ws_kd, int64_t ws_kh, int64_t ws_kw,
                                                      const T* __restrict__ x, const T* __restrict__ w,
                                                      const T* __restrict__ bias, T* __restrict__ y) {
  const int od = id * kd, oh = ih * kh, ow = iw * kw;
  const int64_t total = (int64_t)n * od * oh * ow * cout;
  int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int co = (int)(idx % cout);
  int64_t m = idx / cout;
  const int xw = (int)(m % ow); m /= ow;
  const int xh = (int)(m % oh); m /= oh;
  const int xd = (int)(m % od);
  const int nb = (int)(m / od);
  const T* xp = x + ((((int64_t)nb * id + xd / kd) * ih + xh / kh) * iw + xw / kw) * cin;
  const T* wp = w + (int64_t)co * ws_co + (int64_t)(xd % kd) * ws_kd + (int64_t)(xh % kh) * ws_kh + (int64_t)(xw % kw) * ws_kw;
  float acc = 0.f;
  for (int ci = 0; ci < cin; ++ci) acc = fmaf(to_float(xp[ci]), to_float(wp[(int64_t)ci * ws_ci]), acc);
  if (bias != nullptr) acc += to_float(bias[co]);
  y[idx] = elem<T>::from_float(acc);
}

template <typename T>
static int launch_gather(const DirectConvArgs& a, const void* x, const void* w, const void* bias, void* y, hipStream_t st) {
  const int64_t total = (int64_t)a.n * a.od * a.oh * a.ow * a.cout;
  if (total == 0) return SFH_OK;
  const int64_t blocks = cdiv(total, 256);
  if (blocks > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "direct conv: %lld outputs exceed the grid limit", (long long)total);
  hipLaunchKernelGGL(conv3d_direct_gather<T>, dim3((unsigned)blocks), dim3(256), 0, st, a, (const T*)x, (const T*)w,
                     (const T*)bias, (T*)y);
  return check_launch("conv3d_direct_gather");
}

int direct_conv_gather(const DirectConvArgs& a, int dtype, const void* x, const void* w, const void* bias, void* y,
                       hipStream_t st) {
  switch (dtype) {
    case SFH_BF16: return launch_gather<bf16_t>(a, x, w, bias, y, st);
    case SFH_FP16: return launch_gather<fp16_t>(a, x, w, bias, y, st);
    default: return launch_gather<float>(a, x, w, bias, y, st);
  }
}

template <typename T>
static int launch_wgrad(const DirectConvArgs& a, const void* x, const void* gy, void* gw, hipStream_t st) {
  int cb = 1;
  while (cb < a.cin && cb < 256) cb <<= 1;
  const int64_t blocks = (int64_t)a.cout * a.kd * a.kh * a.kw;
  hipLaunchKernelGGL(conv3d_direct_wgrad<T>, dim3((unsigned)blocks), dim3(256), 0, st, a, cb, (const T*)x, (const T*)gy,
                     (T*)gw);
  return check_launch("conv3d_direct_wgrad");
}

int direct_conv_wgrad(const DirectConvArgs& a, int dtype, const void* x, const void* gy, void* gw, hipStream_t st) {
  switch (dtype) {
    case SFH_BF16: return launch_wgrad<bf16_t>(a, x, gy, gw, st);
    case SFH_FP16: return launch_wgrad<fp16_t>(a, x, gy, gw, st);
    default: return launch_wgrad<float>(a, x, gy, gw, st);
  }
}

template <typename T>
static int launch_convT(const sfh_convT3d_desc& p, const int64_t* ws, const void* x, const void* w, const void* bias, void* y,
                        hipStream_t st) {
  const int64_t total = (int64_t)p.n * p.in_d * p.kd * p.in_h * p.kh * p.in_w * p.kw * p.cout;
  if (total == 0) return SFH_OK;
  const int64_t blocks = cdiv(total, 256);
  if (blocks > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "direct convT: %lld outputs exceed the grid limit", (long long)total);
  hipLaunchKernelGGL(convT3d_direct<T>, dim3((unsigned)blocks), dim3(256), 0, st, p.n, p.cin, p.in_d, p.in_h, p.in_w, p.cout,
                     p.kd, p.kh, p.kw, ws[0], ws[1], ws[2], ws[3], ws[4], (const T*)x, (const T*)w, (const T*)bias, (T*)y);
  return check_launch("convT3d_direct");
}

int direct_convT(const sfh_convT3d_desc& p, int dtype, const int64_t* w_stride, const void* x, const void* w, const void* bias,
                 void* y, hipStream_t st) {
  switch (dtype) {
    case SFH_BF16: return launch_convT<bf16_t>(p, w_stride, x, w, bias, y, st);
    case SFH_FP16: return launch_convT<fp16_t>(p, w_stride, x, w, bias, y, st);
    default: return launch_convT<float>(p, w_stride, x, w, bias, y, st);
  }
}

}  // namespace sfh
