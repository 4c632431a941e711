// Host-side interface of the direct convolution kernels.
#pragma once
#include "common.hpp"

namespace sfh {

// A gather convolution y[m, co] = sum_{tap, ci} x[m (+) tap, ci] * w[co, ci, tap]. The data
// gradient is expressed in the same terms (channel roles swapped through the strides, taps
// flipped, padding dil*(k-1)-p), which is how the reference obtains it
// (triton_conv3d/bwd_data.py:344-363).
struct DirectConvArgs {
  int n, cin, id, ih, iw;  // reduction channels and input extents
  int cout, od, oh, ow;    // produced channels and output extents
  int kd, kh, kw, sd, sh, sw, pd, ph, pw, dd, dh, dw;
  int flip;                                    // 1: consume the taps mirrored in all three axes
  int64_t ws_co, ws_ci, ws_kd, ws_kh, ws_kw;   // weight element strides in the roles above
};

int direct_conv_gather(const DirectConvArgs& a, int dtype, const void* x, const void* w, const void* bias, void* y,
                       hipStream_t st);
int direct_conv_wgrad(const DirectConvArgs& a, int dtype, const void* x, const void* gy, void* gw, hipStream_t st);
int direct_convT(const sfh_convT3d_desc& p, int dtype, const int64_t* w_stride, const void* x, const void* w,
                 const void* bias, void* y, hipStream_t st);

}  // namespace sfh
