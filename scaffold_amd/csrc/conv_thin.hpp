// Host-side interface of the thin-channel convolution kernels (one channel count below MFMA tile size).
#pragma once
#include "common.hpp"
#include "gn_stats.hpp"

namespace sfh {

// Iterated volume (n, od, oh, ow) with a WIDE tensor of cw channels sampled at the iterated voxel,
// and J THIN samples per voxel:
//   K == 0: the J == ct channels of a thin tensor at the same voxel (1x1x1, stride 1, no padding);
//   K == 2 or 3: the K^3 taps of a one-channel tensor (ct == 1) of extents (td, th, tw) at
//                voxel*stride + tap*dilation - padding, zero outside.
struct ThinArgs {
  int n, od, oh, ow;
  int cw;
  int K, J, ct;
  int td, th, tw;
  int sd, sh, sw, pd, ph, pw, dd, dh, dw;
  // element strides of the weight for the wide channel, the thin channel (K == 0) and the taps
  int64_t ws_wide, ws_thin, ws_kd, ws_kh, ws_kw;
  // element strides of the weight gradient for the wide channel and the thin sample j
  int64_t so_wide, so_thin;
};

bool thin_supported(const ThinArgs& a, int dtype);
// out[v][c] = bias[c] + sum_j s_j(v) * W[j][c]
// `gn` (optional): also leave GroupNorm partials of the rounded output (gn_stats.hpp), gn->records per sample as
// thin_wide_out_gn_records says (0: this problem's kernel does not offer them).
int thin_wide_out_gn_records(const ThinArgs& a, int dtype, int groups);
int thin_wide_out(const ThinArgs& a, int dtype, const void* thin, const void* wt, const void* bias, void* out, hipStream_t st,
                  const GnPartialOut* gn = nullptr);
// out[v][j] = bias[j] + sum_c wide[v][c] * W[j][c]
int thin_out(const ThinArgs& a, int dtype, const void* wide, const void* wt, const void* bias, void* out, hipStream_t st);
// G[j][c] = sum_v s_j(v) * wide[v][c], through fp32 partial slices in `ws`
int thin_reduce_splits(const ThinArgs& a);
size_t thin_reduce_workspace_bytes(const ThinArgs& a, bool with_thin_sums = false);
// `thin_sums` (optional, where thin_reduce_offers_thin_sums says so): also the J sums of the thin tensor over all voxels,
// in gw's dtype, from the same pass (the bias gradient, when the thin tensor is the output gradient of a 1x1x1 convolution).
bool thin_reduce_offers_thin_sums(const ThinArgs& a, int dtype);
int thin_reduce(const ThinArgs& a, int dtype, const void* thin, const void* wide, void* gw, int gw_dtype, void* ws, hipStream_t st,
                void* thin_sums = nullptr);

}  // namespace sfh
