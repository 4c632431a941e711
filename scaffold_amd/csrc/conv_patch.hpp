// Host-side interface of the MFMA kernels for 2x2x2, stride-2, unpadded convolutions: the U-Net's
// transposed up-convolution and its two gradients (bf16 / fp16).
#pragma once
#include "common.hpp"

namespace sfh {

// A BIG volume (cbig channels, extents bd x bh x bw) and a SMALL one (csmall channels, extents
// sd x sh x sw, 2 * s? <= b?): small voxel v and tap (a,b,c) in {0,1}^3 meet big voxel 2v + tap.
//   gather  : small[v][cs] = bias[cs] + sum_{tap,cb} big[2v+tap][cb] * W(cs, cb, tap)     (conv, stride 2)
//   scatter : big[2v+tap][cb] = bias[cb] + sum_cs small[v][cs] * W(cs, cb, tap)            (transposed conv)
//   reduce  : G[cs][tap][cb] = sum_v small[v][cs] * big[2v+tap][cb]                         (weight gradient)
struct PatchArgs {
  int n;
  int cbig, bd, bh, bw;
  int csmall, sd, sh, sw;
};

bool patch_supported(const PatchArgs& a, int dtype);         // gather and scatter
bool patch_reduce_supported(const PatchArgs& a, int dtype);
// `packed` holds the weight in MFMA fragment order [produced/32][reduced/32][tap][kstep][lane][8]
// (mfma_pack_weight): produced = csmall for gather, cbig for scatter.
int patch_gather(const PatchArgs& a, int dtype, const void* big, const void* packed, const void* bias, void* small, hipStream_t st);
// `halo_elems` > 0 (one sample): big is the interior of a depth slab with that many elements of face on either side,
// which the launch zeroes too.
int patch_scatter(const PatchArgs& a, int dtype, const void* small, const void* packed, const void* bias, void* big, hipStream_t st,
                  int64_t halo_elems = 0);
int patch_reduce_splits(const PatchArgs& a);
size_t patch_reduce_workspace_bytes(const PatchArgs& a, bool with_bias = false);
// g: dense [csmall][8][cbig] in the element type, from fp32 partial slices in ws summed in split order.
// gb (optional, big extents exactly twice the small ones): also the sum of `big` over all voxels per channel, cbig
// elements of g's type -- the bias gradient of the transposed convolution -- from the same pass over `big`.
int patch_reduce(const PatchArgs& a, int dtype, const void* small, const void* big, void* g, int g_dtype, void* ws, hipStream_t st,
                 void* gb = nullptr);

}  // namespace sfh
