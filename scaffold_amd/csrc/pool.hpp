// 2x2x2, stride-2 max pooling of channels-last volumes (the U-Net's down-sampling step) and its gradient.
#pragma once
#include "common.hpp"

namespace sfh {

// y[n][od][oh][ow][c] = max over the 2x2x2 cell; idx holds, per output element, which of the cell's eight voxels
// (kd * 4 + kh * 2 + kw) supplied it. Odd trailing planes, rows and columns are dropped.
// `halo_elems` > 0 (one sample): y is the interior of a depth slab with that many elements of face on either side,
// which the launch zeroes too.
int maxpool2_fwd(const sfh_pool_desc& p, int dtype, const void* x, void* y, uint8_t* idx, hipStream_t st, int64_t halo_elems = 0);

// gx = gy routed to the voxel idx names, zero elsewhere (including dropped odd planes). Writes all of gx.
// gx = the pooling gradient (+ `add`, a tensor of the input's shape, when given)
int maxpool2_bwd(const sfh_pool_desc& p, int dtype, const void* gy, const uint8_t* idx, const void* add, void* gx, hipStream_t st);

}  // namespace sfh
