// Assembly of a depth shard's halo-extended slab: [planes from the lower neighbour | the shard | planes from the upper one].
#pragma once
#include "common.hpp"

namespace sfh {

// out (N, D + 2*halo, H, W, C) <- lo (N, halo, H, W, C) or zeros | x (N, D, H, W, C) | hi or zeros; all dense NDHWC.
int halo_assemble(const sfh_halo_desc& p, int dtype, const void* x, const void* lo, const void* hi, void* out, hipStream_t st);

}  // namespace sfh
