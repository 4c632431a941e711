// Assembly of a depth shard's halo-extended slab: [planes from the lower neighbour | the shard | planes from the upper one].
#pragma once
#include "common.hpp"

namespace sfh {

// out (N, D + 2*halo, H, W, C) <- lo (N, halo, H, W, C) or zeros | x (N, D, H, W, C) | hi or zeros; all dense NDHWC.
int halo_assemble(const sfh_halo_desc& p, int dtype, const void* x, const void* lo, const void* hi, void* out, hipStream_t st);

// lo_out (N, halo, H, W, C) <- x[:, :halo], hi_out <- x[:, D - halo:] for x (N, D, H, W, C); either output may be null.
int halo_pack(const sfh_halo_desc& p, int dtype, const void* x, void* lo_out, void* hi_out, hipStream_t st);

// In place on g (N, D, H, W, C): g[:, :halo] += lo_in, g[:, D - halo:] += hi_in; either input may be null. D >= 2 * halo.
int halo_accumulate(const sfh_halo_desc& p, int dtype, void* g, const void* lo_in, const void* hi_in, hipStream_t st);

}  // namespace sfh
