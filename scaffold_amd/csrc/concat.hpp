// The skip connection's channel concatenation, written straight into the slab the next convolution reads.
#pragma once
#include "common.hpp"

namespace sfh {

// out (N, halo_rows + rows + halo_rows, Ca + Cb) <- [a (N, rows, Ca) | b (N, rows, Cb)] in the interior, zeros in the faces.
// Both channel counts must fill whole 16-byte pieces and all pointers must be 16-byte aligned.
bool concat_supported(const sfh_concat_desc& p, int dtype);
int concat_forward(const sfh_concat_desc& p, int dtype, const void* a, const void* b, void* out, hipStream_t st);
// ga (N, rows, Ca), gb (N, rows, Cb) <- the two channel ranges of the interior of g (same layout as `out` above).
int concat_backward(const sfh_concat_desc& p, int dtype, const void* g, void* ga, void* gb, hipStream_t st);

}  // namespace sfh
