// Deterministic reductions shared by the weight-gradient kernels, and the bias gradient.
#pragma once
#include "common.hpp"

namespace sfh {

// out[e] = sum over s < splits, in index order within fixed groups, of part[s * nelem + e]; one rounding to `dtype`.
int sum_slices(int dtype, const float* part, void* out, int64_t nelem, int splits, hipStream_t st);
// Two such sums from one launch (same bits as two calls of sum_slices).
int sum_slices_two(int dtype, const float* part_a, void* out_a, int64_t nelem_a, int splits_a, const float* part_b, void* out_b,
                   int64_t nelem_b, int splits_b, hipStream_t st);

// out[e] = bias[e % channels] + sum over s < splits, in index order, of part[s * nelem + e]; nelem a multiple of 4.
// `out2` (optional): the result as two tensors cut at channel out2->first of every row of `channels`.
int sum_slices_bias(int dtype, const float* part, const void* bias, void* out, int64_t nelem, int channels, int splits,
                    hipStream_t st, const ChannelPair* out2 = nullptr);

// The same with GroupNorm partials of the rounded result (gn_stats.hpp) for n samples of sample_elems elements each:
// `records` per sample as sum_slices_bias_stats_records says (0: not offered for this shape; 16-bit outputs only).
struct GnPartialOut;
int sum_slices_bias_stats_records(int64_t sample_elems, int channels, int groups);
int sum_slices_bias_stats(int dtype, const float* part, const void* bias, void* out, int n, int64_t sample_elems, int channels,
                          int splits, const GnPartialOut& gn, hipStream_t st);

// gb[c] = sum over rows of g[row * channels + c] for a dense (rows, channels) tensor of `dtype`; fp32
// accumulation through partial slices in `ws`, result rounded once to `out_dtype`.
size_t bias_grad_workspace_bytes(int64_t rows, int channels);
int bias_grad(int dtype, int out_dtype, const void* g, int64_t rows, int channels, void* gb, void* ws, hipStream_t st);

}  // namespace sfh
