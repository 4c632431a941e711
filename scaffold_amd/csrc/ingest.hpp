// A dataset shard as it lies on disk, turned into what the first convolution and the loss read.
#pragma once
#include "common.hpp"

namespace sfh {

constexpr int kIngestMaxChannels = 4;

// x (N, halo_rows + rows + halo_rows, C) of `dtype` <- volume (N, C, rows) fp32, interior rows; zeros in the faces.
// labels (N, rows) int64 <- mask (N, rows) of 16-bit integers (unsigned or signed), when both are given.
int shard_ingest(const sfh_ingest_desc& p, int dtype, const float* volume, const void* mask, void* x, int64_t* labels,
                 hipStream_t st);

}  // namespace sfh
