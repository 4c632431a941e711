// Host-side interface of the fused cross-entropy + soft-Dice loss head.
#pragma once
#include "common.hpp"

namespace sfh {

bool loss_supported(const sfh_loss_desc& p);
size_t loss_workspace_bytes(const sfh_loss_desc& p);
// stats (N * 3 * C + 2 floats): inter[N][C] | psum[N][C] | tsum[N][C] | ce_sum | normaliser -- what the backward needs.
int loss_forward(const sfh_loss_desc& p, int dtype, const void* logits, const int64_t* labels, const float* class_weight,
                 float* loss, float* stats, void* ws, hipStream_t st);
int loss_backward(const sfh_loss_desc& p, int dtype, const void* logits, const int64_t* labels, const float* class_weight,
                  const float* stats, const float* grad_loss, void* dlogits, hipStream_t st);

}  // namespace sfh
