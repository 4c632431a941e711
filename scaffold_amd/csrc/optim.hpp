// Gradient-norm clipping and the Adam update of many fp32 tensors in two passes over the gradients' and the
// parameters' bytes.
#pragma once
#include "common.hpp"

namespace sfh {

constexpr int kOptimChunk = 8192;  // elements one workgroup handles

// Number of fp32 slots pass 1 writes (one per chunk of every tensor).
int64_t optim_chunks(int ntensors, const int64_t* numel);

// Pass 1: slot[c] = sum of g^2 over chunk c, chunks numbered tensor by tensor. Also advances *step by one.
int optim_grad_sumsq(int ntensors, const float* const* grads, const int64_t* numel, float* slots, float* step, hipStream_t st);

// Pass 2: every workgroup adds the slots in a fixed order, derives the clipping factor
// min(1, max_norm / (sqrt(sum) + 1e-6)) (1 when max_norm <= 0), and applies Adam to its chunk. shadow (may be null,
// entries may be null) receives the updated parameter rounded to shadow_dtype. grad_norm (may be null) gets sqrt(sum).
int optim_clip_adam(const sfh_adam_desc& d, int ntensors, float* const* params, const float* const* grads, float* const* exp_avg,
                    float* const* exp_avg_sq, void* const* shadow, const int64_t* numel, const float* slots, int nslots,
                    const float* step, float* grad_norm, hipStream_t st);

}  // namespace sfh
