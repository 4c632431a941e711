// Loss head of the U-Net train step, fused: fp32 log-softmax over the class logits of every voxel, the
// (optionally class-weighted) cross-entropy sum with its normaliser, and the soft-Dice sums per (sample, class)
// in ONE pass over the logits; the backward is one more pass. This is the block ScaFFold/utils/trainer.py:634-663
// builds from torch ops (log_softmax -> nll_loss(reduction="none").sum() / normaliser, ScaFFold/utils/losses.py:
// 119-214; exp -> Dice sums -> (2I + eps) / (P + T + eps), ScaFFold/utils/dice_score.py:101-136; loss =
// CE + 1 - mean foreground Dice, trainer.py:331-333,660-663). It is bandwidth-bound: 22 B of bf16 logits and an
// 8-byte label per voxel at 11 classes.
//
// No atomics: every workgroup leaves its partial sums in its own slot and one workgroup adds the slots in a
// fixed order (the reference avoids the atomic fused reduction for the same reason, losses.py:156-160).
#include "loss.hpp"

namespace sfh {
namespace {

constexpr int kBlock = 256;

template <typename T> __device__ __forceinline__ float ld(const T* p) { return to_float(*p); }

__device__ __forceinline__ float wave_sum_all(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;  // lane 0 holds the sum
}

// A tile's logits are one contiguous byte range whatever the class count (11 classes: 22-byte rows): it moves between
// global memory and LDS in 16-byte pieces when the range starts on a 16-byte boundary (`vec`), element by element else.
template <typename T>
__device__ __forceinline__ void tile_in(T* tile, const T* __restrict__ src, int nelem, bool vec) {
  const int tid = threadIdx.x;
  if (vec) {
    constexpr int E = 16 / (int)sizeof(T);
    const int npiece = nelem / E;
    for (int i = tid; i < npiece; i += kBlock) reinterpret_cast<uint4*>(tile)[i] = reinterpret_cast<const uint4*>(src)[i];
    for (int i = npiece * E + tid; i < nelem; i += kBlock) tile[i] = src[i];
  } else {
    for (int i = tid; i < nelem; i += kBlock) tile[i] = src[i];
  }
}
template <typename T>
__device__ __forceinline__ void tile_out(T* __restrict__ dst, const T* tile, int nelem, bool vec) {
  const int tid = threadIdx.x;
  if (vec) {
    constexpr int E = 16 / (int)sizeof(T);
    const int npiece = nelem / E;
    for (int i = tid; i < npiece; i += kBlock) reinterpret_cast<uint4*>(dst)[i] = reinterpret_cast<const uint4*>(tile)[i];
    for (int i = npiece * E + tid; i < nelem; i += kBlock) dst[i] = tile[i];
  } else {
    for (int i = tid; i < nelem; i += kBlock) dst[i] = tile[i];
  }
}

// Quantities per sample: inter[c], psum[c], tsum[c] (3 * C), then the two launch-wide ones: ce_sum, normaliser.
template <typename T, int CMAX>
__global__ void __launch_bounds__(kBlock) ce_dice_partial(const T* __restrict__ logits, const int64_t* __restrict__ labels,
                                                          const float* __restrict__ cw, float* __restrict__ part, int64_t S, int C,
                                                          int nsplit, int64_t per_split, int vec) {
  extern __shared__ __align__(16) char smem_raw[];
  T* tile = reinterpret_cast<T*>(smem_raw);  // kBlock voxels x C logits
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = blockIdx.y, split = blockIdx.x;
  const T* src = logits + (int64_t)n * S * C;
  const int64_t* lab = labels + (int64_t)n * S;
  float inter[CMAX], psum[CMAX], tsum[CMAX], ce = 0.f, norm = 0.f;
#pragma unroll
  for (int c = 0; c < CMAX; ++c) inter[c] = psum[c] = tsum[c] = 0.f;
  const int64_t begin = (int64_t)split * per_split;
  int64_t end = begin + per_split;
  if (end > S) end = S;
  for (int64_t v0 = begin; v0 < end; v0 += kBlock) {
    const int nv = (int)((end - v0) < kBlock ? (end - v0) : kBlock);
    __syncthreads();
    tile_in<T>(tile, src + v0 * C, nv * C, vec != 0);
    __syncthreads();
    if (tid < nv) {
      float x[CMAX];
      float m = -INFINITY;
#pragma unroll
      for (int c = 0; c < CMAX; ++c) {
        x[c] = c < C ? to_float(tile[tid * C + c]) : -INFINITY;
        m = fmaxf(m, x[c]);
      }
      float s = 0.f;
#pragma unroll
      for (int c = 0; c < CMAX; ++c) {
        x[c] = c < C ? expf(x[c] - m) : 0.f;  // x now holds exp(logit - max)
        s += x[c];
      }
      const float inv = 1.f / s, logs = logf(s);
      const int64_t y = lab[v0 + tid];
      const bool valid = y >= 0 && y < C;
#pragma unroll
      for (int c = 0; c < CMAX; ++c) {
        const float p = x[c] * inv;
        const bool hit = valid && c == (int)y;
        psum[c] += p;
        inter[c] += hit ? p : 0.f;
        tsum[c] += hit ? 1.f : 0.f;
      }
      if (valid) {
        const float w = cw != nullptr ? cw[y] : 1.f;
        // -log p_y = log(sum) - (logit_y - max)
        ce += w * (logs - (to_float(tile[tid * C + (int)y]) - m));
        norm += w;
      }
    }
  }
  // workgroup totals: every quantity through the wavefront tree, the wave totals parked in LDS, then one thread per
  // quantity adds the four wave totals in order (one barrier for all 3 C + 2 quantities)
  float* dst = part + ((int64_t)n * nsplit + split) * (3 * C + 2);
  __syncthreads();  // the tile is consumed: its LDS holds the wave totals now
  float* wave_tot = reinterpret_cast<float*>(smem_raw);  // [4][3 * CMAX + 2]
  constexpr int Q = 3 * CMAX + 2;
  auto park = [&](float v, int slot) {
    v = wave_sum_all(v);
    if (lane == 0) wave_tot[wave * Q + slot] = v;
  };
#pragma unroll
  for (int c = 0; c < CMAX; ++c) {
    park(inter[c], c);
    park(psum[c], CMAX + c);
    park(tsum[c], 2 * CMAX + c);
  }
  park(ce, 3 * CMAX);
  park(norm, 3 * CMAX + 1);
  __syncthreads();
  if (tid < Q) {
    const int q = tid < 3 * CMAX ? tid / CMAX : 3, c = tid < 3 * CMAX ? tid % CMAX : tid - 3 * CMAX;
    if (q == 3 || c < C) {
      const float t = (wave_tot[tid] + wave_tot[Q + tid]) + (wave_tot[2 * Q + tid] + wave_tot[3 * Q + tid]);
      dst[q == 3 ? 3 * C + c : q * C + c] = t;
    }
  }
}

// Slots lane, lane + 64, ... of a quantity (stride `q` floats between slots), added in that order with sixteen loads in
// flight at a time (one slot per trip to memory made a launch of 1024 slots sixteen trips long).
__device__ __forceinline__ float lane_slots_sum(const float* __restrict__ src, int slots, int q, int lane) {
  float s = 0.f;
  int sp = lane;
  for (; sp + 15 * 64 < slots; sp += 16 * 64) {
    float v[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) v[k] = src[(int64_t)(sp + 64 * k) * q];
#pragma unroll
    for (int k = 0; k < 16; ++k) s += v[k];
  }
  for (; sp < slots; sp += 64) s += src[(int64_t)sp * q];
  return s;
}

// One 64-lane workgroup per quantity: lane l adds slots l, l + 64, ... and the lane totals meet in a fixed tree.
// stats: inter[N][C] | psum[N][C] | tsum[N][C] | ce_sum | normaliser
__global__ void __launch_bounds__(64) ce_dice_sum(const float* __restrict__ part, float* __restrict__ stats, int N, int C, int nsplit,
                                                  int unweighted, float count) {
  const int Q = 3 * C + 2;
  const int b = blockIdx.x, lane = threadIdx.x;
  float s = 0.f;
  int dst;
  if (b < N * 3 * C) {
    const int n = b / (3 * C), q = b - n * 3 * C;
    s = lane_slots_sum(part + (int64_t)n * nsplit * Q + q, nsplit, Q, lane);
    dst = (q / C) * N * C + n * C + q % C;
  } else {
    const int q = 3 * C + (b - N * 3 * C);  // ce_sum or normaliser, over all samples
    s = lane_slots_sum(part + q, N * nsplit, Q, lane);
    dst = b;
  }
  s = wave_sum_all(s);
  if (lane == 0) {
    if (b == N * 3 * C + 1 && unweighted) s = count;  // the normaliser of the unweighted mean is the voxel count
    stats[dst] = s;
  }
}

__global__ void __launch_bounds__(64) ce_dice_scalar(const float* __restrict__ stats, float* __restrict__ loss, int N, int C, float eps) {
  // one lane per (sample, foreground class) pass; the Dice terms meet in the fixed wavefront tree
  const float* inter = stats;
  const float* psum = stats + N * C;
  const float* tsum = stats + 2 * N * C;
  // (asked for now: thread 0 needs them after the tree)
  const float ce_sum = stats[N * 3 * C], normaliser = stats[N * 3 * C + 1];
  float dice = 0.f;
  for (int i = threadIdx.x; i < N * C; i += 64) {
    const int c = i % C;
    if (c >= 1) {
      const float two_i = 2.f * inter[i];
      float sets = psum[i] + tsum[i];
      if (sets == 0.f) sets = two_i;
      dice += (two_i + eps) / (sets + eps);
    }
  }
  dice = wave_sum_all(dice);
  if (threadIdx.x == 0) {
    dice /= (float)(N * (C - 1));
    const float ce = ce_sum / fmaxf(normaliser, 1.1920929e-07f);
    loss[0] = ce + (1.f - dice);
  }
}

// dlogits[v][j] = gl * ( w_y / normaliser * (p_j - [j == y])  +  p_j * (g_j - sum_c g_c p_c) ),
// g_c = -(1 / (N (C-1))) * d dice_c / d p_c = -(1 / (N (C-1))) * ([c == y] * 2 / den_c - (2 I_c + eps) / den_c^2), g_0 = 0.
template <typename T, int CMAX>
__global__ void __launch_bounds__(kBlock) ce_dice_backward(const T* __restrict__ logits, const int64_t* __restrict__ labels,
                                                           const float* __restrict__ cw, const float* __restrict__ stats,
                                                           const float* __restrict__ grad_loss, T* __restrict__ dlogits, int64_t S,
                                                           int N, int C, float eps, int64_t per_split, int vec) {
  extern __shared__ __align__(16) char smem_raw[];
  T* tile = reinterpret_cast<T*>(smem_raw);
  __shared__ float ca[CMAX], cb[CMAX];
  const int tid = threadIdx.x;
  const int n = blockIdx.y, split = blockIdx.x;
  const float gl = grad_loss[0];
  if (tid < CMAX) {
    float a = 0.f, b = 0.f;
    if (tid >= 1 && tid < C) {
      const float two_i = 2.f * stats[n * C + tid];
      float sets = stats[N * C + n * C + tid] + stats[2 * N * C + n * C + tid];
      if (sets == 0.f) sets = two_i;
      const float den = sets + eps, k = -gl / (float)(N * (C - 1));
      a = k * 2.f / den;
      b = k * (two_i + eps) / (den * den);
    }
    ca[tid] = a;
    cb[tid] = b;
  }
  const float ce_scale = gl / fmaxf(stats[N * 3 * C + 1], 1.1920929e-07f);
  const T* src = logits + (int64_t)n * S * C;
  T* dst = dlogits + (int64_t)n * S * C;
  const int64_t* lab = labels + (int64_t)n * S;
  const int64_t begin = (int64_t)split * per_split;
  int64_t end = begin + per_split;
  if (end > S) end = S;
  for (int64_t v0 = begin; v0 < end; v0 += kBlock) {
    const int nv = (int)((end - v0) < kBlock ? (end - v0) : kBlock);
    __syncthreads();
    tile_in<T>(tile, src + v0 * C, nv * C, vec != 0);
    __syncthreads();
    if (tid < nv) {
      float p[CMAX];
      float m = -INFINITY;
#pragma unroll
      for (int c = 0; c < CMAX; ++c) {
        p[c] = c < C ? to_float(tile[tid * C + c]) : -INFINITY;
        m = fmaxf(m, p[c]);
      }
      float s = 0.f;
#pragma unroll
      for (int c = 0; c < CMAX; ++c) {
        p[c] = c < C ? expf(p[c] - m) : 0.f;
        s += p[c];
      }
      const float inv = 1.f / s;
      const int64_t y = lab[v0 + tid];
      const bool valid = y >= 0 && y < C;
      float g[CMAX], dot = 0.f, wy = 0.f;
#pragma unroll
      for (int c = 0; c < CMAX; ++c) {
        p[c] *= inv;
        const bool hit = valid && c == (int)y;
        g[c] = (hit ? ca[c] : 0.f) - cb[c];
        dot = fmaf(g[c], p[c], dot);
        if (hit) wy = cw != nullptr ? cw[c] : 1.f;
      }
      const float cs = ce_scale * wy;
#pragma unroll
      for (int c = 0; c < CMAX; ++c) {
        if (c < C) {
          const bool hit = valid && c == (int)y;
          const float d = fmaf(p[c], g[c] - dot, cs * (p[c] - (hit ? 1.f : 0.f)));
          tile[tid * C + c] = elem<T>::from_float(d);
        }
      }
    }
    __syncthreads();
    tile_out<T>(dst + v0 * C, tile, nv * C, vec != 0);
  }
}

struct LossPlan { int nsplit; int64_t per_split; };

LossPlan loss_plan(const sfh_loss_desc& p) {
  LossPlan pl;
  int64_t want = cdiv(4 * kComputeUnits, p.n);
  const int64_t tiles = cdiv(p.spatial, kBlock);
  if (want > tiles) want = tiles;
  if (want < 1) want = 1;
  pl.per_split = cdiv(tiles, want) * kBlock;
  pl.nsplit = (int)cdiv(p.spatial, pl.per_split);
  return pl;
}

// Every tile starts kBlock * classes elements after the previous one and every sample spatial * classes elements after
// the previous one: all tiles start on 16-byte boundaries when those two strides and the base pointers do.
template <typename T>
int tiles_on_16_bytes(const sfh_loss_desc& p, const void* a, const void* b) {
  const bool ok = (reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(b) & 15) == 0 &&
                  ((size_t)kBlock * p.classes * sizeof(T)) % 16 == 0 && (p.n == 1 || ((size_t)p.spatial * p.classes * sizeof(T)) % 16 == 0);
  return ok ? 1 : 0;
}

template <typename T, int CMAX>
int fwd_typed(const sfh_loss_desc& p, const void* logits, const int64_t* labels, const float* cw, float* loss, float* stats,
              float* ws, hipStream_t st) {
  const LossPlan pl = loss_plan(p);
  size_t lds = (size_t)kBlock * p.classes * sizeof(T);
  if (lds < 4 * (3 * CMAX + 2) * sizeof(float)) lds = 4 * (3 * CMAX + 2) * sizeof(float);  // the fold at the end reuses the tile
  hipLaunchKernelGGL((ce_dice_partial<T, CMAX>), dim3(pl.nsplit, p.n), dim3(kBlock), lds, st, (const T*)logits, labels, cw, ws,
                     p.spatial, p.classes, pl.nsplit, pl.per_split, tiles_on_16_bytes<T>(p, logits, nullptr));
  if (int rc = check_launch("ce_dice_partial")) return rc;
  hipLaunchKernelGGL(ce_dice_sum, dim3(p.n * 3 * p.classes + 2), dim3(64), 0, st, ws, stats, p.n, p.classes, pl.nsplit,
                     cw == nullptr ? 1 : 0, (float)p.n * (float)p.spatial);
  if (int rc = check_launch("ce_dice_sum")) return rc;
  hipLaunchKernelGGL(ce_dice_scalar, dim3(1), dim3(64), 0, st, stats, loss, p.n, p.classes, p.eps);
  return check_launch("ce_dice_scalar");
}

template <typename T, int CMAX>
int bwd_typed(const sfh_loss_desc& p, const void* logits, const int64_t* labels, const float* cw, const float* stats,
              const float* grad_loss, void* dlogits, hipStream_t st) {
  const LossPlan pl = loss_plan(p);
  const size_t lds = (size_t)kBlock * p.classes * sizeof(T);
  hipLaunchKernelGGL((ce_dice_backward<T, CMAX>), dim3(pl.nsplit, p.n), dim3(kBlock), lds, st, (const T*)logits, labels, cw, stats,
                     grad_loss, (T*)dlogits, p.spatial, p.n, p.classes, p.eps, pl.per_split, tiles_on_16_bytes<T>(p, logits, dlogits));
  return check_launch("ce_dice_backward");
}

}  // namespace

bool loss_supported(const sfh_loss_desc& p) {
  return p.n >= 1 && p.classes >= 2 && p.classes <= 32 && p.spatial >= 1 && (int64_t)p.n * cdiv(p.spatial, kBlock) < 0x7fffffffLL;
}

size_t loss_workspace_bytes(const sfh_loss_desc& p) {
  return (size_t)p.n * loss_plan(p).nsplit * (3 * p.classes + 2) * sizeof(float);
}

#define SFH_LOSS_DISPATCH(fn, ...)                                               \
  if (p.classes <= 12) {                                                         \
    if (dtype == SFH_BF16) return fn<bf16_t, 12>(__VA_ARGS__);                   \
    if (dtype == SFH_FP16) return fn<fp16_t, 12>(__VA_ARGS__);                   \
    return fn<float, 12>(__VA_ARGS__);                                           \
  }                                                                              \
  if (p.classes <= 16) {                                                         \
    if (dtype == SFH_BF16) return fn<bf16_t, 16>(__VA_ARGS__);                   \
    if (dtype == SFH_FP16) return fn<fp16_t, 16>(__VA_ARGS__);                   \
    return fn<float, 16>(__VA_ARGS__);                                           \
  }                                                                              \
  if (dtype == SFH_BF16) return fn<bf16_t, 32>(__VA_ARGS__);                     \
  if (dtype == SFH_FP16) return fn<fp16_t, 32>(__VA_ARGS__);                     \
  return fn<float, 32>(__VA_ARGS__);

int loss_forward(const sfh_loss_desc& p, int dtype, const void* logits, const int64_t* labels, const float* cw, float* loss,
                 float* stats, void* ws, hipStream_t st) {
  SFH_LOSS_DISPATCH(fwd_typed, p, logits, labels, cw, loss, stats, (float*)ws, st)
}

int loss_backward(const sfh_loss_desc& p, int dtype, const void* logits, const int64_t* labels, const float* cw, const float* stats,
                  const float* grad_loss, void* dlogits, hipStream_t st) {
  SFH_LOSS_DISPATCH(bwd_typed, p, logits, labels, cw, stats, grad_loss, dlogits, st)
}

}  // namespace sfh
