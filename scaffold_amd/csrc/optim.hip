// clip_grad_norm_(max_norm) + Adam over a list of fp32 tensors (ScaFFold/utils/trainer.py:678-694 with the optimizer
// of trainer.py:268-274), as two streaming passes: the squared gradient norm into fixed slots, then one kernel that
// folds the slots in a fixed order, scales the gradient on the fly and updates parameter and both moments. The
// gradients are read twice and never rewritten; parameter, moments are read and written once: 20 B + 12 B per
// element (+2 B for an optional half-precision copy of the parameter that saves the next step's cast).
// Tensor pointers travel by value in the kernel arguments (48 tensors per launch), so a captured graph holds them.
#include "optim.hpp"
#include "vec_io.hpp"

namespace sfh {

namespace {

constexpr int kBlock = 256;
constexpr int kMaxTensors = 64;  // per launch: the table travels in the kernel arguments (4 KiB at most); 64 hold a whole 5-level U-Net

struct SumsqTable {
  const float* g[kMaxTensors];
  int64_t numel[kMaxTensors];
  int chunk_start[kMaxTensors + 1];  // chunks of this launch, numbered from 0
  int n;
};

struct AdamTable {
  float* p[kMaxTensors];
  const float* g[kMaxTensors];
  float* m[kMaxTensors];
  float* v[kMaxTensors];
  void* shadow[kMaxTensors];
  int64_t numel[kMaxTensors];
  int chunk_start[kMaxTensors + 1];
  int n;
};

static_assert(sizeof(AdamTable) + 128 <= 4096, "the table and the other arguments fit the kernel argument segment");

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

// Fixed-order sum over the 256 threads; every thread gets the result.
__device__ __forceinline__ float block_sum(float v, float* red4) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red4[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red4[0] + red4[1]) + (red4[2] + red4[3]);
}

template <typename Table>
__device__ __forceinline__ int find_tensor(const Table& t, int chunk) {
  int i = 0;
  while (i + 1 < t.n && t.chunk_start[i + 1] <= chunk) ++i;
  return i;
}

__global__ void __launch_bounds__(kBlock) grad_sumsq_kernel(SumsqTable t, float* __restrict__ slots, float* step, int bump_step) {
  __shared__ float red4[4];
  const int chunk = blockIdx.x;
  const int ti = find_tensor(t, chunk);
  const int64_t begin = (int64_t)(chunk - t.chunk_start[ti]) * kOptimChunk;
  const int64_t len = min((int64_t)kOptimChunk, t.numel[ti] - begin);
  const float* g = t.g[ti] + begin;
  float s = 0.f;
  if ((reinterpret_cast<uintptr_t>(g) & 15) == 0) {
    const int64_t nvec = len / 4;
    for (int64_t i = threadIdx.x; i < nvec; i += kBlock) {
      const float4 q = reinterpret_cast<const float4*>(g)[i];
      s += (q.x * q.x + q.y * q.y) + (q.z * q.z + q.w * q.w);
    }
    for (int64_t i = nvec * 4 + threadIdx.x; i < len; i += kBlock) s += g[i] * g[i];
  } else {
    for (int64_t i = threadIdx.x; i < len; i += kBlock) s += g[i] * g[i];
  }
  s = block_sum(s, red4);
  if (threadIdx.x == 0) {
    slots[chunk] = s;
    if (bump_step && chunk == 0) *step += 1.f;
  }
}

struct AdamCoef {
  float lr, beta1, beta2, eps, weight_decay, max_norm;
};

template <typename TS>
__device__ __forceinline__ void write_shadow(TS* s, int64_t i, float p) { s[i] = elem<TS>::from_float(p); }

template <int SHADOW>  // 0 none, 1 bf16, 2 fp16
__global__ void __launch_bounds__(kBlock) clip_adam_kernel(AdamTable t, AdamCoef c, const float* __restrict__ slots, int nslots,
                                                           int slot_base, const float* __restrict__ step_ptr, float* grad_norm) {
  __shared__ float red4[4];
  // every workgroup folds all slots, the same way: four loads in flight per lane (one after the other they were a chain
  // of a dozen dependent trips to L2 in front of every workgroup's own work), combined in a fixed order
  float t0 = 0.f, t1 = 0.f, t2 = 0.f, t3 = 0.f;
  int i = threadIdx.x;
  for (; i + 3 * kBlock < nslots; i += 4 * kBlock) {
    const float a0 = slots[i], a1 = slots[i + kBlock], a2 = slots[i + 2 * kBlock], a3 = slots[i + 3 * kBlock];
    t0 += a0; t1 += a1; t2 += a2; t3 += a3;
  }
  for (; i < nslots; i += kBlock) t0 += slots[i];
  float total = block_sum((t0 + t1) + (t2 + t3), red4);
  const float norm = sqrtf(total);
  float scale = 1.f;
  if (c.max_norm > 0.f) scale = fminf(c.max_norm / (norm + 1e-6f), 1.f);
  if (grad_norm != nullptr && blockIdx.x == 0 && slot_base == 0 && threadIdx.x == 0) *grad_norm = norm;

  const float step = *step_ptr;
  const float bc1 = 1.f - powf(c.beta1, step);
  const float bc2_sqrt = sqrtf(1.f - powf(c.beta2, step));
  const float step_size = c.lr / bc1;

  const int chunk = blockIdx.x;
  const int ti = find_tensor(t, chunk);
  const int64_t begin = (int64_t)(chunk - t.chunk_start[ti]) * kOptimChunk;
  const int64_t len = min((int64_t)kOptimChunk, t.numel[ti] - begin);
  float* p = t.p[ti] + begin;
  const float* g = t.g[ti] + begin;
  float* m = t.m[ti] + begin;
  float* v = t.v[ti] + begin;
  void* sh = t.shadow[ti];

  auto update = [&](float& pe, float ge, float& me, float& ve) {
    float grad = ge * scale;
    if (c.weight_decay != 0.f) grad = fmaf(c.weight_decay, pe, grad);
    me = me + (1.f - c.beta1) * (grad - me);
    ve = c.beta2 * ve + (1.f - c.beta2) * grad * grad;
    const float denom = sqrtf(ve) / bc2_sqrt + c.eps;
    pe = pe - step_size * (me / denom);
  };

  const bool aligned = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(m) |
                         reinterpret_cast<uintptr_t>(v)) & 15) == 0 &&
                       (SHADOW == 0 || sh == nullptr || ((reinterpret_cast<uintptr_t>(sh) + 2 * begin) & 7) == 0);
  int64_t done = 0;
  if (aligned) {
    const int64_t nvec = len / 4;
    // Four of a thread's pieces at a time, all sixteen loads in flight before the first update: a launch of a few dozen
    // chunks (the tail of the parameter list) has nothing else on its CUs to cover a trip to memory, and one piece
    // per trip made its chunk of 8192 elements a chain of eight (15.8 us for half a megabyte of parameters).
    constexpr int U = 4;
    for (int64_t i0 = threadIdx.x; i0 < nvec; i0 += U * kBlock) {
      float4 pq[U], gq[U], mq[U], vq[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = i0 + u * kBlock;
        if (i < nvec) {
          pq[u] = reinterpret_cast<float4*>(p)[i];
          gq[u] = reinterpret_cast<const float4*>(g)[i];
          mq[u] = reinterpret_cast<float4*>(m)[i];
          vq[u] = reinterpret_cast<float4*>(v)[i];
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int64_t i = i0 + u * kBlock;
        if (i < nvec) {
          update(pq[u].x, gq[u].x, mq[u].x, vq[u].x);
          update(pq[u].y, gq[u].y, mq[u].y, vq[u].y);
          update(pq[u].z, gq[u].z, mq[u].z, vq[u].z);
          update(pq[u].w, gq[u].w, mq[u].w, vq[u].w);
          reinterpret_cast<float4*>(p)[i] = pq[u];
          reinterpret_cast<float4*>(m)[i] = mq[u];
          reinterpret_cast<float4*>(v)[i] = vq[u];
          if (SHADOW != 0 && sh != nullptr) {
            uint2 pk;
            if (SHADOW == 1) { pk.x = pack_bf16x2(pq[u].x, pq[u].y); pk.y = pack_bf16x2(pq[u].z, pq[u].w); }
            else { pk.x = pack_fp16x2(pq[u].x, pq[u].y); pk.y = pack_fp16x2(pq[u].z, pq[u].w); }
            reinterpret_cast<uint2*>(static_cast<char*>(sh) + 2 * begin)[i] = pk;
          }
        }
      }
    }
    done = nvec * 4;
  }
  for (int64_t i = done + threadIdx.x; i < len; i += kBlock) {
    float pe = p[i], me = m[i], ve = v[i];
    update(pe, g[i], me, ve);
    p[i] = pe; m[i] = me; v[i] = ve;
    if (SHADOW == 1 && sh != nullptr) write_shadow(static_cast<bf16_t*>(sh) + begin, i, pe);
    if (SHADOW == 2 && sh != nullptr) write_shadow(static_cast<fp16_t*>(sh) + begin, i, pe);
  }
}

int64_t chunks_of(int64_t numel) { return cdiv(numel, kOptimChunk); }

}  // namespace

int64_t optim_chunks(int ntensors, const int64_t* numel) {
  int64_t total = 0;
  for (int i = 0; i < ntensors; ++i) total += chunks_of(numel[i]);
  return total;
}

int optim_grad_sumsq(int ntensors, const float* const* grads, const int64_t* numel, float* slots, float* step, hipStream_t st) {
  int64_t slot_base = 0;
  bool first = true;
  for (int base = 0; base < ntensors; base += kMaxTensors) {
    SumsqTable t{};
    t.n = ntensors - base < kMaxTensors ? ntensors - base : kMaxTensors;
    int64_t chunks = 0;
    for (int i = 0; i < t.n; ++i) {
      t.g[i] = grads[base + i];
      t.numel[i] = numel[base + i];
      t.chunk_start[i] = (int)chunks;
      chunks += chunks_of(numel[base + i]);
    }
    t.chunk_start[t.n] = (int)chunks;
    if (chunks > 0x7fffffff) return fail(SFH_ERR_UNSUPPORTED, "adam: too many chunks in one launch");
    hipLaunchKernelGGL(grad_sumsq_kernel, dim3((unsigned)chunks), dim3(kBlock), 0, st, t, slots + slot_base, step, first ? 1 : 0);
    if (int rc = check_launch("grad_sumsq_kernel")) return rc;
    first = false;
    slot_base += chunks;
  }
  return SFH_OK;
}

int optim_clip_adam(const sfh_adam_desc& d, int ntensors, float* const* params, const float* const* grads, float* const* exp_avg,
                    float* const* exp_avg_sq, void* const* shadow, const int64_t* numel, const float* slots, int nslots,
                    const float* step, float* grad_norm, hipStream_t st) {
  const AdamCoef c{d.lr, d.beta1, d.beta2, d.eps, d.weight_decay, d.max_norm};
  int64_t slot_base = 0;
  for (int base = 0; base < ntensors; base += kMaxTensors) {
    AdamTable t{};
    t.n = ntensors - base < kMaxTensors ? ntensors - base : kMaxTensors;
    int64_t chunks = 0;
    for (int i = 0; i < t.n; ++i) {
      t.p[i] = params[base + i];
      t.g[i] = grads[base + i];
      t.m[i] = exp_avg[base + i];
      t.v[i] = exp_avg_sq[base + i];
      t.shadow[i] = shadow != nullptr ? shadow[base + i] : nullptr;
      t.numel[i] = numel[base + i];
      t.chunk_start[i] = (int)chunks;
      chunks += chunks_of(numel[base + i]);
    }
    t.chunk_start[t.n] = (int)chunks;
    if (chunks > 0) {
      const dim3 grid((unsigned)chunks), block(kBlock);
      if (shadow == nullptr || d.shadow_dtype < 0)
        hipLaunchKernelGGL(clip_adam_kernel<0>, grid, block, 0, st, t, c, slots, nslots, (int)slot_base, step, grad_norm);
      else if (d.shadow_dtype == SFH_BF16)
        hipLaunchKernelGGL(clip_adam_kernel<1>, grid, block, 0, st, t, c, slots, nslots, (int)slot_base, step, grad_norm);
      else
        hipLaunchKernelGGL(clip_adam_kernel<2>, grid, block, 0, st, t, c, slots, nslots, (int)slot_base, step, grad_norm);
      if (int rc = check_launch("clip_adam_kernel")) return rc;
    }
    slot_base += chunks;
  }
  return SFH_OK;
}

}  // namespace sfh
