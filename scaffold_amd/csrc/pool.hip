// MaxPool3d(2) on NDHWC tensors, forward and backward. Pure streaming: the forward pass reads the input once and
// writes an eighth of it plus one byte per output element; the backward pass reads those and writes the input
// gradient once. Replaces the stock op the reference's Down block calls (ScaFFold/unet/unet_parts.py:165), with its
// semantics: the running maximum starts at -inf, a voxel replaces it when it is larger or NaN, cells are scanned
// depth-major, so ties go to the first voxel and a NaN cell reports its last NaN.
#include "pool.hpp"
#include "vec_io.hpp"

namespace sfh {

namespace {

constexpr int kBlock = 256;

struct PoolGeom {
  int64_t cvec;  // channel vectors per voxel
  int c, d, h, w, od, oh, ow;
};

template <typename T, int V> struct LdN {
  static __device__ __forceinline__ void run(const T* p, float (&f)[V]) {
    if constexpr (V == 1) f[0] = to_float(p[0]);
    else Ld<T, V>::run(p, f);
  }
};
template <typename T, int V> struct StN {
  static __device__ __forceinline__ void run(T* p, const float (&f)[V]) {
    if constexpr (V == 1) p[0] = elem<T>::from_float(f[0]);
    else St<T, V>::run(p, f);
  }
};

// `face_pieces` > 0: y is the interior of a depth slab whose two faces of that many 16-byte pieces (in front of y and
// behind its last element) the launch zeroes as well, spread over all its threads.
template <typename T, int V>
__global__ void __launch_bounds__(kBlock) maxpool2_fwd_kernel(PoolGeom g, int64_t total, const T* __restrict__ x, T* __restrict__ y,
                                                              uint8_t* __restrict__ idx, int64_t face_pieces) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (face_pieces > 0) {
    uint4* lo = reinterpret_cast<uint4*>(y) - face_pieces;
    uint4* hi = reinterpret_cast<uint4*>(y + total * V);
    for (int64_t p = i; p < face_pieces; p += (int64_t)gridDim.x * kBlock) {
      lo[p] = make_uint4(0, 0, 0, 0);
      hi[p] = make_uint4(0, 0, 0, 0);
    }
  }
  if (i >= total) return;
  const int64_t cv = i % g.cvec;
  int64_t v = i / g.cvec;
  const int ow = (int)(v % g.ow); v /= g.ow;
  const int oh = (int)(v % g.oh); v /= g.oh;
  const int od = (int)(v % g.od);
  const int64_t n = v / g.od;
  const T* src = x + ((((n * g.d + 2 * od) * g.h + 2 * oh) * g.w + 2 * ow) * (int64_t)g.c + cv * V);
  float in[8][V];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int64_t off = (((int64_t)(k >> 2) * g.h + ((k >> 1) & 1)) * g.w + (k & 1)) * g.c;
    LdN<T, V>::run(src + off, in[k]);
  }
  float best[V];
  uint8_t which[V];
#pragma unroll
  for (int e = 0; e < V; ++e) {
    float m = -INFINITY;
    int w = 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float val = in[k][e];
      const bool take = (m < val) | (val != val);
      m = take ? val : m;
      w = take ? k : w;
    }
    best[e] = m;
    which[e] = (uint8_t)w;
  }
  StN<T, V>::run(y + i * V, best);
  if constexpr (V == 8) {
    uint2 pk;
    pk.x = which[0] | (which[1] << 8) | (which[2] << 16) | ((uint32_t)which[3] << 24);
    pk.y = which[4] | (which[5] << 8) | (which[6] << 16) | ((uint32_t)which[7] << 24);
    *reinterpret_cast<uint2*>(idx + i * 8) = pk;
  } else if constexpr (V == 4) {
    *reinterpret_cast<uint32_t*>(idx + i * 4) = which[0] | (which[1] << 8) | (which[2] << 16) | ((uint32_t)which[3] << 24);
  } else {
    idx[i] = which[0];
  }
}

// One thread per (cell, channel vector); cells cover ceil(d/2) x ceil(h/2) x ceil(w/2), so dropped odd planes get
// their zeros from the same pass.
template <typename T, int V>
__global__ void __launch_bounds__(kBlock) maxpool2_bwd_kernel(PoolGeom g, int cd, int ch, int cw, int64_t total,
                                                              const T* __restrict__ gy, const uint8_t* __restrict__ idx,
                                                              const T* __restrict__ add, T* __restrict__ gx) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= total) return;
  const int64_t cv = i % g.cvec;
  int64_t v = i / g.cvec;
  const int ow = (int)(v % cw); v /= cw;
  const int oh = (int)(v % ch); v /= ch;
  const int od = (int)(v % cd);
  const int64_t n = v / cd;
  const bool pooled = (od < g.od) & (oh < g.oh) & (ow < g.ow);
  // gy and idx are read only where a pooled cell exists: with an odd or unit extent some lanes have none, and when the
  // pooled tensor is empty the pointers themselves are not valid, so there is no address to clamp to.
  float grad[V];
  uint8_t which[V];
#pragma unroll
  for (int e = 0; e < V; ++e) { grad[e] = 0.f; which[e] = 8; }
  if (pooled) {
    const int64_t o = (((n * g.od + od) * g.oh + oh) * g.ow + ow) * g.cvec + cv;
    LdN<T, V>::run(gy + o * V, grad);
    if constexpr (V == 8) {
      const uint2 pk = *reinterpret_cast<const uint2*>(idx + o * 8);
#pragma unroll
      for (int e = 0; e < 4; ++e) { which[e] = (pk.x >> (8 * e)) & 0xff; which[4 + e] = (pk.y >> (8 * e)) & 0xff; }
    } else if constexpr (V == 4) {
      const uint32_t pk = *reinterpret_cast<const uint32_t*>(idx + o * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) which[e] = (pk >> (8 * e)) & 0xff;
    } else {
      which[0] = idx[o];
    }
  }
  const int64_t cell = (((n * g.d + 2 * od) * g.h + 2 * oh) * g.w + 2 * ow) * (int64_t)g.c + cv * V;
  T* dst = gx + cell;
  bool inside[8];
  int64_t at[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int kd = k >> 2, kh = (k >> 1) & 1, kw = k & 1;
    inside[k] = (2 * od + kd < g.d) & (2 * oh + kh < g.h) & (2 * ow + kw < g.w);
    at[k] = inside[k] ? (((int64_t)kd * g.h + kh) * g.w + kw) * g.c : 0;  // voxel 0 of the cell always exists
  }
  // The eight reads of `add` are issued together, from voxel 0 of the cell where a voxel lies outside the tensor
  // (under per-lane conditions they wait for one another: eight trips to memory in a row on the small tensors).
  float more[8][V];
  if (add != nullptr) {  // a second gradient of the pooled tensor (its use as a skip connection), summed in fp32
#pragma unroll
    for (int k = 0; k < 8; ++k) LdN<T, V>::run(add + cell + at[k], more[k]);
  }
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    float out[V];
#pragma unroll
    for (int e = 0; e < V; ++e) out[e] = which[e] == k ? grad[e] : 0.f;
    if (add != nullptr) {
#pragma unroll
      for (int e = 0; e < V; ++e) out[e] += more[k][e];
    }
    if (inside[k]) StN<T, V>::run(dst + at[k], out);
  }
}

PoolGeom geom(const sfh_pool_desc& p, int vec) {
  PoolGeom g{};
  g.c = p.c; g.d = p.in_d; g.h = p.in_h; g.w = p.in_w;
  g.od = p.in_d / 2; g.oh = p.in_h / 2; g.ow = p.in_w / 2;
  g.cvec = p.c / vec;
  return g;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T>
int fwd_typed(const sfh_pool_desc& p, const void* x, void* y, uint8_t* idx, int64_t halo_elems, hipStream_t st) {
  constexpr int V = VecOf<T>::N;
  const bool vec = p.c % V == 0 && aligned16(x) && aligned16(y) && (reinterpret_cast<uintptr_t>(idx) & 7) == 0;
  const PoolGeom g = geom(p, vec ? V : 1);
  const int64_t total = (int64_t)p.n * g.od * g.oh * g.ow * g.cvec;
  const int64_t out_bytes = (int64_t)p.n * g.od * g.oh * g.ow * p.c * (int64_t)sizeof(T), halo_bytes = halo_elems * (int64_t)sizeof(T);
  if (halo_elems > 0 && (p.n != 1 || total == 0 || !aligned16(y) || out_bytes % 16 != 0 || halo_bytes % 16 != 0))
    return fail(SFH_ERR_UNSUPPORTED, "maxpool fwd: a slab output needs one sample and 16-byte aligned faces");
  const int64_t face_pieces = halo_elems > 0 ? halo_bytes / 16 : 0;
  if (total == 0) return SFH_OK;
  const int64_t blocks = cdiv(total, kBlock);
  if (blocks > 0x7fffffff) return fail(SFH_ERR_UNSUPPORTED, "maxpool fwd: %lld workgroups exceed the grid limit", (long long)blocks);
  if (vec)
    hipLaunchKernelGGL((maxpool2_fwd_kernel<T, V>), dim3((unsigned)blocks), dim3(kBlock), 0, st, g, total, static_cast<const T*>(x),
                       static_cast<T*>(y), idx, face_pieces);
  else
    hipLaunchKernelGGL((maxpool2_fwd_kernel<T, 1>), dim3((unsigned)blocks), dim3(kBlock), 0, st, g, total, static_cast<const T*>(x),
                       static_cast<T*>(y), idx, face_pieces);
  return check_launch("maxpool2_fwd_kernel");
}

template <typename T>
int bwd_typed(const sfh_pool_desc& p, const void* gy, const uint8_t* idx, const void* add, void* gx, hipStream_t st) {
  constexpr int V = VecOf<T>::N;
  const bool vec = p.c % V == 0 && aligned16(gy) && aligned16(gx) && aligned16(add) && (reinterpret_cast<uintptr_t>(idx) & 7) == 0;
  const PoolGeom g = geom(p, vec ? V : 1);
  const int cd = (p.in_d + 1) / 2, ch = (p.in_h + 1) / 2, cw = (p.in_w + 1) / 2;
  const int64_t total = (int64_t)p.n * cd * ch * cw * g.cvec;
  if (total == 0) return SFH_OK;
  const int64_t blocks = cdiv(total, kBlock);
  if (blocks > 0x7fffffff) return fail(SFH_ERR_UNSUPPORTED, "maxpool bwd: %lld workgroups exceed the grid limit", (long long)blocks);
  if (vec)
    hipLaunchKernelGGL((maxpool2_bwd_kernel<T, V>), dim3((unsigned)blocks), dim3(kBlock), 0, st, g, cd, ch, cw, total,
                       static_cast<const T*>(gy), idx, static_cast<const T*>(add), static_cast<T*>(gx));
  else
    hipLaunchKernelGGL((maxpool2_bwd_kernel<T, 1>), dim3((unsigned)blocks), dim3(kBlock), 0, st, g, cd, ch, cw, total,
                       static_cast<const T*>(gy), idx, static_cast<const T*>(add), static_cast<T*>(gx));
  return check_launch("maxpool2_bwd_kernel");
}

}  // namespace

int maxpool2_fwd(const sfh_pool_desc& p, int dtype, const void* x, void* y, uint8_t* idx, hipStream_t st, int64_t halo_elems) {
  if (dtype == SFH_BF16) return fwd_typed<bf16_t>(p, x, y, idx, halo_elems, st);
  if (dtype == SFH_FP16) return fwd_typed<fp16_t>(p, x, y, idx, halo_elems, st);
  return fwd_typed<float>(p, x, y, idx, halo_elems, st);
}

int maxpool2_bwd(const sfh_pool_desc& p, int dtype, const void* gy, const uint8_t* idx, const void* add, void* gx, hipStream_t st) {
  if (dtype == SFH_BF16) return bwd_typed<bf16_t>(p, gy, idx, add, gx, st);
  if (dtype == SFH_FP16) return bwd_typed<fp16_t>(p, gy, idx, add, gx, st);
  return bwd_typed<float>(p, gy, idx, add, gx, st);
}

}  // namespace sfh
