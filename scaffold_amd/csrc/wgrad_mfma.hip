// MFMA weight gradient of a 3x3x3 stride-1 convolution for gfx950, bf16 / fp16 operands.
//
//   gw[co][kd][kh][kw][ci] = sum over output voxels v of gy[v][co] * x[v + tap - pad][ci]
//
// GEMM view (triton_conv3d/reduce_gemm.py:137-393): M = Cout, N = 27 x Cin, K = output voxels,
// split over workgroups along K, fp32 partial slices at fixed workspace slots and an ordered
// reduction (reduce_gemm.py:396-435) -- no float atomics, split count a pure function of shape.
//
// Both MFMA operands need the contraction index (voxels) contiguous per lane while memory is
// channel-contiguous. The transpose is done ONCE, while staging into LDS: a thread fetches the
// same 8 channels of 4 consecutive W voxels (4 x 16-byte global loads), regroups them with
// byte permutes into 8 x (4 voxels of one channel) and writes 8-byte pieces, so LDS holds
//   G[co][tile voxel]            (gy tile, 256 voxels)
//   X[ci][brick row][w + halo]   (x brick with its one-voxel halo)
// and every fragment is a plain 16-byte ds_read at an immediate offset. The three kw taps of a
// brick row come from one 20-byte window: kw = 0 and kw = 2 are register renames, kw = 1 is four
// funnel shifts. Channel strides are odd multiples of 16 bytes so 16 lanes (16 channels) hit 16
// different bank groups.
//
// A workgroup is four wavefronts; each owns 6-7 of the 27 taps (whole brick rows where possible)
// and all 32x32 (co, ci) outputs of those taps: 112 accumulator registers. Tiles of the
// workgroup's K range are processed one after another; two workgroups per CU overlap one's
// staging with the other's MFMAs.
#include "wgrad_mfma.hpp"
#include "reduce.hpp"

namespace sfh {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
  static __device__ __forceinline__ f32x16_t run(const uint4& a, const uint4& b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
};
template <> struct Mma<fp16_t> {
  static __device__ __forceinline__ f32x16_t run(const uint4& a, const uint4& b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
};

constexpr int kTargetWorkgroups = 2 * kComputeUnits;

constexpr int odd16(int bytes) {  // smallest odd multiple of 16 that is >= bytes
  int u = (bytes + 15) / 16;
  return (u % 2 == 0 ? u + 1 : u) * 16;
}

template <int TD_, int TH_, int TW_>
struct WTile {
  static constexpr int TD = TD_, TH = TH_, TW = TW_;
  static constexpr int BD = TD + 2, BH = TH + 2;
  static constexpr int NBR = BD * BH;                 // brick rows
  static constexpr int XR = (TW + 2 + 7) / 8 * 8;     // elements per stored brick row
  static constexpr int NQX = (TW + 2 + 3) / 4;        // 4-voxel groups staged per brick row
  static constexpr int XC = odd16(NBR * XR * 2);      // bytes per channel of X
  static constexpr int GC = odd16(TD * TH * TW * 2);  // bytes per channel of G
  static constexpr int GOFF = 32 * XC;
  static constexpr int LDS = 32 * XC + 32 * GC;
  static constexpr int NKS = TD * TH * TW / 16;       // k-steps per tile
  static constexpr int XITEMS = NBR * NQX * 4;
  static_assert(TD * TH * TW == 256, "one gy staging item per thread");
  static_assert(TH % 2 == 0, "an 8-voxel row pair must not straddle a depth slice");
  static_assert(LDS <= 80 * 1024, "two workgroups per CU");
};

// Brick row (kd*3 + kh) sets of the four wavefronts; wave w < 3 also owns tap (2,2,kw=w).
template <int WAVE> struct WaveTaps {
  static constexpr int R0 = 2 * WAVE, R1 = 2 * WAVE + 1;
  static constexpr bool EXTRA = WAVE < 3;
  static constexpr int NACC = EXTRA ? 7 : 6;
};

// d0..d3 hold the same channel pair (even channel in the low half) of four consecutive voxels;
// e0 / e1 receive the four voxels of the even / odd channel, voxel 0 in the lowest 16 bits.
__device__ __forceinline__ void transpose4(uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3, uint2& e0, uint2& e1) {
  e0.x = (d0 & 0xffffu) | (d1 << 16);
  e0.y = (d2 & 0xffffu) | (d3 << 16);
  e1.x = (d0 >> 16) | (d1 & 0xffff0000u);
  e1.y = (d2 >> 16) | (d3 & 0xffff0000u);
}

__device__ __forceinline__ uint4 shift_one(const uint4& lo, uint32_t next) {
  // elements 1..8 of the nine-element window {lo (8 x 16 bit), next (low 16 bit)}
  uint4 r;
  r.x = (lo.x >> 16) | (lo.y << 16);
  r.y = (lo.y >> 16) | (lo.z << 16);
  r.z = (lo.z >> 16) | (lo.w << 16);
  r.w = (lo.w >> 16) | (next << 16);
  return r;
}

// Uniform byte offset inside X of the 16-element window of k-step `ks` at brick row offset
// (kd, kh); the per-lane part (channel, k-half) is added by the caller.
template <typename C>
__device__ __forceinline__ constexpr int x_window_off(int ks, int kd, int kh) {
  if (C::TW == 32) {
    const int grow = ks / 2, td = grow / C::TH, th = grow % C::TH;
    return ((td + kd) * C::BH + th + kh) * C::XR * 2 + (ks % 2) * 32;
  } else if (C::TW == 16) {
    const int td = ks / C::TH, th = ks % C::TH;
    return ((td + kd) * C::BH + th + kh) * C::XR * 2;
  } else {
    const int grow = 2 * ks, td = grow / C::TH, th = grow % C::TH;
    return ((td + kd) * C::BH + th + kh) * C::XR * 2;
  }
}

template <typename T, typename C, int WAVE>
__device__ __forceinline__ void wave_compute(const char* lds, int lane, f32x16_t (&acc)[7]) {
  using W = WaveTaps<WAVE>;
  const int i = lane & 31, kg = lane >> 5;
  const int gbase = C::GOFF + i * C::GC + kg * 16;
  // k-half offset inside X: 8 voxels along W, or (TW == 8) the next brick row
  const int xbase = i * C::XC + (C::TW == 8 ? kg * C::XR * 2 : kg * 16);
#pragma unroll
  for (int ks = 0; ks < C::NKS; ++ks) {
    const uint4 af = *reinterpret_cast<const uint4*>(lds + gbase + ks * 32);
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
      const int row = rr == 0 ? W::R0 : W::R1;
      const int off = xbase + x_window_off<C>(ks, row / 3, row % 3);
      const uint4 lo = *reinterpret_cast<const uint4*>(lds + off);
      const uint32_t nx = *reinterpret_cast<const uint32_t*>(lds + off + 16);
      const uint4 f1 = shift_one(lo, nx);
      const uint4 f2 = make_uint4(lo.y, lo.z, lo.w, nx);
      acc[rr * 3 + 0] = Mma<T>::run(af, lo, acc[rr * 3 + 0]);
      acc[rr * 3 + 1] = Mma<T>::run(af, f1, acc[rr * 3 + 1]);
      acc[rr * 3 + 2] = Mma<T>::run(af, f2, acc[rr * 3 + 2]);
    }
    if (W::EXTRA) {
      const int off = xbase + x_window_off<C>(ks, 2, 2);
      const uint4 lo = *reinterpret_cast<const uint4*>(lds + off);
      uint4 f = lo;
      if (WAVE >= 1) {
        const uint32_t nx = *reinterpret_cast<const uint32_t*>(lds + off + 16);
        f = WAVE == 1 ? shift_one(lo, nx) : make_uint4(lo.y, lo.z, lo.w, nx);
      }
      acc[6] = Mma<T>::run(af, f, acc[6]);
    }
  }
}

template <typename C, int WAVE>
__device__ __forceinline__ void wave_store(const f32x16_t (&acc)[7], float* __restrict__ dst, int cin, int lane) {
  using W = WaveTaps<WAVE>;
  const int j = lane & 31, kg = lane >> 5;
#pragma unroll
  for (int t = 0; t < W::NACC; ++t) {
    const int tap = t < 3 ? W::R0 * 3 + t : (t < 6 ? W::R1 * 3 + (t - 3) : 24 + WAVE);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int co = 8 * (r / 4) + 4 * kg + (r % 4);
      dst[((int64_t)co * 27 + tap) * cin + j] = acc[t][r];
    }
  }
}

template <typename T, typename C>
__global__ void __launch_bounds__(256, 2)
wgrad_mfma_kernel(WgradArgs a, const T* __restrict__ x, const T* __restrict__ gy, float* __restrict__ ws, int tiles_d,
                  int tiles_h, int tiles_w, int ntiles, int tiles_per_split, int nblk_ci, int nblk, uint32_t total) {
  __shared__ __attribute__((aligned(16))) char lds[C::LDS];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;

  uint32_t wg = xcd_remap(blockIdx.x, total);
  const int blk = wg % nblk;
  const int split = wg / nblk;
  const int cib = blk % nblk_ci, cob = blk / nblk_ci;

  f32x16_t acc[7];
#pragma unroll
  for (int t = 0; t < 7; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;

  const int t_begin = split * tiles_per_split;
  int t_end = t_begin + tiles_per_split;
  if (t_end > ntiles) t_end = ntiles;

  constexpr int XIT = (C::XITEMS + 255) / 256;
  for (int tile = t_begin; tile < t_end; ++tile) {
    int t = tile;
    const int tw_i = t % tiles_w; t /= tiles_w;
    const int th_i = t % tiles_h; t /= tiles_h;
    const int td_i = t % tiles_d;
    const int n = t / tiles_d;
    const int od0 = td_i * C::TD, oh0 = th_i * C::TH, ow0 = tw_i * C::TW;

    __syncthreads();  // previous tile fully consumed
    // ---- stage gy tile, transposed: one item (tile row, 4-voxel group, 8-channel piece) per thread
    {
      const int piece = tid & 3;
      const int quad = (tid >> 2) % (C::TW / 4);
      const int grow = tid / (C::TW);  // (tid >> 2) / (TW / 4)
      const int td = grow / C::TH, th = grow % C::TH;
      const int od = od0 + td, oh = oh0 + th;
      const bool rowok = od < a.od && oh < a.oh;
      const T* gp = gy + ((((int64_t)n * a.od + od) * a.oh + oh) * a.ow) * a.cout + cob * 32 + piece * 8;
      uint4 v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int ow = ow0 + quad * 4 + k;
        v[k] = make_uint4(0, 0, 0, 0);
        if (rowok && ow < a.ow) v[k] = *reinterpret_cast<const uint4*>(gp + (int64_t)ow * a.cout);
      }
      char* dst = lds + C::GOFF + (piece * 8) * C::GC + grow * C::TW * 2 + quad * 8;
      const uint32_t d0[4] = {v[0].x, v[0].y, v[0].z, v[0].w}, d1[4] = {v[1].x, v[1].y, v[1].z, v[1].w},
                     d2[4] = {v[2].x, v[2].y, v[2].z, v[2].w}, d3[4] = {v[3].x, v[3].y, v[3].z, v[3].w};
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        uint2 e0, e1;
        transpose4(d0[d], d1[d], d2[d], d3[d], e0, e1);
        *reinterpret_cast<uint2*>(dst + (2 * d) * C::GC) = e0;
        *reinterpret_cast<uint2*>(dst + (2 * d + 1) * C::GC) = e1;
      }
    }
    // ---- stage x brick (with halo), transposed
    {
      const int id0 = od0 - a.pd, ih0 = oh0 - a.ph, iw0 = ow0 - a.pw;
      const T* xn = x + (int64_t)n * a.id * a.ih * a.iw * a.cin + cib * 32;
#pragma unroll
      for (int it = 0; it < XIT; ++it) {
        const int item = it * 256 + tid;
        if (item < C::XITEMS) {
          const int piece = item & 3;
          const int quad = (item >> 2) % C::NQX;
          const int brow = (item >> 2) / C::NQX;
          const int bd = brow / C::BH, bh = brow % C::BH;
          const int id = id0 + bd, ih = ih0 + bh;
          const bool rowok = (unsigned)id < (unsigned)a.id && (unsigned)ih < (unsigned)a.ih;
          const T* xp = xn + (((int64_t)id * a.ih + ih) * a.iw) * a.cin + piece * 8;
          uint4 v[4];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const int bw = quad * 4 + k;
            const int iw = iw0 + bw;
            v[k] = make_uint4(0, 0, 0, 0);
            if (rowok && bw < C::TW + 2 && (unsigned)iw < (unsigned)a.iw)
              v[k] = *reinterpret_cast<const uint4*>(xp + (int64_t)iw * a.cin);
          }
          char* dst = lds + (piece * 8) * C::XC + brow * C::XR * 2 + quad * 8;
          const uint32_t d0[4] = {v[0].x, v[0].y, v[0].z, v[0].w}, d1[4] = {v[1].x, v[1].y, v[1].z, v[1].w},
                         d2[4] = {v[2].x, v[2].y, v[2].z, v[2].w}, d3[4] = {v[3].x, v[3].y, v[3].z, v[3].w};
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            uint2 e0, e1;
            transpose4(d0[d], d1[d], d2[d], d3[d], e0, e1);
            *reinterpret_cast<uint2*>(dst + (2 * d) * C::XC) = e0;
            *reinterpret_cast<uint2*>(dst + (2 * d + 1) * C::XC) = e1;
          }
        }
      }
    }
    __syncthreads();

    switch (wave) {
      case 0: wave_compute<T, C, 0>(lds, lane, acc); break;
      case 1: wave_compute<T, C, 1>(lds, lane, acc); break;
      case 2: wave_compute<T, C, 2>(lds, lane, acc); break;
      default: wave_compute<T, C, 3>(lds, lane, acc); break;
    }
  }

  float* dst = ws + ((int64_t)split * a.cout + cob * 32) * 27 * a.cin + cib * 32;
  switch (wave) {
    case 0: wave_store<C, 0>(acc, dst, a.cin, lane); break;
    case 1: wave_store<C, 1>(acc, dst, a.cin, lane); break;
    case 2: wave_store<C, 2>(acc, dst, a.cin, lane); break;
    default: wave_store<C, 3>(acc, dst, a.cin, lane); break;
  }
}

struct Plan {
  int tw;  // 32, 16 or 8
  int tiles_d, tiles_h, tiles_w, ntiles;
  int nblk_ci, nblk;
  int splits, tiles_per_split;
};

Plan make_plan(const WgradArgs& a) {
  Plan p{};
  int td, th;
  if (a.ow > 16) { p.tw = 32; td = 2; th = 4; }
  else if (a.ow > 8) { p.tw = 16; td = 2; th = 8; }
  else { p.tw = 8; td = 4; th = 8; }
  p.tiles_d = (int)cdiv(a.od, td);
  p.tiles_h = (int)cdiv(a.oh, th);
  p.tiles_w = (int)cdiv(a.ow, p.tw);
  p.ntiles = a.n * p.tiles_d * p.tiles_h * p.tiles_w;
  p.nblk_ci = a.cin / 32;
  p.nblk = p.nblk_ci * (a.cout / 32);
  int want = kTargetWorkgroups / p.nblk;
  if (want < 1) want = 1;
  if (want > p.ntiles) want = p.ntiles;
  p.tiles_per_split = (int)cdiv(p.ntiles, want);
  p.splits = (int)cdiv(p.ntiles, p.tiles_per_split);
  return p;
}

template <typename T, typename C>
int launch_tile(const WgradArgs& a, const Plan& p, const void* x, const void* gy, float* ws, hipStream_t st) {
  const int64_t total = (int64_t)p.splits * p.nblk;
  hipLaunchKernelGGL((wgrad_mfma_kernel<T, C>), dim3((unsigned)total), dim3(256), 0, st, a, (const T*)x, (const T*)gy, ws,
                     p.tiles_d, p.tiles_h, p.tiles_w, p.ntiles, p.tiles_per_split, p.nblk_ci, p.nblk, (uint32_t)total);
  return check_launch("wgrad_mfma_kernel");
}

template <typename T>
int launch_typed(const WgradArgs& a, const void* x, const void* gy, void* gw, void* workspace, hipStream_t st) {
  const Plan p = make_plan(a);
  float* ws = (float*)workspace;
  int rc;
  if (p.tw == 32) rc = launch_tile<T, WTile<2, 4, 32>>(a, p, x, gy, ws, st);
  else if (p.tw == 16) rc = launch_tile<T, WTile<2, 8, 16>>(a, p, x, gy, ws, st);
  else rc = launch_tile<T, WTile<4, 8, 8>>(a, p, x, gy, ws, st);
  if (rc != SFH_OK) return rc;
  const int64_t nelem = (int64_t)a.cout * 27 * a.cin;
  return sum_slices(__is_same(T, bf16_t) ? SFH_BF16 : SFH_FP16, ws, gw, nelem, p.splits, st);
}

}  // namespace

bool mfma_wgrad_supported(const WgradArgs& a, int dtype) {
  if (dtype != SFH_BF16 && dtype != SFH_FP16) return false;
  if (a.cin % 32 != 0 || a.cout % 32 != 0) return false;
  if (a.pd < 0 || a.ph < 0 || a.pw < 0 || a.pd > 2 || a.ph > 2 || a.pw > 2) return false;
  if (a.n < 1 || a.od < 1 || a.oh < 1 || a.ow < 1) return false;
  const Plan p = make_plan(a);
  if ((int64_t)a.n * p.tiles_d * p.tiles_h * p.tiles_w > 0x7fffffffLL) return false;
  return true;
}

int mfma_wgrad_splits(const WgradArgs& a) { return make_plan(a).splits; }

size_t mfma_wgrad_workspace_bytes(const WgradArgs& a) {
  const Plan p = make_plan(a);
  return align_up((size_t)p.splits * a.cout * 27 * a.cin * sizeof(float), 256);
}

int mfma_wgrad(const WgradArgs& a, int dtype, const void* x, const void* gy, void* gw, void* workspace, hipStream_t st) {
  if (dtype == SFH_BF16) return launch_typed<bf16_t>(a, x, gy, gw, workspace, st);
  return launch_typed<fp16_t>(a, x, gy, gw, workspace, st);
}

}  // namespace sfh
