// MFMA kernels for 2x2x2, stride-2, unpadded convolutions between a BIG and a SMALL volume: the U-Net's
// transposed up-convolution (triton_conv3d/transposed.py:135-319), its data gradient (a stride-2
// convolution, transposed.py:1073) and its weight gradient (transposed.py:1113).
//
// Windows do not overlap, so there is no halo and nothing to reuse between neighbouring voxels: the
// three kernels are HBM-bound GEMMs with M = small voxels. The gather and the scatter take both MFMA
// operands straight from global memory (a lane's fragment is 8 consecutive channels of one voxel, one
// 16-byte load; the weight is pre-packed in fragment order and stays in L1/L2). The weight gradient
// contracts over voxels, so both operands must be transposed: tiles are staged in LDS in their natural
// [voxel][channel] layout and read with ds_read_b64_tr_b16, which hands each lane four consecutive
// voxels of one channel.
#include "conv_patch.hpp"
#include <type_traits>
#include "mma.hpp"
#include "reduce.hpp"

namespace sfh {
namespace {

constexpr int kTaps = 8;

struct Voxel { int nn, d, h, w; };

__device__ __forceinline__ Voxel decode_small(const PatchArgs& a, int64_t v) {
  Voxel r;
  if (v <= 0x7fffffffLL) {  // 32-bit arithmetic when it fits
    uint32_t t = (uint32_t)v;
    r.w = (int)(t % (uint32_t)a.sw); t /= (uint32_t)a.sw;
    r.h = (int)(t % (uint32_t)a.sh); t /= (uint32_t)a.sh;
    r.d = (int)(t % (uint32_t)a.sd);
    r.nn = (int)(t / (uint32_t)a.sd);
    return r;
  }
  r.w = (int)(v % a.sw);
  int64_t t = v / a.sw;
  r.h = (int)(t % a.sh);
  t /= a.sh;
  r.d = (int)(t % a.sd);
  r.nn = (int)(t / a.sd);
  return r;
}

__device__ __forceinline__ int64_t big_index(const PatchArgs& a, const Voxel& v, int tap) {
  return (((int64_t)v.nn * a.bd + 2 * v.d + (tap >> 2)) * a.bh + 2 * v.h + ((tap >> 1) & 1)) * a.bw + 2 * v.w + (tap & 1);
}


// ---- gather: stride-2 convolution --------------------------------------------------------------
// A wavefront owns 32 small voxels x NB blocks of 32 produced channels. grid = (voxel tiles of 128, groups of NB blocks).
template <typename T, int NB>
__global__ void __launch_bounds__(256) patch_gather_kernel(PatchArgs a, const T* __restrict__ big, const T* __restrict__ packed,
                                                           const T* __restrict__ bias, T* __restrict__ small, int64_t total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kg = lane >> 5;
  const int64_t v = (int64_t)blockIdx.x * 128 + wave * 32 + (lane & 31);
  const bool valid = v < total;
  const Voxel vx = decode_small(a, valid ? v : total - 1);
  const int nchunks = a.cbig / 32;
  const int blk0 = blockIdx.y * NB;
  f32x16_t acc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[b][r] = 0.f;
  for (int tap = 0; tap < kTaps; ++tap) {
    const T* src = big + big_index(a, vx, tap) * a.cbig + kg * 8;
    for (int cc = 0; cc < nchunks; ++cc) {
      uint4 bf[2], wf[2][NB];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        bf[ks] = load16(src + cc * 32 + ks * 16);
#pragma unroll
        for (int b = 0; b < NB; ++b)
          wf[ks][b] = load16(packed + (((((int64_t)(blk0 + b) * nchunks + cc) * kTaps + tap) * 2 + ks) * 64 + lane) * 8);
      }
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int b = 0; b < NB; ++b) acc[b] = Mma32<T>::run(wf[ks][b], bf[ks], acc[b]);
    }
  }
  const int64_t vs = valid ? v : total - 1;
#pragma unroll
  for (int b = 0; b < NB; ++b) store_block<T>(acc[b], small + vs * a.csmall + (blk0 + b) * 32, bias, (blk0 + b) * 32, kg, valid);
}

// The same for launches that would leave most of the chip idle (the U-Net's deepest levels: a few hundred voxels, hundreds
// of channels, where one wavefront's chain of dependent loads sets the time). A workgroup owns 32 small voxels x one block of
// 32 produced channels; its four wavefronts take two taps each, keep the loads of four chunks in flight, and their partial
// blocks are added in wavefront order through LDS. grid = (voxel tiles of 32, csmall / 32).
template <typename T>
__global__ void __launch_bounds__(256) patch_gather_deep_kernel(PatchArgs a, const T* __restrict__ big, const T* __restrict__ packed,
                                                                const T* __restrict__ bias, T* __restrict__ small, int64_t total) {
  __shared__ float part[3][16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kg = lane >> 5;
  const int64_t v = (int64_t)blockIdx.x * 32 + (lane & 31);
  const bool valid = v < total;
  const int64_t vs = valid ? v : total - 1;
  const Voxel vx = decode_small(a, vs);
  const int nchunks = a.cbig / 32;
  const int blk = blockIdx.y;
  f32x16_t acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  for (int tap = 2 * wave; tap < 2 * wave + 2; ++tap) {
    const T* src = big + big_index(a, vx, tap) * a.cbig + kg * 8;
    const T* wsrc = packed + ((((int64_t)blk * nchunks) * kTaps + tap) * 2 * 64 + lane) * 8;
    const int64_t wstep = (int64_t)kTaps * 2 * 64 * 8;  // elements between the fragments of consecutive chunks
    // U chunks per step: all their loads are issued before the first MFMA
    auto step = [&](int cc, auto width) {
      constexpr int U = decltype(width)::value;
      uint4 bf[U][2], wf[U][2];
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          bf[u][ks] = load16(src + (cc + u) * 32 + ks * 16);
          wf[u][ks] = load16(wsrc + (cc + u) * wstep + ks * 64 * 8);
        }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) acc = Mma32<T>::run(wf[u][ks], bf[u][ks], acc);
    };
    int cc = 0;
    for (; cc + 4 <= nchunks; cc += 4) step(cc, std::integral_constant<int, 4>{});
    for (; cc < nchunks; ++cc) step(cc, std::integral_constant<int, 1>{});
  }
  if (wave > 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) part[wave - 1][r][lane] = acc[r];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int w = 0; w < 3; ++w)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] += part[w][r][lane];
    store_block<T>(acc, small + vs * a.csmall + blk * 32, bias, blk * 32, kg, valid);
  }
}

// ---- scatter: transposed convolution -----------------------------------------------------------
// A wavefront owns 32 small voxels x one block of 32 big channels x TS of the 8 taps.
// grid = (voxel tiles of 128, cbig / 32, 8 / TS). TS = 8 reads the small tensor once; TS = 1 and 2 are for launches that
// would otherwise leave most of the chip idle or give a CU a single long chain of dependent loads (the deeper levels):
// more workgroups, each with a shorter chain, and the loads of several k-steps in flight per lane.
// `face_pieces` > 0: `big` is the interior of a depth slab whose two faces of that many 16-byte pieces (in front of it and
// behind its `big_elems` elements) the launch zeroes as well, spread over all its threads.
template <typename T, int TS>
__global__ void __launch_bounds__(256) patch_scatter_kernel(PatchArgs a, const T* __restrict__ small, const T* __restrict__ packed,
                                                            const T* __restrict__ bias, T* __restrict__ big, int64_t total,
                                                            int64_t face_pieces, int64_t big_elems) {
  if (face_pieces > 0) {
    const int64_t nthreads = (int64_t)gridDim.x * gridDim.y * gridDim.z * 256;
    const int64_t me = (((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
    uint4* lo = reinterpret_cast<uint4*>(big) - face_pieces;
    uint4* hi = reinterpret_cast<uint4*>(big + big_elems);
    for (int64_t p = me; p < face_pieces; p += nthreads) {
      lo[p] = make_uint4(0, 0, 0, 0);
      hi[p] = make_uint4(0, 0, 0, 0);
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kg = lane >> 5;
  const int64_t v = (int64_t)blockIdx.x * 128 + wave * 32 + (lane & 31);
  const bool valid = v < total;
  const int64_t vc = valid ? v : total - 1;
  const int nchunks = a.csmall / 32;
  const int blk = blockIdx.y;
  const int tap0 = blockIdx.z * TS;
  f32x16_t acc[TS];
#pragma unroll
  for (int t = 0; t < TS; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
  const T* src = small + vc * a.csmall + kg * 8;
  // U half-chunks (k-steps of 16 channels) per step: all their loads are issued before the first MFMA
  auto step = [&](int k, auto width) {
    constexpr int U = decltype(width)::value;
    uint4 sf[U], wf[U][TS];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int cc = (k + u) >> 1, ks = (k + u) & 1;
      sf[u] = load16(src + cc * 32 + ks * 16);
#pragma unroll
      for (int t = 0; t < TS; ++t)
        wf[u][t] = load16(packed + (((((int64_t)blk * nchunks + cc) * kTaps + tap0 + t) * 2 + ks) * 64 + lane) * 8);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < TS; ++t) acc[t] = Mma32<T>::run(wf[u][t], sf[u], acc[t]);
  };
  int k = 0;
  if constexpr (TS == 1)
    for (; k + 8 <= 2 * nchunks; k += 8) step(k, std::integral_constant<int, 8>{});
  if constexpr (TS == 2)
    for (; k + 4 <= 2 * nchunks; k += 4) step(k, std::integral_constant<int, 4>{});
  if constexpr (TS == 4)
    for (; k + 2 <= 2 * nchunks; k += 2) step(k, std::integral_constant<int, 2>{});
  for (; k < 2 * nchunks; ++k) step(k, std::integral_constant<int, 1>{});
  const Voxel vx = decode_small(a, vc);
#pragma unroll
  for (int t = 0; t < TS; ++t)
    store_block<T>(acc[t], big + big_index(a, vx, tap0 + t) * a.cbig + blk * 32, bias, blk * 32, kg, valid);
}

// ---- reduce: weight gradient -------------------------------------------------------------------
constexpr int kVx = 32;             // voxels staged per round (two k-steps of 16)
constexpr int kSmallTile = 64;      // small channels per workgroup (two row blocks)
constexpr int kSRow = kSmallTile + 8;  // LDS row strides in elements: 16-byte aligned, off the 128-byte period
constexpr int kBRow = 32 + 8;

// Operand fragment (32 channels x 16 voxels) from a natural-layout LDS tile: `tile` points at the first
// of the 16 voxel rows, channel 0 of the block. Within each group of 16 lanes the transposing read takes
// lane m's address as (voxel m / 4, channels 4 * (m % 4) .. + 3) and returns to lane m channel m of the
// four voxels, so two reads give a lane its 8 voxels of the k-step.
template <typename T>
__device__ __forceinline__ uint4 tr_fragment(const T* tile, int row_stride, int lane) {
  typedef short v4s __attribute__((__vector_size__(4 * sizeof(short))));
  const int g = lane >> 4, m = lane & 15;
  const T* p0 = tile + ((g >> 1) * 8 + (m >> 2)) * row_stride + (g & 1) * 16 + 4 * (m & 3);
  const T* p1 = p0 + 4 * row_stride;
  const v4s r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)(p0));
  const v4s r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s*)(p1));
  uint4 out;
  out.x = __builtin_bit_cast(uint2, r0).x; out.y = __builtin_bit_cast(uint2, r0).y;
  out.z = __builtin_bit_cast(uint2, r1).x; out.w = __builtin_bit_cast(uint2, r1).y;
  return out;
}

// grid = (splits, csmall / 64, cbig / 32). Wavefront w accumulates taps 2w and 2w + 1 for both row blocks.
// BIAS: the workgroups of the first small-channel tile also add up the big tensor itself over the voxels -- the bias
// gradient of the transposed convolution whose weight gradient this is (every big voxel is a tap of exactly one small
// voxel there) -- as one more MFMA row block of ones: bias_part[split][tap][cb], the same fixed order as the weights'.
template <typename T, bool BIAS>
__global__ void __launch_bounds__(256) patch_reduce_kernel(PatchArgs a, const T* __restrict__ small, const T* __restrict__ big,
                                                           float* __restrict__ part, int64_t total, int64_t per_split,
                                                           float* __restrict__ bias_part) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(16))) T s_tile[kVx * kSRow];
  __shared__ __attribute__((aligned(16))) T b_tile[kTaps * kVx * kBRow];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cs0 = blockIdx.y * kSmallTile, cb0 = blockIdx.z * 32;
  const int64_t begin = (int64_t)blockIdx.x * per_split;
  int64_t end = begin + per_split;
  if (end > total) end = total;
  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  f32x16_t bacc[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) bacc[j][r] = 0.f;
  const bool sums_big = BIAS && blockIdx.y == 0;
  const uint32_t one2 = sizeof(T) == 2 && std::is_same<T, bf16_t>::value ? 0x3f803f80u : 0x3c003c00u;  // two ones of T
  const uint4 ones = make_uint4(one2, one2, one2, one2);
  const int s_vox = tid >> 3, s_piece = tid & 7;          // small tile: 32 voxels x 8 pieces of 16 bytes
  const int b_vox = (tid >> 2) & 31, b_piece = tid & 3;   // big tiles: 4 taps (tid/128, +2, +4, +6) of one voxel
  const int b_tap0 = tid >> 7;
  const uint4 zero = make_uint4(0, 0, 0, 0);
  for (int64_t v0 = begin; v0 < end; v0 += kVx) {
    uint4 sv = zero, bv[4] = {zero, zero, zero, zero};
    if (v0 + s_vox < end) sv = load16(small + (v0 + s_vox) * a.csmall + cs0 + s_piece * 8);
    if (v0 + b_vox < end) {
      const Voxel vx = decode_small(a, v0 + b_vox);
#pragma unroll
      for (int i = 0; i < 4; ++i) bv[i] = load16(big + big_index(a, vx, b_tap0 + 2 * i) * a.cbig + cb0 + b_piece * 8);
    }
    __syncthreads();  // the previous round's reads are done
    *reinterpret_cast<uint4*>(s_tile + s_vox * kSRow + s_piece * 8) = sv;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<uint4*>(b_tile + ((b_tap0 + 2 * i) * kVx + b_vox) * kBRow + b_piece * 8) = bv[i];
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      uint4 af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) af[i] = tr_fragment<T>(s_tile + ks * 16 * kSRow + i * 32, kSRow, lane);
#pragma unroll
      for (int j = 0; j < 2; ++j) bf[j] = tr_fragment<T>(b_tile + ((2 * wave + j) * kVx + ks * 16) * kBRow, kBRow, lane);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = Mma32<T>::run(af[i], bf[j], acc[i][j]);
      if constexpr (BIAS) {
        if (sums_big) {  // every row of the block is the column sum
#pragma unroll
          for (int j = 0; j < 2; ++j) bacc[j] = Mma32<T>::run(ones, bf[j], bacc[j]);
        }
      }
    }
  }
  // part[split][cs][tap][cb]: a lane holds column cb = lane % 32 and 16 rows of each block
  float* dst = part + (int64_t)blockIdx.x * a.csmall * kTaps * a.cbig;
  const int col = lane & 31, kg = lane >> 5;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int cs = cs0 + i * 32 + 8 * (r >> 2) + 4 * kg + (r & 3);
        dst[((int64_t)cs * kTaps + 2 * wave + j) * a.cbig + cb0 + col] = acc[i][j][r];
      }
  if constexpr (BIAS) {
    if (sums_big && kg == 0) {
#pragma unroll
      for (int j = 0; j < 2; ++j) bias_part[((int64_t)blockIdx.x * kTaps + 2 * wave + j) * a.cbig + cb0 + col] = bacc[j][0];
    }
  }
#endif
}

int64_t small_voxels(const PatchArgs& a) { return (int64_t)a.n * a.sd * a.sh * a.sw; }

// Produced-channel blocks per wavefront: as many as keep at least two wavefronts per SIMD busy.
int gather_blocks(const PatchArgs& a) {
  const int nblk = a.csmall / 32;
  const int64_t wave_tiles = cdiv(small_voxels(a), 32);
  int nb = 8;
  while (nb > 1 && (nblk % nb != 0 || wave_tiles * (nblk / nb) < 2048)) nb >>= 1;
  return nb;
}

template <typename T>
int launch_gather(const PatchArgs& a, const void* big, const void* packed, const void* bias, void* small, hipStream_t st) {
  const int64_t total = small_voxels(a);
  const int nb = gather_blocks(a);
  const dim3 grid((unsigned)cdiv(total, 128), (unsigned)(a.csmall / 32 / nb));
  if (nb == 1 && (int64_t)grid.x * grid.y < kComputeUnits) {  // under one workgroup per CU (no gain measured above that)
    hipLaunchKernelGGL((patch_gather_deep_kernel<T>), dim3((unsigned)cdiv(total, 32), (unsigned)(a.csmall / 32)), dim3(256), 0, st, a,
                       (const T*)big, (const T*)packed, (const T*)bias, (T*)small, total);
    return check_launch("patch_gather_deep_kernel");
  }
#define SFH_PATCH_GATHER(NB)                                                                                              \
  hipLaunchKernelGGL((patch_gather_kernel<T, NB>), grid, dim3(256), 0, st, a, (const T*)big, (const T*)packed, (const T*)bias, \
                     (T*)small, total)
  if (nb == 8) SFH_PATCH_GATHER(8);
  else if (nb == 4) SFH_PATCH_GATHER(4);
  else if (nb == 2) SFH_PATCH_GATHER(2);
  else SFH_PATCH_GATHER(1);
#undef SFH_PATCH_GATHER
  return check_launch("patch_gather_kernel");
}

template <typename T>
int launch_scatter(const PatchArgs& a, const void* small, const void* packed, const void* bias, void* big, hipStream_t st,
                   int64_t halo_elems) {
  const int64_t total = small_voxels(a);
  const int64_t big_elems = (int64_t)a.n * a.bd * a.bh * a.bw * a.cbig;
  if (halo_elems > 0 && (a.n != 1 || (reinterpret_cast<uintptr_t>(big) & 15) != 0 || (big_elems * (int64_t)sizeof(T)) % 16 != 0 ||
                         (halo_elems * (int64_t)sizeof(T)) % 16 != 0))
    return fail(SFH_ERR_UNSUPPORTED, "convT3d fwd: a slab output needs one sample and 16-byte aligned faces");
  const int64_t face_pieces = halo_elems > 0 ? halo_elems * (int64_t)sizeof(T) / 16 : 0;
  dim3 grid((unsigned)cdiv(total, 128), (unsigned)(a.cbig / 32));
  const int64_t wgs = (int64_t)grid.x * grid.y;
  if (wgs < kComputeUnits) {  // under one workgroup per CU: one tap per workgroup
    grid.z = kTaps;
    hipLaunchKernelGGL((patch_scatter_kernel<T, 1>), grid, dim3(256), 0, st, a, (const T*)small, (const T*)packed, (const T*)bias,
                       (T*)big, total, face_pieces, big_elems);
  } else if (wgs < 4 * kComputeUnits) {  // under four per CU: two taps (the big voxels next to each other along W)
    grid.z = kTaps / 2;
    hipLaunchKernelGGL((patch_scatter_kernel<T, 2>), grid, dim3(256), 0, st, a, (const T*)small, (const T*)packed, (const T*)bias,
                       (T*)big, total, face_pieces, big_elems);
  } else {
    // four taps (one big depth plane of the 2 x 2 x 2 patch) per workgroup: eight taps need 295 registers a lane, i.e. one
    // wavefront per SIMD walking four dependent trips to memory each (31 us at 64 -> 32 on 32 x 64 x 64); with half the
    // accumulators three wavefronts share a SIMD, and the small tensor read twice costs less than that gains
    grid.z = 2;
    hipLaunchKernelGGL((patch_scatter_kernel<T, 4>), grid, dim3(256), 0, st, a, (const T*)small, (const T*)packed, (const T*)bias,
                       (T*)big, total, face_pieces, big_elems);
  }
  return check_launch("patch_scatter_kernel");
}

struct ReducePlan { int splits; int64_t per_split; };

ReducePlan reduce_plan(const PatchArgs& a) {
  const int64_t total = small_voxels(a);
  const int64_t tiles = (int64_t)(a.csmall / kSmallTile) * (a.cbig / 32);
  const int64_t rounds = cdiv(total, kVx);
  int64_t splits = cdiv(2 * kComputeUnits, tiles);  // every split writes a whole fp32 slice: more would be write-bound
  if (splits > rounds) splits = rounds;
  if (splits < 1) splits = 1;
  ReducePlan p;
  p.per_split = cdiv(rounds, splits) * kVx;
  p.splits = (int)cdiv(total, p.per_split);
  return p;
}

template <typename T>
int launch_reduce(const PatchArgs& a, const void* small, const void* big, void* g, int g_dtype, void* ws, hipStream_t st, void* gb) {
  const ReducePlan p = reduce_plan(a);
  const int64_t total = small_voxels(a);
  const dim3 grid((unsigned)p.splits, (unsigned)(a.csmall / kSmallTile), (unsigned)(a.cbig / 32));
  const int64_t nelem = (int64_t)a.csmall * kTaps * a.cbig;
  float* bias_part = (float*)ws + (int64_t)p.splits * nelem;  // behind the weight slices
  if (gb != nullptr)
    hipLaunchKernelGGL((patch_reduce_kernel<T, true>), grid, dim3(256), 0, st, a, (const T*)small, (const T*)big, (float*)ws, total,
                       p.per_split, bias_part);
  else
    hipLaunchKernelGGL((patch_reduce_kernel<T, false>), grid, dim3(256), 0, st, a, (const T*)small, (const T*)big, (float*)ws, total,
                       p.per_split, (float*)nullptr);
  if (int rc = check_launch("patch_reduce_kernel")) return rc;
  if (gb == nullptr) return sum_slices(g_dtype, (const float*)ws, g, nelem, p.splits, st);
  // both sums in one launch; the bias partials are [split][tap][channel]: slices of cbig elements
  return sum_slices_two(g_dtype, (const float*)ws, g, nelem, p.splits, bias_part, gb, a.cbig, p.splits * kTaps, st);
}

bool geometry_ok(const PatchArgs& a, int dtype) {
  if (dtype != SFH_BF16 && dtype != SFH_FP16) return false;
  if (a.n < 1 || a.sd < 1 || a.sh < 1 || a.sw < 1) return false;
  if (a.bd < 2 * a.sd || a.bh < 2 * a.sh || a.bw < 2 * a.sw) return false;
  if (cdiv(small_voxels(a), 128) > 0x7fffffffLL) return false;
  return true;
}

}  // namespace

bool patch_supported(const PatchArgs& a, int dtype) {
  return geometry_ok(a, dtype) && a.cbig % 32 == 0 && a.csmall % 32 == 0 && a.cbig / 32 <= 65535 && a.csmall / 32 <= 65535;
}

bool patch_reduce_supported(const PatchArgs& a, int dtype) {
  return geometry_ok(a, dtype) && a.cbig % 32 == 0 && a.csmall % kSmallTile == 0 && a.cbig / 32 <= 65535 &&
         a.csmall / kSmallTile <= 65535;
}

int patch_gather(const PatchArgs& a, int dtype, const void* big, const void* packed, const void* bias, void* small, hipStream_t st) {
  if (dtype == SFH_BF16) return launch_gather<bf16_t>(a, big, packed, bias, small, st);
  return launch_gather<fp16_t>(a, big, packed, bias, small, st);
}

int patch_scatter(const PatchArgs& a, int dtype, const void* small, const void* packed, const void* bias, void* big, hipStream_t st,
                  int64_t halo_elems) {
  if (dtype == SFH_BF16) return launch_scatter<bf16_t>(a, small, packed, bias, big, st, halo_elems);
  return launch_scatter<fp16_t>(a, small, packed, bias, big, st, halo_elems);
}

int patch_reduce_splits(const PatchArgs& a) { return reduce_plan(a).splits; }

size_t patch_reduce_workspace_bytes(const PatchArgs& a, bool with_bias) {
  const size_t splits = (size_t)reduce_plan(a).splits;
  return splits * a.csmall * kTaps * a.cbig * sizeof(float) + (with_bias ? splits * kTaps * a.cbig * sizeof(float) : 0);
}

int patch_reduce(const PatchArgs& a, int dtype, const void* small, const void* big, void* g, int g_dtype, void* ws, hipStream_t st,
                 void* gb) {
  if (gb != nullptr && (a.bd != 2 * a.sd || a.bh != 2 * a.sh || a.bw != 2 * a.sw))
    return fail(SFH_ERR_UNSUPPORTED, "2x2x2 weight gradient: the bias gradient needs every big voxel under a tap");
  if (dtype == SFH_BF16) return launch_reduce<bf16_t>(a, small, big, g, g_dtype, ws, st, gb);
  return launch_reduce<fp16_t>(a, small, big, g, g_dtype, ws, st, gb);
}

}  // namespace sfh
