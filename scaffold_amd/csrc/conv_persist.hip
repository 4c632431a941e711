// Persistent MFMA implicit-GEMM convolution for gfx950 (3x3x3, stride 1, bf16 / fp16).
//
// One workgroup of four wavefronts per CU, resident for the whole launch, walks a contiguous range
// of output bricks. It is built so that the matrix pipe never waits for memory:
//
//   * One wavefront per SIMD may use all 512 vector registers. The 54 weight fragments of a
//     (32 out-channel, 32 reduction-channel) slab -- 216 registers -- therefore stay RESIDENT in
//     registers; with 32 reduction channels they are fetched once per workgroup. With more
//     reduction channels the slab of the next 32-channel chunk is streamed into the same registers,
//     each fragment re-requested right after its last use, one whole chunk (~7k cycles) ahead.
//   * LDS holds TWO input bricks (with halo). While the MFMAs of a step read one, the brick of the
//     next step streams into the other straight from memory (buffer_load ... lds, 16 bytes per
//     lane, no register staging); voxels outside the input are out-of-range buffer offsets and
//     arrive as zeros. Everything a step needs was requested during the previous step, and one
//     barrier per step separates the two roles of a buffer.
//   * A brick is stored as four 16-byte channel planes (conflict-free ds_read_b128 at immediate
//     offsets, see conv_mfma.hip): one direct load instruction fills 64 consecutive voxels of one
//     plane.
//
// Work item = (32-channel output block, brick); workgroup g owns items of ONE output block so its
// weight slab never changes when there is a single reduction chunk.
#include <stdlib.h>

#include "conv_mfma.hpp"
#include "mma.hpp"

namespace sfh {
namespace {

typedef uint32_t sfh_u32x2_t __attribute__((ext_vector_type(2)));

typedef mma_frag_t sfh_i32x4_t;

constexpr int plane_bytes(int voxels) {  // smallest size >= voxels*16 that is 64 modulo 256
  return ((voxels * 16 - 64 + 255) / 256) * 256 + 64;
}

template <int TD_, int TH_, int TW_>
struct PTile {
  static constexpr int TD = TD_, TH = TH_, TW = TW_;
  static constexpr int BD = TD + 2, BH = TH + 2, BW = TW + 2;
  static constexpr int BV = BD * BH * BW;
  static constexpr int PLANE = plane_bytes(BV);
  static constexpr int BRICK = 4 * PLANE;
  static constexpr int LDS = 2 * BRICK;
  static constexpr int NGROUP = (BV + 63) / 64;       // 64-voxel groups of a plane
  static constexpr int GPW = (NGROUP + 3) / 4;        // groups staged by each wavefront
  static constexpr int MS = TD * TH * TW / 128;       // 32-voxel sub-tiles per wavefront
  static constexpr int NIT = 27 * 2;                  // (tap, k-step) iterations per 32-channel chunk
  static constexpr int NVEC = 27;                     // weight fragments kept in vector registers
  static constexpr int PIECES = BV * 4;
  static constexpr int PITER = (PIECES + 255) / 256;  // staging pieces per thread
  static_assert(TD * TH * TW == 512, "four wavefronts of four 32-voxel sub-tiles");
  static_assert(2 * PLANE + (2 * BH * BW + 2 * BW + 2) * 16 < 65536, "ds_read immediate range");
  static_assert(LDS <= 160 * 1024, "LDS of a CU");
};

template <typename C>
__device__ __forceinline__ constexpr int lds_off(int it) {
  const int tap = it / 2, ks = it % 2;
  const int kd = tap / 9, kh = (tap / 3) % 3, kw = tap % 3;
  return ((kd * C::BH + kh) * C::BW + kw) * 16 + ks * 2 * C::PLANE;
}

struct TileCoord { int n, d, h, w; };

struct PersistGeom {
  int tiles_d, tiles_h, tiles_w, ntiles;  // bricks per output block (batch folded in)
  int nblocks, wgs_per_block, items_per_wg;
  int blocked;  // brick order, see decode_tile
};

// Brick order. Plain: (n, d, h, w), w fastest. Blocked (brick counts along d and h divisible by 4): 4 x 4 groups of
// bricks in (d, h), d fastest inside a group, then the groups along d, along h, then w, then n -- a workgroup's run of
// 16 bricks is then a compact 16 x 16 rows region of one w column instead of a 4-row slab across the whole width, and
// consecutive bricks share two of their six input planes: fewer halo voxels are fetched twice (1.34x against 1.7x
// of the input at 128^3) and the re-fetched ones were read one step ago.
__device__ __forceinline__ TileCoord decode_tile(int tile, const PersistGeom& gm) {
  TileCoord tc;
  if (gm.blocked) {
    const int din = tile & 3, hin = (tile >> 2) & 3;
    tile >>= 4;
    const int gd = gm.tiles_d >> 2, gh = gm.tiles_h >> 2;
    tc.d = (tile % gd) * 4 + din; tile /= gd;
    tc.h = (tile % gh) * 4 + hin; tile /= gh;
    tc.w = tile % gm.tiles_w;
    tc.n = tile / gm.tiles_w;
    return tc;
  }
  tc.w = tile % gm.tiles_w; tile /= gm.tiles_w;
  tc.h = tile % gm.tiles_h; tile /= gm.tiles_h;
  tc.d = tile % gm.tiles_d;
  tc.n = tile / gm.tiles_d;
  return tc;
}

// The brick after `tc` in the order of decode_tile: increments with carries, no divisions.
__device__ __forceinline__ TileCoord next_tile(TileCoord tc, const PersistGeom& gm) {
  if (gm.blocked) {
    if ((++tc.d & 3) != 0) return tc;
    tc.d -= 4;
    if ((++tc.h & 3) != 0) return tc;
    tc.h -= 4;
    tc.d += 4;  // next group along d
    if (tc.d != gm.tiles_d) return tc;
    tc.d = 0;
    tc.h += 4;  // next group along h
    if (tc.h != gm.tiles_h) return tc;
    tc.h = 0;
    if (++tc.w == gm.tiles_w) { tc.w = 0; ++tc.n; }
    return tc;
  }
  if (++tc.w == gm.tiles_w) {
    tc.w = 0;
    if (++tc.h == gm.tiles_h) {
      tc.h = 0;
      if (++tc.d == gm.tiles_d) { tc.d = 0; ++tc.n; }
    }
  }
  return tc;
}

// s_waitcnt immediate (gfx9 encoding) that waits for vmcnt <= n and nothing else.
constexpr int waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// Staging loads address the input through a buffer descriptor of kRange bytes based at the brick
// origin: offsets of real voxels are below it, kRange itself (and anything above) reads as zero.
constexpr int kRange = 0x40000000;

// Streams a whole brick at once (used for the first brick of a workgroup). voff: per 64-voxel group the lane's
// buffer offset (out of range = zero fill), or -1 in lanes past the brick's end.
template <typename T, typename C>
__device__ __forceinline__ void fetch_brick(char* dst, int wave, const T* origin, const int (&voff)[C::GPW]) {
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(origin), 0, kRange, 0x00020000);
#pragma unroll
  for (int k = 0; k < C::GPW; ++k)
    if (voff[k] != -1) {
#pragma unroll
      for (int p = 0; p < 4; ++p)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + (wave + 4 * k) * 1024 + p * C::PLANE),
                                                 16, voff[k] + p * 16, 0, 0, 0);
    }
}

// Launch-constant geometry of a lane, and what it needs to know about the input.
template <typename C>
struct LaneGeom {
  int lbase[C::MS];   // LDS byte offset of the lane's A-fragment voxel, per sub-tile
  int gcoord[C::GPW]; // staging: packed brick coordinates of the lane's voxel per group, -1 past the brick
  int grel[C::GPW];   // staging: byte offset of that voxel from the brick origin in the input
  int vcoord[C::MS];  // output: packed tile coordinates of the lane's voxel per sub-tile
  int vrel[C::MS];    // output: byte offset of the lane's first channel from the tile origin in y
};

// Offsets of the brick of tile `tc` for this lane's groups; returns the (possibly virtual) brick origin. Lanes whose
// voxel lies outside the input use an out-of-range offset and receive zeros; `live` false turns the whole brick
// into such lanes (the step after the last has nothing to fetch).
template <typename T, typename C>
__device__ __forceinline__ const T* brick_origin(const MfmaConvArgs& a, const T* x, const TileCoord& tc) {
  const int id0 = tc.d * C::TD - a.pd, ih0 = tc.h * C::TH - a.ph, iw0 = tc.w * C::TW - a.pw;
  return x + ((((int64_t)tc.n * a.id + id0) * a.ih + ih0) * a.iw + iw0) * a.cred;
}
template <typename C>
__device__ __forceinline__ int brick_group_offset(const MfmaConvArgs& a, const TileCoord& tc, bool live, int gcoord, int grel) {
  const int id0 = tc.d * C::TD - a.pd, ih0 = tc.h * C::TH - a.ph, iw0 = tc.w * C::TW - a.pw;
  const int bd = gcoord & 0xff, bh = (gcoord >> 8) & 0xff, bw = (gcoord >> 16) & 0xff;
  const int inside = ((unsigned)(id0 + bd) < (unsigned)a.id) & ((unsigned)(ih0 + bh) < (unsigned)a.ih) &
                     ((unsigned)(iw0 + bw) < (unsigned)a.iw) & (int)live;
  return gcoord < 0 ? -1 : (inside ? grel : kRange);
}
// Byte offset of the lane's output piece of sub-tile voxel `vcoord` from the tile origin, or out of range when the
// voxel lies past the ragged edge of the output (such stores are dropped by the buffer bounds check).
template <typename C>
__device__ __forceinline__ int store_offset(const MfmaConvArgs& a, const TileCoord& tc, int vcoord, int vrel) {
  const int td = vcoord & 0xff, th = (vcoord >> 8) & 0xff, tw = vcoord >> 16;
  const int ok = (tc.d * C::TD + td < a.od) & (tc.h * C::TH + th < a.oh) & (tc.w * C::TW + tw < a.ow);
  return ok ? vrel : kRange;
}
// `row`: channels per voxel of the tensor written, `c0`: the workgroup's first channel in it.
template <typename T, typename C>
__device__ __forceinline__ T* tile_origin(const MfmaConvArgs& a, T* y, const TileCoord& tc, int row, int c0) {
  return y + ((((int64_t)tc.n * a.od + tc.d * C::TD) * a.oh + tc.h * C::TH) * a.ow + tc.w * C::TW) * row + c0;
}

// Output of a finished brick, rounded, waiting to be stored during the next step. Accumulator register 4g+t of a
// lane is output channel 8g + 4*kg + t of voxel j of the sub-tile, so the two k-half lanes of a voxel (lanes j and
// j + 32) hold interleaved runs of four channels. They trade runs (v_permlane32_swap) so that the kg = 0 lane ends
// up with channels 0-7 and 16-23 and the kg = 1 lane with 8-15 and 24-31: each then stores two 16-byte pieces, and
// one store instruction covers 32 contiguous bytes of every voxel instead of 16.
typedef uint32_t sfh_u32x4_t __attribute__((ext_vector_type(4)));
template <typename C>
struct PendingStore {
  sfh_u32x4_t data[C::MS][2];
};

// With GN, the rounded values of the voxels inside the output are also added to the lane's GroupNorm sums. Their shift
// is picked at the first brick whose first voxel of this wavefront lies inside the output (`have_shift`, wave-uniform):
// a workgroup's run of bricks may start on one that a ragged edge cuts off from this wavefront.
template <typename T, typename C, bool BIAS, bool GN>
__device__ __forceinline__ void round_brick(const f32x16_t (&acc)[C::MS], const float (&bias)[16], PendingStore<C>& ps,
                                            const MfmaConvArgs& a, const TileCoord& tc, const LaneGeom<C>& lg, RunSums& sums,
                                            int& have_shift) {
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) {
    uint32_t run[4][2];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float v[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) v[t] = BIAS ? acc[ms][4 * g + t] + bias[4 * g + t] : acc[ms][4 * g + t];
      run[g][0] = Mma32<T>::pack2(v[0], v[1]);
      run[g][1] = Mma32<T>::pack2(v[2], v[3]);
    }
    if constexpr (GN) {
      const bool inside = store_offset<C>(a, tc, lg.vcoord[ms], lg.vrel[ms]) != kRange;
      bool first = false;
      if (ms == 0 && !have_shift) {
        first = __builtin_amdgcn_readfirstlane((int)inside) != 0;  // lane 0 holds the wavefront's first voxel of the brick
        have_shift = first ? 1 : 0;
      }
      sums.template add<T>(run, inside, first);
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      // lanes 32-63 of run 2h <-> lanes 0-31 of run 2h+1
      const auto lo = __builtin_amdgcn_permlane32_swap(run[2 * h][0], run[2 * h + 1][0], false, false);
      const auto hi = __builtin_amdgcn_permlane32_swap(run[2 * h][1], run[2 * h + 1][1], false, false);
      ps.data[ms][h] = sfh_u32x4_t{lo[0], hi[0], lo[1], hi[1]};
    }
  }
}

// One step = one output brick. While the 54 x MS MFMAs run over the brick in `cur`, the wavefront also issues, a
// little in every iteration so that the matrix pipe never waits behind a block of other work:
//   * the direct-to-LDS loads of the next brick into `nxt` (even iterations),
//   * the stores of the PREVIOUS brick's rounded result (odd ones); lanes past a ragged edge carry an out-of-range
//     offset and the buffer bounds check drops their store, so there is no branch,
//   * the fetch offsets of the brick after the next and the store offsets of this brick (late odd iterations),
//     written over the ones this step has finished using.
template <typename T, typename C>
__device__ __forceinline__ void persist_step(const MfmaConvArgs& a, const char* cur, char* nxt, int wave, const LaneGeom<C>& lg,
                                             const uint4 (&wq)[C::NVEC], const sfh_i32x4_t (&wa)[C::NIT - C::NVEC],
                                             f32x16_t (&acc)[C::MS], const PendingStore<C>& ps,
                                             const T* fetch_origin, int (&voff)[C::GPW],
                                             __amdgpu_buffer_rsrc_t done_rsrc, int (&done_off)[C::MS],
                                             const TileCoord& plan_tc, bool plan_live, const TileCoord& tc) {
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(fetch_origin), 0, kRange, 0x00020000);
  constexpr int NLOAD = C::GPW * 4;
  constexpr int NSTORE = C::MS * 2;
  // group k's offsets are overwritten in place, so its planning must come after its last load (iteration 8k + 6)
  constexpr int PLAN0 = 6 * (C::GPW - 1) + 9;       // first (odd) iteration that plans a group
  constexpr int OFF0 = PLAN0 + 2 * C::GPW;          // first (odd) iteration that computes a store offset
  static_assert(2 * NLOAD <= C::NIT && OFF0 + 2 * C::MS <= C::NIT + 1 && PLAN0 > 2 * NSTORE, "one piece of side work per iteration");
  // activation fragments are requested ADEPTH iterations ahead of the MFMAs that consume them
  constexpr int ADEPTH = 2;
  uint4 aq[ADEPTH + 1][C::MS];
#pragma unroll
  for (int d = 0; d < ADEPTH; ++d)
#pragma unroll
    for (int ms = 0; ms < C::MS; ++ms) aq[d][ms] = *reinterpret_cast<const uint4*>(cur + lg.lbase[ms] + lds_off<C>(d));
#pragma unroll
  for (int it = 0; it < C::NIT; ++it) {
    __builtin_amdgcn_sched_barrier(0);
    // The activation fragments of iteration it + ADEPTH are requested BETWEEN this iteration's MFMAs, one behind each: a
    // ds_read issued while the matrix pipe is busy costs nothing, a block of them in front of the MFMAs leaves the pipe
    // idle for as long as they take to issue.
    f32x16_t zero;
#pragma unroll
    for (int r = 0; r < 16; ++r) zero[r] = 0.f;
#pragma unroll
    for (int ms = 0; ms < C::MS; ++ms) {
      // a brick starts from zero: the first MFMA takes a zero addend instead of a clearing pass
      if (it == 0) acc[ms] = Mma32<T>::run(wq[it], aq[it % (ADEPTH + 1)][ms], zero);
      else if (it < C::NVEC) acc[ms] = Mma32<T>::run(wq[it], aq[it % (ADEPTH + 1)][ms], acc[ms]);
      else Mma32Pinned<T>::run_row_in_acc(wa[it - C::NVEC], aq[it % (ADEPTH + 1)][ms], acc[ms]);
      __builtin_amdgcn_sched_barrier(0);
      if (it + ADEPTH < C::NIT)
        aq[(it + ADEPTH) % (ADEPTH + 1)][ms] = *reinterpret_cast<const uint4*>(cur + lg.lbase[ms] + lds_off<C>(it + ADEPTH));
      __builtin_amdgcn_sched_barrier(0);
      // one piece of side work per iteration, behind the first MFMA
      if (ms == 0) {
        if (it % 2 == 0 && it / 2 < NLOAD) {
          const int k = (it / 2) / 4, p = (it / 2) % 4;
          // only the last group of a wavefront can have lanes past the end of the brick
          const bool full = (3 + 4 * k) * 64 + 63 < C::BV;
          if (full || voff[k] != -1)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(nxt + (wave + 4 * k) * 1024 + p * C::PLANE),
                                                     16, voff[k] + p * 16, 0, 0, 0);
        }
        if (it % 2 == 1 && it / 2 < NSTORE) {
          const int ms = (it / 2) / 2, h = (it / 2) % 2;
          __builtin_amdgcn_raw_buffer_store_b128(ps.data[ms][h], done_rsrc, done_off[ms] + 32 * h, 0, 0);
        }
        if (it % 2 == 1 && it >= PLAN0 && (it - PLAN0) / 2 < C::GPW) {
          const int k = (it - PLAN0) / 2;
          voff[k] = brick_group_offset<C>(a, plan_tc, plan_live, lg.gcoord[k], lg.grel[k]);  // group k's loads are all issued
        }
        if (it % 2 == 1 && it >= OFF0 && (it - OFF0) / 2 < C::MS) {
          const int ms = (it - OFF0) / 2;
          done_off[ms] = store_offset<C>(a, tc, lg.vcoord[ms], lg.vrel[ms]);  // the previous brick's pieces are all stored
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <typename T, typename C, bool BIAS, bool GN>
__global__ void __launch_bounds__(256, 1)
conv_persist_kernel(MfmaConvArgs a, const T* __restrict__ x, const T* __restrict__ wp, const T* __restrict__ bias_ptr,
                    T* __restrict__ y, PersistGeom gm, GnPartialOut gn, T* __restrict__ y1, int c_first) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses LDS address-space builtins the host pass cannot type-check
  __shared__ __attribute__((aligned(16))) char buf0[C::BRICK];
  __shared__ __attribute__((aligned(16))) char buf1[C::BRICK];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: LDS destinations become scalar
  const int j = lane & 31, kg = lane >> 5;

  const int wg = (int)xcd_remap(blockIdx.x, gridDim.x);
  const int nb = wg / gm.wgs_per_block;
  const int tile_begin = (wg - nb * gm.wgs_per_block) * gm.items_per_wg;
  int tile_end = tile_begin + gm.items_per_wg;
  if (tile_end > gm.ntiles) tile_end = gm.ntiles;
  if (nb >= gm.nblocks || tile_begin >= tile_end) return;
  const int nsteps = tile_end - tile_begin;

  // Where this workgroup's 32 output channels go: into y, or -- an output handed over as two tensors whose channels
  // follow each other, the first c_first in y and the rest in y1 -- into the one that holds them. Fixed for the launch.
  T* yout = y;
  int yrow = a.cout, yc0 = nb * 32;
  if (y1 != nullptr) {
    const bool second = nb * 32 >= c_first;
    yout = second ? y1 : y;
    yrow = second ? a.cout - c_first : c_first;
    yc0 = second ? nb * 32 - c_first : nb * 32;
  }

  LaneGeom<C> lg;
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) {
    const int v = (wave * C::MS + ms) * 32 + j;
    const int tw = v % C::TW, th = (v / C::TW) % C::TH, td = v / (C::TW * C::TH);
    lg.lbase[ms] = kg * C::PLANE + ((td * C::BH + th) * C::BW + tw) * 16;
    lg.vcoord[ms] = td | (th << 8) | (tw << 16);
    lg.vrel[ms] = (((td * a.oh + th) * a.ow + tw) * yrow + 8 * kg) * 2;
  }
  // Staging role of this lane, fixed for the whole launch: wave w fills the 64-voxel groups w, w+4, ... of every
  // plane; the lane's voxel inside the brick and its byte offset from the brick origin in the input tensor.
#pragma unroll
  for (int k = 0; k < C::GPW; ++k) {
    const int vox = (wave + 4 * k) * 64 + lane;
    const int bw = vox % C::BW, bh = (vox / C::BW) % C::BH, bd = vox / (C::BW * C::BH);
    lg.gcoord[k] = vox < C::BV ? (bd | (bh << 8) | (bw << 16)) : -1;
    lg.grel[k] = (((bd * a.ih + bh) * a.iw + bw) * a.cred) * 2;
  }

  constexpr int FRAG = 512;
  const T* wblock = wp + (int64_t)nb * C::NIT * FRAG + lane * 8;
  // The first NVEC fragments live in vector registers, the rest in accumulation registers (there are not 216 + the
  // activation fragments' worth of vector registers; the MFMA reads its row operand from either file).
  uint4 wq[C::NVEC];
  sfh_i32x4_t wa[C::NIT - C::NVEC];
#pragma unroll
  for (int it = 0; it < C::NVEC; ++it) wq[it] = *reinterpret_cast<const uint4*>(wblock + it * FRAG);
#pragma unroll
  for (int it = C::NVEC; it < C::NIT; ++it) wa[it - C::NVEC] = *reinterpret_cast<const sfh_i32x4_t*>(wblock + it * FRAG);
  float bias[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) bias[r] = BIAS ? to_float(bias_ptr[nb * 32 + 8 * (r / 4) + 4 * kg + (r % 4)]) : 0.f;

  // Bricks in flight: `tc` is computed in this step, `tc1` is fetched during it, `tc2` is planned during it.
  TileCoord tc = decode_tile(tile_begin, gm);
  int voff[C::GPW];
#pragma unroll
  for (int k = 0; k < C::GPW; ++k) voff[k] = brick_group_offset<C>(a, tc, true, lg.gcoord[k], lg.grel[k]);
  fetch_brick<T, C>(buf0, wave, brick_origin<T, C>(a, x, tc), voff);
  TileCoord tc1 = next_tile(tc, gm);
#pragma unroll
  for (int k = 0; k < C::GPW; ++k) voff[k] = brick_group_offset<C>(a, tc1, nsteps > 1, lg.gcoord[k], lg.grel[k]);
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // this wave's part of the first brick has landed
  __syncthreads();

  f32x16_t acc[C::MS];
  PendingStore<C> ps;
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms)
#pragma unroll
    for (int h = 0; h < 2; ++h) ps.data[ms][h] = sfh_u32x4_t{0u, 0u, 0u, 0u};
  int done_off[C::MS];
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) done_off[ms] = kRange;  // nothing to store during the first step
  T* done_origin = yout;
  RunSums gn_sums;  // GroupNorm statistics of this workgroup's rounded outputs (GN)
  gn_sums.clear();
  int gn_have_shift = 0;

  for (int step = 0; step < nsteps; ++step) {
    const TileCoord tc2 = next_tile(tc1, gm);
    const bool live2 = step + 2 < nsteps;
    const T* fetch_origin = brick_origin<T, C>(a, x, tc1);
    const __amdgpu_buffer_rsrc_t done_rsrc = __builtin_amdgcn_make_buffer_rsrc(done_origin, 0, kRange, 0x00020000);
    if (step & 1) persist_step<T, C>(a, buf1, buf0, wave, lg, wq, wa, acc, ps, fetch_origin, voff, done_rsrc, done_off, tc2, live2, tc);
    else persist_step<T, C>(a, buf0, buf1, wave, lg, wq, wa, acc, ps, fetch_origin, voff, done_rsrc, done_off, tc2, live2, tc);
    asm volatile("s_nop 15\n\ts_nop 15");  // the last MFMAs are inline asm: the compiler does not know their result latency
    round_brick<T, C, BIAS, GN>(acc, bias, ps, a, tc, lg, gn_sums, gn_have_shift);  // its stores ride along with the next step's MFMAs
    done_origin = tile_origin<T, C>(a, yout, tc, yrow, yc0);
    tc = tc1;
    tc1 = tc2;
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // this wave's part of the next brick has landed
    __syncthreads();                            // ... and every wave is done reading the current one
  }
  // the last brick's result
  const __amdgpu_buffer_rsrc_t done_rsrc = __builtin_amdgcn_make_buffer_rsrc(done_origin, 0, kRange, 0x00020000);
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms)
#pragma unroll
    for (int h = 0; h < 2; ++h) __builtin_amdgcn_raw_buffer_store_b128(ps.data[ms][h], done_rsrc, done_off[ms] + 32 * h, 0, 0);
  if constexpr (GN) {
    // one record per workgroup (one sample): the loop's last barrier has freed the LDS
    const int per_wg = gn.cg > 32 ? gn.cg / 32 : 1;  // output blocks that share a group
    RunSums one[1] = {gn_sums};
    write_group_partials<4, 1>(one, reinterpret_cast<float*>(buf0), gn, 0, (wg - nb * gm.wgs_per_block) * per_wg + nb % per_wg, nb * 32, tid);
  }
#endif
}

PersistGeom persist_geom(const MfmaConvArgs& a, int td, int th, int tw) {
  PersistGeom gm{};
  gm.tiles_d = (int)cdiv(a.od, td);
  gm.tiles_h = (int)cdiv(a.oh, th);
  gm.tiles_w = (int)cdiv(a.ow, tw);
  const int64_t ntiles = (int64_t)a.n * gm.tiles_d * gm.tiles_h * gm.tiles_w;
  gm.ntiles = ntiles > 0x7fffffffLL ? -1 : (int)ntiles;
  gm.blocked = (gm.tiles_d % 4 == 0 && gm.tiles_h % 4 == 0) ? 1 : 0;
  gm.nblocks = a.cout / 32;
  int per_block = kComputeUnits / gm.nblocks;
  if (per_block < 1) per_block = 1;
  if (per_block > gm.ntiles) per_block = gm.ntiles;
  if (gm.ntiles > 0) {
    gm.items_per_wg = (int)cdiv(gm.ntiles, per_block);
    gm.wgs_per_block = (int)cdiv(gm.ntiles, gm.items_per_wg);
  }
  return gm;
}
PersistGeom persist_geom(const MfmaConvArgs& a) {
  if (a.ow > 16) return persist_geom(a, 4, 4, 32);
  if (a.ow > 8) return persist_geom(a, 4, 8, 16);
  return persist_geom(a, 8, 8, 8);
}

template <typename T, typename C>
int launch_tile(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                const GnPartialOut& gn, const ChannelPair& out2) {
  const PersistGeom gm = persist_geom(a, C::TD, C::TH, C::TW);
  if (gm.ntiles < 0) return fail(SFH_ERR_UNSUPPORTED, "conv mfma: too many bricks");
  if (gm.ntiles == 0) return SFH_OK;
  const unsigned grid = (unsigned)(gm.wgs_per_block * gm.nblocks);
#define SFH_PERSIST(BIAS, GN)                                                                                                    \
  hipLaunchKernelGGL((conv_persist_kernel<T, C, BIAS, GN>), dim3(grid), dim3(256), 0, st, a, (const T*)x, (const T*)packed, \
                     (const T*)bias, (T*)y, gm, gn, (T*)out2.second, out2.first)
  if (bias != nullptr) {
    if (gn.part != nullptr) SFH_PERSIST(true, true);
    else SFH_PERSIST(true, false);
  } else {
    if (gn.part != nullptr) SFH_PERSIST(false, true);
    else SFH_PERSIST(false, false);
  }
#undef SFH_PERSIST
  return check_launch("conv_persist_kernel");
}

template <typename T>
int launch_typed(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                 const GnPartialOut& gn, const ChannelPair& out2) {
  if (a.ow > 16) return launch_tile<T, PTile<4, 4, 32>>(a, x, packed, bias, y, st, gn, out2);
  if (a.ow > 8) return launch_tile<T, PTile<4, 8, 16>>(a, x, packed, bias, y, st, gn, out2);
  return launch_tile<T, PTile<8, 8, 8>>(a, x, packed, bias, y, st, gn, out2);
}

}  // namespace

// Rows of more than 16 voxels take the column-walking form of the persistent kernel.
static bool ring_serves(const MfmaConvArgs& a) {
  return mfma_conv_ring_applies(a) && a.od > 0 && a.n > 0;
}

// The persistent kernel pays off when the weight slab stays in registers for the whole launch, i.e. with a
// single 32-channel reduction chunk; wider reductions run the brick-per-workgroup kernel. A brick (at most
// 10 x 10 input rows deep and high) must also span less than kRange bytes of the input, a tile (at most 8 x 8 output
// rows) less than kRange bytes of the output.
bool mfma_conv_persist_applies(const MfmaConvArgs& a) {
  return a.cred == 32 && ((int64_t)10 * a.ih + 10) * a.iw * a.cred * 2 + 64 < kRange &&
         ((int64_t)8 * a.oh + 8) * a.ow * a.cout * 2 + 64 < kRange;
}

MfmaConvGeometry mfma_conv_geometry(const MfmaConvArgs& a) {
  if (!mfma_conv_persist_applies(a)) return mfma_conv_gather_geometry(a);
  return MfmaConvGeometry{kKernelPersist, 512, 1, 1};
}

// One record per workgroup, so one sample only (a workgroup's run of bricks may cross samples).
int mfma_conv_gn_records(const MfmaConvArgs& a, int groups) {
  if (!mfma_conv_persist_applies(a)) return mfma_conv_gather_gn_records(a, groups);
  if (a.n != 1 || !gn_partials_fit(a.cout, groups, 32)) return 0;
  const int cg = a.cout / groups;
  if (ring_serves(a)) return mfma_conv_ring_workgroups_per_block(a) * (cg > 32 ? cg / 32 : 1);
  const PersistGeom gm = persist_geom(a);
  if (gm.ntiles <= 0) return 0;
  return gm.wgs_per_block * (cg > 32 ? cg / 32 : 1);
}

// A persistent workgroup owns one 32-channel output block for the whole launch: any cut of the OUTPUT at a multiple of
// 32 channels falls between workgroups (a tile of either tensor spans less than the kernel's addressing range a
// fortiori). Its 32 reduction channels cannot be cut.
bool mfma_conv_pair_ok(const MfmaConvArgs& a, int first, bool as_output) {
  if (!mfma_conv_persist_applies(a)) return mfma_conv_gather_pair_ok(a, first, as_output);
  return as_output && first > 0 && first < a.cout && first % 32 == 0;
}

int mfma_conv_persist(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y,
                      void* partial, hipStream_t st, const GnPartialOut* gn, const ChannelPair* in2, const ChannelPair* out2) {
  if (!mfma_conv_persist_applies(a)) return mfma_conv_gather(a, dtype, x, packed, bias, y, partial, st, gn, in2, out2);
  if (in2 != nullptr) return fail(SFH_ERR_UNSUPPORTED, "conv persist: 32 reduction channels cannot be a pair of tensors");
  if (out2 != nullptr && (out2->second == nullptr || !mfma_conv_pair_ok(a, out2->first, true)))
    return fail(SFH_ERR_UNSUPPORTED, "conv persist: the output cannot be cut at channel %d of %d", out2->first, a.cout);
  const ChannelPair pair = out2 != nullptr ? *out2 : ChannelPair{nullptr, 0};
  GnPartialOut out{nullptr, 0, 0, 0};
  if (gn != nullptr && gn->part != nullptr) {
    if (gn->records == 0 || gn->records != mfma_conv_gn_records(a, gn->groups))
      return fail(SFH_ERR_INVALID, "conv persist: GroupNorm partials asked for %d records, this launch leaves %d", gn->records,
                  mfma_conv_gn_records(a, gn->groups));
    out = *gn;
    out.cg = a.cout / gn->groups;
  }
  if (ring_serves(a)) return mfma_conv_ring(a, dtype, x, packed, bias, y, st, out, pair);
  if (dtype == SFH_BF16) return launch_typed<bf16_t>(a, x, packed, bias, y, st, out, pair);
  return launch_typed<fp16_t>(a, x, packed, bias, y, st, out, pair);
}

}  // namespace sfh
