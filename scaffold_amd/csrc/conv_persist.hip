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
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }
};
template <> struct Mma<fp16_t> {
  static __device__ __forceinline__ f32x16_t run(const uint4& a, const uint4& b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) { return pack_fp16x2(lo, hi); }
};

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
};

__device__ __forceinline__ TileCoord decode_tile(int tile, const PersistGeom& gm) {
  TileCoord tc;
  tc.w = tile % gm.tiles_w; tile /= gm.tiles_w;
  tc.h = tile % gm.tiles_h; tile /= gm.tiles_h;
  tc.d = tile % gm.tiles_d;
  tc.n = tile / gm.tiles_d;
  return tc;
}

// The brick after `tc` in (n, d, h, w) order, w fastest: increments with carries, no divisions.
__device__ __forceinline__ TileCoord next_tile(TileCoord tc, const PersistGeom& gm) {
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

// What a wavefront streams into the other brick buffer during a step: for each of its 64-voxel
// groups the per-lane buffer offset (out of range = zero fill), or -1 in lanes past the brick's end.
template <typename C>
struct BrickFetch {
  int voff[C::GPW];
};

// Output of the previous brick, already rounded, waiting to be stored during the next step.
template <typename C>
struct PendingStore {
  uint2 data[C::MS][4];
  int64_t off[C::MS];  // element offset of the lane's voxel row in y, or -1
};

// Streams a whole brick at once (used for the first brick of a workgroup).
template <typename T, typename C>
__device__ __forceinline__ void fetch_brick(char* dst, int wave, const T* origin, const BrickFetch<C>& bf) {
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(origin), 0, kRange, 0x00020000);
#pragma unroll
  for (int k = 0; k < C::GPW; ++k)
    if (bf.voff[k] != -1) {
#pragma unroll
      for (int p = 0; p < 4; ++p)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + (wave + 4 * k) * 1024 + p * C::PLANE),
                                                 16, bf.voff[k] + p * 16, 0, 0, 0);
    }
}

// One step: MFMAs over the brick in `cur`; interleaved with them, one instruction at a time so that
// neither the memory pipe nor the matrix pipe sees a burst: the direct-to-LDS loads of the next brick
// (even iterations), the stores of the previous brick's output (odd iterations) and, when STREAM, the
// weight fragments of the next chunk (each right after its last use).
template <typename T, typename C, bool STREAM>
__device__ __forceinline__ void persist_step(const char* cur, char* nxt, int wave, const int (&lbase)[C::MS], uint4 (&wq)[C::NIT],
                                             f32x16_t (&acc)[C::MS], const T* wnext, const T* origin, const BrickFetch<C>& bf,
                                             const PendingStore<C>& ps, bool have_store, T* __restrict__ y) {
  constexpr int FRAG = 512;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(origin), 0, kRange, 0x00020000);
  constexpr int NLOAD = C::GPW * 4;
  constexpr int NSTORE = C::MS * 4;
  static_assert(2 * NLOAD <= C::NIT && 2 * NSTORE <= C::NIT, "one memory instruction per iteration");
  // activation fragments are requested ADEPTH iterations ahead of the MFMAs that consume them
  constexpr int ADEPTH = 2;
  uint4 aq[ADEPTH + 1][C::MS];
#pragma unroll
  for (int d = 0; d < ADEPTH; ++d)
#pragma unroll
    for (int ms = 0; ms < C::MS; ++ms) aq[d][ms] = *reinterpret_cast<const uint4*>(cur + lbase[ms] + lds_off<C>(d));
#pragma unroll
  for (int it = 0; it < C::NIT; ++it) {
    if (it + ADEPTH < C::NIT) {
#pragma unroll
      for (int ms = 0; ms < C::MS; ++ms)
        aq[(it + ADEPTH) % (ADEPTH + 1)][ms] = *reinterpret_cast<const uint4*>(cur + lbase[ms] + lds_off<C>(it + ADEPTH));
    }
    if (it % 2 == 0 && it / 2 < NLOAD) {
      const int k = (it / 2) / 4, p = (it / 2) % 4;
      if (bf.voff[k] != -1)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(nxt + (wave + 4 * k) * 1024 + p * C::PLANE),
                                                 16, bf.voff[k] + p * 16, 0, 0, 0);
    }
    if (it % 2 == 1 && it / 2 < NSTORE) {
      const int ms = (it / 2) / 4, g = (it / 2) % 4;
      if (have_store && ps.off[ms] >= 0) *reinterpret_cast<uint2*>(y + ps.off[ms] + 8 * g) = ps.data[ms][g];
    }
    __builtin_amdgcn_sched_barrier(0);
    if (it == 0 && !STREAM) {
      // a single-chunk brick starts from zero: the first MFMA takes a zero addend instead of a clearing pass
      f32x16_t zero;
#pragma unroll
      for (int r = 0; r < 16; ++r) zero[r] = 0.f;
#pragma unroll
      for (int ms = 0; ms < C::MS; ++ms) acc[ms] = Mma<T>::run(wq[it], aq[it % (ADEPTH + 1)][ms], zero);
    } else {
#pragma unroll
      for (int ms = 0; ms < C::MS; ++ms) acc[ms] = Mma<T>::run(wq[it], aq[it % (ADEPTH + 1)][ms], acc[ms]);
    }
    if (STREAM) wq[it] = *reinterpret_cast<const uint4*>(wnext + it * FRAG);
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <typename T, typename C, bool STREAM>
__global__ void __launch_bounds__(256, 1)
conv_persist_kernel(MfmaConvArgs a, const T* __restrict__ x, const T* __restrict__ wp, const T* __restrict__ bias,
                    T* __restrict__ y, PersistGeom gm) {
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
  const int ncc = a.cred / 32;
  const int nsteps = (tile_end - tile_begin) * ncc;

  int lbase[C::MS];
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) {
    const int v = (wave * C::MS + ms) * 32 + j;
    const int tw = v % C::TW, th = (v / C::TW) % C::TH, td = v / (C::TW * C::TH);
    lbase[ms] = kg * C::PLANE + ((td * C::BH + th) * C::BW + tw) * 16;
  }

  // Staging role of this lane, fixed for the whole launch: wave w fills the 64-voxel groups
  // w, w+4, ... of every plane; the lane's voxel inside the brick and its byte offset from the
  // brick origin in the input tensor.
  int gcoord[C::GPW], grel[C::GPW];
#pragma unroll
  for (int k = 0; k < C::GPW; ++k) {
    const int vox = (wave + 4 * k) * 64 + lane;
    const int bw = vox % C::BW, bh = (vox / C::BW) % C::BH, bd = vox / (C::BW * C::BH);
    gcoord[k] = vox < C::BV ? (bd | (bh << 8) | (bw << 16)) : -1;
    grel[k] = (((bd * a.ih + bh) * a.iw + bw) * a.cred) * 2;
  }

  constexpr int FRAG = 512;
  const int64_t slab = (int64_t)C::NIT * FRAG;  // elements per (output block, chunk) weight slab
  const T* wblock = wp + (int64_t)nb * ncc * slab + lane * 8;

  uint4 wq[C::NIT];
#pragma unroll
  for (int it = 0; it < C::NIT; ++it) wq[it] = *reinterpret_cast<const uint4*>(wblock + it * FRAG);

  // Buffer descriptor and per-lane offsets of the brick of (tile, chunk). The descriptor is based at the
  // (possibly virtual) voxel at the brick origin; lanes whose voxel lies outside the input never
  // dereference it: they use an out-of-range offset and receive zeros.
  auto plan_brick = [&](const TileCoord& tc, int cc, BrickFetch<C>& bf) -> const T* {
    const int tw_i = tc.w, th_i = tc.h, td_i = tc.d, n = tc.n;
    const int id0 = td_i * C::TD - a.pd, ih0 = th_i * C::TH - a.ph, iw0 = tw_i * C::TW - a.pw;
    const T* origin = x + ((((int64_t)n * a.id + id0) * a.ih + ih0) * a.iw + iw0) * a.cred + cc * 32;
#pragma unroll
    for (int k = 0; k < C::GPW; ++k) {
      const int bd = gcoord[k] & 0xff, bh = (gcoord[k] >> 8) & 0xff, bw = (gcoord[k] >> 16) & 0xff;
      const bool inside = (unsigned)(id0 + bd) < (unsigned)a.id && (unsigned)(ih0 + bh) < (unsigned)a.ih &&
                          (unsigned)(iw0 + bw) < (unsigned)a.iw;
      bf.voff[k] = gcoord[k] < 0 ? -1 : (inside ? grel[k] : kRange);
    }
    return origin;
  };

  BrickFetch<C> bf;
  TileCoord tc = decode_tile(tile_begin, gm);
  const T* origin = plan_brick(tc, 0, bf);
  fetch_brick<T, C>(buf0, wave, origin, bf);
  __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // this wave's part of the brick has landed
  __syncthreads();

  // Output position of this lane's voxel of every sub-tile relative to the brick origin: coordinates (for the
  // ragged-edge test) and element offset, fixed for the whole launch.
  int vcoord[C::MS], vrel[C::MS];
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) {
    const int v = (wave * C::MS + ms) * 32 + j;
    const int tw = v % C::TW, th = (v / C::TW) % C::TH, td = v / (C::TW * C::TH);
    vcoord[ms] = td | (th << 8) | (tw << 16);
    vrel[ms] = ((td * a.oh + th) * a.ow + tw) * a.cout + 4 * kg;
  }

  f32x16_t acc[C::MS];
  PendingStore<C> ps;
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) ps.off[ms] = -1;
  bool have_store = false;
  int cc = 0;
  for (int step = 0; step < nsteps; ++step) {
    TileCoord ntc = tc;
    int ncc_next = cc + 1;
    if (ncc_next == ncc) { ncc_next = 0; ntc = next_tile(tc, gm); }
    const bool has_next = step + 1 < nsteps;
    // On the last step the current brick is fetched once more (into the idle buffer) rather than
    // branching around every interleaved load.
    origin = plan_brick(has_next ? ntc : tc, has_next ? ncc_next : cc, bf);
    // slab to stream into the weight registers during this step (the current one again at the end)
    const T* wnext = wblock + (int64_t)(has_next ? ncc_next : cc) * slab;

    if (STREAM && cc == 0) {
#pragma unroll
      for (int ms = 0; ms < C::MS; ++ms)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[ms][r] = 0.f;
    }

    if (step & 1) persist_step<T, C, STREAM>(buf1, buf0, wave, lbase, wq, acc, wnext, origin, bf, ps, have_store, y);
    else persist_step<T, C, STREAM>(buf0, buf1, wave, lbase, wq, acc, wnext, origin, bf, ps, have_store, y);
    have_store = false;

    if (cc == ncc - 1) {
      // Round the finished brick now; its stores ride along with the next step's MFMAs. Accumulator
      // register 4g+t of a lane is output channel 8g + 4*kg + t of voxel j of the sub-tile: the two
      // k-half lanes of a voxel write adjacent 8-byte halves of a 16-byte piece.
      const int od0 = tc.d * C::TD, oh0 = tc.h * C::TH, ow0 = tc.w * C::TW;
      const int64_t tile_off = ((((int64_t)tc.n * a.od + od0) * a.oh + oh0) * a.ow + ow0) * a.cout + nb * 32;  // wave-uniform
#pragma unroll
      for (int ms = 0; ms < C::MS; ++ms) {
        const int td = vcoord[ms] & 0xff, th = (vcoord[ms] >> 8) & 0xff, tw = vcoord[ms] >> 16;
        const bool ok = od0 + td < a.od && oh0 + th < a.oh && ow0 + tw < a.ow;
        ps.off[ms] = ok ? tile_off + vrel[ms] : -1;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          if (bias != nullptr) {
            const T* bp = bias + nb * 32 + 8 * g + 4 * kg;
            ps.data[ms][g].x = Mma<T>::pack2(acc[ms][4 * g] + to_float(bp[0]), acc[ms][4 * g + 1] + to_float(bp[1]));
            ps.data[ms][g].y = Mma<T>::pack2(acc[ms][4 * g + 2] + to_float(bp[2]), acc[ms][4 * g + 3] + to_float(bp[3]));
          } else {
            ps.data[ms][g].x = Mma<T>::pack2(acc[ms][4 * g], acc[ms][4 * g + 1]);
            ps.data[ms][g].y = Mma<T>::pack2(acc[ms][4 * g + 2], acc[ms][4 * g + 3]);
          }
        }
      }
      have_store = true;
    }

    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // this wave's part of the next brick has landed
    __syncthreads();                            // ... and every wave is done reading the current one
    tc = ntc;
    cc = ncc_next;
  }
  if (have_store) {
#pragma unroll
    for (int ms = 0; ms < C::MS; ++ms)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        if (ps.off[ms] >= 0) *reinterpret_cast<uint2*>(y + ps.off[ms] + 8 * g) = ps.data[ms][g];
  }
#endif
}

template <typename T, typename C>
int launch_tile(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st) {
  PersistGeom gm{};
  gm.tiles_d = (int)cdiv(a.od, C::TD);
  gm.tiles_h = (int)cdiv(a.oh, C::TH);
  gm.tiles_w = (int)cdiv(a.ow, C::TW);
  const int64_t ntiles = (int64_t)a.n * gm.tiles_d * gm.tiles_h * gm.tiles_w;
  if (ntiles > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "conv mfma: too many bricks");
  gm.ntiles = (int)ntiles;
  gm.nblocks = a.cout / 32;
  int per_block = kComputeUnits / gm.nblocks;
  if (per_block < 1) per_block = 1;
  if (per_block > gm.ntiles) per_block = gm.ntiles;
  gm.items_per_wg = (int)cdiv(gm.ntiles, per_block);
  gm.wgs_per_block = (int)cdiv(gm.ntiles, gm.items_per_wg);
  const unsigned grid = (unsigned)(gm.wgs_per_block * gm.nblocks);
  if (a.cred == 32)
    hipLaunchKernelGGL((conv_persist_kernel<T, C, false>), dim3(grid), dim3(256), 0, st, a, (const T*)x, (const T*)packed,
                       (const T*)bias, (T*)y, gm);
  else
    hipLaunchKernelGGL((conv_persist_kernel<T, C, true>), dim3(grid), dim3(256), 0, st, a, (const T*)x, (const T*)packed,
                       (const T*)bias, (T*)y, gm);
  return check_launch("conv_persist_kernel");
}

template <typename T>
int launch_typed(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st) {
  if (a.ow > 16) return launch_tile<T, PTile<4, 4, 32>>(a, x, packed, bias, y, st);
  if (a.ow > 8) return launch_tile<T, PTile<4, 8, 16>>(a, x, packed, bias, y, st);
  return launch_tile<T, PTile<8, 8, 8>>(a, x, packed, bias, y, st);
}

}  // namespace

int mfma_conv_persist(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y,
                      void* partial, hipStream_t st) {
  // The persistent kernel pays off when the weight slab stays in registers for the whole launch, i.e. with a
  // single 32-channel reduction chunk; wider reductions run the brick-per-workgroup kernel. A brick (at most
  // 10 x 10 input rows deep and high) must also span less than kRange bytes of the input.
  if (a.cred != 32 || ((int64_t)10 * a.ih + 10) * a.iw * a.cred * 2 + 64 >= kRange)
    return mfma_conv_gather(a, dtype, x, packed, bias, y, partial, st);
  if (dtype == SFH_BF16) return launch_typed<bf16_t>(a, x, packed, bias, y, st);
  return launch_typed<fp16_t>(a, x, packed, bias, y, st);
}

}  // namespace sfh
