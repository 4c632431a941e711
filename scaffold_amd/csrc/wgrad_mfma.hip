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
// and all 32x32 (co, ci) outputs of those taps: 112 accumulator registers. One workgroup per CU
// walks the tiles of its K range; the next tile's operands are fetched into registers before the
// current tile's MFMAs start, so global-memory latency is hidden behind the compute.
#include "wgrad_mfma.hpp"
#include <type_traits>

#include "mma.hpp"
#include "reduce.hpp"

namespace sfh {
namespace {

constexpr int kTargetWorkgroups = kComputeUnits;

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
  static_assert(2 * LDS <= 160 * 1024, "two buffers in the 160 KB LDS of a CU");
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

// Fragments of one k-step for a wavefront: the gy fragment, the nine-element windows of its two brick rows,
// and the window of its extra tap (already positioned on that tap's first element pair).
struct KFrags {
  uint4 af;
  uint4 lo0, lo1;
  uint32_t nx0, nx1;
  uint4 lox;
  uint32_t nxx;
};

template <typename C>
__device__ __forceinline__ KFrags load_frags(const char* gsrc, const char* row0, const char* row1, const char* rowx, int ks) {
  const int koff = x_window_off<C>(ks, 0, 0);
  KFrags f;
  f.af = *reinterpret_cast<const uint4*>(gsrc + ks * 32);
  f.lo0 = *reinterpret_cast<const uint4*>(row0 + koff);
  f.nx0 = *reinterpret_cast<const uint32_t*>(row0 + koff + 16);
  f.lo1 = *reinterpret_cast<const uint4*>(row1 + koff);
  f.nx1 = *reinterpret_cast<const uint32_t*>(row1 + koff + 16);
  f.lox = *reinterpret_cast<const uint4*>(rowx + koff);
  f.nxx = *reinterpret_cast<const uint32_t*>(rowx + koff + 16);
  return f;
}

// All four wavefronts run this one straight-line code path; what differs per wavefront (its two brick rows
// and the kw of its extra tap) enters through addresses and one shift amount, so there are no branches and
// the accumulators stay in place across the tile loop. Wavefront 3 has no 27th tap: it repeats tap (2,2,0)
// into an accumulator that is never stored (it would otherwise idle at the barrier). The fragments of
// k-step ks+1 are read from LDS before the MFMAs of k-step ks are issued: with one wavefront per SIMD
// nothing else hides the LDS latency.
template <typename T, typename C>
__device__ __forceinline__ void wave_compute(const char* lds, int lane, int wave, f32x16_t (&acc)[7]) {
  const int i = lane & 31, kg = lane >> 5;
  const char* gsrc = lds + C::GOFF + i * C::GC + kg * 16;
  // k-half offset inside X: 8 voxels along W, or (TW == 8) the next brick row
  const int xbase = i * C::XC + (C::TW == 8 ? kg * C::XR * 2 : kg * 16);
  const int r0 = 2 * wave, r1 = 2 * wave + 1;
  const char* row0 = lds + xbase + ((r0 / 3) * C::BH + r0 % 3) * C::XR * 2;
  const char* row1 = lds + xbase + ((r1 / 3) * C::BH + r1 % 3) * C::XR * 2;
  // extra tap (2, 2, kw): kw = 1 is a 16-bit funnel shift, kw = 2 takes the next dword (wave-uniform selects)
  const int kwx = wave < 3 ? wave : 0;
  const char* rowx = lds + xbase + (2 * C::BH + 2) * C::XR * 2;
  const uint32_t shx = kwx == 1 ? 16u : 0u;
  const bool next_dword = kwx == 2;
  KFrags cur = load_frags<C>(gsrc, row0, row1, rowx, 0);
#pragma unroll
  for (int ks = 0; ks < C::NKS; ++ks) {
    // first MFMA of this k-step, then the LDS reads of the next one, then the other six MFMAs: the wait for
    // this k-step's fragments comes before any younger read is in flight
    __builtin_amdgcn_sched_barrier(0);
    acc[0] = Mma32<T>::run(cur.af, cur.lo0, acc[0]);
    __builtin_amdgcn_sched_barrier(0);
    KFrags nxt = cur;
    if (ks + 1 < C::NKS) nxt = load_frags<C>(gsrc, row0, row1, rowx, ks + 1);
    __builtin_amdgcn_sched_barrier(0);
    acc[1] = Mma32<T>::run(cur.af, shift_one(cur.lo0, cur.nx0), acc[1]);
    acc[2] = Mma32<T>::run(cur.af, make_uint4(cur.lo0.y, cur.lo0.z, cur.lo0.w, cur.nx0), acc[2]);
    acc[3] = Mma32<T>::run(cur.af, cur.lo1, acc[3]);
    acc[4] = Mma32<T>::run(cur.af, shift_one(cur.lo1, cur.nx1), acc[4]);
    acc[5] = Mma32<T>::run(cur.af, make_uint4(cur.lo1.y, cur.lo1.z, cur.lo1.w, cur.nx1), acc[5]);
    uint4 fx;
    fx.x = next_dword ? cur.lox.y : __builtin_amdgcn_alignbit(cur.lox.y, cur.lox.x, shx);
    fx.y = next_dword ? cur.lox.z : __builtin_amdgcn_alignbit(cur.lox.z, cur.lox.y, shx);
    fx.z = next_dword ? cur.lox.w : __builtin_amdgcn_alignbit(cur.lox.w, cur.lox.z, shx);
    fx.w = next_dword ? cur.nxx : __builtin_amdgcn_alignbit(cur.nxx, cur.lox.w, shx);
    acc[6] = Mma32<T>::run(cur.af, fx, acc[6]);
    __builtin_amdgcn_sched_barrier(0);
    cur = nxt;
  }
}

template <typename C>
__device__ __forceinline__ void wave_store(const f32x16_t (&acc)[7], float* __restrict__ dst, int cin, int lane, int wave) {
  const int j = lane & 31, kg = lane >> 5;
#pragma unroll
  for (int t = 0; t < 7; ++t) {
    if (t == 6 && wave == 3) break;
    const int tap = t < 3 ? 6 * wave + t : (t < 6 ? 6 * wave + t : 24 + wave);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int co = 8 * (r / 4) + 4 * kg + (r % 4);
      dst[((int64_t)co * 27 + tap) * cin + j] = acc[t][r];
    }
  }
}

// A staging item is (8-channel piece, 4-voxel slot). Within a wavefront the 16 lanes of a quarter share the
// piece and take 16 consecutive slots: their transposed 8-byte LDS writes to one channel row are then
// contiguous, and the two pieces of a half-wave land 128 bytes apart (mod 256), i.e. on disjoint banks.
__device__ __forceinline__ int item_piece(int item) { return (item >> 4) & 3; }
__device__ __forceinline__ int item_slot(int item) { return ((item >> 6) << 4) | (item & 15); }

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
constexpr uint32_t kOob = 0x80000000u;   // a byte offset no sample reaches: the buffer load returns zeros
constexpr int kWaitLgkm0 = 0xC07F;       // s_waitcnt immediate (gfx9): lgkmcnt(0), vmcnt and expcnt untouched

// Per-thread staging geometry, fixed for the whole kernel. Slot 0 is the thread's gy item, slots 1..XIT its x
// items; an item is four consecutive W voxels x 8 channels.
template <typename C>
struct Slots {
  // slots are handed out 16 per wavefront pass of 64 items
  static constexpr int XIT = ((C::NBR * C::NQX + 15) / 16 * 64 + 255) / 256;
  static constexpr int N = 1 + XIT;
  int dst[N];  // LDS byte offset (inside one buffer) of the item's first channel row; -1: the thread has no such item
  int off[N];  // byte offset of the item's first voxel from the tile origin
  int crd[N];  // row coordinates relative to the tile origin and first W position: r0 | r1 << 8 | w0 << 16
  uint4 raw[N][4];
};

struct TileOrigin { int n, od0, oh0, ow0; };

__device__ __forceinline__ TileOrigin decode_tile(int tile, int tiles_d, int tiles_h, int tiles_w, int td, int th, int tw) {
  TileOrigin o;
  int t = tile;
  o.ow0 = (t % tiles_w) * tw; t /= tiles_w;
  o.oh0 = (t % tiles_h) * th; t /= tiles_h;
  o.od0 = (t % tiles_d) * td;
  o.n = t / tiles_d;
  return o;
}

template <typename C>
__device__ __forceinline__ void init_slots(const WgradArgs& a, int tid, Slots<C>& sl) {
  {
    const int piece = item_piece(tid), q = item_slot(tid);
    const int quad = q % (C::TW / 4), grow = q / (C::TW / 4);
    const int td = grow / C::TH, th = grow % C::TH, w0 = quad * 4;
    sl.dst[0] = C::GOFF + (piece * 8) * C::GC + grow * C::TW * 2 + quad * 8;
    sl.off[0] = ((td * a.oh + th) * a.ow + w0) * a.cout * 2 + piece * 16;
    sl.crd[0] = td | (th << 8) | (w0 << 16);
  }
#pragma unroll
  for (int it = 0; it < Slots<C>::XIT; ++it) {
    const int item = it * 256 + tid;
    const int piece = item_piece(item), q = item_slot(item);
    const int quad = q % C::NQX, brow = q / C::NQX;
    const int bd = brow / C::BH, bh = brow % C::BH, w0 = quad * 4;
    sl.dst[1 + it] = q < C::NBR * C::NQX ? (piece * 8) * C::XC + brow * C::XR * 2 + quad * 8 : -1;
    sl.off[1 + it] = ((bd * a.ih + bh) * a.iw + w0) * a.cin * 2 + piece * 16;
    sl.crd[1 + it] = bd | (bh << 8) | (w0 << 16);
  }
}

// Issues the four 16-byte loads of slot S for the tile at `o`. Voxels outside the tensor (padding, ragged tiles)
// get an out-of-range offset, for which the buffer load returns zeros.
template <typename T, typename C, int S>
__device__ __forceinline__ void fetch_slot(const WgradArgs& a, const T* __restrict__ x, const T* __restrict__ gy, const TileOrigin& o,
                                           int cib, int cob, Slots<C>& sl) {
  const int r0 = sl.crd[S] & 0xff, r1 = (sl.crd[S] >> 8) & 0xff, w0 = sl.crd[S] >> 16;
  if (S == 0) {
    const int64_t sample = (int64_t)a.od * a.oh * a.ow * a.cout;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(gy + o.n * sample), 0, (int)(sample * 2), 0x00020000);
    const int org = ((o.od0 * a.oh + o.oh0) * a.ow + o.ow0) * a.cout * 2 + cob * 64;
    // plain integer masks (no short-circuit), so that the selection stays a select and never becomes a branch
    const int rowok = (int)(o.od0 + r0 < a.od) & (int)(o.oh0 + r1 < a.oh);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int ok = rowok & (int)(o.ow0 + w0 + k < a.ow);
      const uint32_t voff = ok != 0 ? (uint32_t)(org + sl.off[0] + k * a.cout * 2) : kOob;
      sl.raw[0][k] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, voff, 0, 0));
    }
  } else {
    const int64_t sample = (int64_t)a.id * a.ih * a.iw * a.cin;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(x + o.n * sample), 0, (int)(sample * 2), 0x00020000);
    const int id0 = o.od0 - a.pd, ih0 = o.oh0 - a.ph, iw0 = o.ow0 - a.pw;
    const int org = ((id0 * a.ih + ih0) * a.iw + iw0) * a.cin * 2 + cib * 64;
    const int rowok = (int)(sl.dst[S] >= 0) & (int)((unsigned)(id0 + r0) < (unsigned)a.id) & (int)((unsigned)(ih0 + r1) < (unsigned)a.ih);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int ok = rowok & (int)(w0 + k < C::TW + 2) & (int)((unsigned)(iw0 + w0 + k) < (unsigned)a.iw);
      const uint32_t voff = ok != 0 ? (uint32_t)(org + sl.off[S] + k * a.cin * 2) : kOob;
      sl.raw[S][k] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, voff, 0, 0));
    }
  }
}

// Transposes four voxels x 8 channels (v[k] = voxel k) into 8 channel rows of 4 voxels at dst, dst + stride, ...
__device__ __forceinline__ void store_transposed(char* dst, int stride, const uint4 (&v)[4]) {
  const uint32_t d0[4] = {v[0].x, v[0].y, v[0].z, v[0].w}, d1[4] = {v[1].x, v[1].y, v[1].z, v[1].w},
                 d2[4] = {v[2].x, v[2].y, v[2].z, v[2].w}, d3[4] = {v[3].x, v[3].y, v[3].z, v[3].w};
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    uint2 e0, e1;
    transpose4(d0[d], d1[d], d2[d], d3[d], e0, e1);
    *reinterpret_cast<uint2*>(dst + (2 * d) * stride) = e0;
    *reinterpret_cast<uint2*>(dst + (2 * d + 1) * stride) = e1;
  }
}

template <typename C, int S>
__device__ __forceinline__ void stage_slot(char* buf, const Slots<C>& sl) {
  if (S == 0 || sl.dst[S] >= 0) store_transposed(buf + sl.dst[S], S == 0 ? C::GC : C::XC, sl.raw[S]);
}

template <typename T, typename C, int S>
struct SlotLoop {
  static __device__ __forceinline__ void fetch_all(const WgradArgs& a, const T* x, const T* gy, const TileOrigin& o, int cib, int cob,
                                                   Slots<C>& sl) {
    fetch_slot<T, C, S>(a, x, gy, o, cib, cob, sl);
    if constexpr (S + 1 < Slots<C>::N) SlotLoop<T, C, S + 1>::fetch_all(a, x, gy, o, cib, cob, sl);
  }
  static __device__ __forceinline__ void stage_all(char* buf, const Slots<C>& sl) {
    stage_slot<C, S>(buf, sl);
    if constexpr (S + 1 < Slots<C>::N) SlotLoop<T, C, S + 1>::stage_all(buf, sl);
  }
  // Slot by slot: the raw data fetched one tile ago goes to the idle LDS buffer and the registers are refilled
  // with the tile after next.
  static __device__ __forceinline__ void stage_and_refill(char* idle, const WgradArgs& a, const T* x, const T* gy,
                                                          const TileOrigin& o2, int cib, int cob, Slots<C>& sl) {
    stage_slot<C, S>(idle, sl);
    fetch_slot<T, C, S>(a, x, gy, o2, cib, cob, sl);
    if constexpr (S + 1 < Slots<C>::N) SlotLoop<T, C, S + 1>::stage_and_refill(idle, a, x, gy, o2, cib, cob, sl);
  }
};

// One 8-wavefront workgroup per CU, two LDS buffers, two kinds of wavefront (one of each per SIMD):
//   * wavefronts 0..3 only compute: LDS fragment reads, the kw shifts and 112 MFMAs per tile;
//   * wavefronts 4..7 only stage: while tile t is being computed out of one buffer they transpose tile t+1
//     (which they fetched into registers during tile t-1) into the other buffer and refill their registers
//     with tile t+2, so global-memory latency has a whole tile period to hide in.
// A SIMD issues one vector-ALU instruction per four cycles whatever the number of wavefronts; keeping the
// staging arithmetic out of the MFMA wavefront's instruction stream (and the two streams on different
// wavefronts, which issue to different ports concurrently) is what lets the MFMA pipe stay busy.
// One barrier per tile joins all eight wavefronts.
template <typename T, typename C>
__global__ void __launch_bounds__(512)
wgrad_mfma_kernel(WgradArgs a, const T* __restrict__ x, const T* __restrict__ gy, float* __restrict__ ws, int tiles_d,
                  int tiles_h, int tiles_w, int ntiles, int tiles_per_split, int nblk_ci, int nblk, uint32_t total,
                  const T* __restrict__ x1, int c_first) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(16))) char buf0[C::LDS];
  __shared__ __attribute__((aligned(16))) char buf1[C::LDS];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  uint32_t wg = xcd_remap(blockIdx.x, total);
  const int blk = wg % nblk;
  const int split = wg / nblk;
  const int cib = blk % nblk_ci, cob = blk / nblk_ci;

  const int t_begin = split * tiles_per_split;
  int t_end = t_begin + tiles_per_split;
  if (t_end > ntiles) t_end = ntiles;

  if (wave >= 4) {
    // ---- staging wavefronts ----
    if (t_begin >= t_end) return;
    // An input handed over as two tensors whose channels follow each other (the first c_first in x, the rest in x1):
    // the workgroup's 32 input channels lie in one of them, and from here on that tensor IS the input -- its channel
    // count in `as`, the block's index inside it in `cis`. Only the gradient's own indexing keeps a.cin and cib.
    WgradArgs as = a;
    const T* xs = x;
    int cis = cib;
    if (x1 != nullptr) {
      const bool second = cib * 32 >= c_first;
      xs = second ? x1 : x;
      as.cin = second ? a.cin - c_first : c_first;
      cis = second ? cib - c_first / 32 : cib;
    }
    Slots<C> sl;
    init_slots<C>(as, tid - 256, sl);
    auto origin = [&](int tile) {
      return decode_tile(tile < t_end ? tile : t_end - 1, tiles_d, tiles_h, tiles_w, C::TD, C::TH, C::TW);
    };
    SlotLoop<T, C, 0>::fetch_all(as, xs, gy, origin(t_begin), cis, cob, sl);
    SlotLoop<T, C, 0>::stage_all(buf0, sl);
    SlotLoop<T, C, 0>::fetch_all(as, xs, gy, origin(t_begin + 1), cis, cob, sl);
    __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
    __builtin_amdgcn_s_barrier();
    for (int tile = t_begin; tile < t_end; ++tile) {
      char* idle = ((tile - t_begin) & 1) ? buf0 : buf1;
      // On the last tiles the staged / fetched data is never used; doing the work anyway keeps the loop free of
      // branches (the fetch is clamped to the split's last tile).
      const TileOrigin o2 = origin(tile + 2);
      SlotLoop<T, C, 0>::stage_and_refill(idle, as, xs, gy, o2, cis, cob, sl);
      __builtin_amdgcn_s_waitcnt(kWaitLgkm0);  // the LDS writes of the next tile have landed
      __builtin_amdgcn_s_barrier();            // ... and the compute wavefronts are done reading the current one
    }
    return;
  }

  // ---- compute wavefronts ----
  f32x16_t acc[7];
#pragma unroll
  for (int t = 0; t < 7; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
  if (t_begin < t_end) {
    __builtin_amdgcn_s_barrier();  // the first tile is staged
    for (int tile = t_begin; tile < t_end; ++tile) {
      const char* cur = ((tile - t_begin) & 1) ? buf1 : buf0;
      asm volatile("" ::: "memory");  // LDS changes behind this wavefront's back: reload every tile
      wave_compute<T, C>(cur, lane, wave, acc);
      __builtin_amdgcn_s_barrier();
    }
  }
  float* dst = ws + ((int64_t)split * a.cout + cob * 32) * 27 * a.cin + cib * 32;
  wave_store<C>(acc, dst, a.cin, lane, wave);
#endif
}

// ---- several small-volume weight gradients in one launch ----------------------------------------------------------------------
// The deep levels of a U-Net have many 32 x 32 blocks and few tiles under each (8 tiles at 8 x 16 x 16, one at
// 4 x 8 x 8): launched one problem at a time every workgroup walks a handful of tiles, writes a slice and a sum pass
// follows -- 23-44 us for 4-29 GFLOP. In a batch the UNITS -- (problem, block) with all its tiles -- of all problems lie
// on one line of cost (tiles + kUnitCost each), workgroup w of W takes the units that start in
// [w total / W, (w + 1) total / W), walks each from its first tile to its last and stores the finished block straight
// into the gradient: no slices, no sum pass, and the order of additions of a block is that of its tiles, whatever else
// is in the list. The two tile shapes (rows of 16 and of 8 voxels) share a launch.
constexpr int kUnitCost = 2;          // what starting and storing a unit costs, in tiles (1 .. 5 measure alike)
constexpr int kBatchMaxTiles = 32;    // longer units would not balance: such problems are launched alone

struct WTileBatchEntry {
  WgradArgs a;
  const void* x;
  const void* x1;
  const void* gy;
  void* gw;
  int c_first;
  int tw;                              // 16 or 8
  int tiles_d, tiles_h, tiles_w, ntiles;
  int nblk_ci, nblk;
  int pos_begin;
};

struct WTileBatch {
  int count, wgs, total;
  WTileBatchEntry e[kWgradBatchMax];
};

template <typename C, typename TOut>
__device__ __forceinline__ void wave_store_block(const f32x16_t (&acc)[7], TOut* __restrict__ dst, int cin, int lane, int wave) {
  const int j = lane & 31;
  int kg = lane >> 5;
  // (opaque to the optimiser: in the loop over units it would otherwise compute all 112 store offsets ahead of the loop
  // and keep them in scratch memory)
  asm volatile("" : "+v"(kg));
#pragma unroll
  for (int t = 0; t < 7; ++t) {
    if (t == 6 && wave == 3) break;
    const int tap = t < 3 ? 6 * wave + t : (t < 6 ? 6 * wave + t : 24 + wave);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int co = 8 * (r / 4) + 4 * kg + (r % 4);
      dst[((int64_t)co * 27 + tap) * cin + j] = elem<TOut>::from_float(acc[t][r]);
    }
  }
}

// One unit: all tiles of block (cob, cib) of a problem, the finished block stored at gw. The staging wavefronts and
// the compute wavefronts meet at 1 + ntiles barriers, as in the kernel above.
template <typename T, typename C, typename TOut>
__device__ __forceinline__ void wtile_unit(const WgradArgs& a, const T* __restrict__ x, const T* __restrict__ x1, int c_first,
                                           const T* __restrict__ gy, TOut* __restrict__ gw, int tiles_d, int tiles_h, int tiles_w,
                                           int ntiles, int cib, int cob, char* buf0, char* buf1, int tid) {
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (wave >= 4) {
    WgradArgs as = a;
    const T* xs = x;
    int cis = cib;
    if (x1 != nullptr) {
      const bool second = cib * 32 >= c_first;
      xs = second ? x1 : x;
      as.cin = second ? a.cin - c_first : c_first;
      cis = second ? cib - c_first / 32 : cib;
    }
    Slots<C> sl;
    init_slots<C>(as, tid - 256, sl);
    auto origin = [&](int tile) { return decode_tile(tile < ntiles ? tile : ntiles - 1, tiles_d, tiles_h, tiles_w, C::TD, C::TH, C::TW); };
    SlotLoop<T, C, 0>::fetch_all(as, xs, gy, origin(0), cis, cob, sl);
    SlotLoop<T, C, 0>::stage_all(buf0, sl);
    SlotLoop<T, C, 0>::fetch_all(as, xs, gy, origin(1), cis, cob, sl);
    __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
    __builtin_amdgcn_s_barrier();
    for (int tile = 0; tile < ntiles; ++tile) {
      char* idle = (tile & 1) ? buf0 : buf1;
      SlotLoop<T, C, 0>::stage_and_refill(idle, as, xs, gy, origin(tile + 2), cis, cob, sl);
      __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
      __builtin_amdgcn_s_barrier();
    }
  } else {
    f32x16_t acc[7];
#pragma unroll
    for (int t = 0; t < 7; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
    __builtin_amdgcn_s_barrier();  // the first tile is staged
    for (int tile = 0; tile < ntiles; ++tile) {
      const char* cur = (tile & 1) ? buf1 : buf0;
      asm volatile("" ::: "memory");  // LDS changes behind this wavefront's back: reload every tile
      wave_compute<T, C>(cur, lane, wave, acc);
      __builtin_amdgcn_s_barrier();
    }
    wave_store_block<C, TOut>(acc, gw + ((int64_t)cob * 32 * 27) * a.cin + cib * 32, a.cin, lane, wave);
  }
}

typedef WTile<2, 8, 16> WTile16;
typedef WTile<4, 8, 8> WTile8;
constexpr int kBatchLds = WTile16::LDS > WTile8::LDS ? WTile16::LDS : WTile8::LDS;

__host__ __device__ __forceinline__ int tile_batch_cut(int w, int total, int wgs) { return (int)((uint32_t)w * (uint32_t)total / (uint32_t)wgs); }

template <typename T, typename TOut>
__global__ void __launch_bounds__(512) wgrad_mfma_batch_kernel(WTileBatch b) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(16))) char buf0[kBatchLds];
  __shared__ __attribute__((aligned(16))) char buf1[kBatchLds];
  const int tid = threadIdx.x;
  const int w = (int)xcd_remap(blockIdx.x, (uint32_t)b.wgs);
  const int hi = tile_batch_cut(w + 1, b.total, b.wgs);
  int pos = tile_batch_cut(w, b.total, b.wgs);
  while (pos < hi) {
    int p = 0;
    for (int k = 1; k < b.count; ++k)
      if (pos >= b.e[k].pos_begin) p = k;
    const int ntiles = b.e[p].ntiles, cost = ntiles + kUnitCost;
    const int unit = (pos - b.e[p].pos_begin + cost - 1) / cost;  // the first unit that starts at or behind pos
    if (unit >= b.e[p].nblk) {  // none left in this problem: on to the next one's first unit
      pos = p + 1 < b.count ? b.e[p + 1].pos_begin : hi;
      continue;
    }
    const int start = b.e[p].pos_begin + unit * cost;
    if (start >= hi) break;
    const WgradArgs a = b.e[p].a;
    const int nblk_ci = b.e[p].nblk_ci;
    const int cib = unit % nblk_ci, cob = unit / nblk_ci;
    if (b.e[p].tw == 16)
      wtile_unit<T, WTile16, TOut>(a, (const T*)b.e[p].x, (const T*)b.e[p].x1, b.e[p].c_first, (const T*)b.e[p].gy, (TOut*)b.e[p].gw,
                                   b.e[p].tiles_d, b.e[p].tiles_h, b.e[p].tiles_w, ntiles, cib, cob, buf0, buf1, tid);
    else
      wtile_unit<T, WTile8, TOut>(a, (const T*)b.e[p].x, (const T*)b.e[p].x1, b.e[p].c_first, (const T*)b.e[p].gy, (TOut*)b.e[p].gw,
                                  b.e[p].tiles_d, b.e[p].tiles_h, b.e[p].tiles_w, ntiles, cib, cob, buf0, buf1, tid);
    pos = start + cost;
  }
#endif
}

struct Plan {
  int tw;  // 32, 16 or 8
  int tiles_d, tiles_h, tiles_w, ntiles;
  int nblk_ci, nblk;
  int splits, tiles_per_split;
};

// Rows of more than 16 voxels take the column-walking kernel.
bool ring_serves(const WgradArgs& a) { return mfma_wgrad_ring_applies(a); }

Plan make_plan(const WgradArgs& a) {
  Plan p{};
  if (ring_serves(a)) {
    p.tw = 32;
    p.splits = mfma_wgrad_ring_splits(a);
    return p;
  }
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
  // Slices along the voxel range: at most one workgroup per CU; from there the count is halved while a cost estimate
  // says that pays. A workgroup's time is its tiles (2.4 us each at this kernel's rate); every slice of every 32 x 32
  // block is 108 KiB of fp32 that is written and, when there is more than one slice, read again by the ordered sum
  // (a launch of its own). Units of 0.01 us, constants fitted to timings of the U-Net's levels: the small-volume
  // levels (8 tiles for 64-128 blocks) are cheaper with 1-4 slices than with one per CU.
  int target = kTargetWorkgroups;
  int want = target / p.nblk;
  if (want < 1) want = 1;
  if (want > p.ntiles) want = p.ntiles;
  int64_t best = -1;
  for (int s = want; s >= 1; s /= 2) {
    const int tps = (int)cdiv(p.ntiles, s), eff = (int)cdiv(p.ntiles, tps);
    const int64_t cost = eff > 1 ? 240LL * tps + 1000 + 64LL * eff * p.nblk / 10 : 240LL * tps + 600 + 32LL * p.nblk / 10;
    if (best < 0 || cost < best) {
      best = cost;
      p.tiles_per_split = tps;
      p.splits = eff;
    }
  }
  return p;
}

template <typename T, typename C>
int launch_tile(const WgradArgs& a, const Plan& p, const void* x, const void* gy, float* ws, hipStream_t st, const ChannelPair& x2) {
  const int64_t total = (int64_t)p.splits * p.nblk;
  hipLaunchKernelGGL((wgrad_mfma_kernel<T, C>), dim3((unsigned)total), dim3(512), 0, st, a, (const T*)x, (const T*)gy, ws,
                     p.tiles_d, p.tiles_h, p.tiles_w, p.ntiles, p.tiles_per_split, p.nblk_ci, p.nblk, (uint32_t)total,
                     (const T*)x2.second, x2.first);
  return check_launch("wgrad_mfma_kernel");
}

template <typename T>
int launch_typed(const WgradArgs& a, const void* x, const void* gy, void* gw, int gw_dtype, void* workspace, hipStream_t st,
                 const ChannelPair& x2) {
  const Plan p = make_plan(a);
  // One slice and an fp32 gradient (the deepest levels under fp32 master weights): the kernel's slice IS the
  // gradient, so it is written in place and no sum pass follows.
  const bool direct = p.splits == 1 && gw_dtype == SFH_FP32;
  float* ws = direct ? (float*)gw : (float*)workspace;
  int rc;
  if (ring_serves(a)) rc = mfma_wgrad_ring(a, std::is_same<T, bf16_t>::value ? SFH_BF16 : SFH_FP16, x, gy, ws, st, x2);
  else if (p.tw == 32) rc = launch_tile<T, WTile<2, 4, 32>>(a, p, x, gy, ws, st, x2);
  else if (p.tw == 16) rc = launch_tile<T, WTile<2, 8, 16>>(a, p, x, gy, ws, st, x2);
  else rc = launch_tile<T, WTile<4, 8, 8>>(a, p, x, gy, ws, st, x2);
  if (rc != SFH_OK || direct) return rc;
  const int64_t nelem = (int64_t)a.cout * 27 * a.cin;
  return sum_slices(gw_dtype, ws, gw, nelem, p.splits, st);
}

bool tile_batch_plan(const WgradBatchItem* items, int count, WTileBatch& b) {
  if (count < 1 || count > kWgradBatchMax) return false;
  b = WTileBatch{};
  b.count = count;
  int64_t pos = 0;
  for (int i = 0; i < count; ++i) {
    const WgradArgs& a = items[i].a;
    if (ring_serves(a)) return false;
    const Plan p = make_plan(a);
    if (p.tw == 32 || p.ntiles > kBatchMaxTiles) return false;
    WTileBatchEntry& e = b.e[i];
    e.a = a;
    e.x = items[i].x; e.x1 = items[i].x1; e.c_first = items[i].c_first; e.gy = items[i].gy; e.gw = items[i].gw;
    e.tw = p.tw;
    e.tiles_d = p.tiles_d; e.tiles_h = p.tiles_h; e.tiles_w = p.tiles_w; e.ntiles = p.ntiles;
    e.nblk_ci = p.nblk_ci; e.nblk = p.nblk;
    e.pos_begin = (int)pos;
    pos += (int64_t)p.nblk * (p.ntiles + kUnitCost);
    if (pos > 0x7fffff) return false;  // 32-bit cuts
  }
  b.total = (int)pos;
  b.wgs = b.total < kTargetWorkgroups ? b.total : kTargetWorkgroups;
  return true;
}

template <typename T>
int launch_tile_batch(const WTileBatch& b, int gw_dtype, hipStream_t st) {
  if (b.total == 0) return SFH_OK;
  if (gw_dtype == SFH_FP32) hipLaunchKernelGGL((wgrad_mfma_batch_kernel<T, float>), dim3((unsigned)b.wgs), dim3(512), 0, st, b);
  else hipLaunchKernelGGL((wgrad_mfma_batch_kernel<T, T>), dim3((unsigned)b.wgs), dim3(512), 0, st, b);
  return check_launch("wgrad_mfma_batch_kernel");
}

}  // namespace

bool mfma_wgrad_supported(const WgradArgs& a, int dtype) {
  if (dtype != SFH_BF16 && dtype != SFH_FP16) return false;
  if (a.cin % 32 != 0 || a.cout % 32 != 0) return false;
  if (a.pd < 0 || a.ph < 0 || a.pw < 0 || a.pd > 2 || a.ph > 2 || a.pw > 2) return false;
  if (a.n < 1 || a.od < 1 || a.oh < 1 || a.ow < 1) return false;
  // staging addresses one sample with 32-bit byte offsets
  const int64_t limit = 0x7ff00000LL;
  if ((int64_t)a.id * a.ih * a.iw * a.cin * 2 > limit || (int64_t)a.od * a.oh * a.ow * a.cout * 2 > limit) return false;
  const Plan p = make_plan(a);
  if ((int64_t)a.n * p.tiles_d * p.tiles_h * p.tiles_w > 0x7fffffffLL) return false;
  return true;
}

int mfma_wgrad_splits(const WgradArgs& a) { return make_plan(a).splits; }

size_t mfma_wgrad_workspace_bytes(const WgradArgs& a) {
  const Plan p = make_plan(a);
  return align_up((size_t)p.splits * a.cout * 27 * a.cin * sizeof(float), 256);
}

bool mfma_wgrad_pair_ok(const WgradArgs& a, int first) { return first > 0 && first < a.cin && first % 32 == 0; }

int mfma_wgrad(const WgradArgs& a, int dtype, const void* x, const void* gy, void* gw, int gw_dtype, void* workspace,
               hipStream_t st, const ChannelPair* x2) {
  if (x2 != nullptr && (x2->second == nullptr || !mfma_wgrad_pair_ok(a, x2->first)))
    return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad: the input cannot be cut at channel %d of %d", x2->first, a.cin);
  const ChannelPair pair = x2 != nullptr ? *x2 : ChannelPair{nullptr, 0};
  if (dtype == SFH_BF16) return launch_typed<bf16_t>(a, x, gy, gw, gw_dtype, workspace, st, pair);
  return launch_typed<fp16_t>(a, x, gy, gw, gw_dtype, workspace, st, pair);
}

// ---- a list of problems: the ring-served ones in one launch + sum pass, the small-volume ones in one launch -------------
namespace {
bool tile_batch_applies(const WgradArgs& a) {
  if (ring_serves(a)) return false;
  const Plan p = make_plan(a);
  return p.tw != 32 && p.ntiles <= kBatchMaxTiles;
}
// Splits a list by family, keeping the order inside each.
int split_list(const WgradBatchItem* items, int count, WgradBatchItem* ring, int& nring, WgradBatchItem* tile, int& ntile) {
  nring = ntile = 0;
  for (int i = 0; i < count; ++i) {
    if (ring_serves(items[i].a)) ring[nring++] = items[i];
    else if (tile_batch_applies(items[i].a)) tile[ntile++] = items[i];
    else return SFH_ERR_UNSUPPORTED;
  }
  return SFH_OK;
}
}  // namespace

bool mfma_wgrad_batch_applies(const WgradArgs& a, int dtype) {
  return mfma_wgrad_supported(a, dtype) && (ring_serves(a) || tile_batch_applies(a));
}

size_t mfma_wgrad_batch_workspace_bytes(const WgradBatchItem* items, int count, int max_wgs) {
  if (count < 1 || count > kWgradBatchMax) return 0;
  WgradBatchItem ring[kWgradBatchMax], tile[kWgradBatchMax];
  int nring, ntile;
  if (split_list(items, count, ring, nring, tile, ntile) != SFH_OK) return 0;
  WTileBatch tb;
  if (ntile > 0 && !tile_batch_plan(tile, ntile, tb)) return 0;
  if (nring == 0) return 256;  // (nothing is needed; a non-zero answer says the list is taken)
  const size_t bytes = mfma_wgrad_ring_batch_workspace_bytes(ring, nring, max_wgs);
  return bytes;
}

int mfma_wgrad_batch(const WgradBatchItem* items, int count, int dtype, int gw_dtype, void* workspace, size_t workspace_bytes,
                     hipStream_t st, int max_wgs) {
  if (count < 1 || count > kWgradBatchMax) return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad batch: 1 .. %d problems a call", kWgradBatchMax);
  WgradBatchItem ring[kWgradBatchMax], tile[kWgradBatchMax];
  int nring, ntile;
  if (split_list(items, count, ring, nring, tile, ntile) != SFH_OK)
    return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad batch: a problem of the list is served only by a launch of its own");
  WTileBatch tb;
  if (ntile > 0 && !tile_batch_plan(tile, ntile, tb)) return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad batch: the small-volume problems cannot share a launch");
  if (nring > 0)
    if (int rc = mfma_wgrad_ring_batch(ring, nring, dtype, gw_dtype, workspace, workspace_bytes, st, max_wgs)) return rc;
  if (ntile > 0) return dtype == SFH_BF16 ? launch_tile_batch<bf16_t>(tb, gw_dtype, st) : launch_tile_batch<fp16_t>(tb, gw_dtype, st);
  return SFH_OK;
}

}  // namespace sfh
