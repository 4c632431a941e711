// Wide-tile MFMA implicit-GEMM convolution for gfx950 (3x3x3, stride 1, bf16 / fp16): forward and data gradient with
// 64 or more reduction channels (GEMM view as triton_conv3d/gather_gemm.py:112-341: M = output voxels, N = produced
// channels, K = taps x reduction channels).
//
// What bounds such a kernel on this chip is operand delivery, not the matrix pipe: a ds_read_b128 of a wavefront moves
// 1 KiB and the LDS delivers 128 bytes per clock, so one LDS operand read per 32-cycle MFMA from each of the four SIMDs
// already saturates it. The tile is therefore shaped for reuse out of registers:
//
//   * One workgroup of four wavefronts per CU (all 512 registers per lane), each wavefront holding an MS x NSUB grid of
//     32-voxel x 32-channel accumulator blocks (16 blocks = 256 registers): per tap it reads MS activation fragments
//     and NSUB weight fragments for MS x NSUB MFMAs -- 0.5 (4 x 4) or 0.625 (8 x 2) LDS reads per MFMA instead of
//     1.25.
//   * The reduction runs in chunks of 16 channels (one MFMA k-step): the input brick of a chunk, halo included, sits
//     in LDS as two 16-byte channel planes (conflict-free ds_read_b128 at immediate tap offsets), double-buffered, and
//     is fetched with direct-to-LDS buffer loads (no register staging; voxels outside the input are out-of-range
//     offsets and arrive as zeros) while the MFMAs of the previous chunk run.
//   * The weight fragments are SHARED through LDS: the packed weight is already in fragment order, so a fragment is
//     one 1 KiB direct-to-LDS load; the 12 fragments of a step (12 / NSUB taps) arrive one step ahead in a two-slot
//     ring.
//   * Every wavefront fetches a quarter of both: three weight fragments at a step's barrier, then its share of the
//     next chunk's brick one load per tap. A wavefront's loads complete in order, so the wait for the next step's
//     weights allows exactly the brick loads issued after them to stay in flight.
//   * One barrier per step, placed before the step's LAST tap: the operands of that tap are already in registers, so
//     its MFMAs cover the latency of the first reads after the barrier. The operand reads of the next tap are issued
//     BETWEEN the MFMAs of the current one: a ds_read issued while the matrix pipe is busy costs nothing, a block of
//     them in front of the MFMAs leaves the pipe idle for as long as they take to issue.
//
// The data gradient runs this kernel with the weight packed transposed and tap-flipped and padding k-1-p
// (triton_conv3d/bwd_data.py:344-363). Launch geometry is a pure function of the shape.
#include <stdlib.h>

#include <type_traits>
#include <utility>

#include "conv_mfma.hpp"
#include "mma.hpp"

namespace sfh {
namespace {

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): an unrolled loop whose index is a constant
// expression (instruction immediates: ds_read offsets, s_waitcnt counts).
template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

typedef mma_frag_t frag_t;  // one MFMA operand fragment of a lane (8 x 16 bit)

// LDS operand reads are issued as inline asm and waited for by hand (lgkmcnt): the compiler cannot tell which
// direct-to-LDS loads in flight a ds_read depends on and would otherwise wait for all of them (vmcnt(0)) before the
// first read that follows one -- the pipeline below keeps several in flight on purpose.
template <int OFFSET>
__device__ __forceinline__ frag_t lds_read_frag(int addr) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "ds_read immediate range");
  frag_t v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET) : "memory");
  return v;
}
// The MFMAs are the inline-asm form with the accumulator pinned to accumulation registers: left to the compiler, the 256
// accumulator values of a lane wander between the two register files around the loop and push the addresses the loop
// needs out to scratch memory. An accumulator block is reused only every MS x NSUB MFMAs, so no wait states are needed
// between them; the epilogue waits out the last ones by hand.
__device__ __forceinline__ void zero_pinned(f32x16_t& c) {
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float z;
    asm volatile("v_accvgpr_write_b32 %0, 0" : "=a"(z));
    c[r] = z;
  }
}

// Orders every later use of `v` behind the preceding s_waitcnt (an empty asm: no instruction).
__device__ __forceinline__ void landed(frag_t& v) { asm volatile("" : "+v"(v)); }

constexpr int plane_bytes(int voxels) {  // smallest size >= voxels*16 that is 64 modulo 256
  return ((voxels * 16 - 64 + 255) / 256) * 256 + 64;
}
// s_waitcnt immediate (gfx9 encoding) that waits for vmcnt <= n and nothing else.
constexpr int waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }
// ... for vmcnt <= n and lgkmcnt == 0
constexpr int waitcnt_vm_lgkm0(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (0 << 8); }

// Staging loads address the input through a buffer descriptor of kRange bytes based at the brick origin: offsets of
// real voxels are below it, kRange itself (and anything above) reads as zero.
constexpr int kRange = 0x40000000;
constexpr int kTaps = 27;
constexpr int kFragBytes = 1024;                 // one packed (32 channels x 16 reduction channels) fragment
constexpr int kFragsPerStep = 12;                // weight fragments the four wavefronts fetch per step (3 each)
constexpr int kPairBytes = kTaps * 2 * kFragBytes;  // packed bytes of one (32-channel block, 32-reduction-channel pair)

template <int TD_, int TH_, int TW_, int NSUB_>
struct WTile {
  static constexpr int TD = TD_, TH = TH_, TW = TW_, NSUB = NSUB_;
  static constexpr int BD = TD + 2, BH = TH + 2, BW = TW + 2;
  static constexpr int BV = BD * BH * BW;            // brick voxels
  static constexpr int PLANE = plane_bytes(BV);
  static constexpr int BRICK = 2 * PLANE;            // one 16-channel chunk of the brick
  static constexpr int NGROUP = (BV + 63) / 64;      // 64-voxel groups of a plane
  static constexpr int GPW = NGROUP / 4;             // groups fetched by each wavefront
  static constexpr int NLOAD = 2 * GPW;              // brick loads of a wavefront per chunk
  static constexpr int MS = TD * TH * TW / 128;      // 32-voxel sub-tiles per wavefront
  static constexpr int TPS = kFragsPerStep / NSUB;   // taps per step
  static constexpr int SPC = (kTaps + TPS - 1) / TPS;  // steps per chunk
  static constexpr int WSLOT = kFragsPerStep * kFragBytes;
  static constexpr int LDS = 2 * BRICK + 2 * WSLOT;
  static constexpr int NM = MS * NSUB;               // MFMAs of a wavefront per tap
  static constexpr int NREAD = MS + NSUB;            // operand reads of a wavefront per tap
  static_assert(TD * TH * TW % 128 == 0 && NM <= 16, "accumulator blocks per wavefront");
  static_assert(SPC % 2 == 1, "the ring slot of a step alternates with the chunk");
  static_assert(LDS <= 160 * 1024, "LDS of a CU");
  static_assert(PLANE + (2 * BH * BW + 2 * BW + 2) * 16 < 65536, "ds_read immediate range");
  // brick loads of the next chunk issued per wavefront in the window of step u (none in the last step of a chunk)
  static constexpr int window_loads(int u) { return u >= SPC - 1 ? 0 : NLOAD / (SPC - 1) + (u < NLOAD % (SPC - 1) ? 1 : 0); }
  static constexpr int window_first(int u) {  // index of the window's first load in the wavefront's list
    int s = 0;
    for (int i = 0; i < u; ++i) s += window_loads(i);
    return s;
  }
  static_assert(NGROUP % 4 == 0, "every wavefront issues the same number of brick loads");
  static_assert(window_loads(0) <= TPS, "one brick load per tap");
};

constexpr int waitcnt_lgkm0() { return 15 | (3 << 14) | (7 << 4) | (0 << 8); }  // lgkmcnt == 0 and nothing else

template <typename C>
__device__ __forceinline__ constexpr int tap_off(int tap) {
  const int kd = tap / 9, kh = (tap / 3) % 3, kw = tap % 3;
  return ((kd * C::BH + kh) * C::BW + kw) * 16;
}

struct WideGeom {
  int tiles_d, tiles_h, tiles_w, nblocks;
  uint32_t total;
};

// What a lane knows for the whole launch.
template <typename T, typename C>
struct WideCtx {
  int lane, wave, nb, ncc32, c_end;
  int lbase[C::MS];  // LDS byte offset of the lane's activation fragment voxel at tap (0,0,0), per sub-tile
  int voff[C::GPW];  // staging: byte offset of the lane's voxel from the brick origin; kRange outside the input, -1 past the brick
  __amdgpu_buffer_rsrc_t xrsrc, wrsrc;
  // an input given as two tensors of equal channel counts: the second one's descriptor and its first 16-channel chunk
  __amdgpu_buffer_rsrc_t xrsrc1;
  int chunk1;
};

typedef __attribute__((address_space(3))) void* lds_ptr;
typedef __attribute__((address_space(3))) char* lds_bytes;
typedef const __attribute__((address_space(3))) uint4* lds_u4;

// byte offset in the packed weight of the fragment (block nb*NSUB + ns, 16-channel chunk, tap)
template <typename T, typename C>
__device__ __forceinline__ int frag_offset(const WideCtx<T, C>& k, int ns, int chunk, int tap) {
  return ((k.nb * C::NSUB + ns) * k.ncc32 + (chunk >> 1)) * kPairBytes + (tap * 2 + (chunk & 1)) * kFragBytes;
}
// I-th brick load of this wavefront for chunk `chunk` into the brick buffer `dst`: wavefront w fills the 64-voxel
// groups w, w + 4, ... of both planes
template <typename T, typename C, int I, bool PAIR>
__device__ __forceinline__ void brick_load(const WideCtx<T, C>& k, int chunk, lds_bytes dst) {
  constexpr int g = I >> 1, p = I & 1;
  constexpr bool full = (3 + 4 * g) * 64 + 63 < C::BV;  // only a wavefront's last group can have lanes past the brick
  // (the instruction's immediate offset would move the LDS destination as well: the plane's 16 bytes go into the scalar offset)
  if (full || k.voff[g] != -1) {
    if (PAIR && chunk >= k.chunk1)  // the chunk lies in the second tensor (same voxel offsets: equal channel counts)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(k.xrsrc1, (lds_ptr)(dst + p * C::PLANE + (k.wave + 4 * g) * 1024), 16, k.voff[g],
                                               (chunk - k.chunk1) * 32 + p * 16, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(k.xrsrc, (lds_ptr)(dst + p * C::PLANE + (k.wave + 4 * g) * 1024), 16, k.voff[g],
                                               chunk * 32 + p * 16, 0, 0);
  }
}
// this wavefront's three fragments of step `u` of chunk `chunk` into the ring slot `dst`
template <typename T, typename C>
__device__ __forceinline__ void weight_loads(const WideCtx<T, C>& k, int chunk, int u, lds_bytes dst) {
#pragma unroll
  for (int i = 0; i < kFragsPerStep / 4; ++i) {
    const int f = k.wave * (kFragsPerStep / 4) + i;
    const int tap = u * C::TPS + f / C::NSUB, ns = f % C::NSUB;
    if (tap < kTaps)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(k.wrsrc, (lds_ptr)(dst + f * kFragBytes), 16, k.lane * 16,
                                               __builtin_amdgcn_readfirstlane(frag_offset<T, C>(k, ns, chunk, tap)), 0, 0);
  }
}

// PAIR: the input is two tensors of a.cred / 2 channels each whose channels follow each other (x, then x1).
template <typename T, typename C, bool PAIR>
__global__ void __launch_bounds__(256, 1)
conv_wide_kernel(MfmaConvArgs a, const T* __restrict__ x, const T* __restrict__ wp, const T* __restrict__ bias, T* __restrict__ y,
                 WideGeom gm, GnPartialOut gn, const T* __restrict__ x1) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses LDS address-space builtins the host pass cannot type-check
  __shared__ __attribute__((aligned(16))) char brick0_[C::BRICK];
  __shared__ __attribute__((aligned(16))) char brick1_[C::BRICK];
  __shared__ __attribute__((aligned(16))) char wslot0_[C::WSLOT];
  __shared__ __attribute__((aligned(16))) char wslot1_[C::WSLOT];
  const lds_bytes brick0 = (lds_bytes)brick0_, brick1 = (lds_bytes)brick1_, wslot0 = (lds_bytes)wslot0_, wslot1 = (lds_bytes)wslot1_;
  const int tid = threadIdx.x;
  WideCtx<T, C> k;
  k.lane = tid & 63;
  k.wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: LDS destinations become scalar
  const int j = k.lane & 31, kg = k.lane >> 5;

  uint32_t t = xcd_remap(blockIdx.x, gm.total);
  const int nb = t % gm.nblocks; t /= gm.nblocks;
  const int tw_i = t % gm.tiles_w; t /= gm.tiles_w;
  const int th_i = t % gm.tiles_h; t /= gm.tiles_h;
  const int td_i = t % gm.tiles_d;
  const int n = t / gm.tiles_d;
  const int od0 = td_i * C::TD, oh0 = th_i * C::TH, ow0 = tw_i * C::TW;
  const int id0 = od0 - a.pd, ih0 = oh0 - a.ph, iw0 = ow0 - a.pw;

  const int c_begin = 0;
  k.c_end = a.cred / 16;
  k.nb = nb;
  k.ncc32 = a.cred / 32;
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) {
    const int v = (k.wave * C::MS + ms) * 32 + j;
    const int tw = v % C::TW, th = (v / C::TW) % C::TH, td = v / (C::TW * C::TH);
    k.lbase[ms] = kg * C::PLANE + ((td * C::BH + th) * C::BW + tw) * 16;
  }
  // Staging role of the lane: byte offset of its voxel of group wave + 4g from the (possibly virtual) brick origin,
  // kRange when the voxel lies outside the input (such loads return zeros), -1 past the brick.
  const int row = PAIR ? a.cred / 2 : a.cred;  // channels per voxel of the tensor(s) read
#pragma unroll
  for (int g = 0; g < C::GPW; ++g) {
    const int vox = (k.wave + 4 * g) * 64 + k.lane;
    const int bw = vox % C::BW, bh = (vox / C::BW) % C::BH, bd = vox / (C::BW * C::BH);
    const bool inside = (unsigned)(id0 + bd) < (unsigned)a.id && (unsigned)(ih0 + bh) < (unsigned)a.ih && (unsigned)(iw0 + bw) < (unsigned)a.iw;
    k.voff[g] = vox >= C::BV ? -1 : (inside ? (((bd * a.ih + bh) * a.iw + bw) * row) * 2 : kRange);
  }
  const int64_t origin = ((((int64_t)n * a.id + id0) * a.ih + ih0) * a.iw + iw0) * row;
  k.xrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(x + origin), 0, kRange, 0x00020000);
  k.xrsrc1 = k.xrsrc;
  k.chunk1 = 0;
  if constexpr (PAIR) {
    k.xrsrc1 = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(x1 + origin), 0, kRange, 0x00020000);
    k.chunk1 = row / 16;
  }
  k.wrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(wp), 0, 0x7fffffff, 0x00020000);

  f32x16_t acc[C::MS][C::NSUB];
  {
    // ---- prologue: the first chunk's brick, the first step's weights -------------------------------------------
    static_for<C::NLOAD>([&](auto i_c) { brick_load<T, C, decltype(i_c)::value, PAIR>(k, c_begin, brick0); });
    weight_loads<T, C>(k, c_begin, 0, wslot0);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
    __syncthreads();
    weight_loads<T, C>(k, c_begin, 1, wslot1);  // the second step's (the ring has two slots)
#pragma unroll
    for (int ms = 0; ms < C::MS; ++ms)
#pragma unroll
      for (int ns = 0; ns < C::NSUB; ++ns) zero_pinned(acc[ms][ns]);
    frag_t a_cur[C::MS], b_cur[C::NSUB];
#pragma unroll
    for (int ms = 0; ms < C::MS; ++ms) a_cur[ms] = lds_read_frag<tap_off<C>(0)>((int)(uintptr_t)brick0 + k.lbase[ms]);
    static_for<C::NSUB>([&](auto ns_c) {
      constexpr int ns = decltype(ns_c)::value;
      b_cur[ns] = lds_read_frag<ns * kFragBytes>((int)(uintptr_t)wslot0 + k.lane * 16);
    });
    // One 16-channel chunk: 27 taps x MS x NSUB MFMAs out of the brick `cur`, while the next chunk's brick streams
    // into `nxt`. `w_even` / `w_odd` are the ring slots of the chunk's even / odd steps (they trade places from chunk
    // to chunk because a chunk has an odd number of steps).
    auto wide_chunk = [&](int c, lds_bytes cur, lds_bytes nxt, lds_bytes w_even, lds_bytes w_odd) {
      const bool more = c + 1 < k.c_end;
      int acur[C::MS], anxt[C::MS];
#pragma unroll
      for (int ms = 0; ms < C::MS; ++ms) {
        acur[ms] = (int)(uintptr_t)cur + k.lbase[ms];
        anxt[ms] = (int)(uintptr_t)nxt + k.lbase[ms];
      }
      const int wl_even = (int)(uintptr_t)w_even + k.lane * 16, wl_odd = (int)(uintptr_t)w_odd + k.lane * 16;
      static_for<kTaps>([&](auto tap_c) {
        constexpr int tap = decltype(tap_c)::value;
        constexpr int u = tap / C::TPS;
        constexpr bool last_of_step = (tap % C::TPS == C::TPS - 1) || tap == kTaps - 1;
        constexpr bool last_of_chunk = tap == kTaps - 1;
        if constexpr (last_of_step) {
          // Behind the barrier: the next step's weights (fetched during this step by all four wavefronts) are
          // visible, this step's ring slot and -- at the end of a chunk -- this chunk's brick buffer are free, and
          // the next chunk's brick has landed. Loads that may stay in flight: the brick loads issued in this step's
          // window (they follow the weight loads this barrier is about; none without a next chunk).
          if (more) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(C::window_loads(u)));
          else __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
          __builtin_amdgcn_s_barrier();
          // weights of the step after next into the slot this step used
          constexpr int u2 = (u + 2) % C::SPC;
          const int c2 = c + (u + 2) / C::SPC;
          if (c2 < k.c_end) weight_loads<T, C>(k, c2, u2, (u & 1) ? w_odd : w_even);
        } else {
          __builtin_amdgcn_s_waitcnt(waitcnt_lgkm0());  // this tap's fragments (requested during the previous tap) have landed
        }
#pragma unroll
        for (int ms = 0; ms < C::MS; ++ms) landed(a_cur[ms]);
#pragma unroll
        for (int ns = 0; ns < C::NSUB; ++ns) landed(b_cur[ns]);
        // brick loads of the next chunk: window u starts at the first tap of step u, one load per tap
        if constexpr ((tap - u * C::TPS) < C::window_loads(u)) {
          if (more) brick_load<T, C, C::window_first(u) + tap - u * C::TPS, PAIR>(k, c + 1, nxt);
        }
        // This tap's MFMAs with the operand reads of the next tap spread between them.
        frag_t a_nxt[C::MS], b_nxt[C::NSUB];
        static_for<C::NM>([&](auto i_c) {
          constexpr int i = decltype(i_c)::value;
          constexpr int ms = i / C::NSUB, ns = i % C::NSUB;
          Mma32Pinned<T>::run(b_cur[ns], a_cur[ms], acc[ms][ns]);
          // reads [i * NREAD / NM, (i + 1) * NREAD / NM) of the next tap: the weight fragments first, then the activations
          static_for<(i + 1) * C::NREAD / C::NM - i * C::NREAD / C::NM>([&](auto q_c) {
            constexpr int r = i * C::NREAD / C::NM + decltype(q_c)::value;
            if constexpr (r < C::NSUB) {
              if constexpr (!last_of_chunk) {
                constexpr int u1 = (tap + 1) / C::TPS, i1 = (tap + 1) % C::TPS;
                b_nxt[r] = lds_read_frag<(i1 * C::NSUB + r) * kFragBytes>((u1 & 1) ? wl_odd : wl_even);
              } else {
                b_nxt[r] = lds_read_frag<r * kFragBytes>(wl_odd);  // first tap of the next chunk (unused after the last)
              }
            } else {
              constexpr int m = r - C::NSUB;
              if constexpr (!last_of_chunk) a_nxt[m] = lds_read_frag<tap_off<C>(tap + 1)>(acur[m]);
              else a_nxt[m] = lds_read_frag<tap_off<C>(0)>(anxt[m]);
            }
          });
        });
#pragma unroll
        for (int ms = 0; ms < C::MS; ++ms) a_cur[ms] = a_nxt[ms];
#pragma unroll
        for (int ns = 0; ns < C::NSUB; ++ns) b_cur[ns] = b_nxt[ns];
      });
      __builtin_amdgcn_s_waitcnt(waitcnt_lgkm0());  // nothing in flight into registers when the chunk ends
    };
    for (int c = c_begin; c < k.c_end; c += 2) {
      wide_chunk(c, brick0, brick1, wslot0, wslot1);
      if (c + 1 < k.c_end) wide_chunk(c + 1, brick1, brick0, wslot1, wslot0);
    }
    asm volatile("s_nop 15\n\ts_nop 15");  // the last MFMAs are inline asm: the compiler does not know their result latency
  }

  // ---- epilogue. Accumulator register r of a lane is output channel 8*(r/4) + 4*kg + r%4 of the sub-tile's voxel j ----
  // The lane's position is derived again from a thread id the compiler cannot equate with the first one: otherwise the
  // output addresses are computed before the main loop (they share the sub-tile arithmetic of its set-up) and
  // occupy a hundred registers across it.
  int tid_out = tid;
  asm volatile("" : "+v"(tid_out));
  const int wave_out = tid_out >> 6, j_out = tid_out & 31, kg_out = (tid_out >> 5) & 1;
  RunSums gn_sums[C::NSUB];  // GroupNorm statistics of the rounded output, when the caller wants them
#pragma unroll
  for (int ns = 0; ns < C::NSUB; ++ns) {
    gn_sums[ns].clear();
  }
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) {
    const int v = (wave_out * C::MS + ms) * 32 + j_out;
    const int tw = v % C::TW, th = (v / C::TW) % C::TH, td = v / (C::TW * C::TH);
    const int od = od0 + td, oh = oh0 + th, ow = ow0 + tw;
    const bool inside = od < a.od && oh < a.oh && ow < a.ow;
    const int64_t vox = (((int64_t)n * a.od + od) * a.oh + oh) * a.ow + ow;
    T* yp = y + vox * a.cout + nb * C::NSUB * 32;
#pragma unroll
    for (int ns = 0; ns < C::NSUB; ++ns) {
      store_block<T>(acc[ms][ns], yp + ns * 32, bias, (nb * C::NSUB + ns) * 32, kg_out, inside, gn_sums[ns], gn.part != nullptr, ms == 0);
      // one block at a time: left to itself the scheduler reads many accumulator blocks out ahead of their stores and
      // runs out of vector registers (all 256 accumulation registers are taken by the 8 x 2 grid)
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if (gn.part != nullptr) {
    __syncthreads();  // every wave is done with the bricks: the LDS is free
    constexpr int SPAN = 32 * C::NSUB;
    const int per_tile = gn.cg > SPAN ? gn.cg / SPAN : 1;  // workgroups that share a group of this tile
    const int tile = (td_i * gm.tiles_h + th_i) * gm.tiles_w + tw_i;
    write_group_partials<4, C::NSUB>(gn_sums, reinterpret_cast<float*>(brick0_), gn, n, tile * per_tile + nb % per_tile, nb * SPAN,
                                     tid_out);
  }
#endif
}

struct WidePlan {
  bool use;
  int shape;   // 0: 4x4x32 tile with 4 channel blocks, 1: 8x4x32 with 2, 2: 8x4x32 with 1, 3: 4x4x32 with 2, 4: 4x4x32 with 1
};

int64_t wide_tiles(const MfmaConvArgs& a, int td) { return (int64_t)a.n * cdiv(a.od, td) * cdiv(a.oh, 4) * cdiv(a.ow, 32); }

// workgroups of accumulator grid `shape` before any split of the reduction
int64_t wide_workgroups(const MfmaConvArgs& a, int shape) {
  static const int td[5] = {4, 8, 8, 4, 4}, nsub[5] = {4, 2, 1, 2, 1};
  return wide_tiles(a, td[shape]) * (a.cout / (32 * nsub[shape]));
}

// Launch geometry, a pure function of the problem. Rows of more than 16 voxels only (32-voxel sub-tiles are one row).
WidePlan wide_plan(const MfmaConvArgs& a) {
  WidePlan p{false, 0};
  if (a.kd != 3 || a.kh != 3 || a.kw != 3 || a.cred < 64 || a.cred % 32 != 0 || a.cout % 32 != 0 || a.ow <= 16) return p;
  // a brick (at most 10 input planes and 6 rows) must span less than kRange bytes of the input
  if (((int64_t)10 * a.ih + 6) * a.iw * a.cred * 2 + 64 >= kRange) return p;
  int shape = -1;
  // Measured against the brick-per-workgroup kernel on every shape of the U-Net and of the cube configurations, this
  // kernel wins where a 64-channel output meets 128 or more reduction channels (one workgroup then produces all of a
  // voxel's channels from one staged brick): 8 x 2 accumulator blocks per wavefront when such workgroups fill the
  // chip, else 4 x 2. Everything else stays with the other kernels.
  if (a.cout == 64 && a.cred >= 128) {
    if (wide_workgroups(a, 1) >= kComputeUnits) shape = 1;
    else if (wide_workgroups(a, 3) >= kComputeUnits) shape = 3;
  }
  if (shape < 0) return p;
  p.use = true;
  p.shape = shape;
  return p;
}

template <typename T, typename C>
int launch_wide(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                const GnPartialOut& gn, const void* x1) {
  WideGeom gm{};
  gm.tiles_d = (int)cdiv(a.od, C::TD);
  gm.tiles_h = (int)cdiv(a.oh, C::TH);
  gm.tiles_w = (int)cdiv(a.ow, C::TW);
  gm.nblocks = a.cout / (32 * C::NSUB);
  const int64_t total = (int64_t)a.n * gm.tiles_d * gm.tiles_h * gm.tiles_w * gm.nblocks;
  if (total == 0) return SFH_OK;
  if (total > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "conv wide: %lld workgroups exceed the grid limit", (long long)total);
  gm.total = (uint32_t)total;
  if (x1 != nullptr)
    hipLaunchKernelGGL((conv_wide_kernel<T, C, true>), dim3((unsigned)total), dim3(256), 0, st, a, (const T*)x, (const T*)packed,
                       (const T*)bias, (T*)y, gm, gn, (const T*)x1);
  else
    hipLaunchKernelGGL((conv_wide_kernel<T, C, false>), dim3((unsigned)total), dim3(256), 0, st, a, (const T*)x, (const T*)packed,
                       (const T*)bias, (T*)y, gm, gn, (const T*)nullptr);
  return check_launch("conv_wide_kernel");
}

template <typename T>
int launch_typed(const MfmaConvArgs& a, const WidePlan& p, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                 const GnPartialOut& gn, const void* x1) {
  switch (p.shape) {
    case 1: return launch_wide<T, WTile<8, 4, 32, 2>>(a, x, packed, bias, y, st, gn, x1);
    case 3: return launch_wide<T, WTile<4, 4, 32, 2>>(a, x, packed, bias, y, st, gn, x1);
    default: return fail(SFH_ERR_UNSUPPORTED, "conv wide: no kernel for accumulator grid %d", p.shape);
  }
}

}  // namespace

bool mfma_conv_wide_applies(const MfmaConvArgs& a) { return wide_plan(a).use; }

MfmaConvGeometry mfma_conv_wide_geometry(const MfmaConvArgs& a) {
  static const int td[5] = {4, 8, 8, 4, 4}, nsub[5] = {4, 2, 1, 2, 1};
  const WidePlan p = wide_plan(a);
  return MfmaConvGeometry{kKernelWide, td[p.shape] * 4 * 32, nsub[p.shape], 1};
}

int mfma_conv_wide_gn_records(const MfmaConvArgs& a, int groups) {
  const WidePlan p = wide_plan(a);
  if (!p.use) return 0;
  const MfmaConvGeometry g = mfma_conv_wide_geometry(a);
  const int span = 32 * g.blocks;
  if (!gn_partials_fit(a.cout, groups, span)) return 0;
  const int cg = a.cout / groups;
  const int64_t tiles = (int64_t)cdiv(a.od, g.voxels / 128) * cdiv(a.oh, 4) * cdiv(a.ow, 32);
  const int64_t records = tiles * (cg > span ? cg / span : 1);
  return records <= 0x7fffffff ? (int)records : 0;
}

// The staging offsets of a lane are those of one tensor: a pair must be two tensors of the same channel count.
bool mfma_conv_wide_pair_ok(const MfmaConvArgs& a, int first) { return wide_plan(a).use && first * 2 == a.cred && first % 16 == 0; }

int mfma_conv_wide(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                   const GnPartialOut* gn, const ChannelPair* in2) {
  const WidePlan p = wide_plan(a);
  if (!p.use) return fail(SFH_ERR_UNSUPPORTED, "conv wide: not applicable to this problem");
  if (in2 != nullptr && (in2->second == nullptr || !mfma_conv_wide_pair_ok(a, in2->first)))
    return fail(SFH_ERR_UNSUPPORTED, "conv wide: the input cannot be cut at channel %d of %d", in2->first, a.cred);
  const void* x1 = in2 != nullptr ? in2->second : nullptr;
  GnPartialOut out{nullptr, 0, 0, 0};
  if (gn != nullptr && gn->part != nullptr) {
    if (gn->records == 0 || gn->records != mfma_conv_wide_gn_records(a, gn->groups))
      return fail(SFH_ERR_INVALID, "conv wide: GroupNorm partials asked for %d records, this launch leaves %d", gn->records,
                  mfma_conv_wide_gn_records(a, gn->groups));
    out = *gn;
    out.cg = a.cout / gn->groups;
  }
  if (dtype == SFH_BF16) return launch_typed<bf16_t>(a, p, x, packed, bias, y, st, out, x1);
  return launch_typed<fp16_t>(a, p, x, packed, bias, y, st, out, x1);
}

}  // namespace sfh
