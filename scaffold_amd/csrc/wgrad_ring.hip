// MFMA weight gradient of a 3x3x3 stride-1 convolution for gfx950 (bf16 / fp16, rows of more than 16 voxels) that
// stages both operands in LDS exactly as they lie in memory and lets the LDS do the transposition.
//
//   gw[co][kd][kh][kw][ci] = sum over output voxels v of gy[v][co] * x[v + tap - pad][ci]
//
// GEMM view (triton_conv3d/reduce_gemm.py:137-393): M = Cout, N = 27 x Cin, K = output voxels, split over workgroups
// along K, fp32 partial slices at fixed workspace slots and an ordered reduction (reduce_gemm.py:396-435) -- no float
// atomics, split count a pure function of shape.
//
// Both MFMA operands need the contraction index (voxels) along a lane's register while memory is channel-contiguous.
// gfx950's ds_read_b64_tr_b16 does that transposition on the way out of LDS (within 16 lanes: lane m gives the address
// of 4 channels of voxel m / 4 and receives channel m of the four voxels), so nothing is transposed by hand:
//   * a workgroup (four wavefronts, one per SIMD) walks a column 4 rows high and 32 voxels wide along depth, two
//     planes per step, as the persistent forward kernel does (conv_ring.hip): LDS holds a ring of three input plane
//     PAIRS (2 x 6 x 34 voxels with the halo) and three gy tiles (2 x 4 x 32 voxels); while the MFMAs of a step read two
//     pairs and one tile, the next step's new pair and tile stream in straight from memory (buffer_load ... lds);
//   * every voxel is stored as four 16-byte channel pieces in four piece planes (the forward kernel's layout), which
//     makes the transposing reads bank-conflict free at any voxel offset: a tap's shift along W is an address offset,
//     not a funnel shift;
//   * wavefront (s, g) owns the half-rows s (16 voxels = one MFMA k-step) and the tap group g (14 / 13 of the 27 taps):
//     224 accumulation registers. Its gy fragments of the step (8) stay in registers; it walks the input rows of the
//     step once, and an input-row fragment (plane D, row H, shift kw) feeds up to six MFMAs -- the taps (kd, kh) under
//     which that row is seen from the step's output rows: 0.8 LDS reads per MFMA, no vector-ALU work between them;
//   * at the end the two wavefronts that hold the same taps add their accumulators through LDS in a fixed order and
//     the workgroup writes one fp32 slice.
#include <utility>

#include "mma.hpp"
#include "reduce.hpp"
#include "wgrad_mfma.hpp"

namespace sfh {
namespace {

constexpr int kTD = 2, kTH = 4, kTW = 32;             // output voxels of a step
constexpr int kBH = kTH + 2, kBW = kTW + 2;           // rows / voxels per row of an input plane with its halo
constexpr int kXVoxels = 2 * kBH * kBW;               // voxels of an input plane pair (408)
constexpr int kGVoxels = kTD * kTH * kTW;             // voxels of a gy tile (256)
constexpr int wring_piece_bytes(int voxels) { return ((voxels * 16 - 64 + 255) / 256) * 256 + 64; }  // 64 modulo 256
constexpr int kXPiece = wring_piece_bytes(kXVoxels), kXPair = 4 * kXPiece;
constexpr int kGPiece = wring_piece_bytes(kGVoxels), kGTile = 4 * kGPiece;
constexpr int kXGroups = (kXVoxels + 63) / 64;        // 64-voxel groups a pair is fetched in (7, the last one partial)
constexpr int kXGroupsPerWave = (kXGroups + 3) / 4;   // 2
constexpr int kLoads = (kXGroupsPerWave + 1) * 4;     // load instructions per wavefront and step (x groups + one gy group)
constexpr int kRange = 0x40000000;                    // buffer range: offsets at or above it read as zero
constexpr int kTaps0 = 14, kTaps1 = 13;               // taps of the two groups
static_assert(3 * kXPair + 3 * kGTile <= 160 * 1024, "three plane pairs and three gy tiles in the LDS of a CU");
static_assert(kGVoxels == 4 * 64, "one gy group per wavefront");
constexpr int kHandTaps = kXPair / 4096, kHandRounds = (kTaps0 + kHandTaps - 1) / kHandTaps;  // accumulators (4 KiB per tap) handed over per round
constexpr int kWaitLgkm0 = 0xC07F;  // s_waitcnt immediate (gfx9): lgkmcnt(0), vmcnt and expcnt untouched

// Tap (kd, kh, kw) -> group and accumulator. Group 0: kw = 0, and kw = 1 for the first five (kd, kh); group 1: kw = 2, and
// kw = 1 for the other four.
constexpr int tap_group(int t9, int kw) { return kw == 0 ? 0 : (kw == 2 ? 1 : (t9 < 5 ? 0 : 1)); }
constexpr int tap_slot(int t9, int kw) { return kw == 0 ? t9 : (kw == 2 ? t9 : (t9 < 5 ? 9 + t9 : 9 + t9 - 5)); }

// ---- the compile-time schedule of a step, per tap group ---------------------------------------------------------------------
// The input rows of the step are visited in the order (H = 0..5, D = 0..3, kw); fragment X(D, H, kw) is requested if the
// group has a tap that sees it, and then feeds the MFMAs acc[(kd, kh, kw)] += gy(d, h) x X for all (d, kd = D - d),
// (h, kh = H - h) of the group.
struct WSchedule {
  static constexpr int kMaxMfmas = 8 * kTaps0, kMaxFrags = 72, kLead = 4, kBuffers = 4;
  int nm, nf;
  int mf_frag[kMaxMfmas], mf_acc[kMaxMfmas], mf_gy[kMaxMfmas];
  int fr_d[kMaxFrags], fr_h[kMaxFrags], fr_kw[kMaxFrags], fr_first[kMaxFrags], fr_last[kMaxFrags];
  int issue_after[kMaxFrags], buffer[kMaxFrags], request_at[kMaxMfmas];
  int gy_first[kTD * kTH], gy_issue[kTD * kTH], gy_request_at[kMaxMfmas];  // the same for the gy fragment of output row r
  int buffers_used, min_acc_distance;
  bool early_in_lo;  // every fragment requested before the step's first MFMA lies in the step's first plane pair
};

constexpr WSchedule make_wschedule(int g) {
  WSchedule s{};
  for (int h = 0; h < kBH; ++h)
    for (int d = 0; d < 4; ++d)
      for (int kw = 0; kw < 3; ++kw) {
        int first = -1;
        for (int dd = 0; dd < kTD; ++dd)
          for (int hh = 0; hh < kTH; ++hh) {
            const int kd = d - dd, kh = h - hh;
            if (kd < 0 || kd > 2 || kh < 0 || kh > 2 || tap_group(kd * 3 + kh, kw) != g) continue;
            if (first < 0) {
              first = s.nm;
              s.fr_d[s.nf] = d; s.fr_h[s.nf] = h; s.fr_kw[s.nf] = kw; s.fr_first[s.nf] = s.nm;
            }
            s.mf_frag[s.nm] = s.nf;
            s.mf_acc[s.nm] = tap_slot(kd * 3 + kh, kw);
            s.mf_gy[s.nm] = dd * kTH + hh;
            s.fr_last[s.nf] = s.nm;
            ++s.nm;
          }
        if (first >= 0) ++s.nf;
      }
  int next = s.nm;
  for (int f = s.nf - 1; f >= 0; --f) {
    int at = s.fr_first[f] - WSchedule::kLead;
    if (at >= next) at = next - 1;
    s.issue_after[f] = at;
    next = at;
  }
  // what is requested ahead of the step's first MFMA must lie in its first plane pair (the second may still be on its
  // way when the requests go out): such fragments of the second pair move behind the first MFMAs instead
  int taken = -1;
  for (int f = 0; f < s.nf; ++f) {
    if (s.issue_after[f] < 0 && s.fr_d[f] < 2) continue;
    if (s.issue_after[f] <= taken) s.issue_after[f] = taken + 1;
    taken = s.issue_after[f];
  }
  for (int k = 0; k < WSchedule::kMaxMfmas; ++k) s.request_at[k] = -1;
  for (int f = 0; f < s.nf; ++f)
    if (s.issue_after[f] >= 0) s.request_at[s.issue_after[f]] = f;
  int busy_until[WSchedule::kMaxFrags] = {};
  int nb = 0;
  for (int f = 0; f < s.nf; ++f) {
    int pick = -1;
    for (int b = 0; b < nb && pick < 0; ++b)
      if (busy_until[b] <= s.issue_after[f]) pick = b;
    if (pick < 0) pick = nb++;
    busy_until[pick] = s.fr_last[f];
    s.buffer[f] = pick;
  }
  s.buffers_used = nb;
  // gy fragments: requested a little before their first use as well (in order of first use, never two behind one MFMA)
  for (int r = 0; r < kTD * kTH; ++r) s.gy_first[r] = -1;
  for (int i = 0; i < s.nm; ++i)
    if (s.gy_first[s.mf_gy[i]] < 0) s.gy_first[s.mf_gy[i]] = i;
  for (int k = 0; k < WSchedule::kMaxMfmas; ++k) s.gy_request_at[k] = -1;
  int gnext = s.nm;
  for (int pass = 0; pass < kTD * kTH; ++pass) {
    int r = -1;  // the row with the latest first use among those not placed yet
    for (int q = 0; q < kTD * kTH; ++q)
      if (s.gy_issue[q] == 0 && s.gy_first[q] >= 0 && (r < 0 || s.gy_first[q] > s.gy_first[r])) r = q;
    if (r < 0) break;
    int at = s.gy_first[r] - WSchedule::kLead - 1;
    if (at >= gnext) at = gnext - 1;
    if (at == 0) at = -1;  // 0 marks "not placed" above
    s.gy_issue[r] = at;
    gnext = at;
    if (at > 0) s.gy_request_at[at] = r;
  }
  s.early_in_lo = true;
  for (int f = 0; f < s.nf; ++f)
    if (s.issue_after[f] < 0 && s.fr_d[f] >= 2) s.early_in_lo = false;
  s.min_acc_distance = s.nm;
  for (int i = 0; i < s.nm; ++i)
    for (int k = i + 1; k < s.nm && k < i + 8; ++k)
      if (s.mf_acc[i] == s.mf_acc[k] && k - i < s.min_acc_distance) s.min_acc_distance = k - i;
  return s;
}

constexpr WSchedule kWSched0 = make_wschedule(0), kWSched1 = make_wschedule(1);
static_assert(kWSched0.nm == 8 * kTaps0 && kWSched1.nm == 8 * kTaps1, "every (row, tap) of the group exactly once");
static_assert(kWSched0.buffers_used <= WSchedule::kBuffers && kWSched1.buffers_used <= WSchedule::kBuffers, "fragment registers");
static_assert(kWSched0.min_acc_distance >= 2 && kWSched1.min_acc_distance >= 2, "no two MFMAs in a row on one accumulator");
static_assert(kWSched0.early_in_lo && kWSched1.early_in_lo, "the fragments requested ahead of a step lie in the pair that is already resident");
constexpr bool wschedule_requests_in_time(const WSchedule& s) {
  for (int f = 0; f < s.nf; ++f)
    if (s.issue_after[f] >= s.fr_first[f] - 1) return false;
  return true;
}
static_assert(wschedule_requests_in_time(kWSched0) && wschedule_requests_in_time(kWSched1), "every fragment is requested ahead of its first use");

// A load rides behind every sixth MFMA from the step's start. (Measured: where in the step the loads sit, and whether
// the wavefronts issue theirs at the same or at staggered MFMAs, changes the step time by less than 2 %.)
constexpr int kSidePeriod = 6, kSidePhase = 1;
static_assert((8 * kTaps1 - kSidePhase + kSidePeriod - 1) / kSidePeriod >= kLoads, "a slot per load");

constexpr int wring_waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

struct WRingGeom {
  int tiles_h, tiles_w, steps, segs, seg_steps;
  int nblk_ci, nblk;                       // 32 x 32 blocks of (co, ci)
  int items, splits, items_per_split;      // items = columns x segments; a workgroup (split) takes consecutive ones
};

struct WRingLane {
  int xrel[kXGroupsPerWave], xcoord[kXGroupsPerWave];  // staging of x: byte offset from the pair's first voxel; dl | bh << 8 | bw << 16 or -1
  int grel, gcoord;                                    // staging of gy: byte offset from the tile's first voxel; d | h << 8 | w << 16
  int xread, gread;                                    // transposing reads: per-lane byte offset inside a pair / a tile
};

struct WRingColumn { int n, h0, w0; };

__device__ __forceinline__ WRingColumn wring_column(int col, int tiles_h, int tiles_w) {
  WRingColumn c;
  c.w0 = (col % tiles_w) * kTW; col /= tiles_w;
  c.h0 = (col % tiles_h) * kTH;
  c.n = col / tiles_h;
  return c;
}

// Buffer offsets of the lane's voxels of the input pair whose first plane is `plane`, and of the gy tile whose first
// plane is `d0`: out-of-range (zeros) for whatever lies outside the tensors; `live` false does that to all of it.
__device__ __forceinline__ void wring_offsets(const WgradArgs& a, const WRingColumn& c, const WRingLane& ln, int plane, int d0, bool live,
                                              int (&xoff)[kXGroupsPerWave], int& goff) {
  const int ih0 = c.h0 - a.ph, iw0 = c.w0 - a.pw;
#pragma unroll
  for (int k = 0; k < kXGroupsPerWave; ++k) {
    const int dl = ln.xcoord[k] & 0xff, bh = (ln.xcoord[k] >> 8) & 0xff, bw = (ln.xcoord[k] >> 16) & 0xff;
    const int inside = (int)((unsigned)(plane + dl) < (unsigned)a.id) & (int)((unsigned)(ih0 + bh) < (unsigned)a.ih) &
                       (int)((unsigned)(iw0 + bw) < (unsigned)a.iw) & (int)live;
    xoff[k] = ln.xcoord[k] < 0 ? -1 : (inside ? ln.xrel[k] : kRange);
  }
  const int d = ln.gcoord & 0xff, h = (ln.gcoord >> 8) & 0xff, w = (ln.gcoord >> 16) & 0xff;
  const int inside = (int)(d0 + d < a.od) & (int)(c.h0 + h < a.oh) & (int)(c.w0 + w < a.ow) & (int)live;
  goff = inside ? ln.grel : kRange;
}

template <typename T>
__device__ __forceinline__ void wring_fetch(char* xdst, char* gdst, int wave, const T* xorigin, const T* gorigin,
                                            const int (&xoff)[kXGroupsPerWave], int goff) {
  const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(xorigin), 0, kRange, 0x00020000);
#pragma unroll
  for (int k = 0; k < kXGroupsPerWave; ++k)
    if (xoff[k] != -1) {
#pragma unroll
      for (int p = 0; p < 4; ++p)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (__attribute__((address_space(3))) void*)(xdst + (wave + 4 * k) * 1024 + p * kXPiece), 16,
                                                 xoff[k] + p * 16, 0, 0, 0);
    }
  if (gdst != nullptr) {
    const __amdgpu_buffer_rsrc_t gr = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(gorigin), 0, kRange, 0x00020000);
#pragma unroll
    for (int p = 0; p < 4; ++p)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(gr, (__attribute__((address_space(3))) void*)(gdst + wave * 1024 + p * kGPiece), 16, goff + p * 16,
                                               0, 0, 0);
  }
}

typedef short wring_v4s __attribute__((__vector_size__(4 * sizeof(short))));

// A 32-channel x 16-voxel operand fragment from the piece planes at `p` (the lane's address of its first four voxels).
__device__ __forceinline__ uint4 wring_fragment(const char* p) {
  const wring_v4s r0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) wring_v4s*)(p));
  const wring_v4s r1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) wring_v4s*)(p + 64));
  uint4 out;
  out.x = __builtin_bit_cast(uint2, r0).x; out.y = __builtin_bit_cast(uint2, r0).y;
  out.z = __builtin_bit_cast(uint2, r1).x; out.w = __builtin_bit_cast(uint2, r1).y;
  return out;
}

// One step of wavefront (s, G): the MFMAs of tap group G over the pairs `lo` (planes 0, 1) and `hi` (planes 2, 3) and the
// gy tile `gt`, with the loads of the next step's pair and of the gy tile after next riding along. The fragments a step
// needs for its first MFMAs are requested by early() BEFORE the barrier that ends the step in front of it (they lie in
// the pair and the tile that are already resident), so the LDS latency hides behind that barrier.
template <int G>
struct WRingFrags {
  static constexpr const WSchedule& S = G == 0 ? kWSched0 : kWSched1;
  const char* xlo;
  const char* xhi;
  const char* gt;
  uint4 (&gyf)[kTD * kTH];
  uint4 (&fr)[WSchedule::kBuffers];

  template <int F>
  __device__ __forceinline__ void request() {
    constexpr int d = S.fr_d[F], h = S.fr_h[F], kw = S.fr_kw[F];
    constexpr int off = (((d % 2) * kBH + h) * kBW + kw) * 16;
    fr[S.buffer[F]] = wring_fragment((d < 2 ? xlo : xhi) + off);
  }
  template <int R>
  __device__ __forceinline__ void request_gy() { gyf[R] = wring_fragment(gt + R * kTW * 16); }
  template <int F>
  __device__ __forceinline__ void request_if_early() {
    if constexpr (F < S.nf) {
      if constexpr (S.issue_after[F] < 0) request<F>();
    }
  }
  template <int R>
  __device__ __forceinline__ void request_gy_if_early() {
    if constexpr (S.gy_issue[R] < 0) request_gy<R>();
  }
  // Only xlo and gt are read.
  template <int... Fs, int... Rs>
  __device__ __forceinline__ void early(std::integer_sequence<int, Fs...>, std::integer_sequence<int, Rs...>) {
    (request_gy_if_early<Rs>(), ...);
    (request_if_early<Fs>(), ...);
  }
};

template <typename T, int G>
struct WRingStep {
  static constexpr const WSchedule& S = G == 0 ? kWSched0 : kWSched1;
  static constexpr int NACC = G == 0 ? kTaps0 : kTaps1;
  WRingFrags<G> fg;
  char* xfill;
  char* gfill;
  int wave;
  f32x16_t (&acc)[NACC];
  const int (&xoff)[kXGroupsPerWave];
  int goff;
  __amdgpu_buffer_rsrc_t xrsrc, grsrc;

  template <int M>
  __device__ __forceinline__ void mfma() {
    if constexpr (M < S.nm) {
      constexpr int f = S.mf_frag[M], ac = S.mf_acc[M], r = S.mf_gy[M];
      __builtin_amdgcn_sched_barrier(0);
      acc[ac] = Mma32<T>::run(fg.gyf[r], fg.fr[S.buffer[f]], acc[ac]);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (S.request_at[M] >= 0) {
        fg.template request<S.request_at[M]>();
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (S.gy_request_at[M] >= 0) {
        fg.template request_gy<S.gy_request_at[M]>();
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (M % kSidePeriod == kSidePhase && M / kSidePeriod < kLoads) {
        constexpr int slot = M / kSidePeriod;
        if constexpr (slot < kXGroupsPerWave * 4) {
          constexpr int k = slot / 4, p = slot % 4;
          if (xoff[k] != -1)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(xrsrc, (__attribute__((address_space(3))) void*)(xfill + (wave + 4 * k) * 1024 + p * kXPiece),
                                                     16, xoff[k] + p * 16, 0, 0, 0);
        } else {
          constexpr int p = slot - kXGroupsPerWave * 4;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(grsrc, (__attribute__((address_space(3))) void*)(gfill + wave * 1024 + p * kGPiece), 16,
                                                   goff + p * 16, 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  template <int... Ms>
  __device__ __forceinline__ void run(std::integer_sequence<int, Ms...>) {
    (mfma<Ms>(), ...);
  }
};

// The per-lane constants of a problem: where the lane's voxels of a staged pair / tile lie in memory and in LDS.
__device__ __forceinline__ WRingLane wring_lane(const WgradArgs& a, int x_cin, int tid) {
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int seg16 = wave & 1;  // which 16 voxels of every row this wavefront contracts over
  WRingLane ln;
#pragma unroll
  for (int k = 0; k < kXGroupsPerWave; ++k) {
    const int vox = (wave + 4 * k) * 64 + lane;
    const int dl = vox / (kBH * kBW), r = vox % (kBH * kBW), bh = r / kBW, bw = r % kBW;
    ln.xcoord[k] = vox < kXVoxels ? (dl | (bh << 8) | (bw << 16)) : -1;
    ln.xrel[k] = ((dl * a.ih + bh) * a.iw + bw) * x_cin * 2;
  }
  {
    const int vox = wave * 64 + lane;
    const int d = vox / (kTH * kTW), h = (vox / kTW) % kTH, w = vox % kTW;
    ln.gcoord = d | (h << 8) | (w << 16);
    ln.grel = ((d * a.oh + h) * a.ow + w) * a.cout * 2;
  }
  {
    // transposing read: 16-lane group q supplies channels 16 (q & 1) .. + 15 of voxels 8 (q >> 1) .. + 7; inside it lane m
    // gives the address of channels 4 (m & 3) .. + 3 of voxel m >> 2
    const int q = lane >> 4, m = lane & 15;
    const int piece = 2 * (q & 1) + ((m & 3) >> 1);
    const int vox = 8 * (q >> 1) + (m >> 2) + 16 * seg16;
    ln.xread = piece * kXPiece + vox * 16 + (m & 1) * 8;
    ln.gread = piece * kGPiece + vox * 16 + (m & 1) * 8;
  }
  return ln;
}

// The LDS of a workgroup: a ring of three input plane pairs and three gy tiles.
struct WRingLds {
  char *xp0, *xp1, *xp2, *gt0, *gt1, *gt2;
};

// Steps s_begin .. s_begin + nsteps - 1 of column `col` of the 32 x 32 block (cob, cib), added to acc. `x` is the tensor
// that holds the block's input channels, moved so that the block's index in the whole input addresses them; x_cin its
// channel count.
template <typename T, int G>
__device__ __forceinline__ void wring_segment(const WgradArgs& a, const T* __restrict__ x, const T* __restrict__ gy, const WRingColumn& col,
                                              int s_begin, int nsteps, int cib, int cob, int x_cin, const WRingLane& ln, int wave,
                                              f32x16_t (&acc)[G == 0 ? kTaps0 : kTaps1], uint4 (&gyf)[kTD * kTH],
                                              uint4 (&fr)[WSchedule::kBuffers], const WRingLds& m) {
  int xoff[kXGroupsPerWave];
  int goff;
  const int plane0 = kTD * s_begin - a.pd;
  auto xorigin = [&](int plane) {
    return x + ((((int64_t)col.n * a.id + plane) * a.ih + (col.h0 - a.ph)) * a.iw + (col.w0 - a.pw)) * x_cin + cib * 32;
  };
  auto gorigin = [&](int d0) { return gy + ((((int64_t)col.n * a.od + d0) * a.oh + col.h0) * a.ow + col.w0) * a.cout + cob * 32; };

  // the first step's two pairs, and the gy tiles of the first two steps (gy runs two steps ahead of the MFMAs)
  wring_offsets(a, col, ln, plane0, kTD * s_begin, true, xoff, goff);
  wring_fetch<T>(m.xp0, m.gt0, wave, xorigin(plane0), gorigin(kTD * s_begin), xoff, goff);
  wring_offsets(a, col, ln, plane0 + 2, kTD * (s_begin + 1), true, xoff, goff);
  if (nsteps < 2) goff = kRange;
  wring_fetch<T>(m.xp1, m.gt1, wave, xorigin(plane0 + 2), gorigin(kTD * (s_begin + 1)), xoff, goff);
  __builtin_amdgcn_s_waitcnt(wring_waitcnt_vm(0));
  __builtin_amdgcn_s_barrier();
  {
    WRingFrags<G> first{m.xp0 + ln.xread, nullptr, m.gt0 + ln.gread, gyf, fr};
    first.early(std::make_integer_sequence<int, WSchedule::kMaxFrags>{}, std::make_integer_sequence<int, kTD * kTH>{});
  }

  // step i: MFMAs over pairs (lo, hi) and tile gt; the pair after them streams into xfill, the gy tile of step i + 2
  // into gfill; gt_next is the (resident) tile of step i + 1
  auto step = [&](int i, const char* lo, const char* hi, const char* gt, char* xfill, char* gfill, const char* gt_next) {
    const int plane = plane0 + 2 * i + 4, d_ahead = kTD * (s_begin + i + 2);
    wring_offsets(a, col, ln, plane, d_ahead, i + 1 < nsteps, xoff, goff);
    if (i + 2 >= nsteps) goff = kRange;
    WRingStep<T, G> st{WRingFrags<G>{lo + ln.xread, hi + ln.xread, gt + ln.gread, gyf, fr}, xfill, gfill, wave, acc, xoff, goff,
                       __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(xorigin(plane)), 0, kRange, 0x00020000),
                       __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(gorigin(d_ahead)), 0, kRange, 0x00020000)};
    st.run(std::make_integer_sequence<int, WSchedule::kMaxMfmas>{});
    if (i + 1 < nsteps) {  // the next step's first fragments: its first pair is this step's second one
      WRingFrags<G> next{hi + ln.xread, nullptr, gt_next + ln.gread, gyf, fr};
      next.early(std::make_integer_sequence<int, WSchedule::kMaxFrags>{}, std::make_integer_sequence<int, kTD * kTH>{});
    }
    __builtin_amdgcn_s_waitcnt(wring_waitcnt_vm(0));  // this wavefront's part of the next pair and tile has landed
    __builtin_amdgcn_s_barrier();                     // ... and every wavefront is done reading this step's
  };
  for (int i = 0; i < nsteps; i += 3) {
    step(i, m.xp0, m.xp1, m.gt0, m.xp2, m.gt2, m.gt1);
    if (i + 1 < nsteps) step(i + 1, m.xp1, m.xp2, m.gt1, m.xp0, m.gt0, m.gt2);
    if (i + 2 < nsteps) step(i + 2, m.xp2, m.xp0, m.gt2, m.xp1, m.gt1, m.gt0);
  }
}

// The wavefronts (0, G) and (1, G) hold sums over different voxels for the same taps: the second hands its
// accumulators over through LDS (the last barrier has freed it), kHandTaps taps at a time through the group's own
// array, the first adds them -- a fixed order -- and writes the block's part of a slice: dst points at element
// (co = first of the block, tap 0, ci = first of the block) of a [Cout][27][cin] slice. IN_LOOP (the batch, where a
// workgroup hands over in the middle of its range, while the others stream): dst is the block's own 27 x 1024 floats
// of a slice, written as they lie in the registers -- [tap][r4][lane][4]: lane (kg, j) holds output channels
// 8 r4 + 4 kg .. + 3 at input channel j -- in 16-byte stores, a quarter of the store instructions; the batch's sum
// pass puts them in place.
template <int G, bool IN_LOOP>
__device__ __forceinline__ void wring_handover(const f32x16_t (&acc)[G == 0 ? kTaps0 : kTaps1], float* __restrict__ dst, int cin, int tid,
                                               const WRingLds& m) {
  constexpr int NACC = G == 0 ? kTaps0 : kTaps1;
  const int lane = tid & 63;
  const int seg16 = __builtin_amdgcn_readfirstlane(tid >> 6) & 1;
  char* handover = G == 0 ? m.xp0 : m.xp1;
  const int j = lane & 31;
  int kg = lane >> 5;
  // (opaque to the optimiser where the call sits in a loop over blocks: it would otherwise compute all 224 store offsets
  // ahead of the loop and keep them in scratch memory)
  if constexpr (IN_LOOP) asm volatile("" : "+v"(kg));
  float4* dst4 = reinterpret_cast<float4*>(dst) + lane;
  if constexpr (IN_LOOP) asm volatile("" : "+v"(dst4));
#pragma unroll
  for (int round = 0; round < kHandRounds; ++round) {
    if (seg16 == 1) {
#pragma unroll
      for (int t = round * kHandTaps; t < (round + 1) * kHandTaps; ++t) {
        if (t >= NACC) continue;
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4)
          *reinterpret_cast<float4*>(handover + ((t - round * kHandTaps) * 4 + r4) * 1024 + lane * 16) =
              make_float4(acc[t][4 * r4], acc[t][4 * r4 + 1], acc[t][4 * r4 + 2], acc[t][4 * r4 + 3]);
      }
    }
    __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
    __builtin_amdgcn_s_barrier();
    if (seg16 == 0) {
#pragma unroll
      for (int t9 = 0; t9 < 9; ++t9)
#pragma unroll
        for (int kw = 0; kw < 3; ++kw) {
          if (tap_group(t9, kw) != G) continue;
          const int t = tap_slot(t9, kw), tap = t9 * 3 + kw;
          if (t < round * kHandTaps || t >= (round + 1) * kHandTaps) continue;
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const float4 o = *reinterpret_cast<const float4*>(handover + ((t - round * kHandTaps) * 4 + r4) * 1024 + lane * 16);
            const float v[4] = {acc[t][4 * r4] + o.x, acc[t][4 * r4 + 1] + o.y, acc[t][4 * r4 + 2] + o.z, acc[t][4 * r4 + 3] + o.w};
            if constexpr (IN_LOOP) {
              dst4[(tap * 4 + r4) * 64] = make_float4(v[0], v[1], v[2], v[3]);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const int co = 8 * r4 + 4 * kg + e;
                dst[((int64_t)co * 27 + tap) * cin + j] = v[e];
              }
            }
          }
        }
    }
    __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
    __builtin_amdgcn_s_barrier();  // the array is free for the next round
  }
}

template <typename T, int G>
__device__ __forceinline__ void wring_run(const WgradArgs& a, const T* __restrict__ x, const T* __restrict__ gy, float* __restrict__ ws,
                                          const WRingGeom& gm, int split, int cib, int cob, int x_cin, int tid, const WRingLds& m) {
  constexpr int NACC = G == 0 ? kTaps0 : kTaps1;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const WRingLane ln = wring_lane(a, x_cin, tid);

  f32x16_t acc[NACC];
#pragma unroll
  for (int t = 0; t < NACC; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
  uint4 gyf[kTD * kTH];            // gy fragments of the step's eight output rows (this wavefront's 16 voxels of each)
  uint4 fr[WSchedule::kBuffers];   // input-row fragments in rotation

  const int item_begin = split * gm.items_per_split;
  int item_end = item_begin + gm.items_per_split;
  if (item_end > gm.items) item_end = gm.items;
  const int ncols = gm.items / gm.segs;
  for (int item = item_begin; item < item_end; ++item) {
    const int seg = item / ncols;
    const WRingColumn col = wring_column(item - seg * ncols, gm.tiles_h, gm.tiles_w);
    const int s_begin = seg * gm.seg_steps;
    int s_end = s_begin + gm.seg_steps;
    if (s_end > gm.steps) s_end = gm.steps;
    if (s_end <= s_begin) continue;
    wring_segment<T, G>(a, x, gy, col, s_begin, s_end - s_begin, cib, cob, x_cin, ln, wave, acc, gyf, fr, m);
  }
  wring_handover<G, false>(acc, ws + ((int64_t)split * a.cout + cob * 32) * 27 * a.cin + cib * 32, a.cin, tid, m);
}

// ---- several weight gradients in one launch ------------------------------------------------------------------------------------
// A launch of the kernel above costs the same whatever the problem: every workgroup fetches its first two steps at once
// (all CUs asking together: 4.4 us), at the end every workgroup writes its 110 KB slice at once (6-7 us), a sum pass
// reads the 256 slices back (6 us), and two launches start. A batch pays that once for all its problems. All blocks of
// all problems lie on one line of cost -- problem after problem, inside a problem in UNITS (a chunk of columns of one
// 32 x 32 block, see batch_unit), inside a unit column after column, a column being kFillCost positions for the ring's
// start and one per step -- and workgroup w of W takes the positions [w total / W, (w + 1) total / W): whole columns,
// parts of columns, units of several blocks and problems. For every unit it touches it walks its steps of the unit's
// columns, hands its accumulators over and writes a slice of the unit's block: slice number (the block's slices from
// earlier units) + w - (the first workgroup that touches the unit). The sum pass knows from the same arithmetic how
// many slices a block has. The cut is a pure function of the list of problems; nothing is added atomically.
constexpr int kFillCost = 4;  // (the captured U-Net step: 2 -> 4 is 20 us faster, 4, 6 and 8 are alike)

struct WRingBatchEntry {
  WgradArgs a;
  const void* x;
  const void* x1;       // second tensor of the input (channels c_first ..), or null
  const void* gy;
  float* ws;            // this problem's slices: [slices][block][27 x 1024 floats in register order, see wring_handover]
  void* gw;
  int c_first;
  int tiles_h, tiles_w, steps, nblk_ci, nblk;
  int ncols;            // columns of a block
  int chunk;            // columns of a unit: the line runs [chunk of columns][block][column], see batch_unit
  int pos_begin;        // the problem's first position on the line
  int slices;           // the most slices any of its blocks gets
  int quad_begin;       // the problem's first float4 in the sum pass (a multiple of 256)
};

struct WRingBatch {
  int count, wgs, total, quads;
  WRingBatchEntry e[kWgradBatchMax];
};

// (32-bit arithmetic: wring_batch_plan refuses a line of kBatchMaxTotal positions or more)
constexpr int kBatchMaxTotal = 0x7fffff;
__host__ __device__ __forceinline__ int batch_cut(int w, int total, int wgs) { return (int)((uint32_t)w * (uint32_t)total / (uint32_t)wgs); }
// The workgroup whose range holds position q (total >= wgs: ranges are never empty).
__host__ __device__ __forceinline__ int batch_owner(int q, int total, int wgs) {
  int w = (int)((uint32_t)q * (uint32_t)wgs / (uint32_t)total);
  if (batch_cut(w + 1, total, wgs) <= q) ++w;
  return w;
}

// Inside a problem the line runs chunk of columns after chunk, inside a chunk block after block, inside a block's
// chunk -- a UNIT -- column after column. A chunk is about one workgroup's range, so the workgroups that walk the same
// columns for the problem's different 32 x 32 blocks are neighbours (same XCD) and do it at the same time: what one
// fetches of a 128-byte line of a 64-channel tensor, the other finds in L2. (Block after block over all columns, the
// launch fetched 1.9 times the bytes of the one-problem launches, FETCH_SIZE, and ran its level-1 steps a third slower.)
struct WUnit {
  int blk, col0, cols, begin;  // block, first column, columns, first position
};
__host__ __device__ __forceinline__ WUnit batch_unit(int rel, int pos_begin, int nblk, int ncols, int chunk, int colcost) {
  const int nfull = ncols / chunk, uc = chunk * colcost, span = nfull * nblk * uc;
  WUnit u;
  if (rel < span) {
    const int i = rel / uc;
    u.blk = i % nblk; u.col0 = (i / nblk) * chunk; u.cols = chunk; u.begin = pos_begin + i * uc;
  } else {
    const int rest = ncols - nfull * chunk, ur = rest * colcost, i = (rel - span) / ur;
    u.blk = i; u.col0 = nfull * chunk; u.cols = rest; u.begin = pos_begin + span + i * ur;
  }
  return u;
}
// Slices of block `blk` that belong to its first `chunks` units: each unit has one slice per workgroup that touches it.
__host__ __device__ __forceinline__ int batch_slices_before(int blk, int chunks, int pos_begin, int nblk, int ncols, int chunk, int colcost,
                                                            int total, int wgs) {
  const int nfull = ncols / chunk, uc = chunk * colcost;
  int n = 0;
  for (int k = 0; k < chunks; ++k) {
    const int cols = k < nfull ? chunk : ncols - nfull * chunk;
    const int begin = k < nfull ? pos_begin + (k * nblk + blk) * uc : pos_begin + nfull * nblk * uc + blk * cols * colcost;
    n += batch_owner(begin + cols * colcost - 1, total, wgs) - batch_owner(begin, total, wgs) + 1;
  }
  return n;
}

template <typename T, int G>
__device__ __forceinline__ void wring_batch_run(const WRingBatch& b, int w, int tid, const WRingLds& m) {
  constexpr int NACC = G == 0 ? kTaps0 : kTaps1;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  f32x16_t acc[NACC];
  uint4 gyf[kTD * kTH];
  uint4 fr[WSchedule::kBuffers];
  const int hi = batch_cut(w + 1, b.total, b.wgs);
  int pos = batch_cut(w, b.total, b.wgs);
  while (pos < hi) {
    int p = 0;
    for (int k = 1; k < b.count; ++k)
      if (pos >= b.e[k].pos_begin) p = k;
    const WgradArgs a = b.e[p].a;
    const int steps = b.e[p].steps, nblk_ci = b.e[p].nblk_ci, tiles_h = b.e[p].tiles_h, tiles_w = b.e[p].tiles_w;
    const int colcost = steps + kFillCost, chunk = b.e[p].chunk;
    const WUnit u = batch_unit(pos - b.e[p].pos_begin, b.e[p].pos_begin, b.e[p].nblk, b.e[p].ncols, chunk, colcost);
    const int blk = u.blk, b0 = u.begin, unit_end = u.begin + u.cols * colcost;
    const int seg_hi = hi < unit_end ? hi : unit_end;
    const int cib = blk % nblk_ci, cob = blk / nblk_ci;
    const T* xs = (const T*)b.e[p].x;
    int x_cin = a.cin, cis = cib;
    if (b.e[p].x1 != nullptr) {
      const int c_first = b.e[p].c_first;
      const bool second = cib * 32 >= c_first;
      xs = second ? (const T*)b.e[p].x1 : xs;
      x_cin = second ? a.cin - c_first : c_first;
      cis = second ? cib - c_first / 32 : cib;
    }
    const T* gy = (const T*)b.e[p].gy;
    const WRingLane ln = wring_lane(a, x_cin, tid);
#pragma unroll
    for (int t = 0; t < NACC; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
    for (int q = pos; q < seg_hi;) {
      const int c = (q - b0) / colcost, first_step = b0 + c * colcost + kFillCost;  // the position of the column's step 0
      int s_begin = q - first_step, s_end = seg_hi - first_step;
      if (s_begin < 0) s_begin = 0;
      if (s_end > steps) s_end = steps;
      if (s_end > s_begin)
        wring_segment<T, G>(a, xs + (cis - cib) * 32, gy, wring_column(u.col0 + c, tiles_h, tiles_w), s_begin, s_end - s_begin, cib, cob,
                            x_cin, ln, wave, acc, gyf, fr, m);
      q = first_step + steps;
    }
    const int slice = batch_slices_before(blk, u.col0 / chunk, b.e[p].pos_begin, b.e[p].nblk, b.e[p].ncols, chunk, colcost, b.total, b.wgs) +
                      (w - batch_owner(b0, b.total, b.wgs));
    wring_handover<G, true>(acc, b.e[p].ws + ((int64_t)slice * b.e[p].nblk + blk) * (27 * 1024), a.cin, tid, m);
    pos = seg_hi;
  }
}

template <typename T>
__global__ void __launch_bounds__(256, 1) wgrad_ring_batch_kernel(WRingBatch b) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(16))) char xp0[kXPair];
  __shared__ __attribute__((aligned(16))) char xp1[kXPair];
  __shared__ __attribute__((aligned(16))) char xp2[kXPair];
  __shared__ __attribute__((aligned(16))) char gt0[kGTile];
  __shared__ __attribute__((aligned(16))) char gt1[kGTile];
  __shared__ __attribute__((aligned(16))) char gt2[kGTile];
  const WRingLds m{xp0, xp1, xp2, gt0, gt1, gt2};
  const int tid = threadIdx.x;
  const int w = (int)xcd_remap(blockIdx.x, (uint32_t)b.wgs);
  if (__builtin_amdgcn_readfirstlane(tid >> 6) < 2) wring_batch_run<T, 0>(b, w, tid, m);
  else wring_batch_run<T, 1>(b, w, tid, m);
#endif
}

// The sum over the slices of every block of every problem of a batch, in slice order (eight, four, two loads in
// flight), one rounding to the gradient's dtype. A slice holds its blocks one after the other, each as the kernel's
// registers held it ([tap][r4][lane][4], see wring_handover); a thread owns one float4 of a block -- four consecutive
// output channels at one input channel of one tap -- and the lanes of a wavefront write rows of 32 input channels.
template <typename TOut>
__global__ void __launch_bounds__(256) wgrad_ring_batch_sum(WRingBatch b) {
  const int q0 = blockIdx.x * 256;  // a workgroup's 256 float4s lie in one problem (quad_begin is a multiple of 256)
  int p = 0;
  for (int k = 1; k < b.count; ++k)
    if (q0 >= b.e[k].quad_begin) p = k;
  const int q = q0 + threadIdx.x;
  const int cin = b.e[p].a.cin, cout = b.e[p].a.cout;
  const uint32_t nelem = (uint32_t)cout * 27u * (uint32_t)cin;  // below 2^31 (wring_batch_plan)
  const uint32_t el = (uint32_t)(q - b.e[p].quad_begin) * 4u;
  if (el >= nelem) return;
  const uint32_t quad = el / 4u;
  const int lane = (int)(quad % 64u), r4 = (int)(quad / 64u % 4u), tap = (int)(quad / 256u % 27u), blk = (int)(quad / (256u * 27u));
  const int ci = (blk % b.e[p].nblk_ci) * 32 + (lane & 31), co = (blk / b.e[p].nblk_ci) * 32 + 8 * r4 + 4 * (lane >> 5);
  const int chunk = b.e[p].chunk, ncols = b.e[p].ncols;
  const int n = batch_slices_before(blk, (ncols + chunk - 1) / chunk, b.e[p].pos_begin, b.e[p].nblk, ncols, chunk, b.e[p].steps + kFillCost,
                                    b.total, b.wgs);
  const float* part = b.e[p].ws + el;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  int sp = 0;
  for (; sp + 7 < n; sp += 8) {
    float4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = *reinterpret_cast<const float4*>(part + (int64_t)(sp + k) * nelem);
#pragma unroll
    for (int k = 0; k < 8; ++k) { s.x += v[k].x; s.y += v[k].y; s.z += v[k].z; s.w += v[k].w; }
  }
  for (; sp + 3 < n; sp += 4) {
    float4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = *reinterpret_cast<const float4*>(part + (int64_t)(sp + k) * nelem);
#pragma unroll
    for (int k = 0; k < 4; ++k) { s.x += v[k].x; s.y += v[k].y; s.z += v[k].z; s.w += v[k].w; }
  }
  for (; sp + 1 < n; sp += 2) {
    const float4 v0 = *reinterpret_cast<const float4*>(part + (int64_t)sp * nelem);
    const float4 v1 = *reinterpret_cast<const float4*>(part + (int64_t)(sp + 1) * nelem);
    s.x += v0.x; s.y += v0.y; s.z += v0.z; s.w += v0.w;
    s.x += v1.x; s.y += v1.y; s.z += v1.z; s.w += v1.w;
  }
  for (; sp < n; ++sp) {
    const float4 v = *reinterpret_cast<const float4*>(part + (int64_t)sp * nelem);
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  TOut* out = (TOut*)b.e[p].gw + ((int64_t)co * 27 + tap) * cin + ci;
  const int64_t row = (int64_t)27 * cin;
  out[0] = elem<TOut>::from_float(s.x);
  out[row] = elem<TOut>::from_float(s.y);
  out[2 * row] = elem<TOut>::from_float(s.z);
  out[3 * row] = elem<TOut>::from_float(s.w);
}

template <typename T>
__global__ void __launch_bounds__(256, 1)
wgrad_ring_kernel(WgradArgs a, const T* __restrict__ x, const T* __restrict__ gy, float* __restrict__ ws, WRingGeom gm, uint32_t total,
                  const T* __restrict__ x1, int c_first) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(16))) char xp0[kXPair];
  __shared__ __attribute__((aligned(16))) char xp1[kXPair];
  __shared__ __attribute__((aligned(16))) char xp2[kXPair];
  __shared__ __attribute__((aligned(16))) char gt0[kGTile];
  __shared__ __attribute__((aligned(16))) char gt1[kGTile];
  __shared__ __attribute__((aligned(16))) char gt2[kGTile];
  const WRingLds m{xp0, xp1, xp2, gt0, gt1, gt2};
  const int tid = threadIdx.x;
  const uint32_t wg = xcd_remap(blockIdx.x, total);
  const int blk = wg % gm.nblk, split = wg / gm.nblk;
  int cib = blk % gm.nblk_ci;
  const int cob = blk / gm.nblk_ci;
  // An input handed over as two tensors whose channels follow each other (the first c_first in x, the rest in x1): the
  // workgroup's 32 input channels lie in one of them, and that tensor is the one staged; the gradient's own indexing
  // keeps a.cin and the block's index in the whole.
  const T* xs = x;
  int x_cin = a.cin, cis = cib;
  if (x1 != nullptr) {
    const bool second = cib * 32 >= c_first;
    xs = second ? x1 : x;
    x_cin = second ? a.cin - c_first : c_first;
    cis = second ? cib - c_first / 32 : cib;
  }
  // wavefronts 0, 1 hold tap group 0, wavefronts 2, 3 tap group 1 (wave-uniform branch)
  WgradArgs as = a;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  float* wsb = ws;
  if (wave < 2) {
    // (the slice is indexed with the whole tensor's cin and block index)
    wring_run<T, 0>(as, xs + (cis - cib) * 32, gy, wsb, gm, split, cib, cob, x_cin, tid, m);
  } else {
    wring_run<T, 1>(as, xs + (cis - cib) * 32, gy, wsb, gm, split, cib, cob, x_cin, tid, m);
  }
#endif
}

WRingGeom wring_geom(const WgradArgs& a) {
  WRingGeom gm{};
  gm.tiles_h = (int)cdiv(a.oh, kTH);
  gm.tiles_w = (int)cdiv(a.ow, kTW);
  gm.steps = (int)cdiv(a.od, kTD);
  gm.nblk_ci = a.cin / 32;
  gm.nblk = gm.nblk_ci * (a.cout / 32);
  const int64_t ncols = (int64_t)a.n * gm.tiles_h * gm.tiles_w;
  int want = kComputeUnits / gm.nblk;  // workgroups per block: at most one workgroup per CU over all blocks
  if (want < 1) want = 1;
  int64_t segs = ncols >= want ? 1 : cdiv(want, ncols);
  if (segs > gm.steps) segs = gm.steps;
  gm.seg_steps = (int)cdiv(gm.steps, segs);
  gm.segs = (int)cdiv(gm.steps, gm.seg_steps);
  const int64_t items = ncols * gm.segs;
  gm.items = items > 0x7fffffffLL ? -1 : (int)items;
  if (gm.items > 0) {
    if (want > gm.items) want = gm.items;
    gm.items_per_split = (int)cdiv(gm.items, want);
    gm.splits = (int)cdiv(gm.items, gm.items_per_split);
  }
  return gm;
}

template <typename T>
int launch_wring(const WgradArgs& a, const WRingGeom& gm, const void* x, const void* gy, float* ws, hipStream_t st, const ChannelPair& x2) {
  const int64_t total = (int64_t)gm.splits * gm.nblk;
  hipLaunchKernelGGL((wgrad_ring_kernel<T>), dim3((unsigned)total), dim3(256), 0, st, a, (const T*)x, (const T*)gy, ws, gm, (uint32_t)total,
                     (const T*)x2.second, x2.first);
  return check_launch("wgrad_ring_kernel");
}

// The line of cost and the slices of a batch; ws_bytes: the workspace all problems need together. False when the batch
// cannot be laid out (too many problems, too much work for 32-bit positions).
bool wring_batch_plan(const WgradBatchItem* items, int count, WRingBatch& b, size_t& ws_bytes, int max_wgs) {
  if (count < 1 || count > kWgradBatchMax) return false;
  b = WRingBatch{};
  b.count = count;
  int64_t pos = 0, quads = 0;
  for (int i = 0; i < count; ++i) {
    const WgradArgs& a = items[i].a;
    WRingBatchEntry& e = b.e[i];
    e.a = a;
    e.x = items[i].x; e.x1 = items[i].x1; e.c_first = items[i].c_first; e.gy = items[i].gy; e.gw = items[i].gw;
    e.tiles_h = (int)cdiv(a.oh, kTH);
    e.tiles_w = (int)cdiv(a.ow, kTW);
    e.steps = (int)cdiv(a.od, kTD);
    e.nblk_ci = a.cin / 32;
    e.nblk = e.nblk_ci * (a.cout / 32);
    const int64_t ncols = (int64_t)a.n * e.tiles_h * e.tiles_w;
    const int64_t cost = (int64_t)e.nblk * ncols * (e.steps + kFillCost);
    if (ncols > kBatchMaxTotal || cost > kBatchMaxTotal) return false;
    e.ncols = (int)ncols;
    e.pos_begin = (int)pos;
    e.quad_begin = (int)quads;
    pos += cost;
    quads += (int64_t)a.cout * 27 * a.cin / 4;  // a multiple of 256 (Cout and Cin in blocks of 32)
    if ((int64_t)a.cout * 27 * a.cin > 0x7fffffffLL) return false;
    if (pos > kBatchMaxTotal || quads > 0x3fffffffLL) return false;
  }
  b.total = (int)pos;
  b.quads = (int)quads;
  // one workgroup per CU, fewer when that would leave a workgroup less than two columns' start cost of positions (a range
  // without a step still costs its block a slice of zeros)
  b.wgs = b.total / (2 * kFillCost);
  if (b.wgs > kComputeUnits) b.wgs = kComputeUnits;
  // (a launch meant to run beside other work takes fewer workgroups: one to a CU, the CUs it leaves alone are the others')
  if (max_wgs > 0 && b.wgs > max_wgs) b.wgs = max_wgs;
  if (b.wgs < 1) b.wgs = 1;
  ws_bytes = 0;
  for (int i = 0; i < count; ++i) {
    WRingBatchEntry& e = b.e[i];
    // a chunk of columns costs about one workgroup's range (a problem of one block is a single run of columns either way;
    // bending the column-start cost of a problem so that its units are exactly a range long was measured: no better)
    const int colcost = e.steps + kFillCost, range = b.total / b.wgs;
    int chunk = (range + colcost / 2) / colcost;
    if (chunk < 1) chunk = 1;
    if (chunk > e.ncols || e.nblk == 1) chunk = e.ncols;
    e.chunk = chunk;
    int most = 1;
    for (int blk = 0; blk < e.nblk; ++blk) {
      const int n = batch_slices_before(blk, (e.ncols + chunk - 1) / chunk, e.pos_begin, e.nblk, e.ncols, chunk, colcost, b.total, b.wgs);
      if (n > most) most = n;
    }
    e.slices = most;
    ws_bytes += align_up((size_t)most * e.a.cout * 27 * e.a.cin * sizeof(float), 256);
  }
  return true;
}

}  // namespace

// Rows of more than 16 voxels; a plane pair with its halo and a gy tile must span less than the buffer range.
bool mfma_wgrad_ring_applies(const WgradArgs& a) {
  if (a.ow <= 16 || a.od < 1 || a.oh < 1 || a.n < 1) return false;
  if (((int64_t)(a.ih + kBH) * a.iw + kBW) * a.cin * 2 + 64 >= kRange || ((int64_t)(a.oh + kTH) * a.ow + kTW) * a.cout * 2 + 64 >= kRange)
    return false;
  return wring_geom(a).items > 0;
}

int mfma_wgrad_ring_splits(const WgradArgs& a) { return wring_geom(a).splits; }

int mfma_wgrad_ring(const WgradArgs& a, int dtype, const void* x, const void* gy, float* ws, hipStream_t st, const ChannelPair& x2) {
  const WRingGeom gm = wring_geom(a);
  if (dtype == SFH_BF16) return launch_wring<bf16_t>(a, gm, x, gy, ws, st, x2);
  return launch_wring<fp16_t>(a, gm, x, gy, ws, st, x2);
}

size_t mfma_wgrad_ring_batch_workspace_bytes(const WgradBatchItem* items, int count, int max_wgs) {
  WRingBatch b;
  size_t bytes = 0;
  return wring_batch_plan(items, count, b, bytes, max_wgs) ? bytes : 0;
}

int mfma_wgrad_ring_batch(const WgradBatchItem* items, int count, int dtype, int gw_dtype, void* workspace, size_t workspace_bytes,
                          hipStream_t st, int max_wgs) {
  WRingBatch b;
  size_t need = 0;
  if (!wring_batch_plan(items, count, b, need, max_wgs)) return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad batch: %d problems cannot share a launch", count);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(SFH_ERR_WORKSPACE, "conv3d wgrad batch: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
  char* ws = (char*)workspace;
  for (int i = 0; i < count; ++i) {
    b.e[i].ws = (float*)ws;
    ws += align_up((size_t)b.e[i].slices * b.e[i].a.cout * 27 * b.e[i].a.cin * sizeof(float), 256);
  }
  if (b.total == 0) return SFH_OK;
  if (dtype == SFH_BF16) hipLaunchKernelGGL((wgrad_ring_batch_kernel<bf16_t>), dim3((unsigned)b.wgs), dim3(256), 0, st, b);
  else hipLaunchKernelGGL((wgrad_ring_batch_kernel<fp16_t>), dim3((unsigned)b.wgs), dim3(256), 0, st, b);
  if (int rc = check_launch("wgrad_ring_batch_kernel")) return rc;
  const unsigned sum_grid = (unsigned)cdiv(b.quads, 256);
  if (gw_dtype == SFH_FP32) hipLaunchKernelGGL((wgrad_ring_batch_sum<float>), dim3(sum_grid), dim3(256), 0, st, b);
  else if (gw_dtype == SFH_BF16) hipLaunchKernelGGL((wgrad_ring_batch_sum<bf16_t>), dim3(sum_grid), dim3(256), 0, st, b);
  else hipLaunchKernelGGL((wgrad_ring_batch_sum<fp16_t>), dim3(sum_grid), dim3(256), 0, st, b);
  return check_launch("wgrad_ring_batch_sum");
}

}  // namespace sfh
