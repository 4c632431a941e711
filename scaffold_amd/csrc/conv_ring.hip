// Persistent MFMA implicit-GEMM convolution for gfx950 (3x3x3, stride 1, 32 reduction channels, bf16 / fp16, rows of
// more than 16 voxels) that walks COLUMNS of the volume along depth and keeps the input planes it has already fetched.
//
// A workgroup (four wavefronts, one per CU, 512 registers per lane, the 54 weight fragments resident in registers) owns
// a column 8 rows high and 32 voxels wide and produces it two depth planes at a time. A step of 2 x 8 x 32 output
// voxels reads the four input planes d-1 .. d+2 (10 x 34 voxels each with the halo); the next step needs d+1 .. d+4,
// of which two are already in LDS. LDS therefore holds a ring of three plane PAIRS: two are read by the MFMAs of the
// current step while the third receives the next step's two new planes straight from memory (buffer_load ... lds).
// Per step a workgroup fetches 680 voxels for 512 outputs (1.33x) in 44 load instructions (12, 12, 12 and 8 over its four
// wavefronts), where a brick with its own halo in all three directions needs 1224 voxels (2.39x) and 80: global-memory instructions are what this
// kernel's matrix pipe waits for most.
//
// Each wavefront owns a 2 x 2 block of the step's rows (two planes x two rows of 32 voxels). An activation fragment --
// 32 voxels of one input row, shifted by kw, one k-step -- then serves up to four MFMAs (the taps (kd, kh) under which
// the row is seen from the wavefront's four output rows) and is read from LDS once: 96 reads for 216 MFMAs. The order
// of MFMAs and reads is a compile-time schedule (RingSchedule): the same order of taps for every output voxel, the four
// accumulators in turn, every fragment requested several MFMAs ahead of its first use.
//
// The three plane pairs are three separate LDS arrays and the ring position is a template parameter of the step: the
// compiler then sees that the MFMA operands never alias the array being filled, and every LDS address is an immediate
// offset from one of three per-lane bases.
#include <utility>

#include "conv_mfma.hpp"
#include "mma.hpp"

namespace sfh {
namespace {

typedef uint32_t ring_u32x4_t __attribute__((ext_vector_type(4)));
typedef mma_frag_t ring_i32x4_t;

constexpr int kTD = 2, kTH = 8, kTW = 32;         // output voxels of a step
constexpr int kBH = kTH + 2, kBW = kTW + 2;       // rows / voxels per row of an input plane with its halo
constexpr int kPairVoxels = 2 * kBH * kBW;        // voxels of a plane pair (680)
constexpr int ring_piece_bytes(int voxels) { return ((voxels * 16 - 64 + 255) / 256) * 256 + 64; }  // 64 modulo 256
constexpr int kPiece = ring_piece_bytes(kPairVoxels);  // one 8-channel piece of every voxel of a pair
constexpr int kPair = 4 * kPiece;                      // a plane pair: four pieces = 32 channels
constexpr int kGroups = (kPairVoxels + 63) / 64;       // 64-voxel groups a pair is fetched in (11, the last one partial)
constexpr int kGroupsPerWave = (kGroups + 3) / 4;      // 3
constexpr int kLoads = kGroupsPerWave * 4;             // load instructions per wavefront and step
constexpr int kStores = 8;                             // store instructions per wavefront and step (4 sub-tiles x 2)
constexpr int kRange = 0x40000000;                     // buffer range: offsets at or above it read as zero / are not stored
constexpr int kWeightFrags = 54;                       // (tap, k-step) fragments of a 32-channel output block, 1 KiB each
constexpr int kWeightInPair = kPair / 1024;            // ... of which the third pair's array holds this many while the kernel starts
constexpr int kWeightSpare = (kWeightFrags - kWeightInPair) * 1024;  // and a small array of its own the rest
static_assert(3 * kPair + kWeightSpare <= 160 * 1024, "three plane pairs and the rest of the weights in the LDS of a CU");
static_assert(kGroups * 1024 - kPiece < 64 * 16 && kPiece >= kPairVoxels * 16, "only the last group runs past a piece, by masked lanes");

// ---- the compile-time schedule of a step ---------------------------------------------------------------------------------------
// Block b = 0..5 handles kw = b % 3 and k-step ks = b / 3 (the first three blocks use the weight fragments held in vector
// registers, the last three those in accumulation registers). Inside a block the nine taps (kd, kh) come in row-major
// order, and each is applied to the wavefront's four accumulators (dd, hl) in turn: accumulator (dd, hl) under tap
// (kd, kh) reads input-row fragment F(D, H) = (kd + dd, kh + hl) -- plane D = 0..3 of the step, row H = 0..3 of the
// wavefront's two output rows with halo. Every output voxel therefore accumulates its 54 products in the same order
// whatever its place in the step (results do not depend on where a tensor's planes fall in the walk: a depth shard's
// slab and the padded volume give the same bits), two MFMAs on one accumulator are always four apart, and a fragment is
// read from LDS once and kept until the last tap that sees it.
struct RingSchedule {
  static constexpr int kFragsPerBlock = 16, kMfmasPerBlock = 36, kBlocks = 6;
  static constexpr int kFrags = kFragsPerBlock * kBlocks, kMfmas = kMfmasPerBlock * kBlocks;
  static constexpr int kLead = 5;      // a fragment is requested at least this many MFMAs before its first use
  static constexpr int kBuffers = 8;   // fragment registers (the schedule's need is checked against it)
  int frag_d[kFragsPerBlock], frag_h[kFragsPerBlock];  // in order of first use
  int mf_frag[kMfmasPerBlock], mf_acc[kMfmasPerBlock], mf_tap9[kMfmasPerBlock];
  int first_use[kFragsPerBlock], last_use[kFragsPerBlock];
  int issue_after[kFrags];  // global MFMA index after which fragment f is requested (negative: before the loop)
  int buffer[kFrags];       // the register set fragment f is read into
  int request_at[kMfmas];   // the fragment requested behind MFMA m, or -1
  int buffers_used;
};

constexpr RingSchedule make_ring_schedule() {
  RingSchedule s{};
  int slot_of[4][4] = {{-1, -1, -1, -1}, {-1, -1, -1, -1}, {-1, -1, -1, -1}, {-1, -1, -1, -1}};
  int nf = 0, m = 0;
  for (int kd = 0; kd < 3; ++kd)
    for (int kh = 0; kh < 3; ++kh)
      for (int dd = 0; dd < 2; ++dd)
        for (int hl = 0; hl < 2; ++hl) {
          const int d = kd + dd, h = kh + hl;
          if (slot_of[d][h] < 0) {
            slot_of[d][h] = nf;
            s.frag_d[nf] = d;
            s.frag_h[nf] = h;
            s.first_use[nf] = m;
            ++nf;
          }
          s.mf_frag[m] = slot_of[d][h];
          s.mf_acc[m] = dd * 2 + hl;
          s.mf_tap9[m] = kd * 3 + kh;
          s.last_use[slot_of[d][h]] = m;
          ++m;
        }
  // request times, latest first: as late as the lead allows, never two after the same MFMA
  int next = RingSchedule::kMfmas;
  for (int f = RingSchedule::kFrags - 1; f >= 0; --f) {
    const int use = (f / 16) * 36 + s.first_use[f % 16];
    int at = use - RingSchedule::kLead;
    if (at >= next) at = next - 1;
    s.issue_after[f] = at;
    next = at;
  }
  for (int k = 0; k < RingSchedule::kMfmas; ++k) s.request_at[k] = -1;
  for (int f = 0; f < RingSchedule::kFrags; ++f)
    if (s.issue_after[f] >= 0) s.request_at[s.issue_after[f]] = f;
  // register sets: a set is free again once the MFMA of its fragment's last use has been issued
  int busy_until[RingSchedule::kFrags] = {};
  int nb = 0;
  for (int f = 0; f < RingSchedule::kFrags; ++f) {
    const int last = (f / 16) * 36 + s.last_use[f % 16];
    int pick = -1;
    for (int b = 0; b < nb && pick < 0; ++b)
      if (busy_until[b] <= s.issue_after[f]) pick = b;
    if (pick < 0) pick = nb++;
    busy_until[pick] = last;
    s.buffer[f] = pick;
  }
  s.buffers_used = nb;
  return s;
}

constexpr RingSchedule kSched = make_ring_schedule();

constexpr bool ring_schedule_ok() {
  // the first four MFMAs touch the four accumulators (they start from zero); afterwards the accumulators take turns
  for (int i = 0; i < 36; ++i)
    if (kSched.mf_acc[i] != i % 4) return false;
  // every fragment is requested ahead of its first use
  for (int f = 0; f < RingSchedule::kFrags; ++f)
    if (kSched.issue_after[f] > (f / 16) * 36 + kSched.first_use[f % 16] - 2) return false;
  return kSched.buffers_used <= RingSchedule::kBuffers;
}
static_assert(ring_schedule_ok(), "step schedule");

// Side work of a step rides behind every tenth MFMA: first the loads of the next pair (they need the rest of the step to
// arrive), then the stores of the previous step's rounded result. Measured against closer spacings and interleaved
// orders: the kernel is insensitive to it within 2 %, spreading the memory instructions out is marginally the best.
constexpr int kSidePeriod = 10, kSidePhase = 3;
constexpr int side_kind(int slot) { return slot < kLoads + kStores ? slot : -1; }  // which load (0 ..) or store (kLoads ..) a slot carries
static_assert((RingSchedule::kMfmas - kSidePhase + kSidePeriod - 1) / kSidePeriod >= kLoads + kStores, "a slot per load and store");

// s_waitcnt immediate (gfx9 encoding) that waits for vmcnt <= n and nothing else.
constexpr int ring_waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

struct RingGeom {
  int tiles_h, tiles_w;       // columns per sample
  int steps;                  // steps of a whole column: ceil(od / 2)
  int segs, seg_steps;        // a column is cut into `segs` segments of `seg_steps` steps (the last one shorter)
  int nblocks;                // 32-channel output blocks
  int items, wgs_per_block, items_per_wg;  // items = columns x segments; each workgroup takes items_per_wg consecutive ones
};

// What a lane needs to know for the whole launch.
struct RingLane {
  int rbase;                     // LDS read: byte offset of (k-half, first row of the wavefront, voxel j) inside a pair
  int grel[kGroupsPerWave];      // staging: byte offset of the lane's voxel from the pair's first voxel in the input
  int gcoord[kGroupsPerWave];    // staging: dl | bh << 8 | bw << 16, or -1 past the pair's end
  int vrel[4];                   // output: byte offset of the lane's piece from the step's first voxel in y
};

// Output of a finished step, rounded, waiting to be stored during the next one (see conv_persist.hip: the two lanes of
// a voxel trade channel runs so that each stores two 16-byte pieces).
struct RingPending {
  ring_u32x4_t data[4][2];
};

struct RingColumn {
  int n, h0, w0;  // sample, first output row and voxel of the column
};

__device__ __forceinline__ RingColumn ring_column(int col, const RingGeom& gm) {
  RingColumn c;
  c.w0 = (col % gm.tiles_w) * kTW; col /= gm.tiles_w;
  c.h0 = (col % gm.tiles_h) * kTH;
  c.n = col / gm.tiles_h;
  return c;
}

// Buffer offsets of the lane's voxels of the plane pair whose first plane is input plane `plane` (may be negative or past
// the end: such planes, like rows and voxels outside the input, get an out-of-range offset and arrive as zeros).
// `live` false turns the whole pair into such lanes. -1: the lane has no voxel in this group.
__device__ __forceinline__ void ring_pair_offsets(const MfmaConvArgs& a, const RingColumn& c, const RingLane& ln, int plane, bool live,
                                                  int (&voff)[kGroupsPerWave]) {
  const int ih0 = c.h0 - a.ph, iw0 = c.w0 - a.pw;
#pragma unroll
  for (int k = 0; k < kGroupsPerWave; ++k) {
    const int dl = ln.gcoord[k] & 0xff, bh = (ln.gcoord[k] >> 8) & 0xff, bw = (ln.gcoord[k] >> 16) & 0xff;
    const int inside = (int)((unsigned)(plane + dl) < (unsigned)a.id) & (int)((unsigned)(ih0 + bh) < (unsigned)a.ih) &
                       (int)((unsigned)(iw0 + bw) < (unsigned)a.iw) & (int)live;
    voff[k] = ln.gcoord[k] < 0 ? -1 : (inside ? ln.grel[k] : kRange);
  }
}

// The (possibly virtual) address of voxel (plane, first row, first voxel) of the column's input with halo.
template <typename T>
__device__ __forceinline__ const T* ring_pair_origin(const MfmaConvArgs& a, const T* x, const RingColumn& c, int plane) {
  return x + ((((int64_t)c.n * a.id + plane) * a.ih + (c.h0 - a.ph)) * a.iw + (c.w0 - a.pw)) * a.cred;
}

// Issues the whole pair at once (a segment's first two pairs).
template <typename T>
__device__ __forceinline__ void ring_fetch_pair(char* dst, int wave, const T* origin, const int (&voff)[kGroupsPerWave]) {
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(origin), 0, kRange, 0x00020000);
#pragma unroll
  for (int k = 0; k < kGroupsPerWave; ++k)
    if (voff[k] != -1) {
#pragma unroll
      for (int p = 0; p < 4; ++p)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(dst + (wave + 4 * k) * 1024 + p * kPiece), 16,
                                                 voff[k] + p * 16, 0, 0, 0);
    }
}

// Byte offset inside a pair of fragment F(D % 2, H) shifted by kw, k-step ks, relative to RingLane::rbase.
__device__ __forceinline__ constexpr int ring_frag_off(int dl, int h, int kw, int ks) {
  return ks * 2 * kPiece + ((dl * kBH + h) * kBW + kw) * 16;
}

// One step: 216 MFMAs over the pairs `lo` (planes 0, 1 of the step) and `hi` (planes 2, 3), with the loads of the next
// step's new pair into `fill` and the stores of the previous step's result riding along. Everything the schedule decides
// is a template argument, so that every register array is indexed by constants.
template <typename T>
struct RingStep {
  using S = RingSchedule;
  const char* lane_lo;
  const char* lane_hi;
  char* fill;
  int wave;
  const uint4 (&wq)[27];
  const ring_i32x4_t (&wa)[27];
  f32x16_t (&acc)[4];
  const RingPending& ps;
  const int (&voff)[kGroupsPerWave];
  __amdgpu_buffer_rsrc_t rsrc, done_rsrc;
  const int (&done_off)[4];
  uint4 fr[S::kBuffers];

  template <int F>
  __device__ __forceinline__ void request() {
    constexpr int b = F / 16, fi = F % 16;
    constexpr int d = kSched.frag_d[fi], h = kSched.frag_h[fi];
    constexpr int off = ring_frag_off(d % 2, h, b % 3, b / 3);
    fr[kSched.buffer[F]] = *reinterpret_cast<const uint4*>((d < 2 ? lane_lo : lane_hi) + off);
  }
  template <int F>
  __device__ __forceinline__ void request_if_early() {
    if constexpr (kSched.issue_after[F] < 0) request<F>();
  }
  template <int... Fs>
  __device__ __forceinline__ void prologue(std::integer_sequence<int, Fs...>) {
    (request_if_early<Fs>(), ...);
  }

  template <int M>
  __device__ __forceinline__ void mfma() {
    constexpr int b = M / 36, i = M % 36;
    constexpr int kw = b % 3, ks = b / 3;
    constexpr int f = b * 16 + kSched.mf_frag[i], ac = kSched.mf_acc[i];
    constexpr int tap = kSched.mf_tap9[i] * 3 + kw;
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (ks == 0) {
      if constexpr (M < 4) {  // a step starts from zero: the first MFMA on an accumulator takes a zero addend
        f32x16_t zero;
#pragma unroll
        for (int r = 0; r < 16; ++r) zero[r] = 0.f;
        acc[ac] = Mma32<T>::run(wq[tap], fr[kSched.buffer[f]], zero);
      } else {
        acc[ac] = Mma32<T>::run(wq[tap], fr[kSched.buffer[f]], acc[ac]);
      }
    } else {
      Mma32Pinned<T>::run_row_in_acc(wa[tap], fr[kSched.buffer[f]], acc[ac]);
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (kSched.request_at[M] >= 0) {  // at most one fragment request behind an MFMA
      request<kSched.request_at[M]>();
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (M % kSidePeriod == kSidePhase) {
      constexpr int kind = side_kind(M / kSidePeriod);
      if constexpr (kind >= 0 && kind < kLoads) {
        constexpr int k = kind / 4, p = kind % 4;
        if (voff[k] != -1)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(fill + (wave + 4 * k) * 1024 + p * kPiece), 16,
                                                   voff[k] + p * 16, 0, 0, 0);
      } else if constexpr (kind >= kLoads) {
        constexpr int ms = (kind - kLoads) / 2, h = (kind - kLoads) % 2;
        __builtin_amdgcn_raw_buffer_store_b128(ps.data[ms][h], done_rsrc, done_off[ms] + 32 * h, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  template <int... Ms>
  __device__ __forceinline__ void run(std::integer_sequence<int, Ms...>) {
    (mfma<Ms>(), ...);
  }
};

template <typename T>
__device__ __forceinline__ void ring_step(const char* lo, const char* hi, char* fill, int wave, const RingLane& ln,
                                          const uint4 (&wq)[27], const ring_i32x4_t (&wa)[27], f32x16_t (&acc)[4],
                                          const RingPending& ps, const T* fetch_origin, const int (&voff)[kGroupsPerWave],
                                          __amdgpu_buffer_rsrc_t done_rsrc, const int (&done_off)[4]) {
  RingStep<T> st{lo + ln.rbase, hi + ln.rbase, fill, wave, wq, wa, acc, ps, voff,
                 __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(fetch_origin), 0, kRange, 0x00020000), done_rsrc, done_off, {}};
  st.prologue(std::make_integer_sequence<int, RingSchedule::kFrags>{});
  st.run(std::make_integer_sequence<int, RingSchedule::kMfmas>{});
}

// Rounds the step's accumulators into `ps` (stored during the next step) and works out where they go: `tc` = the step's
// first output plane, the column in `c`. With GN the rounded values inside the output are added to the GroupNorm sums.
template <typename T, bool BIAS, bool GN>
__device__ __forceinline__ void ring_round(const f32x16_t (&acc)[4], const float (&bias)[16], RingPending& ps, int (&done_off)[4],
                                           const MfmaConvArgs& a, const RingColumn& c, int d0, int wave, int j, const RingLane& ln,
                                           RunSums& sums, int& have_shift) {
#pragma unroll
  for (int ms = 0; ms < 4; ++ms) {
    const int dd = ms / 2, hl = ms % 2;
    const int ok = (int)(d0 + dd < a.od) & (int)(c.h0 + 2 * wave + hl < a.oh) & (int)(c.w0 + j < a.ow);
    done_off[ms] = ok ? ln.vrel[ms] : kRange;
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
      bool first = false;
      if (ms == 0 && !have_shift) {
        first = __builtin_amdgcn_readfirstlane(ok) != 0;  // lane 0 holds the wavefront's first voxel of the step
        have_shift = first ? 1 : 0;
      }
      sums.template add<T>(run, ok != 0, first);
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const auto lo = __builtin_amdgcn_permlane32_swap(run[2 * h][0], run[2 * h + 1][0], false, false);
      const auto hi = __builtin_amdgcn_permlane32_swap(run[2 * h][1], run[2 * h + 1][1], false, false);
      ps.data[ms][h] = ring_u32x4_t{lo[0], hi[0], lo[1], hi[1]};
    }
  }
}

template <typename T, bool BIAS, bool GN>
__global__ void __launch_bounds__(256, 1)
conv_ring_kernel(MfmaConvArgs a, const T* __restrict__ x, const T* __restrict__ wp, const T* __restrict__ bias_ptr, T* __restrict__ y,
                 RingGeom gm, GnPartialOut gn, T* __restrict__ y1, int c_first) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(16))) char pair0[kPair];
  __shared__ __attribute__((aligned(16))) char pair1[kPair];
  __shared__ __attribute__((aligned(16))) char pair2[kPair];
  __shared__ __attribute__((aligned(16))) char wrest[kWeightSpare];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 31, kg = lane >> 5;

  const int wg = (int)xcd_remap(blockIdx.x, gridDim.x);
  const int nb = wg / gm.wgs_per_block;
  const int wg_in_block = wg - nb * gm.wgs_per_block;
  const int item_begin = wg_in_block * gm.items_per_wg;
  int item_end = item_begin + gm.items_per_wg;
  if (item_end > gm.items) item_end = gm.items;
  if (nb >= gm.nblocks || item_begin >= item_end) return;

  // Where this workgroup's 32 output channels go (an output handed over as two tensors: see conv_persist.hip).
  T* yout = y;
  int yrow = a.cout, yc0 = nb * 32;
  if (y1 != nullptr) {
    const bool second = nb * 32 >= c_first;
    yout = second ? y1 : y;
    yrow = second ? a.cout - c_first : c_first;
    yc0 = second ? nb * 32 - c_first : nb * 32;
  }

  RingLane ln;
  ln.rbase = kg * kPiece + ((2 * wave) * kBW + j) * 16;
#pragma unroll
  for (int k = 0; k < kGroupsPerWave; ++k) {
    const int vox = (wave + 4 * k) * 64 + lane;
    const int dl = vox / (kBH * kBW), r = vox % (kBH * kBW), bh = r / kBW, bw = r % kBW;
    ln.gcoord[k] = vox < kPairVoxels ? (dl | (bh << 8) | (bw << 16)) : -1;
    ln.grel[k] = (((dl * a.ih + bh) * a.iw + bw) * a.cred) * 2;
  }
#pragma unroll
  for (int ms = 0; ms < 4; ++ms) {
    const int dd = ms / 2, hl = ms % 2;
    ln.vrel[ms] = (((dd * a.oh + 2 * wave + hl) * a.ow + j) * yrow + 8 * kg) * 2;
  }

  constexpr int FRAG = 512;
  uint4 wq[27];
  ring_i32x4_t wa[27];
  // The block's 54 fragments come into LDS once per workgroup (direct-to-LDS loads, a quarter per wavefront: the packed
  // weight is in fragment order, a fragment is 1 KiB as it lies) and every wavefront takes its copy from there: four
  // copies straight from memory cost the CU's address path 216 KiB beside the first plane pairs' 86. They land in the
  // third pair's array, which nothing reads before the first step fills it, and in `wrest`.
  {
    const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(wp + (int64_t)nb * kWeightFrags * FRAG), 0,
                                                                            kWeightFrags * 1024, 0x00020000);
#pragma unroll
    for (int k = 0; k < (kWeightFrags + 3) / 4; ++k) {
      const int f = wave + 4 * k;  // wave-uniform
      if (f < kWeightFrags) {
        char* dst = f < kWeightInPair ? pair2 + f * 1024 : wrest + (f - kWeightInPair) * 1024;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(wrsrc, (__attribute__((address_space(3))) void*)dst, 16, f * 1024 + lane * 16, 0, 0, 0);
      }
    }
  }
  float bias[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) bias[r] = BIAS ? to_float(bias_ptr[nb * 32 + 8 * (r / 4) + 4 * kg + (r % 4)]) : 0.f;

  RunSums gn_sums;
  gn_sums.clear();
  int gn_have_shift = 0;
  f32x16_t acc[4];
  RingPending ps;
  int done_off[4];
  int voff[kGroupsPerWave];

  auto run_item = [&](int item, auto with_weights) {
    // item = segment * columns + column: the workgroups of an XCD work on neighbouring columns over the same depth range
    const int ncols = gm.items / gm.segs;
    const int seg = item / ncols;
    const RingColumn col = ring_column(item - seg * ncols, gm);
    const int s_begin = seg * gm.seg_steps;
    int s_end = s_begin + gm.seg_steps;
    if (s_end > gm.steps) s_end = gm.steps;
    const int nsteps = s_end - s_begin;
    const int plane0 = 2 * s_begin - a.pd;  // first input plane of the segment's first step (every segment has at least one)

    // the first step's four planes
    ring_pair_offsets(a, col, ln, plane0, true, voff);
    ring_fetch_pair<T>(pair0, wave, ring_pair_origin<T>(a, x, col, plane0), voff);
    ring_pair_offsets(a, col, ln, plane0 + 2, true, voff);
    ring_fetch_pair<T>(pair1, wave, ring_pair_origin<T>(a, x, col, plane0 + 2), voff);
#pragma unroll
    for (int ms = 0; ms < 4; ++ms) {
#pragma unroll
      for (int h = 0; h < 2; ++h) ps.data[ms][h] = ring_u32x4_t{0u, 0u, 0u, 0u};
      done_off[ms] = kRange;  // nothing to store during the segment's first step
    }
    T* done_origin = yout;
    __builtin_amdgcn_s_waitcnt(ring_waitcnt_vm(0));
    __syncthreads();
    if constexpr (decltype(with_weights)::value) {
      // the weights have landed with the first pairs: k-step 0 of every tap into vector registers, k-step 1 into
      // accumulation registers (the MFMA reads its row operand from either file; there are not 216 vector registers to
      // spare beside the activation fragments)
#pragma unroll
      for (int tap = 0; tap < 27; ++tap) {
        const int f0 = 2 * tap, f1 = 2 * tap + 1;
        wq[tap] = *reinterpret_cast<const uint4*>((f0 < kWeightInPair ? pair2 + f0 * 1024 : wrest + (f0 - kWeightInPair) * 1024) + lane * 16);
        wa[tap] = *reinterpret_cast<const ring_i32x4_t*>((f1 < kWeightInPair ? pair2 + f1 * 1024 : wrest + (f1 - kWeightInPair) * 1024) + lane * 16);
      }
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the copies are in registers ...
      __syncthreads();                     // ... in every wavefront, before the first step's loads may overwrite them
    }

    auto step = [&](int i, const char* lo, const char* hi, char* fill) {
      // the pair after this step's: planes plane0 + 2 i + 4, + 5
      const int plane = plane0 + 2 * i + 4;
      ring_pair_offsets(a, col, ln, plane, i + 1 < nsteps, voff);
      const __amdgpu_buffer_rsrc_t done_rsrc = __builtin_amdgcn_make_buffer_rsrc(done_origin, 0, kRange, 0x00020000);
      ring_step<T>(lo, hi, fill, wave, ln, wq, wa, acc, ps, ring_pair_origin<T>(a, x, col, plane), voff, done_rsrc, done_off);
      asm volatile("s_nop 15\n\ts_nop 15");  // the last MFMAs are inline asm: the compiler does not know their result latency
      const int d0 = 2 * (s_begin + i);
      ring_round<T, BIAS, GN>(acc, bias, ps, done_off, a, col, d0, wave, j, ln, gn_sums, gn_have_shift);
      done_origin = yout + ((((int64_t)col.n * a.od + d0) * a.oh + col.h0) * a.ow + col.w0) * yrow + yc0;
      __builtin_amdgcn_s_waitcnt(ring_waitcnt_vm(0));  // this wavefront's part of the next pair has landed
      __syncthreads();                                 // ... and every wavefront is done reading this step's pairs
    };
    for (int i = 0; i < nsteps; i += 3) {
      step(i, pair0, pair1, pair2);
      if (i + 1 < nsteps) step(i + 1, pair1, pair2, pair0);
      if (i + 2 < nsteps) step(i + 2, pair2, pair0, pair1);
    }
    // the segment's last result
    const __amdgpu_buffer_rsrc_t done_rsrc = __builtin_amdgcn_make_buffer_rsrc(done_origin, 0, kRange, 0x00020000);
#pragma unroll
    for (int ms = 0; ms < 4; ++ms)
#pragma unroll
      for (int h = 0; h < 2; ++h) __builtin_amdgcn_raw_buffer_store_b128(ps.data[ms][h], done_rsrc, done_off[ms] + 32 * h, 0, 0);
  };
  // the workgroup's first item also takes the weights out of LDS (a copy of the item's code of its own: the register
  // arrays they go to are then defined on every path into the steps)
  run_item(item_begin, std::true_type{});
  for (int item = item_begin + 1; item < item_end; ++item) run_item(item, std::false_type{});
  if constexpr (GN) {
    // one record per workgroup (one sample): the last barrier has freed the LDS
    const int per_wg = gn.cg > 32 ? gn.cg / 32 : 1;  // output blocks that share a group
    RunSums one[1] = {gn_sums};
    write_group_partials<4, 1>(one, reinterpret_cast<float*>(pair0), gn, 0, wg_in_block * per_wg + nb % per_wg, nb * 32, tid);
  }
#endif
}

RingGeom ring_geom(const MfmaConvArgs& a) {
  RingGeom gm{};
  gm.tiles_h = (int)cdiv(a.oh, kTH);
  gm.tiles_w = (int)cdiv(a.ow, kTW);
  gm.steps = (int)cdiv(a.od, kTD);
  gm.nblocks = a.cout / 32;
  const int64_t ncols = (int64_t)a.n * gm.tiles_h * gm.tiles_w;
  int per_block = kComputeUnits / gm.nblocks;
  if (per_block < 1) per_block = 1;
  // segments per column: enough for every workgroup of the block to have one, no more than there are steps
  int64_t segs = ncols >= per_block ? 1 : cdiv(per_block, ncols);
  if (segs > gm.steps) segs = gm.steps;
  gm.seg_steps = (int)cdiv(gm.steps, segs);
  gm.segs = (int)cdiv(gm.steps, gm.seg_steps);
  const int64_t items = ncols * gm.segs;
  gm.items = items > 0x7fffffffLL ? -1 : (int)items;
  if (gm.items > 0) {
    if (per_block > gm.items) per_block = gm.items;
    gm.items_per_wg = (int)cdiv(gm.items, per_block);
    gm.wgs_per_block = (int)cdiv(gm.items, gm.items_per_wg);
  }
  return gm;
}

template <typename T>
int launch_ring(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                const GnPartialOut& gn, const ChannelPair& out2) {
  const RingGeom gm = ring_geom(a);
  if (gm.items < 0) return fail(SFH_ERR_UNSUPPORTED, "conv mfma: too many columns");
  if (gm.items == 0) return SFH_OK;
  const unsigned grid = (unsigned)(gm.wgs_per_block * gm.nblocks);
#define SFH_RING(BIAS, GN)                                                                                                  \
  hipLaunchKernelGGL((conv_ring_kernel<T, BIAS, GN>), dim3(grid), dim3(256), 0, st, a, (const T*)x, (const T*)packed, \
                     (const T*)bias, (T*)y, gm, gn, (T*)out2.second, out2.first)
  if (bias != nullptr) {
    if (gn.part != nullptr) SFH_RING(true, true);
    else SFH_RING(true, false);
  } else {
    if (gn.part != nullptr) SFH_RING(false, true);
    else SFH_RING(false, false);
  }
#undef SFH_RING
  return check_launch("conv_ring_kernel");
}

}  // namespace

// Rows of more than 16 voxels, 32 reduction channels, a 3x3x3 kernel; a plane pair with its halo (10 rows) must span
// less than the buffer range in the input, a step (2 planes of 8 rows) less than it in the output.
bool mfma_conv_ring_applies(const MfmaConvArgs& a) {
  return a.cred == 32 && a.kd == 3 && a.kh == 3 && a.kw == 3 && a.ow > 16 &&
         ((int64_t)(a.ih + kBH) * a.iw + kBW) * a.cred * 2 + 64 < kRange && ((int64_t)(a.oh + kTH) * a.ow + kTW) * a.cout * 2 + 64 < kRange;
}

int mfma_conv_ring_workgroups_per_block(const MfmaConvArgs& a) { return ring_geom(a).wgs_per_block; }

int mfma_conv_ring(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                   const GnPartialOut& gn, const ChannelPair& out2) {
  if (dtype == SFH_BF16) return launch_ring<bf16_t>(a, x, packed, bias, y, st, gn, out2);
  return launch_ring<fp16_t>(a, x, packed, bias, y, st, gn, out2);
}

}  // namespace sfh
