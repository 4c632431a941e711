// MFMA implicit-GEMM convolution for gfx950: stride 1, dilation 1, kernel extents <= 3,
// bf16 / fp16 operands, fp32 accumulation, one rounding on store.
//
// GEMM view (triton_conv3d/gather_gemm.py:112-341): M = output voxels, N = produced channels,
// K = taps x reduction channels. What is different here is where the operands live:
//
//   * A workgroup owns a TD x TH x TW brick of output voxels and stages the matching input
//     brick INCLUDING its halo in LDS once per 32-channel chunk; all taps then read it at a
//     constant offset, so an input voxel is fetched from memory once per brick instead of once
//     per tap.
//   * LDS layout is four "planes" per chunk, plane p holding channels [8p, 8p+8) of every brick
//     voxel as one 16-byte unit. A wavefront's activation fragment for 32 consecutive voxels is
//     then 512 contiguous bytes per half-wave: ds_read_b128 without bank conflicts, no padding
//     between voxels, and every (tap, k-step) is an immediate offset from one per-lane base.
//     Planes are spaced 64 bytes (mod 256) apart so the staging writes do not conflict either.
//   * The weight is repacked once per call (a few hundred KB) into MFMA fragment order, so a
//     wavefront fetches the fragment for (tap, k-step) as one contiguous 1 KiB global load that
//     hits in L1/L2; it is reused across the wave's four 32-voxel sub-tiles.
//   * v_mfma_f32_32x32x16 with the WEIGHT as the row operand: a lane then ends up holding, for
//     one voxel, four runs of four consecutive output channels; the two lanes of a voxel trade runs and store
//     16-byte pieces.
//
// The data gradient runs this same kernel with the weight packed transposed and tap-flipped and
// padding k-1-p (triton_conv3d/bwd_data.py:344-363).
#include "conv_mfma.hpp"
#include "mma.hpp"
#include "gn_stats.hpp"
#include "reduce.hpp"

namespace sfh {
namespace {



constexpr int kChunk = 32;  // reduction channels staged per pass (4 planes of 8)

constexpr int plane_bytes(int voxels) {
  // smallest size >= voxels*16 that is 64 modulo 256
  int b = voxels * 16;
  int r = ((b - 64 + 255) / 256) * 256 + 64;
  return r;
}

template <int TD_, int TH_, int TW_, int KD_, int KH_, int KW_, int NSUB_>
struct Tile {
  static constexpr int TD = TD_, TH = TH_, TW = TW_, KD = KD_, KH = KH_, KW = KW_, NSUB = NSUB_;
  static constexpr int BD = TD + KD - 1, BH = TH + KH - 1, BW = TW + KW - 1;
  static constexpr int BV = BD * BH * BW;            // brick voxels
  static constexpr int PLANE = plane_bytes(BV);
  static constexpr int LDS = 4 * PLANE;
  static constexpr int TAPS = KD * KH * KW;
  static constexpr int SUBTILES = TD * TH * TW / 32;  // 32-voxel MFMA column blocks
  static constexpr int MS = SUBTILES / 4;             // per wavefront
  static_assert(TD * TH * TW % 128 == 0, "tile must split into 4 wavefronts of 32-voxel sub-tiles");
  static_assert(LDS <= 80 * 1024, "two workgroups must fit in the 160 KB LDS of a CU");
  static_assert(2 * PLANE + ((KD - 1) * BH * BW + (KH - 1) * BW + KW - 1) * 16 < 65536, "ds_read immediate range");
};

// LDS byte offset, relative to a lane's sub-tile base, of iteration it = tap*2 + kstep.
template <typename C>
__device__ __forceinline__ constexpr int lds_off(int it) {
  const int tap = it / 2, ks = it % 2;
  const int kd = tap / (C::KH * C::KW), kh = (tap / C::KW) % C::KH, kw = tap % C::KW;
  return ((kd * C::BH + kh) * C::BW + kw) * 16 + ks * 2 * C::PLANE;
}

// WQ: weight fragments in flight per wavefront (see the chunk loop).
// PAIR: the input is two tensors whose channels follow each other (the first `c_first` in x, the rest in x1): every
// 32-channel chunk is staged from the one that holds it. Independently, a non-null y1 splits the OUTPUT the same way.
template <typename T, typename C, int WQ, bool PAIR>
__global__ void __launch_bounds__(256, 2)
conv_mfma_kernel(MfmaConvArgs a, const T* __restrict__ x, const T* __restrict__ wp, const T* __restrict__ bias,
                 T* __restrict__ y, float* __restrict__ partial, int tiles_d, int tiles_h, int tiles_w, int nblocks, int ksplit,
                 uint32_t total, GnPartialOut gn, const T* __restrict__ x1, T* __restrict__ y1, int c_first) {
  __shared__ __attribute__((aligned(16))) char lds[C::LDS];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int j = lane & 31, kg = lane >> 5;

  uint32_t t = xcd_remap(blockIdx.x, total);
  const int ksp = t % ksplit; t /= ksplit;  // slice of the reduction channels (1 slice unless the grid would underfill the chip)
  const int nb = t % nblocks; t /= nblocks;
  const int tw_i = t % tiles_w; t /= tiles_w;
  const int th_i = t % tiles_h; t /= tiles_h;
  const int td_i = t % tiles_d;
  const int n = t / tiles_d;
  const int od0 = td_i * C::TD, oh0 = th_i * C::TH, ow0 = tw_i * C::TW;

  // Per-lane LDS byte offset of the sub-tile voxel at tap (0,0,0), in the lane's k-half plane.
  int lbase[C::MS];
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) {
    const int v = (wave * C::MS + ms) * 32 + j;
    const int tw = v % C::TW, th = (v / C::TW) % C::TH, td = v / (C::TW * C::TH);
    lbase[ms] = kg * C::PLANE + ((td * C::BH + th) * C::BW + tw) * 16;
  }

  f32x16_t acc[C::MS][C::NSUB];
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms)
#pragma unroll
    for (int ns = 0; ns < C::NSUB; ++ns)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ms][ns][r] = 0.f;

  const int ncc = a.cred / kChunk;
  const int id0 = od0 - a.pd, ih0 = oh0 - a.ph, iw0 = ow0 - a.pw;
  constexpr int PIECES = C::BV * 4;
  constexpr int ITERS = (PIECES + 255) / 256;
  // staging loads in flight before the first LDS write: all of them when registers allow
  constexpr int BATCH = C::NSUB == 1 ? ITERS : 8;
  constexpr int FRAG = 512;  // elements per packed (tap, k-step) fragment: 64 lanes x 8

  const int cc_begin = (int)((int64_t)ksp * ncc / ksplit), cc_end = (int)((int64_t)(ksp + 1) * ncc / ksplit);
  for (int cc = cc_begin; cc < cc_end; ++cc) {
    // The first weight fragments of this chunk are requested before its brick is staged (one output block per
    // workgroup; with two the staging needs the registers): they depend on nothing in LDS, and a chunk whose weights
    // come from HBM (every chunk, each time a training step reaches the layer) would otherwise start its MFMAs one
    // memory round trip late.
    const T* wcc = wp + ((int64_t)(nb * C::NSUB) * ncc + cc) * (C::TAPS * 2 * FRAG) + lane * 8;
    const int64_t wns = (int64_t)ncc * (C::TAPS * 2 * FRAG);  // next 32-channel output block
    constexpr int NIT = C::TAPS * 2;
    // Weight fragments in flight per wavefront: WQ. A fragment feeds MS x NSUB MFMAs (32 cycles each): the fewer those
    // are, the more fragments must be under way to cover a trip to L2 or HBM -- 4 with two output blocks (registers), 6
    // for 512-voxel tiles, 12 for 256-voxel tiles when the launch is one round of workgroups (each then waits out its
    // own cold misses), 6 when it is several rounds (two resident workgroups cover for each other; the deeper queue
    // only costs registers and cache there).
    constexpr int WWANT = WQ;
    constexpr int WDEPTH = NIT < WWANT ? NIT : WWANT;
    uint4 wq[NIT][C::NSUB];  // fully unrolled: every slot is its own register set, live for WDEPTH iterations
    // a chunk's first weight requests go out ahead of its brick staging; with two output blocks the staging needs the registers
    constexpr bool early = C::NSUB == 1;
    if (early) {
#pragma unroll
      for (int it = 0; it < WDEPTH; ++it) wq[it][0] = *reinterpret_cast<const uint4*>(wcc + it * FRAG);
    }
    __syncthreads();  // every wave is done reading the previous chunk
    {
      // channels per voxel of the tensor this chunk lies in, and the chunk's first channel in the sample
      int row = a.cred;
      const T* xn;
      if constexpr (PAIR) {
        const bool second = cc * kChunk >= c_first;
        row = second ? a.cred - c_first : c_first;
        xn = (second ? x1 : x) + (int64_t)n * a.id * a.ih * a.iw * row + (second ? cc * kChunk - c_first : cc * kChunk);
      } else {
        xn = x + (int64_t)n * a.id * a.ih * a.iw * a.cred + cc * kChunk;
      }
#pragma unroll
      for (int it0 = 0; it0 < ITERS; it0 += BATCH) {
        uint4 v[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
          if (it0 + u < ITERS) {
            // With two output blocks per workgroup registers are short: the brick position is worked out again for
            // every chunk (the empty asm keeps the compiler from hoisting 64-bit addresses out of the chunk loop, where
            // they were spilled and every load waited for the reload of its address), and the load is unconditional
            // from a clamped address, masked afterwards.
            int p = (it0 + u) * 256 + tid;
            if constexpr (C::NSUB > 1) asm volatile("" : "+v"(p));
            const int vox = p >> 2, piece = p & 3;
            const int bw = vox % C::BW, bh = (vox / C::BW) % C::BH, bd = vox / (C::BW * C::BH);
            const int id = id0 + bd, ih = ih0 + bh, iw = iw0 + bw;
            const bool in = p < PIECES && (unsigned)id < (unsigned)a.id && (unsigned)ih < (unsigned)a.ih && (unsigned)iw < (unsigned)a.iw;
            if constexpr (C::NSUB > 1) {
              const int64_t at = in ? (((int64_t)id * a.ih + ih) * a.iw + iw) * row + piece * 8 : 0;
              const uint4 got = *reinterpret_cast<const uint4*>(xn + at);
              v[u] = in ? got : make_uint4(0, 0, 0, 0);
            } else {  // registers to spare: the compiler keeps the addresses across chunks and batches every load
              v[u] = make_uint4(0, 0, 0, 0);
              if (in) v[u] = *reinterpret_cast<const uint4*>(xn + (((int64_t)id * a.ih + ih) * a.iw + iw) * row + piece * 8);
            }
          }
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
          if (it0 + u < ITERS) {
            const int p = (it0 + u) * 256 + tid;
            if (p < PIECES) *reinterpret_cast<uint4*>(lds + (p & 3) * C::PLANE + (p >> 2) * 16) = v[u];
          }
        }
      }
    }
    __syncthreads();

    // Software pipeline over the TAPS*2 (tap, k-step) iterations of this chunk: the weight fragment
    // of iteration it+WDEPTH and the activation fragments of iteration it+1 are requested before the
    // MFMAs of iteration it are issued, so L2 and LDS latency overlap the matrix pipe.
    uint4 aq[2][C::MS];
    if (!early) {
#pragma unroll
      for (int it = 0; it < WDEPTH; ++it)
#pragma unroll
        for (int ns = 0; ns < C::NSUB; ++ns) wq[it][ns] = *reinterpret_cast<const uint4*>(wcc + ns * wns + it * FRAG);
    }
#pragma unroll
    for (int ms = 0; ms < C::MS; ++ms) aq[0][ms] = *reinterpret_cast<const uint4*>(lds + lbase[ms] + lds_off<C>(0));
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      // The requests of later iterations -- the weight fragments of iteration it + WDEPTH, the activation fragments of
      // iteration it + 1 -- are issued BETWEEN this iteration's MFMAs, one behind each: a load issued while the matrix
      // pipe is busy costs nothing, a block of them in front of the MFMAs leaves the pipe idle while they issue.
      constexpr int NM = C::MS * C::NSUB;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < NM; ++m) {
        const int ms = m / C::NSUB, ns = m % C::NSUB;
        acc[ms][ns] = Mma32<T>::run(wq[it][ns], aq[it & 1][ms], acc[ms][ns]);
        __builtin_amdgcn_sched_barrier(0);
        if (m < C::NSUB) {
          if (it + WDEPTH < NIT) wq[it + WDEPTH][m] = *reinterpret_cast<const uint4*>(wcc + m * wns + (it + WDEPTH) * FRAG);
        } else if (m - C::NSUB < C::MS) {
          if (it + 1 < NIT) aq[(it + 1) & 1][m - C::NSUB] = *reinterpret_cast<const uint4*>(lds + lbase[m - C::NSUB] + lds_off<C>(it + 1));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (C::MS + C::NSUB > NM) {  // more requests than MFMAs (one channel block per workgroup): the rest behind the last
#pragma unroll
        for (int k = NM - C::NSUB; k < C::MS; ++k)
          if (it + 1 < NIT) aq[(it + 1) & 1][k] = *reinterpret_cast<const uint4*>(lds + lbase[k] + lds_off<C>(it + 1));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // GroupNorm statistics of the rounded output, when the caller wants them (the reduction is not sliced then).
  RunSums gn_sums[C::NSUB];
#pragma unroll
  for (int ns = 0; ns < C::NSUB; ++ns) {
    gn_sums[ns].clear();
  }

  // Epilogue. Accumulator register r of a lane is output channel 8*(r/4) + 4*kg + r%4 of the
  // sub-tile's voxel j: four runs of four consecutive channels per 32-channel block. For the 16-bit output the two
  // lanes of a voxel trade runs so that each stores two 16-byte pieces (32 contiguous bytes of a voxel per store
  // instruction).
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) {
    const int v = (wave * C::MS + ms) * 32 + j;
    const int tw = v % C::TW, th = (v / C::TW) % C::TH, td = v / (C::TW * C::TH);
    const int od = od0 + td, oh = oh0 + th, ow = ow0 + tw;
    const bool inside = od < a.od && oh < a.oh && ow < a.ow;
    const int64_t vox = (((int64_t)n * a.od + od) * a.oh + oh) * a.ow + ow;
    if (ksplit > 1) {
      if (!inside) continue;
      // fp32 slice of this reduction range; the slices are summed (and the bias added) by sum_slices_bias
      float* pp = partial + ((int64_t)ksp * a.n * a.od * a.oh * a.ow + vox) * a.cout + nb * C::NSUB * 32;
#pragma unroll
      for (int ns = 0; ns < C::NSUB; ++ns)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          *reinterpret_cast<float4*>(pp + ns * 32 + 8 * g + 4 * kg) =
              make_float4(acc[ms][ns][4 * g], acc[ms][ns][4 * g + 1], acc[ms][ns][4 * g + 2], acc[ms][ns][4 * g + 3]);
      continue;
    }
#pragma unroll
    for (int ns = 0; ns < C::NSUB; ++ns) {
      // the 32-channel block's place in the output: in y, or (an output given as two tensors) in the one that holds it
      const int ch = (nb * C::NSUB + ns) * 32;
      T* yp = y + vox * a.cout + ch;
      if (y1 != nullptr) yp = ch >= c_first ? y1 + vox * (a.cout - c_first) + (ch - c_first) : y + vox * c_first + ch;
      uint32_t run[4][2];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int co = ns * 32 + 8 * g + 4 * kg;
        float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
        if (bias != nullptr) {
          const T* bp = bias + nb * C::NSUB * 32 + co;
          b0 = to_float(bp[0]); b1 = to_float(bp[1]); b2 = to_float(bp[2]); b3 = to_float(bp[3]);
        }
        run[g][0] = Mma32<T>::pack2(acc[ms][ns][4 * g] + b0, acc[ms][ns][4 * g + 1] + b1);
        run[g][1] = Mma32<T>::pack2(acc[ms][ns][4 * g + 2] + b2, acc[ms][ns][4 * g + 3] + b3);
      }
      if (gn.part != nullptr) gn_sums[ns].template add<T>(run, inside, ms == 0);
      uint4 piece[2];
      trade_channel_runs(run, piece);  // all lanes take part, also those of voxels past the edge
      if (inside) {
        *reinterpret_cast<uint4*>(yp + 8 * kg) = piece[0];
        *reinterpret_cast<uint4*>(yp + 16 + 8 * kg) = piece[1];
      }
    }
  }
  if (gn.part != nullptr && ksplit == 1) {
    __syncthreads();  // every wave is done reading the brick: the LDS is free
    constexpr int SPAN = 32 * C::NSUB;
    const int per_tile = gn.cg > SPAN ? gn.cg / SPAN : 1;  // workgroups that share a group of this tile
    const int tile = (td_i * tiles_h + th_i) * tiles_w + tw_i;
    write_group_partials<4, C::NSUB>(gn_sums, reinterpret_cast<float*>(lds), gn, n, tile * per_tile + nb % per_tile, nb * SPAN, tid);
  }
}

// One thread per packed 16-byte piece: the 8 consecutive reduction channels of one (output channel, tap, k-half).
// With the reduction channel innermost in memory (forward, channels-last weight) that is one 16-byte load;
// otherwise eight 2-byte loads, each coalesced across the wavefront's 32 consecutive output channels.
struct PackJob {
  const void* w;
  void* packed;
  int cout, cred;
  int taps;  // kd | kh << 8 | kw << 16 | flip << 24 (one word: 48 jobs fit a 4 KB table of kernel arguments)
  int64_t s_out, s_red, s_kd, s_kh, s_kw;
  int64_t pieces;
};

template <typename T>
__device__ __forceinline__ void pack_piece(const PackJob& j, int64_t idx) {
  const T* w = static_cast<const T*>(j.w);
  T* packed = static_cast<T*>(j.packed);
  const int kh = (j.taps >> 8) & 0xff, kw = (j.taps >> 16) & 0xff, flip = j.taps >> 24;
  const int taps = (j.taps & 0xff) * kh * kw;
  int64_t r = idx;
  const int lane = (int)(r % 64); r /= 64;
  const int ks = (int)(r % 2); r /= 2;
  int tap = (int)(r % taps); r /= taps;
  const int ncc = j.cred / kChunk;
  const int cc = (int)(r % ncc);
  const int nblk = (int)(r / ncc);
  const int co = nblk * 32 + (lane & 31);
  const int ci = cc * kChunk + ks * 16 + (lane >> 5) * 8;
  if (flip) tap = taps - 1 - tap;
  const int tkw = tap % kw, tkh = (tap / kw) % kh, tkd = tap / (kw * kh);
  const T* src = w + co * j.s_out + ci * j.s_red + tkd * j.s_kd + tkh * j.s_kh + tkw * j.s_kw;
  uint4 v;
  if (j.s_red == 1 && (reinterpret_cast<uintptr_t>(src) & 15) == 0) {
    v = *reinterpret_cast<const uint4*>(src);
  } else {
    uint16_t h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = *reinterpret_cast<const uint16_t*>(src + e * j.s_red);
    v.x = h[0] | ((uint32_t)h[1] << 16); v.y = h[2] | ((uint32_t)h[3] << 16);
    v.z = h[4] | ((uint32_t)h[5] << 16); v.w = h[6] | ((uint32_t)h[7] << 16);
  }
  *reinterpret_cast<uint4*>(packed + idx * 8) = v;
}

// Up to two packings of one weight (the forward's and the data gradient's) in one launch.
template <typename T>
__global__ void __launch_bounds__(256) pack_weight_kernel(PackJob first, PackJob second) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx < first.pieces) pack_piece<T>(first, idx);
  else if (idx - first.pieces < second.pieces) pack_piece<T>(second, idx - first.pieces);
}

// Many packings in one launch: a workgroup finds its job from the table of first workgroups.
constexpr int kPackBatch = 48;  // (the table stays under 4 KB of kernel arguments)
struct PackBatch {
  PackJob job[kPackBatch];
  int first_block[kPackBatch + 1];
  int njobs;
};
static_assert(sizeof(PackBatch) <= 4096, "kernel arguments");

template <typename T>
__global__ void __launch_bounds__(256) pack_weight_batch_kernel(PackBatch b) {
  int j = 0;
  while (j + 1 < b.njobs && (int)blockIdx.x >= b.first_block[j + 1]) ++j;
  const int64_t idx = (int64_t)((int)blockIdx.x - b.first_block[j]) * 256 + threadIdx.x;
  if (idx < b.job[j].pieces) pack_piece<T>(b.job[j], idx);
}

struct GatherPlan { int shape; int nsub; int ksplit; int64_t tiles; };

// Brick shapes: the row-length class (32-, 16- or 8-voxel rows) times the tile size (512, 256 or 128 output voxels).
constexpr int kTileDims[3][3][3] = {
    {{4, 4, 32}, {2, 4, 32}, {1, 4, 32}},
    {{4, 8, 16}, {2, 8, 16}, {1, 8, 16}},
    {{8, 8, 8}, {4, 8, 8}, {2, 8, 8}},
};

int64_t tiles_of(const MfmaConvArgs& a, int cls, int size) {
  const int* t = kTileDims[cls][size];
  return (int64_t)a.n * cdiv(a.od, t[0]) * cdiv(a.oh, t[1]) * cdiv(a.ow, t[2]);
}

// Launch geometry, a pure function of the problem. The row length picks the brick's row class; then, among 512- and
// 256-voxel tiles with one or two 32-channel output blocks per workgroup, the choice that loads the busiest CU least:
// workgroups are dealt round-robin, so that CU gets ceil(workgroups / CUs) of them, each worth tile voxels x blocks.
// A 256-voxel tile re-stages more halo per output voxel (weight 1.15), two blocks share one staged brick (0.97); both
// weights are fitted to timings of every convolution shape of a five-level U-Net on whole cubes and on depth shards.
// On the depth slab of a shard (D + 2 planes of data gradient) this is what keeps 288 half-empty second rounds of
// 512-voxel tiles from costing a whole round. When even the small tiles leave CUs idle (the deep, small-volume levels)
// the reduction channels are cut into at most 8 slices that are summed afterwards: a power of two, no more than would
// give every CU a workgroup (more slices cost more in fp32 partials than they gain).
GatherPlan gather_plan(const MfmaConvArgs& a) {
  GatherPlan p{};
  const int cls = a.ow > 16 ? 0 : (a.ow > 8 ? 1 : 2);
  const int ncc = a.cred / kChunk;
  int64_t best = -1, best_wgs = 0;
  for (int size = 0; size < 2; ++size) {
    const int* t = kTileDims[cls][size];
    const int64_t tiles = tiles_of(a, cls, size), voxels = (int64_t)t[0] * t[1] * t[2];
    for (int nsub = 1; nsub <= (a.cout % 64 == 0 ? 2 : 1); ++nsub) {
      const int64_t wgs = tiles * (a.cout / (32 * nsub));
      const int64_t cost = cdiv(wgs, kComputeUnits) * voxels * nsub * (size == 1 ? 115 : 100) * (nsub == 2 ? 97 : 100);
      if (best < 0 || cost < best) {
        best = cost; best_wgs = wgs;
        p.shape = cls * 3 + size; p.tiles = tiles; p.nsub = nsub;
      }
    }
  }
  p.ksplit = 1;
  if (best_wgs > 0 && best_wgs < kComputeUnits) {
    const int64_t room = kComputeUnits / best_wgs;
    while (p.ksplit * 2 <= room && p.ksplit * 2 <= ncc && p.ksplit < 8) p.ksplit *= 2;
  }
  return p;
}

struct PairPtrs { const void* x1; void* y1; int first; };

template <typename T, typename C, bool PAIR>
int launch_cfg(const MfmaConvArgs& a, const GatherPlan& p, const void* x, const void* packed, const void* bias, void* y,
               float* partial, hipStream_t st, const GnPartialOut& gn, const PairPtrs& pr) {
  const int tiles_d = (int)cdiv(a.od, C::TD), tiles_h = (int)cdiv(a.oh, C::TH), tiles_w = (int)cdiv(a.ow, C::TW);
  const int nblocks = a.cout / (32 * C::NSUB);
  const int64_t total = (int64_t)a.n * tiles_d * tiles_h * tiles_w * nblocks * p.ksplit;
  if (total == 0) return SFH_OK;
  if (total > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "conv mfma: %lld workgroups exceed the grid limit", (long long)total);
#define SFH_BRICK(WQ)                                                                                                      \
  hipLaunchKernelGGL((conv_mfma_kernel<T, C, WQ, PAIR>), dim3((unsigned)total), dim3(256), 0, st, a, (const T*)x,       \
                     (const T*)packed, (const T*)bias, (T*)y, partial, tiles_d, tiles_h, tiles_w, nblocks, p.ksplit,       \
                     (uint32_t)total, gn, (const T*)pr.x1, (T*)pr.y1, pr.first)
  if constexpr (C::NSUB > 1) SFH_BRICK(4);
  else if constexpr (C::MS >= 4) SFH_BRICK(6);
  else if (total <= 2 * kComputeUnits) SFH_BRICK(12);
  else SFH_BRICK(6);
#undef SFH_BRICK
  return check_launch("conv_mfma_kernel");
}

template <typename T, int NSUB, bool PAIR>
int launch_k333(const MfmaConvArgs& a, const GatherPlan& p, const void* x, const void* packed, const void* bias, void* y,
                float* partial, hipStream_t st, const GnPartialOut& gn, const PairPtrs& pr) {
  // Brick shape follows the row length: 32-voxel sub-tiles are one, two or four W rows.
  switch (p.shape) {
    case 0: return launch_cfg<T, Tile<4, 4, 32, 3, 3, 3, NSUB>, PAIR>(a, p, x, packed, bias, y, partial, st, gn, pr);
    case 3: return launch_cfg<T, Tile<4, 8, 16, 3, 3, 3, NSUB>, PAIR>(a, p, x, packed, bias, y, partial, st, gn, pr);
    case 6: return launch_cfg<T, Tile<8, 8, 8, 3, 3, 3, NSUB>, PAIR>(a, p, x, packed, bias, y, partial, st, gn, pr);
    case 1: return launch_cfg<T, Tile<2, 4, 32, 3, 3, 3, NSUB>, PAIR>(a, p, x, packed, bias, y, partial, st, gn, pr);
    case 4: return launch_cfg<T, Tile<2, 8, 16, 3, 3, 3, NSUB>, PAIR>(a, p, x, packed, bias, y, partial, st, gn, pr);
    case 7: return launch_cfg<T, Tile<4, 8, 8, 3, 3, 3, NSUB>, PAIR>(a, p, x, packed, bias, y, partial, st, gn, pr);
    default: return fail(SFH_ERR_UNSUPPORTED, "conv mfma: no kernel for brick shape %d", p.shape);
  }
}

// Records of GroupNorm partials per sample the launch of plan p leaves for `groups` groups (0: not offered).
int gather_gn_records(const MfmaConvArgs& a, const GatherPlan& p, int groups) {
  if (p.ksplit > 1) return sum_slices_bias_stats_records((int64_t)a.od * a.oh * a.ow * a.cout, a.cout, groups);
  const int span = 32 * p.nsub;
  if (!gn_partials_fit(a.cout, groups, span)) return 0;
  const int cg = a.cout / groups;
  const int64_t records = p.tiles / a.n * (cg > span ? cg / span : 1);
  return records <= 0x7fffffff ? (int)records : 0;
}

// The brick kernel takes any cut of its input, or of its output, at a multiple of the 32-channel chunk (when the
// reduction is sliced it is the sum of the slices that writes the two tensors).
bool gather_pair_ok(const MfmaConvArgs& a, int first, bool as_output) {
  const int channels = as_output ? a.cout : a.cred;
  return first > 0 && first < channels && first % 32 == 0;
}

template <typename T>
int launch_typed(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y, void* partial,
                 hipStream_t st, const GnPartialOut* gn, const ChannelPair* in2, const ChannelPair* out2) {
  const GatherPlan p = gather_plan(a);
  if (p.ksplit > 1 && partial == nullptr) return fail(SFH_ERR_WORKSPACE, "conv mfma: the reduction split needs its workspace");
  if (in2 != nullptr && out2 != nullptr) return fail(SFH_ERR_UNSUPPORTED, "conv mfma: input and output cannot both be pairs");
  if (out2 != nullptr && gn != nullptr && gn->part != nullptr)
    return fail(SFH_ERR_UNSUPPORTED, "conv mfma: no GroupNorm partials of an output written as two tensors");
  if (in2 != nullptr && (in2->second == nullptr || !gather_pair_ok(a, in2->first, false)))
    return fail(SFH_ERR_UNSUPPORTED, "conv mfma: the input cannot be cut at channel %d of %d", in2->first, a.cred);
  if (out2 != nullptr && (out2->second == nullptr || !gather_pair_ok(a, out2->first, true)))
    return fail(SFH_ERR_UNSUPPORTED, "conv mfma: the output cannot be cut at channel %d of %d", out2->first, a.cout);
  const PairPtrs pr{in2 != nullptr ? in2->second : nullptr, (out2 != nullptr && p.ksplit == 1) ? out2->second : nullptr,
                    in2 != nullptr ? in2->first : (out2 != nullptr ? out2->first : 0)};
  GnPartialOut out{nullptr, 0, 0, 0};
  if (gn != nullptr && gn->part != nullptr) {
    if (gn->records != gather_gn_records(a, p, gn->groups) || gn->records == 0)
      return fail(SFH_ERR_INVALID, "conv mfma: GroupNorm partials asked for %d records, this launch leaves %d", gn->records,
                  gather_gn_records(a, p, gn->groups));
    out = *gn;
    out.cg = a.cout / gn->groups;
  }
  const GnPartialOut none{nullptr, 0, 0, 0};
  const GnPartialOut& in_kernel = p.ksplit == 1 ? out : none;
  int rc;
  if (in2 != nullptr)
    rc = p.nsub == 2 ? launch_k333<T, 2, true>(a, p, x, packed, bias, y, (float*)partial, st, in_kernel, pr)
                     : launch_k333<T, 1, true>(a, p, x, packed, bias, y, (float*)partial, st, in_kernel, pr);
  else
    rc = p.nsub == 2 ? launch_k333<T, 2, false>(a, p, x, packed, bias, y, (float*)partial, st, in_kernel, pr)
                     : launch_k333<T, 1, false>(a, p, x, packed, bias, y, (float*)partial, st, in_kernel, pr);
  if (rc != SFH_OK || p.ksplit == 1) return rc;
  const int64_t sample = (int64_t)a.od * a.oh * a.ow * a.cout;
  if (out.part != nullptr) return sum_slices_bias_stats(dtype, (const float*)partial, bias, y, a.n, sample, a.cout, p.ksplit, out, st);
  return sum_slices_bias(dtype, (const float*)partial, bias, y, a.n * sample, a.cout, p.ksplit, st, out2);
}

}  // namespace

bool mfma_conv_supported(const MfmaConvArgs& a, int dtype) {
  if (dtype != SFH_BF16 && dtype != SFH_FP16) return false;
  if (a.kd != 3 || a.kh != 3 || a.kw != 3) return false;
  if (a.cred % kChunk != 0 || a.cout % 32 != 0) return false;
  if (a.pd < 0 || a.ph < 0 || a.pw < 0 || a.pd > 2 || a.ph > 2 || a.pw > 2) return false;
  if (a.n < 1 || a.od < 1 || a.oh < 1 || a.ow < 1) return false;
  return true;
}

size_t mfma_conv_packed_weight_bytes(const MfmaConvArgs& a) {
  return align_up((size_t)a.cout * a.cred * a.kd * a.kh * a.kw * 2, 256);
}

namespace {
PackJob pack_job(const MfmaConvArgs& a, const void* w, int64_t s_out, int64_t s_red, int64_t s_kd, int64_t s_kh, int64_t s_kw, int flip,
                 void* packed) {
  PackJob j{};
  j.w = w; j.packed = packed;
  j.cout = a.cout; j.cred = a.cred; j.taps = a.kd | (a.kh << 8) | (a.kw << 16) | ((flip ? 1 : 0) << 24);  // (kernel extents are at most 3)
  j.s_out = s_out; j.s_red = s_red; j.s_kd = s_kd; j.s_kh = s_kh; j.s_kw = s_kw;
  j.pieces = (int64_t)a.cout * a.cred * a.kd * a.kh * a.kw / 8;  // 16-byte pieces
  return j;
}
int launch_pack(int dtype, const PackJob& first, const PackJob& second, hipStream_t st) {
  const int64_t total = first.pieces + second.pieces;
  if (total <= 0) return SFH_OK;
  const unsigned blocks = (unsigned)cdiv(total, 256);
  if (dtype == SFH_BF16) hipLaunchKernelGGL(pack_weight_kernel<bf16_t>, dim3(blocks), dim3(256), 0, st, first, second);
  else hipLaunchKernelGGL(pack_weight_kernel<fp16_t>, dim3(blocks), dim3(256), 0, st, first, second);
  return check_launch("pack_weight_kernel");
}
}  // namespace

int mfma_pack_weight(const MfmaConvArgs& a, int dtype, const void* w, int64_t s_out, int64_t s_red, int64_t s_kd, int64_t s_kh,
                     int64_t s_kw, int flip, void* packed, hipStream_t st) {
  PackJob none{};
  return launch_pack(dtype, pack_job(a, w, s_out, s_red, s_kd, s_kh, s_kw, flip, packed), none, st);
}

int mfma_pack_weight_batch(const MfmaPackItem* items, int n, int dtype, hipStream_t st) {
  for (int i0 = 0; i0 < n; i0 += kPackBatch) {
    PackBatch b{};
    int64_t blocks = 0;
    for (int i = i0; i < n && i < i0 + kPackBatch; ++i) {
      const MfmaPackItem& it = items[i];
      const PackJob job = pack_job(it.a, it.w, it.s_out, it.s_red, it.s_kd, it.s_kh, it.s_kw, it.flip, it.packed);
      if (job.pieces <= 0) continue;
      b.job[b.njobs] = job;
      b.first_block[b.njobs] = (int)blocks;
      blocks += cdiv(job.pieces, 256);
      ++b.njobs;
      if (blocks > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "conv3d pack: batch too large");
    }
    b.first_block[b.njobs] = (int)blocks;
    if (b.njobs == 0) continue;
    if (dtype == SFH_BF16) hipLaunchKernelGGL(pack_weight_batch_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, st, b);
    else hipLaunchKernelGGL(pack_weight_batch_kernel<fp16_t>, dim3((unsigned)blocks), dim3(256), 0, st, b);
    if (int rc = check_launch("pack_weight_batch_kernel")) return rc;
  }
  return SFH_OK;
}

size_t mfma_conv_partial_bytes(const MfmaConvArgs& a) {
  if (mfma_conv_wide_applies(a) || mfma_conv_split_applies(a)) return 0;
  const GatherPlan p = gather_plan(a);
  if (a.cred == kChunk || p.ksplit == 1) return 0;
  return align_up((size_t)p.ksplit * a.n * a.od * a.oh * a.ow * a.cout * sizeof(float), 256);
}

MfmaConvGeometry mfma_conv_gather_geometry(const MfmaConvArgs& a) {
  if (mfma_conv_wide_applies(a)) return mfma_conv_wide_geometry(a);
  if (mfma_conv_split_applies(a)) return mfma_conv_split_geometry(a);
  const GatherPlan p = gather_plan(a);
  const int* t = kTileDims[p.shape / 3][p.shape % 3];
  return MfmaConvGeometry{kKernelBrick, t[0] * t[1] * t[2], p.nsub, p.ksplit};
}

int mfma_conv_gather_gn_records(const MfmaConvArgs& a, int groups) {
  if (mfma_conv_wide_applies(a)) return mfma_conv_wide_gn_records(a, groups);
  if (mfma_conv_split_applies(a)) return mfma_conv_split_gn_records(a, groups);
  return gather_gn_records(a, gather_plan(a), groups);
}

int mfma_conv_gather(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y,
                     void* partial, hipStream_t st, const GnPartialOut* gn, const ChannelPair* in2, const ChannelPair* out2) {
  if (mfma_conv_wide_applies(a)) {
    if (out2 != nullptr) return fail(SFH_ERR_UNSUPPORTED, "conv wide: the output cannot be a pair of tensors");
    return mfma_conv_wide(a, dtype, x, packed, bias, y, st, gn, in2);
  }
  if (mfma_conv_split_applies(a)) return mfma_conv_split(a, dtype, x, packed, bias, y, st, gn, in2, out2);
  if (dtype == SFH_BF16) return launch_typed<bf16_t>(a, dtype, x, packed, bias, y, partial, st, gn, in2, out2);
  return launch_typed<fp16_t>(a, dtype, x, packed, bias, y, partial, st, gn, in2, out2);
}

bool mfma_conv_gather_pair_ok(const MfmaConvArgs& a, int first, bool as_output) {
  if (mfma_conv_wide_applies(a)) return !as_output && mfma_conv_wide_pair_ok(a, first);
  if (mfma_conv_split_applies(a)) return mfma_conv_split_pair_ok(a, first, as_output);
  return gather_pair_ok(a, first, as_output);
}

}  // namespace sfh
