// MFMA implicit-GEMM convolution for the small volumes of a deep network level (3x3x3, stride 1, bf16 / fp16, 64 or
// more reduction channels): forward and data gradient (GEMM view as triton_conv3d/gather_gemm.py:112-341: M = output
// voxels, N = produced channels, K = taps x reduction channels).
//
// A level of 16 x 32 x 32 voxels or fewer has too few 256-voxel bricks to give every CU a workgroup unless the
// reduction is cut into slices, and slices that meet in memory cost fp32 partial tiles written and read plus a launch
// of their own. Here the reduction is cut INSIDE the workgroup:
//
//   * A workgroup owns a brick of only 2 x 4 x 8 = 64 output voxels and 64 produced channels -- four 32-voxel x
//     32-channel accumulator blocks -- so even a level of 2048 voxels has 32 x Cout/64 of them.
//   * Its four wavefronts split the REDUCTION, not the voxels: a round stages the halo bricks of R 32-channel chunks
//     (R = 4, or 2 when there are only two) side by side in LDS, and every wavefront runs all four accumulator blocks
//     over its own share -- one chunk each, or half a chunk's k-steps each when R = 2. A weight fragment then feeds
//     four MFMAs (two in the brick kernel at this size), every fragment of the workgroup is fetched by exactly one
//     wavefront (the brick kernel's four wavefronts fetch the same ones), and the chunks of a round are staged with
//     one trip to memory instead of one per chunk.
//   * At the end the wavefronts' partial accumulators meet in LDS: wavefront u collects block u from the other three
//     in wavefront order (a fixed order: the same bits on every run), adds the bias, rounds once, leaves the GroupNorm
//     records of what it stores (gn_stats.hpp) and writes 16-byte pieces.
//
// LDS layout per chunk as in conv_mfma.hip (four 16-byte channel planes, 64 bytes mod 256 apart); chunk slots are a
// further 16 bytes apart so that the staging writes of one voxel's pieces fall into different banks.
// The data gradient runs this kernel with the weight packed transposed and tap-flipped and padding k-1-p
// (triton_conv3d/bwd_data.py:344-363). Launch geometry is a pure function of the shape.
#include "conv_mfma.hpp"
#include "mma.hpp"
#include "gn_stats.hpp"

namespace sfh {
namespace {

constexpr int kChunk = 32;
constexpr int TD = 2, TH = 4, TW = 8;  // output brick: two planes of 4 x 8 voxels, each one MFMA column block
constexpr int BD = TD + 2, BH = TH + 2, BW = TW + 2;
constexpr int BV = BD * BH * BW;  // 240 brick voxels with the halo
constexpr int PLANE = ((BV * 16 - 64 + 255) / 256) * 256 + 64;  // >= BV * 16, 64 modulo 256
constexpr int SLOT = 4 * PLANE + 16;                            // one chunk's brick
constexpr int MS = 2, NSUB = 2;                                 // accumulator blocks: voxel halves x channel halves
constexpr int TAPS = 27, NIT = TAPS * 2, FRAG = 512;
constexpr int RED_BYTES = 4 * 3 * 4096;  // every block from the three wavefronts that do not own it
static_assert(PLANE % 256 == 64 && PLANE >= BV * 16, "plane stride");

// LDS byte offset of (tap, k-step) relative to a lane's voxel at tap (0, 0, 0)
constexpr int tap_off(int tap) { return (((tap / 9) * BH + (tap / 3) % 3) * BW + tap % 3) * 16; }

// R: chunks per round. PAIR: the input is two tensors whose channels follow each other (the first `c_first` in x, the
// rest in x1). Independently, a non-null y1 splits the OUTPUT the same way.
template <typename T, int R, bool PAIR>
__global__ void __launch_bounds__(256, 2)
conv_split_kernel(MfmaConvArgs a, const T* __restrict__ x, const T* __restrict__ wp, const T* __restrict__ bias, T* __restrict__ y,
                  int tiles_d, int tiles_h, int tiles_w, int nblocks, uint32_t total, GnPartialOut gn, const T* __restrict__ x1,
                  T* __restrict__ y1, int c_first) {
  constexpr int LDS = R * SLOT > RED_BYTES ? R * SLOT : RED_BYTES;
  __shared__ __attribute__((aligned(16))) char lds[LDS];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int j = lane & 31, kg = lane >> 5;

  uint32_t t = xcd_remap(blockIdx.x, total);
  const int nb = t % nblocks; t /= nblocks;
  const int tw_i = t % tiles_w; t /= tiles_w;
  const int th_i = t % tiles_h; t /= tiles_h;
  const int td_i = t % tiles_d;
  const int n = t / tiles_d;
  const int od0 = td_i * TD, oh0 = th_i * TH, ow0 = tw_i * TW;

  // This wavefront's share of a round: chunk slot `slot`; with R = 2 also one of the two k-steps of every tap.
  const int slot = R == 4 ? wave : wave >> 1;
  const int khalf = R == 4 ? 0 : wave & 1;
  constexpr int NITS = R == 4 ? NIT : TAPS;  // iterations of a wavefront per round
  constexpr int WSTEP = R == 4 ? FRAG : 2 * FRAG;
  int abase[MS];  // LDS byte address of the lane's voxel of block row ms at tap (0, 0, 0), in its k-half plane
#pragma unroll
  for (int ms = 0; ms < MS; ++ms) {
    const int tw = j % TW, th = j / TW;
    abase[ms] = slot * SLOT + (kg + 2 * khalf) * PLANE + ((ms * BH + th) * BW + tw) * 16;
  }
  auto a_off = [](int k) constexpr { return R == 4 ? tap_off(k / 2) + (k % 2) * 2 * PLANE : tap_off(k); };

  f32x16_t acc[MS][NSUB];
#pragma unroll
  for (int ms = 0; ms < MS; ++ms)
#pragma unroll
    for (int ns = 0; ns < NSUB; ++ns)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ms][ns][r] = 0.f;

  const int ncc = a.cred / kChunk;
  const int id0 = od0 - a.pd, ih0 = oh0 - a.ph, iw0 = ow0 - a.pw;
  constexpr int PIECES = BV * 4 * R;
  constexpr int ITERS = (PIECES + 255) / 256;
  constexpr int WDEPTH = 8;  // weight fragments (per output block) in flight per wavefront
  const int64_t wns = (int64_t)ncc * (NIT * FRAG);  // next 32-channel output block

  for (int c0 = 0; c0 < ncc; c0 += R) {
    // The wavefront's first weight fragments are requested before the bricks are staged: they depend on nothing in LDS.
    const T* wcc = wp + ((int64_t)(nb * NSUB) * ncc + c0 + slot) * (NIT * FRAG) + khalf * FRAG + lane * 8;
    uint4 wq[NITS][NSUB];  // fully unrolled: every slot is its own register set, live for WDEPTH iterations
#pragma unroll
    for (int k = 0; k < WDEPTH; ++k)
#pragma unroll
      for (int ns = 0; ns < NSUB; ++ns) wq[k][ns] = *reinterpret_cast<const uint4*>(wcc + ns * wns + k * WSTEP);
    __syncthreads();  // every wavefront is done reading the previous round
    {
      // A voxel's 4 R pieces (R chunks of 4) are consecutive threads: 64 R contiguous bytes when the chunks lie in one tensor.
      uint4 v[ITERS];
#pragma unroll
      for (int u = 0; u < ITERS; ++u) {
        const int p = u * 256 + tid;
        const int q = p % (4 * R), vox = p / (4 * R);
        const int cc = c0 + (q >> 2), piece = q & 3;
        const int bw = vox % BW, bh = (vox / BW) % BH, bd = vox / (BW * BH);
        const int id = id0 + bd, ih = ih0 + bh, iw = iw0 + bw;
        const bool in = p < PIECES && (unsigned)id < (unsigned)a.id && (unsigned)ih < (unsigned)a.ih && (unsigned)iw < (unsigned)a.iw;
        int row = a.cred, ch = cc * kChunk;
        const T* xb = x;
        if constexpr (PAIR) {
          const bool second = ch >= c_first;
          row = second ? a.cred - c_first : c_first;
          xb = second ? x1 : x;
          ch = second ? ch - c_first : ch;
        }
        v[u] = make_uint4(0, 0, 0, 0);
        if (in) v[u] = *reinterpret_cast<const uint4*>(xb + ((((int64_t)n * a.id + id) * a.ih + ih) * a.iw + iw) * row + ch + piece * 8);
      }
#pragma unroll
      for (int u = 0; u < ITERS; ++u) {
        const int p = u * 256 + tid;
        const int q = p % (4 * R), vox = p / (4 * R);
        if (p < PIECES) *reinterpret_cast<uint4*>(lds + (q >> 2) * SLOT + (q & 3) * PLANE + vox * 16) = v[u];
      }
    }
    __syncthreads();

    // Software pipeline over the wavefront's iterations: the weight fragments of iteration k + WDEPTH and the
    // activation fragments of iteration k + 1 are requested between the MFMAs of iteration k, one behind each.
    uint4 aq[2][MS];
#pragma unroll
    for (int ms = 0; ms < MS; ++ms) aq[0][ms] = *reinterpret_cast<const uint4*>(lds + abase[ms] + a_off(0));
#pragma unroll
    for (int k = 0; k < NITS; ++k) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < MS * NSUB; ++m) {
        const int ms = m / NSUB, ns = m % NSUB;
        acc[ms][ns] = Mma32<T>::run(wq[k][ns], aq[k & 1][ms], acc[ms][ns]);
        __builtin_amdgcn_sched_barrier(0);
        if (m < NSUB) {
          if (k + WDEPTH < NITS) wq[k + WDEPTH][m] = *reinterpret_cast<const uint4*>(wcc + m * wns + (k + WDEPTH) * WSTEP);
        } else {
          if (k + 1 < NITS) aq[(k + 1) & 1][m - NSUB] = *reinterpret_cast<const uint4*>(lds + abase[m - NSUB] + a_off(k + 1));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // The four partial results of every block meet in LDS: wavefront u collects block u = ms * NSUB + ns.
  __syncthreads();  // the bricks are not read any more
  float4* red = reinterpret_cast<float4*>(lds);
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    if (u != wave) {
      const int from = wave < u ? wave : wave - 1;  // this wavefront's place among block u's three senders
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4)
        red[((u * 3 + from) * 4 + r4) * 64 + lane] =
            make_float4(acc[u / NSUB][u % NSUB][4 * r4], acc[u / NSUB][u % NSUB][4 * r4 + 1], acc[u / NSUB][u % NSUB][4 * r4 + 2],
                        acc[u / NSUB][u % NSUB][4 * r4 + 3]);
    }
  }
  __syncthreads();
  f32x16_t tot;
#pragma unroll
  for (int r = 0; r < 16; ++r) tot[r] = 0.f;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    if (u == wave) {
      // wavefronts 0, 1, 2, 3 in that order, this one's own share from its registers
#pragma unroll
      for (int src = 0; src < 4; ++src) {
        f32x16_t part;
        if (src == u) {
          part = acc[u / NSUB][u % NSUB];
        } else {
          const int from = src < u ? src : src - 1;
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const float4 e = red[((u * 3 + from) * 4 + r4) * 64 + lane];
            part[4 * r4] = e.x; part[4 * r4 + 1] = e.y; part[4 * r4 + 2] = e.z; part[4 * r4 + 3] = e.w;
          }
        }
        if (src == 0) tot = part;
        else
#pragma unroll
          for (int r = 0; r < 16; ++r) tot[r] += part[r];
      }
    }
  }

  // Epilogue of block (ms, ns) = (wave / NSUB, wave % NSUB). Accumulator register r of a lane is output channel
  // 8 * (r / 4) + 4 * kg + r % 4 of voxel j of the block row; the two lanes of a voxel trade runs so that each stores
  // two 16-byte pieces.
  const int ms_o = wave / NSUB, ns_o = wave % NSUB;
  const int tw = j % TW, th = j / TW;
  const int od = od0 + ms_o, oh = oh0 + th, ow = ow0 + tw;
  const bool inside = od < a.od && oh < a.oh && ow < a.ow;
  const int64_t vox = (((int64_t)n * a.od + od) * a.oh + oh) * a.ow + ow;
  const int ch = (nb * NSUB + ns_o) * 32;
  T* yp = y + vox * a.cout + ch;
  if (y1 != nullptr) yp = ch >= c_first ? y1 + vox * (a.cout - c_first) + (ch - c_first) : y + vox * c_first + ch;
  uint32_t run[4][2];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
    if (bias != nullptr) {
      const T* bp = bias + ch + 8 * g + 4 * kg;
      b0 = to_float(bp[0]); b1 = to_float(bp[1]); b2 = to_float(bp[2]); b3 = to_float(bp[3]);
    }
    run[g][0] = Mma32<T>::pack2(tot[4 * g] + b0, tot[4 * g + 1] + b1);
    run[g][1] = Mma32<T>::pack2(tot[4 * g + 2] + b2, tot[4 * g + 3] + b3);
  }
  RunSums mine;
  mine.clear();
  if (gn.part != nullptr) mine.template add<T>(run, inside, true);
  uint4 piece[2];
  trade_channel_runs(run, piece);  // all lanes take part, also those of voxels past the edge
  if (inside) {
    *reinterpret_cast<uint4*>(yp + 8 * kg) = piece[0];
    *reinterpret_cast<uint4*>(yp + 16 + 8 * kg) = piece[1];
  }
  if (gn.part != nullptr) {
    // this wavefront's sums belong to channel block ns_o; for the other block it counts nothing
    RunSums rs[NSUB];
#pragma unroll
    for (int ns = 0; ns < NSUB; ++ns) {
      const bool own = ns == ns_o;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        rs[ns].s1[g] = own ? mine.s1[g] : 0.f;
        rs[ns].s2[g] = own ? mine.s2[g] : 0.f;
        rs[ns].k[g] = mine.k[g];
      }
      rs[ns].cnt = own ? mine.cnt : 0.f;
    }
    __syncthreads();  // every wavefront has collected its block: the LDS is free
    constexpr int SPAN = 32 * NSUB;
    const int per_tile = gn.cg > SPAN ? gn.cg / SPAN : 1;  // workgroups that share a group of this tile
    const int tile = (td_i * tiles_h + th_i) * tiles_w + tw_i;
    write_group_partials<4, NSUB>(rs, reinterpret_cast<float*>(lds), gn, n, tile * per_tile + nb % per_tile, nb * SPAN, tid);
  }
}

int64_t split_tiles(const MfmaConvArgs& a) { return (int64_t)a.n * cdiv(a.od, TD) * cdiv(a.oh, TH) * cdiv(a.ow, TW); }

template <typename T, int R, bool PAIR>
int launch_split(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                 const GnPartialOut& gn, const void* x1, void* y1, int first) {
  const int tiles_d = (int)cdiv(a.od, TD), tiles_h = (int)cdiv(a.oh, TH), tiles_w = (int)cdiv(a.ow, TW);
  const int nblocks = a.cout / (32 * NSUB);
  const int64_t total = split_tiles(a) * nblocks;
  if (total == 0) return SFH_OK;
  if (total > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "conv split: %lld workgroups exceed the grid limit", (long long)total);
  hipLaunchKernelGGL((conv_split_kernel<T, R, PAIR>), dim3((unsigned)total), dim3(256), 0, st, a, (const T*)x, (const T*)packed,
                     (const T*)bias, (T*)y, tiles_d, tiles_h, tiles_w, nblocks, (uint32_t)total, gn, (const T*)x1, (T*)y1, first);
  return check_launch("conv_split_kernel");
}

template <typename T>
int launch_split_typed(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                       const GnPartialOut& gn, const void* x1, void* y1, int first) {
  const bool four = (a.cred / kChunk) % 4 == 0;
  if (x1 != nullptr)
    return four ? launch_split<T, 4, true>(a, x, packed, bias, y, st, gn, x1, y1, first)
                : launch_split<T, 2, true>(a, x, packed, bias, y, st, gn, x1, y1, first);
  return four ? launch_split<T, 4, false>(a, x, packed, bias, y, st, gn, x1, y1, first)
              : launch_split<T, 2, false>(a, x, packed, bias, y, st, gn, x1, y1, first);
}

}  // namespace

// Serves 64 or more reduction channels in an even number of 32-channel chunks and produced channels in blocks of 64, on
// planes of at most 32 x 32 voxels whose bricks times block pairs number 24 or more per two planes. Measured against the
// brick kernel on every convolution of a five-level U-Net step: 10-25 % faster at 16 x 32 x 32 and 8 x 16 x 16, where the
// brick kernel runs as one round of workgroups or needs slices; slower on 32 x 64 x 64 (several rounds of bricks overlap
// staging and MFMAs by themselves, and 64-voxel bricks stage 3.75 voxels per output voxel) and at 4 x 8 x 8 (a handful
// of workgroups cannot pull 7-14 MiB of weights fast enough: that level needs the slices over many CUs). For the same
// reason it leaves reductions of 512 channels or more to the slices where its workgroups would number 32 or fewer per
// two planes (8 x 16 x 16 with 256 produced channels: 128 workgroups of 1.7 MiB of weights each, 41 us against 30 with
// the weights cold; eight wavefronts per workgroup instead of four changed nothing, which is how the bound was found).
// The rule does not look at the depth: the data gradient of a depth shard's slab (D + 2 planes) and of the padded volume
// (D planes) must come from the same kernel, or a shard and the whole volume would disagree in the last bit.
constexpr int kSplitMaxPlane = 32 * 32, kSplitMinPerDepth = 24, kSplitFewPerDepth = 32, kSplitFewMaxChunks = 16;

bool mfma_conv_split_applies(const MfmaConvArgs& a) {
  if (a.kd != 3 || a.kh != 3 || a.kw != 3) return false;
  if (a.cred < 2 * kChunk || a.cred % (2 * kChunk) != 0 || a.cout % (32 * NSUB) != 0) return false;
  if ((int64_t)a.oh * a.ow > kSplitMaxPlane) return false;
  const int64_t per_depth = (int64_t)a.n * cdiv(a.oh, TH) * cdiv(a.ow, TW) * (a.cout / (32 * NSUB));
  if (per_depth <= kSplitFewPerDepth && a.cred / kChunk >= kSplitFewMaxChunks) return false;
  return per_depth >= kSplitMinPerDepth;
}

MfmaConvGeometry mfma_conv_split_geometry(const MfmaConvArgs&) { return MfmaConvGeometry{kKernelSplit, TD * TH * TW, NSUB, 1}; }

int mfma_conv_split_gn_records(const MfmaConvArgs& a, int groups) {
  const int span = 32 * NSUB;
  if (!gn_partials_fit(a.cout, groups, span)) return 0;
  const int cg = a.cout / groups;
  const int64_t records = split_tiles(a) / a.n * (cg > span ? cg / span : 1);
  return records <= 0x7fffffff ? (int)records : 0;
}

bool mfma_conv_split_pair_ok(const MfmaConvArgs& a, int first, bool as_output) {
  const int channels = as_output ? a.cout : a.cred;
  return first > 0 && first < channels && first % 32 == 0;
}

int mfma_conv_split(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                    const GnPartialOut* gn, const ChannelPair* in2, const ChannelPair* out2) {
  if (in2 != nullptr && out2 != nullptr) return fail(SFH_ERR_UNSUPPORTED, "conv split: input and output cannot both be pairs");
  if (out2 != nullptr && gn != nullptr && gn->part != nullptr)
    return fail(SFH_ERR_UNSUPPORTED, "conv split: no GroupNorm partials of an output written as two tensors");
  if (in2 != nullptr && (in2->second == nullptr || !mfma_conv_split_pair_ok(a, in2->first, false)))
    return fail(SFH_ERR_UNSUPPORTED, "conv split: the input cannot be cut at channel %d of %d", in2->first, a.cred);
  if (out2 != nullptr && (out2->second == nullptr || !mfma_conv_split_pair_ok(a, out2->first, true)))
    return fail(SFH_ERR_UNSUPPORTED, "conv split: the output cannot be cut at channel %d of %d", out2->first, a.cout);
  GnPartialOut out{nullptr, 0, 0, 0};
  if (gn != nullptr && gn->part != nullptr) {
    if (gn->records != mfma_conv_split_gn_records(a, gn->groups) || gn->records == 0)
      return fail(SFH_ERR_INVALID, "conv split: GroupNorm partials asked for %d records, this launch leaves %d", gn->records,
                  mfma_conv_split_gn_records(a, gn->groups));
    out = *gn;
    out.cg = a.cout / gn->groups;
  }
  const void* x1 = in2 != nullptr ? in2->second : nullptr;
  void* y1 = out2 != nullptr ? out2->second : nullptr;
  const int first = in2 != nullptr ? in2->first : (out2 != nullptr ? out2->first : 0);
  if (dtype == SFH_BF16) return launch_split_typed<bf16_t>(a, x, packed, bias, y, st, out, x1, y1, first);
  return launch_split_typed<fp16_t>(a, x, packed, bias, y, st, out, x1, y1, first);
}

}  // namespace sfh
