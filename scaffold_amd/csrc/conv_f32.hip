// Tiled fp32 convolution on the fp32 matrix pipe of gfx950 (3x3x3, stride 1, dilation 1): forward and data gradient.
//
// The reference runs its fp32 convolutions through the same tiled kernel as the 16-bit ones with the dot product at
// full IEEE fp32 precision (triton_conv3d/gather_gemm.py:1334, input_precision="ieee"). Here that is
// v_mfma_f32_32x32x2_f32: fp32 operands, fp32 products, fp32 accumulation -- no down-conversion anywhere, so the
// 1e-5 bar of the fp32 configuration holds; dense fp32 MFMA peak is 157.3 TFLOP/s.
//
// GEMM view (gather_gemm.py:112-341): M = output voxels, N = produced channels, K = taps x reduction channels.
//   * A workgroup owns a TD x TH x 32 brick of output voxels and one block of 32 produced channels; the input brick
//     with its halo is staged in LDS per chunk of 16 reduction channels as four 16-byte channel planes (plane p =
//     channels 4p .. 4p+3 of every brick voxel; planes 64 bytes apart modulo 256, so a wavefront's ds_read_b128 of 32
//     consecutive voxels is conflict free and every tap is an immediate offset).
//   * One MFMA contracts 2 reduction channels: k-slot kg (= lane / 32) at step kk of a chunk is channel 8 kg + kk, so a
//     lane's operands of the 8 steps of a tap are 8 consecutive channels: two 16-byte LDS reads of activations and two
//     16-byte global loads of the weight, which is repacked once per call into that order
//       packed[cout/32][cred/16][tap][q(2)][lane(64)][4],  lane = cout % 32 + 32 kg,  channel = 16 cc + 8 kg + 4 q + e.
//   * The weight is the ROW operand, so a lane ends up with four runs of four consecutive output channels of one voxel
//     and stores 16-byte pieces.
// The data gradient runs this kernel with the weight packed transposed and tap-flipped and padding k-1-p
// (triton_conv3d/bwd_data.py:344-363).
#include "conv_f32.hpp"
#include "reduce.hpp"

namespace sfh {
namespace {

typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kChunk = 16;  // reduction channels staged per pass (4 planes of 4)
constexpr int kTaps = 27;

constexpr int plane_bytes(int voxels) {  // smallest size >= voxels*16 that is 64 modulo 256
  return ((voxels * 16 - 64 + 255) / 256) * 256 + 64;
}

template <int TD_, int TH_>
struct FTile {
  static constexpr int TD = TD_, TH = TH_, TW = 32;
  static constexpr int BD = TD + 2, BH = TH + 2, BW = TW + 2;
  static constexpr int BV = BD * BH * BW;
  static constexpr int PLANE = plane_bytes(BV);
  static constexpr int LDS = 4 * PLANE;
  static constexpr int MS = TD * TH * TW / 128;  // 32-voxel sub-tiles per wavefront
  static_assert(TD * TH * TW % 128 == 0, "tile must split into 4 wavefronts of 32-voxel sub-tiles");
  static_assert(2 * LDS <= 160 * 1024, "two workgroups in the 160 KB LDS of a CU");
  static_assert(PLANE + (2 * BH * BW + 2 * BW + 2) * 16 < 65536, "ds_read immediate range");
};

template <typename C>
__device__ __forceinline__ constexpr int tap_off(int tap) {
  const int kd = tap / 9, kh = (tap / 3) % 3, kw = tap % 3;
  return ((kd * C::BH + kh) * C::BW + kw) * 16;
}

template <typename C>
__global__ void __launch_bounds__(256, 2)
conv_f32_kernel(MfmaConvArgs a, const float* __restrict__ x, const float* __restrict__ wp, const float* __restrict__ bias,
                float* __restrict__ y, int tiles_d, int tiles_h, int tiles_w, int nblocks, uint32_t total) {
  __shared__ __attribute__((aligned(16))) char lds[C::LDS];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int j = lane & 31, kg = lane >> 5;

  uint32_t t = xcd_remap(blockIdx.x, total);
  const int nb = t % nblocks; t /= nblocks;
  const int tw_i = t % tiles_w; t /= tiles_w;
  const int th_i = t % tiles_h; t /= tiles_h;
  const int td_i = t % tiles_d;
  const int n = t / tiles_d;
  const int od0 = td_i * C::TD, oh0 = th_i * C::TH, ow0 = tw_i * C::TW;
  const int id0 = od0 - a.pd, ih0 = oh0 - a.ph, iw0 = ow0 - a.pw;

  // LDS byte offset of the sub-tile voxel at tap (0,0,0) in the lane's first plane (planes 2 kg and 2 kg + 1 are its)
  int lbase[C::MS];
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) {
    const int v = (wave * C::MS + ms) * 32 + j;
    const int tw = v % C::TW, th = (v / C::TW) % C::TH, td = v / (C::TW * C::TH);
    lbase[ms] = 2 * kg * C::PLANE + ((td * C::BH + th) * C::BW + tw) * 16;
  }
  f32x16_t acc[C::MS];
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[ms][r] = 0.f;

  const int ncc = a.cred / kChunk;
  constexpr int PIECES = C::BV * 4;
  constexpr int ITERS = (PIECES + 255) / 256;
  constexpr int BATCH = 8;  // staging loads in flight before the first LDS write
  const float* xn = x + (int64_t)n * a.id * a.ih * a.iw * a.cred;
  for (int cc = 0; cc < ncc; ++cc) {
    __syncthreads();  // every wave is done reading the previous chunk
#pragma unroll
    for (int it0 = 0; it0 < ITERS; it0 += BATCH) {
      float4 v[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        if (it0 + u < ITERS) {
          // unconditional load from a clamped address, masked afterwards (a load under a branch waits for the one before)
          const int p = (it0 + u) * 256 + tid;
          const int vox = p >> 2, piece = p & 3;
          const int bw = vox % C::BW, bh = (vox / C::BW) % C::BH, bd = vox / (C::BW * C::BH);
          const int id = id0 + bd, ih = ih0 + bh, iw = iw0 + bw;
          const bool in = p < PIECES && (unsigned)id < (unsigned)a.id && (unsigned)ih < (unsigned)a.ih && (unsigned)iw < (unsigned)a.iw;
          const int64_t at = in ? (((int64_t)id * a.ih + ih) * a.iw + iw) * a.cred + cc * kChunk + piece * 4 : 0;
          const float4 got = *reinterpret_cast<const float4*>(xn + at);
          v[u] = in ? got : make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
#pragma unroll
      for (int u = 0; u < BATCH; ++u) {
        if (it0 + u < ITERS) {
          const int p = (it0 + u) * 256 + tid;
          if (p < PIECES) *reinterpret_cast<float4*>(lds + (p & 3) * C::PLANE + (p >> 2) * 16) = v[u];
        }
      }
    }
    __syncthreads();

    // weight fragments of tap t: packed + (((nb * ncc + cc) * 27 + t) * 2 + q) * 256 floats + lane * 4
    const float* wcc = wp + ((int64_t)(nb * ncc + cc) * kTaps * 2) * 256 + lane * 4;
    constexpr int WDEPTH = 3;  // taps requested ahead
    float4 wq[WDEPTH][2];
#pragma unroll
    for (int d = 0; d < WDEPTH; ++d)
#pragma unroll
      for (int q = 0; q < 2; ++q) wq[d][q] = *reinterpret_cast<const float4*>(wcc + (d * 2 + q) * 256);
#pragma unroll
    for (int tap = 0; tap < kTaps; ++tap) {
      float4 wf[2] = {wq[tap % WDEPTH][0], wq[tap % WDEPTH][1]};
      if (tap + WDEPTH < kTaps) {
#pragma unroll
        for (int q = 0; q < 2; ++q) wq[tap % WDEPTH][q] = *reinterpret_cast<const float4*>(wcc + ((tap + WDEPTH) * 2 + q) * 256);
      }
      // the sub-tiles take turns, so consecutive MFMAs do not wait for one another's result
      float4 af[C::MS][2];
#pragma unroll
      for (int ms = 0; ms < C::MS; ++ms) {
        af[ms][0] = *reinterpret_cast<const float4*>(lds + lbase[ms] + tap_off<C>(tap));
        af[ms][1] = *reinterpret_cast<const float4*>(lds + lbase[ms] + C::PLANE + tap_off<C>(tap));
      }
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const float wv[4] = {wf[q].x, wf[q].y, wf[q].z, wf[q].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#pragma unroll
          for (int ms = 0; ms < C::MS; ++ms) {
            const float av[4] = {af[ms][q].x, af[ms][q].y, af[ms][q].z, af[ms][q].w};
            acc[ms] = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[e], av[e], acc[ms], 0, 0, 0);
          }
        }
      }
    }
  }

  // Accumulator register r of a lane is output channel 8 * (r / 4) + 4 * kg + r % 4 of the sub-tile's voxel j.
#pragma unroll
  for (int ms = 0; ms < C::MS; ++ms) {
    const int v = (wave * C::MS + ms) * 32 + j;
    const int tw = v % C::TW, th = (v / C::TW) % C::TH, td = v / (C::TW * C::TH);
    const int od = od0 + td, oh = oh0 + th, ow = ow0 + tw;
    if (od >= a.od || oh >= a.oh || ow >= a.ow) continue;
    float* yp = y + ((((int64_t)n * a.od + od) * a.oh + oh) * a.ow + ow) * a.cout + nb * 32;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int co = 8 * g + 4 * kg;
      float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
      if (bias != nullptr) b = *reinterpret_cast<const float4*>(bias + nb * 32 + co);
      *reinterpret_cast<float4*>(yp + co) =
          make_float4(acc[ms][4 * g] + b.x, acc[ms][4 * g + 1] + b.y, acc[ms][4 * g + 2] + b.z, acc[ms][4 * g + 3] + b.w);
    }
  }
}

// One thread per packed 16-byte piece: the 4 consecutive reduction channels of one (output channel, tap, k-slot, q).
__global__ void __launch_bounds__(256)
pack_f32_kernel(const float* __restrict__ w, float* __restrict__ packed, int cred, int taps_kh_kw, int kw, int flip, int64_t s_out,
                int64_t s_red, int64_t s_kd, int64_t s_kh, int64_t s_kw, int64_t pieces) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= pieces) return;
  int64_t r = idx;
  const int lane = (int)(r % 64); r /= 64;
  const int q = (int)(r % 2); r /= 2;
  int tap = (int)(r % kTaps); r /= kTaps;
  const int ncc = cred / kChunk;
  const int cc = (int)(r % ncc);
  const int nblk = (int)(r / ncc);
  const int co = nblk * 32 + (lane & 31);
  const int ci = cc * kChunk + (lane >> 5) * 8 + q * 4;
  if (flip) tap = kTaps - 1 - tap;
  const int tkw = tap % kw, tkh = (tap / kw) % (taps_kh_kw / kw), tkd = tap / taps_kh_kw;
  const float* src = w + co * s_out + ci * s_red + tkd * s_kd + tkh * s_kh + tkw * s_kw;
  *reinterpret_cast<float4*>(packed + idx * 4) = make_float4(src[0], src[s_red], src[2 * s_red], src[3 * s_red]);
}

template <typename C>
int launch(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st) {
  const int tiles_d = (int)cdiv(a.od, C::TD), tiles_h = (int)cdiv(a.oh, C::TH), tiles_w = (int)cdiv(a.ow, C::TW);
  const int nblocks = a.cout / 32;
  const int64_t total = (int64_t)a.n * tiles_d * tiles_h * tiles_w * nblocks;
  if (total == 0) return SFH_OK;
  if (total > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "conv fp32: %lld workgroups exceed the grid limit", (long long)total);
  hipLaunchKernelGGL((conv_f32_kernel<C>), dim3((unsigned)total), dim3(256), 0, st, a, (const float*)x, (const float*)packed,
                     (const float*)bias, (float*)y, tiles_d, tiles_h, tiles_w, nblocks, (uint32_t)total);
  return check_launch("conv_f32_kernel");
}

// ---- weight gradient ---------------------------------------------------------------------------------------------
//   gw[co][tap][ci] = sum over output voxels v of gy[v][co] * x[v + tap - pad][ci]
// GEMM view (triton_conv3d/reduce_gemm.py:137-393): M = Cout, N = 27 x Cin, K = output voxels. One fp32 MFMA contracts
// TWO voxels and a lane supplies ONE value per operand: row operand gy[voxel 2s + kg][co = lane % 32], column operand
// x[that voxel + tap][ci = lane % 32] -- both are 32 consecutive floats of a channels-last row, so unlike the 16-bit
// kernel nothing has to be transposed and the operands come straight from global memory (L1 / L2 serve the 27-fold
// reuse of x). A workgroup owns one (32 co, 32 ci) block and a contiguous range of output rows; its four wavefronts
// split the 27 taps 7 / 7 / 7 / 6. Split-K over the rows: fp32 partial slices [Cout][27][Cin] at fixed workspace slots,
// summed in fixed order afterwards (reduce_gemm.py:396-435) -- no float atomics, split count a pure function of shape.
constexpr int kPairsPerPass = 4;  // voxel pairs whose loads are issued before the first MFMA of a pass

__global__ void __launch_bounds__(256, 2)
wgrad_f32_kernel(WgradArgs a, const float* __restrict__ x, const float* __restrict__ gy, float* __restrict__ partial, int nsplit, int cibs) {
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int i = lane & 31, kg = lane >> 5;
  int b = blockIdx.x;
  const int split = b % nsplit; b /= nsplit;
  const int cib = b % cibs, cob = b / cibs;
  const int64_t rows = (int64_t)a.n * a.od * a.oh;
  const int64_t r_begin = split * rows / nsplit, r_end = (split + 1) * rows / nsplit;
  const int ntaps = wave < 3 ? 7 : 6;
  const int tap0 = wave * 7;

  f32x16_t acc[7];
#pragma unroll
  for (int t = 0; t < 7; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;

  const float* gyb = gy + cob * 32 + i;
  const float* xb = x + cib * 32 + i;
  for (int64_t row = r_begin; row < r_end; ++row) {
    const int oh = (int)(row % a.oh);
    const int od = (int)((row / a.oh) % a.od);
    const int n = (int)(row / ((int64_t)a.oh * a.od));
    const float* gyr = gyb + row * a.ow * a.cout;
    // per tap of this wavefront: pointer to x at (n, od + kd - pd, oh + kh - ph, kw - pw) or null when that input row is padding
    const float* xr[7];
#pragma unroll
    for (int t = 0; t < 7; ++t) {
      const int tap = tap0 + t;
      const int kd = tap / 9, kh = (tap / 3) % 3, kw = tap % 3;
      const int id = od + kd - a.pd, ih = oh + kh - a.ph;
      const bool ok = t < ntaps && (unsigned)id < (unsigned)a.id && (unsigned)ih < (unsigned)a.ih;
      xr[t] = ok ? xb + ((((int64_t)n * a.id + id) * a.ih + ih) * a.iw + (kw - a.pw)) * a.cin : nullptr;
    }
    for (int w0 = 0; w0 < a.ow; w0 += 2 * kPairsPerPass) {
      float av[kPairsPerPass], bv[kPairsPerPass][7];
#pragma unroll
      for (int u = 0; u < kPairsPerPass; ++u) {
        const int w = w0 + 2 * u + kg;  // this lane's voxel of pair u
        const bool wok = w < a.ow;
        av[u] = wok ? gyr[(int64_t)w * a.cout] : 0.f;
#pragma unroll
        for (int t = 0; t < 7; ++t) {
          const int kw = (tap0 + t) % 3;
          const int iw = w + kw - a.pw;
          const bool ok = wok && xr[t] != nullptr && (unsigned)iw < (unsigned)a.iw;
          bv[u][t] = ok ? xr[t][(int64_t)w * a.cin] : 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < kPairsPerPass; ++u)
#pragma unroll
        for (int t = 0; t < 7; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[u], bv[u][t], acc[t], 0, 0, 0);
    }
  }
  // result register r of a lane: column ci = lane % 32, row co = 8 * (r / 4) + 4 * kg + r % 4
  float* dst = partial + (int64_t)split * a.cout * kTaps * a.cin + ((int64_t)cob * 32 * kTaps) * a.cin + cib * 32 + i;
#pragma unroll
  for (int t = 0; t < 7; ++t) {
    if (t >= ntaps) break;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int co = 8 * (r / 4) + 4 * kg + (r % 4);
      dst[((int64_t)co * kTaps + tap0 + t) * a.cin] = acc[t][r];
    }
  }
}

}  // namespace

bool f32_conv_supported(const MfmaConvArgs& a) {
  if (a.kd != 3 || a.kh != 3 || a.kw != 3) return false;
  if (a.cred % kChunk != 0 || a.cout % 32 != 0) return false;
  if (a.pd < 0 || a.ph < 0 || a.pw < 0 || a.pd > 2 || a.ph > 2 || a.pw > 2) return false;
  if (a.n < 1 || a.od < 1 || a.oh < 1 || a.ow < 1) return false;
  return true;
}

size_t f32_conv_packed_weight_bytes(const MfmaConvArgs& a) { return align_up((size_t)a.cout * a.cred * kTaps * 4, 256); }

int f32_pack_weight(const MfmaConvArgs& a, const void* w, int64_t s_out, int64_t s_red, int64_t s_kd, int64_t s_kh, int64_t s_kw, int flip,
                    void* packed, hipStream_t st) {
  const int64_t pieces = (int64_t)a.cout * a.cred * kTaps / 4;
  if (pieces <= 0) return SFH_OK;
  hipLaunchKernelGGL(pack_f32_kernel, dim3((unsigned)cdiv(pieces, 256)), dim3(256), 0, st, (const float*)w, (float*)packed, a.cred,
                     a.kh * a.kw, a.kw, flip, s_out, s_red, s_kd, s_kh, s_kw, pieces);
  return check_launch("pack_f32_kernel");
}

int f32_conv(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st) {
  // Launch geometry, a pure function of the shape: 4 x 4 x 32 bricks when they fill the chip, else 2 x 2 x 32.
  const int64_t big = (int64_t)a.n * cdiv(a.od, 4) * cdiv(a.oh, 4) * cdiv(a.ow, 32) * (a.cout / 32);
  if (big >= kComputeUnits) return launch<FTile<4, 4>>(a, x, packed, bias, y, st);
  return launch<FTile<2, 2>>(a, x, packed, bias, y, st);
}

}  // namespace sfh

namespace sfh {

bool f32_wgrad_supported(const WgradArgs& a) {
  return a.cin % 32 == 0 && a.cout % 32 == 0 && a.n >= 1 && a.od >= 1 && a.oh >= 1 && a.ow >= 1 && a.pd >= 0 && a.ph >= 0 && a.pw >= 0;
}

int f32_wgrad_splits(const WgradArgs& a) {
  const int64_t rows = (int64_t)a.n * a.od * a.oh;
  const int64_t blocks = (int64_t)(a.cout / 32) * (a.cin / 32);
  int64_t s = 2 * kComputeUnits / blocks;  // two workgroups per CU
  if (s < 1) s = 1;
  if (s > rows) s = rows;
  return (int)s;
}

size_t f32_wgrad_workspace_bytes(const WgradArgs& a) {
  return align_up((size_t)f32_wgrad_splits(a) * a.cout * kTaps * a.cin * sizeof(float), 256);
}

int f32_wgrad(const WgradArgs& a, const void* x, const void* gy, void* gw, void* workspace, hipStream_t st) {
  const int nsplit = f32_wgrad_splits(a);
  const int cibs = a.cin / 32, cobs = a.cout / 32;
  const int64_t total = (int64_t)nsplit * cibs * cobs;
  if (total > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "conv fp32 wgrad: too many workgroups");
  hipLaunchKernelGGL(wgrad_f32_kernel, dim3((unsigned)total), dim3(256), 0, st, a, (const float*)x, (const float*)gy, (float*)workspace,
                     nsplit, cibs);
  if (int rc = check_launch("wgrad_f32_kernel")) return rc;
  return sum_slices(SFH_FP32, (const float*)workspace, gw, (int64_t)a.cout * kTaps * a.cin, nsplit, st);
}

}  // namespace sfh
