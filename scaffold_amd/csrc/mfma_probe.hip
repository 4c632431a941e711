// Measurement kernels, not part of the convolution path: what the matrix pipe of this chip sustains on
// v_mfma_f32_32x32x16_bf16 under the instruction mix of the persistent convolution, so that a convolution's rate can be
// read against a measured ceiling as well as against the nominal peak. One 4-wavefront workgroup per CU, as the
// persistent kernel runs; a "tile" is its unit of 54 x 4 MFMAs per wavefront on four accumulators.
//   mix 0: nothing but the MFMAs (operands stay in registers);
//   mix 1: one ds_read_b128 per two MFMAs feeding their column operand (the convolution reads 96 fragments for 216 MFMAs):
//          the ceiling of a kernel with this operand traffic and no global memory traffic at all;
//   mix 2: mix 1 plus, per tile and wavefront, 12 direct-to-LDS loads of 1 KiB that stream through `src` and 8 stores of
//          1 KiB that stream through `sink` (the convolution's 44 KiB in / 32 KiB out per 512-voxel step), and a
//          workgroup barrier per tile. Every byte of it comes from and goes to HBM, where the convolution finds its halo
//          rows in L2: a reference point for the cost of the traffic, not a bound.
// The operand values come from the caller's buffers (Gaussian or zero bits: the sustained clock depends on them).
#include "common.hpp"
#include "mma.hpp"

namespace sfh {
namespace {

typedef uint32_t sfh_probe_u32x4_t __attribute__((ext_vector_type(4)));
constexpr int kProbeLdsBytes = 64 * 1024;
constexpr int kProbeLoads = 12;           // direct-to-LDS loads per wavefront and tile in mix 2
constexpr int kProbeTileIn = 4 * kProbeLoads * 1024;  // bytes a workgroup fetches per tile in mix 2
constexpr int kProbeTileOut = 32 * 1024;  // bytes it stores (4 x 8 x 1 KiB)

template <int MIX>
__global__ void __launch_bounds__(256, 1)
mfma_probe_kernel(const uint4* __restrict__ operands, const char* __restrict__ src, uint32_t src_bytes, char* __restrict__ sink,
                  uint32_t sink_bytes, int tiles, float* __restrict__ out) {
#if defined(__HIP_DEVICE_COMPILE__)
  __shared__ __attribute__((aligned(16))) char lds_read[kProbeLdsBytes];
  __shared__ __attribute__((aligned(16))) char lds_fill[kProbeLdsBytes];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // 64 KiB of operand bits into the LDS region the MFMAs read; 8 row-operand fragments into registers
  for (int i = tid; i < kProbeLdsBytes / 16; i += 256) reinterpret_cast<uint4*>(lds_read)[i] = operands[(i * 37 + blockIdx.x) & 4095];
  uint4 a[8], b[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = operands[(tid * 5 + i * 977 + blockIdx.x * 13) & 4095];
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = operands[(tid * 7 + i * 1999 + blockIdx.x * 3) & 4095];
  __syncthreads();
  f32x16_t acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  const __amdgpu_buffer_rsrc_t rs_in = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(src), 0, (int)src_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_out = __builtin_amdgcn_make_buffer_rsrc(sink, 0, (int)sink_bytes, 0x00020000);
  const char* rd = lds_read + lane * 16;
  for (int t = 0; t < tiles; ++t) {
    // where this workgroup's tile t lies in the streams (distinct for every workgroup and tile until the buffers wrap)
    const uint32_t in0 = (uint32_t)(((uint64_t)(blockIdx.x * (uint32_t)tiles + t) * kProbeTileIn) % src_bytes);
    const uint32_t out0 = (uint32_t)(((uint64_t)(blockIdx.x * (uint32_t)tiles + t) * kProbeTileOut) % sink_bytes);
#pragma unroll
    for (int it = 0; it < 54; ++it) {
#pragma unroll
      for (int ms = 0; ms < 4; ++ms) {
        __builtin_amdgcn_sched_barrier(0);
        acc[ms] = Mma32<bf16_t>::run(a[(it + ms) & 7], b[ms], acc[ms]);
        __builtin_amdgcn_sched_barrier(0);
        if (MIX >= 1 && ms % 2 == 0) b[ms] = *reinterpret_cast<const uint4*>(rd + ((it * 4 + ms) * 1024 + wave * 256) % (kProbeLdsBytes - 1024));
        if (MIX >= 2 && ms == 0) {  // a load or a store behind every tenth MFMA or so, loads first (as the convolution issues them)
          if (it % 2 == 0 && it / 2 < kProbeLoads) {
            const uint32_t off = (in0 + (uint32_t)((wave * kProbeLoads + it / 2) * 1024 + lane * 16)) % src_bytes;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_in, (__attribute__((address_space(3))) void*)(lds_fill + ((wave * kProbeLoads + it / 2) % 64) * 1024),
                                                     16, off, 0, 0, 0);
          }
          if (it % 2 == 0 && it / 2 >= kProbeLoads && it / 2 < kProbeLoads + 8) {
            const uint32_t off = (out0 + (uint32_t)((wave * 8 + it / 2 - kProbeLoads) * 1024 + lane * 16)) % sink_bytes;
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(sfh_probe_u32x4_t, a[it % 8]), rs_out, off, 0, 0);
          }
        }
      }
    }
    if (MIX >= 2) {
      __builtin_amdgcn_s_waitcnt(0x0070 | (15 << 8));  // vmcnt(0): this wavefront's loads of the tile have landed
      __syncthreads();
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  if (MIX >= 2) s += (float)reinterpret_cast<const uint32_t*>(lds_fill)[tid];
  out[blockIdx.x * 256 + tid] = s;
#endif
}

}  // namespace
}  // namespace sfh

using namespace sfh;

extern "C" double sfh_mfma_ceiling_probe_flops(int32_t workgroups, int32_t tiles) {
  return (double)workgroups * 4.0 * (double)tiles * 216.0 * 32768.0;
}

extern "C" int sfh_mfma_ceiling_probe(int32_t mix, int32_t workgroups, int32_t tiles, const void* operands, const void* src,
                                      size_t src_bytes, void* sink, size_t sink_bytes, float* out, void* stream) {
  if (mix < 0 || mix > 2 || workgroups < 1 || workgroups > 65535 || tiles < 1 || operands == nullptr || out == nullptr)
    return fail(SFH_ERR_INVALID, "mfma probe: bad arguments");
  if (mix == 2 && (src == nullptr || sink == nullptr || src_bytes < (1u << 20) || sink_bytes < (1u << 20) || src_bytes > 0x7fffffffu ||
                   sink_bytes > 0x7fffffffu || src_bytes % 1024 != 0 || sink_bytes % 1024 != 0))
    return fail(SFH_ERR_INVALID, "mfma probe: the streams must be 1 MiB .. 2 GiB, multiples of 1 KiB");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)workgroups), block(256);
  const uint4* ops = (const uint4*)operands;
  if (mix == 0)
    hipLaunchKernelGGL(mfma_probe_kernel<0>, grid, block, 0, st, ops, (const char*)src, (uint32_t)src_bytes, (char*)sink, (uint32_t)sink_bytes, tiles, out);
  else if (mix == 1)
    hipLaunchKernelGGL(mfma_probe_kernel<1>, grid, block, 0, st, ops, (const char*)src, (uint32_t)src_bytes, (char*)sink, (uint32_t)sink_bytes, tiles, out);
  else
    hipLaunchKernelGGL(mfma_probe_kernel<2>, grid, block, 0, st, ops, (const char*)src, (uint32_t)src_bytes, (char*)sink, (uint32_t)sink_bytes, tiles, out);
  return check_launch("mfma_probe_kernel");
}
