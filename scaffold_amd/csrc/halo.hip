// The local half of the halo exchange of a depth-sharded convolution: one pass that writes the shard between the
// boundary planes received from its neighbours (or zeros where there is no neighbour) into the slab the convolution
// kernel reads at depth padding 0. The reference assembles it with three strided copies after its receives
// (ScaFFold/unet/conv3d.py:769-776); here it is one streaming kernel, 16 bytes per lane, B read + B(1 + 2 halo/D) written.
#include "halo.hpp"

namespace sfh {

namespace {

constexpr int kBlock = 256;

// One thread per 16-byte piece of the output; `plane` = pieces per depth plane, `od` = D + 2 * halo.
__global__ void __launch_bounds__(kBlock) halo_assemble_kernel(const uint4* __restrict__ x, const uint4* __restrict__ lo,
                                                               const uint4* __restrict__ hi, uint4* __restrict__ out, int64_t plane,
                                                               int d, int halo, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= total) return;
  const int od = d + 2 * halo;
  const int64_t row = i / plane, r = i - row * plane;
  const int64_t n = row / od;
  const int z = (int)(row - n * od);
  uint4 v = make_uint4(0u, 0u, 0u, 0u);
  if (z < halo) {
    if (lo != nullptr) v = lo[(n * halo + z) * plane + r];
  } else if (z >= halo + d) {
    if (hi != nullptr) v = hi[(n * halo + (z - halo - d)) * plane + r];
  } else {
    v = x[(n * d + (z - halo)) * plane + r];
  }
  out[i] = v;
}

// Element-wise form for planes that are not a whole number of 16-byte pieces.
template <typename E>
__global__ void __launch_bounds__(kBlock) halo_assemble_scalar(const E* __restrict__ x, const E* __restrict__ lo,
                                                               const E* __restrict__ hi, E* __restrict__ out, int64_t plane, int d,
                                                               int halo, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= total) return;
  const int od = d + 2 * halo;
  const int64_t row = i / plane, r = i - row * plane;
  const int64_t n = row / od;
  const int z = (int)(row - n * od);
  E v = 0;
  if (z < halo) {
    if (lo != nullptr) v = lo[(n * halo + z) * plane + r];
  } else if (z >= halo + d) {
    if (hi != nullptr) v = hi[(n * halo + (z - halo - d)) * plane + r];
  } else {
    v = x[(n * d + (z - halo)) * plane + r];
  }
  out[i] = v;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

int halo_assemble(const sfh_halo_desc& p, int dtype, const void* x, const void* lo, const void* hi, void* out, hipStream_t st) {
  const int64_t plane_bytes = (int64_t)p.h * p.w * p.c * (int64_t)dtype_size(dtype);
  const int64_t rows = (int64_t)p.n * (p.d + 2 * p.halo);
  if (rows == 0 || plane_bytes == 0) return SFH_OK;
  if (plane_bytes % 16 == 0 && aligned16(x) && aligned16(out) && aligned16(lo) && aligned16(hi)) {
    const int64_t plane = plane_bytes / 16, total = rows * plane;
    const int64_t blocks = cdiv(total, kBlock);
    if (blocks > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "halo assemble: slab too large for one launch");
    hipLaunchKernelGGL(halo_assemble_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, st, (const uint4*)x, (const uint4*)lo,
                       (const uint4*)hi, (uint4*)out, plane, p.d, p.halo, total);
    return check_launch("halo_assemble_kernel");
  }
  const int64_t esz = (int64_t)dtype_size(dtype);
  const int64_t plane = plane_bytes / esz, total = rows * plane;
  const int64_t blocks = cdiv(total, kBlock);
  if (blocks > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "halo assemble: slab too large for one launch");
  if (esz == 4)
    hipLaunchKernelGGL(halo_assemble_scalar<uint32_t>, dim3((unsigned)blocks), dim3(kBlock), 0, st, (const uint32_t*)x,
                       (const uint32_t*)lo, (const uint32_t*)hi, (uint32_t*)out, plane, p.d, p.halo, total);
  else
    hipLaunchKernelGGL(halo_assemble_scalar<uint16_t>, dim3((unsigned)blocks), dim3(kBlock), 0, st, (const uint16_t*)x,
                       (const uint16_t*)lo, (const uint16_t*)hi, (uint16_t*)out, plane, p.d, p.halo, total);
  return check_launch("halo_assemble_scalar");
}

}  // namespace sfh
