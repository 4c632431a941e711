// The local steps of the halo exchange of a depth-sharded convolution. Forward: the boundary planes a shard sends are
// gathered into plain buffers (halo_pack), and after the receives one pass writes the shard between the
// boundary planes received from its neighbours (or zeros where there is no neighbour) into the slab the convolution
// kernel reads at depth padding 0. The reference assembles it with three strided copies after its receives
// (ScaFFold/unet/conv3d.py:769-776); here it is one streaming kernel, 16 bytes per lane, B read + B(1 + 2 halo/D) written.
// Backward (conv3d.py:795-841): the outer planes of the slab's gradient are packed the same way, and what comes back
// from the neighbours is added into the shard's own boundary planes in place (halo_accumulate).
#include "halo.hpp"
#include "vec_io.hpp"

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

// The boundary planes a shard sends: lo_out <- planes [0, halo), hi_out <- planes [d - halo, d) of every sample of x
// (N, d, plane). V is the unit moved (16-byte piece or one element). Grid: one thread per unit of one face pair.
template <typename V>
__global__ void __launch_bounds__(kBlock) halo_pack_kernel(const V* __restrict__ x, V* __restrict__ lo_out, V* __restrict__ hi_out,
                                                           int64_t plane, int d, int halo, int64_t per_face) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;  // over N * halo * plane
  if (i >= per_face) return;
  const int64_t face = (int64_t)halo * plane;
  const int64_t n = i / face, r = i - n * face;
  const V* sample = x + n * d * plane;
  if (lo_out != nullptr) lo_out[i] = sample[r];
  if (hi_out != nullptr) hi_out[i] = sample[(int64_t)(d - halo) * plane + r];
}

// The transpose of the above: g (N, d, plane), in place: planes [0, halo) += lo_in, planes [d - halo, d) += hi_in,
// each sum formed in fp32 and rounded once (what Tensor.add_ does). d >= 2 * halo, so the two ranges are disjoint.
template <typename T, int V>
__global__ void __launch_bounds__(kBlock) halo_accumulate_kernel(T* __restrict__ g, const T* __restrict__ lo_in,
                                                                 const T* __restrict__ hi_in, int64_t plane, int d, int halo,
                                                                 int64_t per_face) {
  const int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * V;  // element index over N * halo * plane
  if (i >= per_face) return;
  const int64_t face = (int64_t)halo * plane;
  const int64_t n = i / face, r = i - n * face;
  T* sample = g + n * d * plane;
  auto add_into = [&](T* dst, const T* src) {
    if constexpr (V == 1) {
      dst[0] = elem<T>::from_float(to_float(dst[0]) + to_float(src[0]));
    } else {
      float a[V], b[V];
      Ld<T, V>::run(dst, a);
      Ld<T, V>::run(src, b);
#pragma unroll
      for (int k = 0; k < V; ++k) a[k] += b[k];
      St<T, V>::run(dst, a);
    }
  };
  if (lo_in != nullptr) add_into(sample + r, lo_in + i);
  if (hi_in != nullptr) add_into(sample + (int64_t)(d - halo) * plane + r, hi_in + i);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T>
int accumulate_typed(const sfh_halo_desc& p, void* g, const void* lo_in, const void* hi_in, hipStream_t st) {
  constexpr int V = VecOf<T>::N;
  const int64_t plane = (int64_t)p.h * p.w * p.c;
  const int64_t per_face = (int64_t)p.n * p.halo * plane;
  const bool vec = plane % V == 0 && aligned16(g) && aligned16(lo_in) && aligned16(hi_in);
  const int64_t threads = vec ? per_face / V : per_face;
  const int64_t blocks = cdiv(threads, kBlock);
  if (blocks > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "halo accumulate: faces too large for one launch");
  if (vec)
    hipLaunchKernelGGL((halo_accumulate_kernel<T, V>), dim3((unsigned)blocks), dim3(kBlock), 0, st, (T*)g, (const T*)lo_in,
                       (const T*)hi_in, plane, p.d, p.halo, per_face);
  else
    hipLaunchKernelGGL((halo_accumulate_kernel<T, 1>), dim3((unsigned)blocks), dim3(kBlock), 0, st, (T*)g, (const T*)lo_in,
                       (const T*)hi_in, plane, p.d, p.halo, per_face);
  return check_launch("halo_accumulate_kernel");
}

}  // namespace

int halo_pack(const sfh_halo_desc& p, int dtype, const void* x, void* lo_out, void* hi_out, hipStream_t st) {
  const int64_t esz = (int64_t)dtype_size(dtype);
  const int64_t plane_bytes = (int64_t)p.h * p.w * p.c * esz;
  if ((int64_t)p.n * p.halo * plane_bytes == 0 || (lo_out == nullptr && hi_out == nullptr)) return SFH_OK;
  const bool vec = plane_bytes % 16 == 0 && aligned16(x) && aligned16(lo_out) && aligned16(hi_out);
  const int64_t unit = vec ? 16 : esz;
  const int64_t plane = plane_bytes / unit, per_face = (int64_t)p.n * p.halo * plane;
  const int64_t blocks = cdiv(per_face, kBlock);
  if (blocks > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "halo pack: faces too large for one launch");
  if (vec)
    hipLaunchKernelGGL(halo_pack_kernel<uint4>, dim3((unsigned)blocks), dim3(kBlock), 0, st, (const uint4*)x, (uint4*)lo_out,
                       (uint4*)hi_out, plane, p.d, p.halo, per_face);
  else if (esz == 4)
    hipLaunchKernelGGL(halo_pack_kernel<uint32_t>, dim3((unsigned)blocks), dim3(kBlock), 0, st, (const uint32_t*)x,
                       (uint32_t*)lo_out, (uint32_t*)hi_out, plane, p.d, p.halo, per_face);
  else
    hipLaunchKernelGGL(halo_pack_kernel<uint16_t>, dim3((unsigned)blocks), dim3(kBlock), 0, st, (const uint16_t*)x,
                       (uint16_t*)lo_out, (uint16_t*)hi_out, plane, p.d, p.halo, per_face);
  return check_launch("halo_pack_kernel");
}

int halo_accumulate(const sfh_halo_desc& p, int dtype, void* g, const void* lo_in, const void* hi_in, hipStream_t st) {
  if ((int64_t)p.n * p.halo * p.h * p.w * p.c == 0 || (lo_in == nullptr && hi_in == nullptr)) return SFH_OK;
  switch (dtype) {
    case SFH_BF16: return accumulate_typed<bf16_t>(p, g, lo_in, hi_in, st);
    case SFH_FP16: return accumulate_typed<fp16_t>(p, g, lo_in, hi_in, st);
    case SFH_FP32: return accumulate_typed<float>(p, g, lo_in, hi_in, st);
  }
  return fail(SFH_ERR_INVALID, "halo accumulate: bad dtype %d", dtype);
}

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
