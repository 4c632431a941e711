// Channel concatenation of two channels-last tensors (the U-Net's skip connection, torch.cat([skip, upsampled], 1),
// ScaFFold/unet/unet_parts.py:107-120) and its backward split, as one streaming pass each: a thread moves one
// 16-byte piece of an output row, so consecutive lanes write consecutive addresses and read two contiguous runs.
// With halo rows the result lands in the interior of a depth slab whose faces are zeroed by the same launch: the
// input of a depth shard's convolution, produced without a second copy.
#include "concat.hpp"

namespace sfh {

namespace {

constexpr int kBlock = 256;

// pa / pb: 16-byte pieces per row of a and b. `rows` per sample, `halo` rows on each face of the slab.
template <typename I>
__global__ void __launch_bounds__(kBlock) concat_fwd_kernel(const uint4* __restrict__ a, const uint4* __restrict__ b,
                                                            uint4* __restrict__ out, I pa, I pb, I rows, I halo, I total, I faces) {
  const I i = (I)blockIdx.x * kBlock + threadIdx.x;
  const I p = pa + pb;
  if (i < total) {
    const I row = i / p, piece = i - row * p;  // row counts over all samples
    const I n = row / rows;
    const uint4 v = piece < pa ? a[row * pa + piece] : b[row * pb + (piece - pa)];
    out[(row + (2 * n + 1) * halo) * p + piece] = v;
  }
  // the faces: 2 * halo rows per sample
  for (I f = i; f < faces; f += (I)gridDim.x * kBlock) {
    const I per = 2 * halo * p;
    const I n = f / per, r = f - n * per;
    const I at = r < halo * p ? r : r + rows * p;
    out[n * (rows + 2 * halo) * p + at] = make_uint4(0u, 0u, 0u, 0u);
  }
}

template <typename I>
__global__ void __launch_bounds__(kBlock) concat_bwd_kernel(const uint4* __restrict__ g, uint4* __restrict__ ga,
                                                            uint4* __restrict__ gb, I pa, I pb, I rows, I halo, I total) {
  const I i = (I)blockIdx.x * kBlock + threadIdx.x;
  if (i >= total) return;
  const I p = pa + pb;
  const I row = i / p, piece = i - row * p;
  const I n = row / rows;
  const uint4 v = g[(row + (2 * n + 1) * halo) * p + piece];
  if (piece < pa) ga[row * pa + piece] = v;
  else gb[row * pb + (piece - pa)] = v;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace

bool concat_supported(const sfh_concat_desc& p, int dtype) {
  const int64_t es = (int64_t)dtype_size(dtype);
  return p.n >= 1 && p.c_a >= 1 && p.c_b >= 1 && p.rows >= 1 && p.halo_rows >= 0 && (p.c_a * es) % 16 == 0 && (p.c_b * es) % 16 == 0;
}

int concat_forward(const sfh_concat_desc& p, int dtype, const void* a, const void* b, void* out, hipStream_t st) {
  if (!aligned16(a) || !aligned16(b) || !aligned16(out)) return fail(SFH_ERR_UNSUPPORTED, "skip concat: pointers must be 16-byte aligned");
  const int64_t es = (int64_t)dtype_size(dtype);
  const int64_t pa = p.c_a * es / 16, pb = p.c_b * es / 16;
  const int64_t total = (int64_t)p.n * p.rows * (pa + pb), faces = (int64_t)p.n * 2 * p.halo_rows * (pa + pb);
  const int64_t blocks = cdiv(total, kBlock);
  if (blocks > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "skip concat: tensor too large for one launch");
  if ((int64_t)p.n * (p.rows + 2 * p.halo_rows) * (pa + pb) < 0x7fffffffLL)
    hipLaunchKernelGGL(concat_fwd_kernel<int32_t>, dim3((unsigned)blocks), dim3(kBlock), 0, st, (const uint4*)a, (const uint4*)b,
                       (uint4*)out, (int32_t)pa, (int32_t)pb, (int32_t)p.rows, (int32_t)p.halo_rows, (int32_t)total, (int32_t)faces);
  else
    hipLaunchKernelGGL(concat_fwd_kernel<int64_t>, dim3((unsigned)blocks), dim3(kBlock), 0, st, (const uint4*)a, (const uint4*)b,
                       (uint4*)out, pa, pb, p.rows, p.halo_rows, total, faces);
  return check_launch("concat_fwd_kernel");
}

int concat_backward(const sfh_concat_desc& p, int dtype, const void* g, void* ga, void* gb, hipStream_t st) {
  if (!aligned16(g) || !aligned16(ga) || !aligned16(gb)) return fail(SFH_ERR_UNSUPPORTED, "skip concat: pointers must be 16-byte aligned");
  const int64_t es = (int64_t)dtype_size(dtype);
  const int64_t pa = p.c_a * es / 16, pb = p.c_b * es / 16;
  const int64_t total = (int64_t)p.n * p.rows * (pa + pb);
  const int64_t blocks = cdiv(total, kBlock);
  if (blocks > 0x7fffffffLL) return fail(SFH_ERR_UNSUPPORTED, "skip concat: tensor too large for one launch");
  if ((int64_t)p.n * (p.rows + 2 * p.halo_rows) * (pa + pb) < 0x7fffffffLL)
    hipLaunchKernelGGL(concat_bwd_kernel<int32_t>, dim3((unsigned)blocks), dim3(kBlock), 0, st, (const uint4*)g, (uint4*)ga,
                       (uint4*)gb, (int32_t)pa, (int32_t)pb, (int32_t)p.rows, (int32_t)p.halo_rows, (int32_t)total);
  else
    hipLaunchKernelGGL(concat_bwd_kernel<int64_t>, dim3((unsigned)blocks), dim3(kBlock), 0, st, (const uint4*)g, (uint4*)ga,
                       (uint4*)gb, pa, pb, p.rows, p.halo_rows, total);
  return check_launch("concat_bwd_kernel");
}

}  // namespace sfh
