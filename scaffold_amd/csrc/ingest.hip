// Shard ingest: the step between a dataset file and the network. A volume is stored channels-first as float32
// (C, D, H, W) with its mask as 16-bit integers (D, H, W) (ScaFFold/datagen/volumegen.py:259-292); the trainer moves
// the batch to the device, relays it out channels-last and widens the mask to int64 (ScaFFold/utils/trainer.py:572-589),
// and autocast then rounds the volume to the compute type in front of the first convolution. Here that is one pass:
// a workgroup takes a run of voxels, reads each channel plane coalesced, interleaves the channels through LDS and
// writes whole 16-byte pieces of channels-last rows (rounded once, to nearest even, when the output is 16-bit),
// optionally into the interior of a depth slab whose faces the same launch zeroes; the mask run is widened beside it.
#include "ingest.hpp"

namespace sfh {

namespace {

constexpr int kBlock = 256;
constexpr int kPerThread = 4;
constexpr int kTile = kBlock * kPerThread;  // voxels per workgroup

template <typename T> __device__ __forceinline__ T rounded(float f) { return elem<T>::from_float(f); }

// Grid: (tiles per sample, N). vin: planes can be read as float4 (rows % 4 == 0, 16-byte aligned base);
// vout: the output tile is a whole number of aligned 16-byte pieces.
template <typename T, int C>
__global__ void __launch_bounds__(kBlock) ingest_kernel(const float* __restrict__ volume, const uint16_t* __restrict__ mask,
                                                        T* __restrict__ x, int64_t* __restrict__ labels, int64_t rows,
                                                        int64_t halo, int mask_signed, int vin, int vout) {
  __shared__ __align__(16) T tile[kTile * C];
  const int tid = threadIdx.x;
  const int64_t n = blockIdx.y;
  const int64_t v0 = (int64_t)blockIdx.x * kTile;
  const int64_t left = rows - v0;
  const int nv = left < kTile ? (int)left : kTile;  // voxels of this tile
  const int mine = kPerThread * tid;                // first voxel of this thread inside the tile

  // 1. planes -> registers; every load is issued before the first use, tails read a clamped address
  float f[C][kPerThread];
  const float* plane0 = volume + n * C * rows + v0;
  if (vin) {
    const int at = mine < nv ? mine : 0;
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const float4 q = *reinterpret_cast<const float4*>(plane0 + c * rows + at);
      f[c][0] = q.x; f[c][1] = q.y; f[c][2] = q.z; f[c][3] = q.w;
    }
  } else {
#pragma unroll
    for (int c = 0; c < C; ++c)
#pragma unroll
      for (int j = 0; j < kPerThread; ++j) {
        const int at = mine + j < nv ? mine + j : nv - 1;
        f[c][j] = plane0[c * rows + at];
      }
  }
  // the mask run of this thread
  uint16_t m[kPerThread] = {0, 0, 0, 0};
  if (mask != nullptr) {
    const uint16_t* run = mask + n * rows + v0;
    if (vin) {
      const int at = mine < nv ? mine : 0;
      const uint2 q = *reinterpret_cast<const uint2*>(run + at);
      m[0] = (uint16_t)(q.x & 0xffffu); m[1] = (uint16_t)(q.x >> 16); m[2] = (uint16_t)(q.y & 0xffffu); m[3] = (uint16_t)(q.y >> 16);
    } else {
#pragma unroll
      for (int j = 0; j < kPerThread; ++j) m[j] = run[mine + j < nv ? mine + j : nv - 1];
    }
  }

  // 2. interleave through LDS
#pragma unroll
  for (int j = 0; j < kPerThread; ++j)
#pragma unroll
    for (int c = 0; c < C; ++c) tile[(mine + j) * C + c] = rounded<T>(f[c][j]);
  __syncthreads();

  // 3. the tile's rows are one contiguous range of the output
  T* dst = x + ((n * (rows + 2 * halo) + halo + v0) * C);
  const int elems = nv * C;
  if (vout) {
    constexpr int kPer16 = 16 / (int)sizeof(T);
    const int pieces = elems / kPer16;  // exact: the host checked divisibility
    const uint4* src = reinterpret_cast<const uint4*>(tile);
    uint4* out = reinterpret_cast<uint4*>(dst);
    for (int i = tid; i < pieces; i += kBlock) out[i] = src[i];
  } else {
    for (int i = tid; i < elems; i += kBlock) dst[i] = tile[i];
  }

  // 4. labels
  if (mask != nullptr) {
    int64_t* lab = labels + n * rows + v0;
    int64_t wide[kPerThread];
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) wide[j] = mask_signed ? (int64_t)(int16_t)m[j] : (int64_t)m[j];
    if (vin && mine < nv) {  // rows % 4 == 0: a thread's four voxels are all inside or all outside
      // 32 contiguous bytes per thread; 16-byte aligned because rows % 4 == 0 and the base is checked on the host
      longlong2* o = reinterpret_cast<longlong2*>(lab + mine);
      o[0] = make_longlong2(wide[0], wide[1]);
      o[1] = make_longlong2(wide[2], wide[3]);
    } else if (!vin) {
#pragma unroll
      for (int j = 0; j < kPerThread; ++j)
        if (mine + j < nv) lab[mine + j] = wide[j];
    }
  }

  // 5. the faces of the slab, spread over the workgroups of the sample
  if (halo > 0) {
    const int64_t face = halo * C;  // elements per face
    T* base = x + n * (rows + 2 * halo) * C;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + tid; i < 2 * face; i += stride) {
      const int64_t at = i < face ? i : i + rows * C;
      base[at] = rounded<T>(0.f);
    }
  }
}

bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

template <typename T, int C>
int launch(const sfh_ingest_desc& p, const float* volume, const void* mask, void* x, int64_t* labels, hipStream_t st) {
  const int64_t tiles = cdiv(p.rows, kTile);
  if (tiles > 0x7fffffffLL || p.n > 65535) return fail(SFH_ERR_UNSUPPORTED, "shard ingest: too many tiles or samples for one launch");
  const int64_t es = (int64_t)sizeof(T);
  const int vin = p.rows % 4 == 0 && aligned(volume, 16) && (mask == nullptr || (aligned(mask, 8) && aligned(labels, 16)));
  const int vout = (p.rows * p.c * es) % 16 == 0 && (p.halo_rows * p.c * es) % 16 == 0 && ((int64_t)kTile * p.c * es) % 16 == 0 &&
                   aligned(x, 16);
  hipLaunchKernelGGL((ingest_kernel<T, C>), dim3((unsigned)tiles, (unsigned)p.n), dim3(kBlock), 0, st, volume,
                     (const uint16_t*)mask, (T*)x, labels, p.rows, p.halo_rows, (int)(p.mask_signed != 0), vin, vout);
  return check_launch("ingest_kernel");
}

template <typename T>
int by_channels(const sfh_ingest_desc& p, const float* volume, const void* mask, void* x, int64_t* labels, hipStream_t st) {
  switch (p.c) {
    case 1: return launch<T, 1>(p, volume, mask, x, labels, st);
    case 2: return launch<T, 2>(p, volume, mask, x, labels, st);
    case 3: return launch<T, 3>(p, volume, mask, x, labels, st);
    case 4: return launch<T, 4>(p, volume, mask, x, labels, st);
  }
  return fail(SFH_ERR_UNSUPPORTED, "shard ingest: %d channels (1..%d supported)", p.c, kIngestMaxChannels);
}

}  // namespace

int shard_ingest(const sfh_ingest_desc& p, int dtype, const float* volume, const void* mask, void* x, int64_t* labels,
                 hipStream_t st) {
  switch (dtype) {
    case SFH_BF16: return by_channels<bf16_t>(p, volume, mask, x, labels, st);
    case SFH_FP16: return by_channels<fp16_t>(p, volume, mask, x, labels, st);
    case SFH_FP32: return by_channels<float>(p, volume, mask, x, labels, st);
  }
  return fail(SFH_ERR_INVALID, "shard ingest: bad dtype %d", dtype);
}

}  // namespace sfh
