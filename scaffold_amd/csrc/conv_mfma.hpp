// Host-side interface of the MFMA implicit-GEMM convolution kernels (bf16 / fp16 only).
#pragma once
#include "common.hpp"
#include "gn_stats.hpp"

namespace sfh {

// A stride-1, dilation-1 gather convolution in the roles the kernel sees them: `cred` reduction
// channels (a multiple of 32), `cout` produced channels (a multiple of 32), kernel extents in
// 1..3. The forward passes (Cin, Cout, padding); the data gradient passes (Cout, Cin, k-1-p)
// with the weight packed transposed and tap-flipped.
struct MfmaConvArgs {
  int n, cred, id, ih, iw;
  int cout, od, oh, ow;
  int kd, kh, kw, pd, ph, pw;
};

bool mfma_conv_supported(const MfmaConvArgs& a, int dtype);
// Whether the kernel that serves problem `a` reads its input as a ChannelPair cut at `first` (as_output: writes its
// output as one): a pure function of the shape. The results are the bits of the same launch on the concatenation.
bool mfma_conv_pair_ok(const MfmaConvArgs& a, int first, bool as_output);
size_t mfma_conv_packed_weight_bytes(const MfmaConvArgs& a);
// Repacks the weight into per-wavefront MFMA fragment order:
//   packed[cout/32][cred/32][tap][kstep(2)][lane(64)][8]
// with lane = (cout % 32) + 32 * (cred % 16 / 8). `s_out`, `s_red`, `s_kd/kh/kw` are element
// strides of the source for the produced channel, the reduction channel and the taps.
int mfma_pack_weight(const MfmaConvArgs& a, int dtype, const void* w, int64_t s_out, int64_t s_red, int64_t s_kd,
                     int64_t s_kh, int64_t s_kw, int flip, void* packed, hipStream_t st);
// Any number of packings (of any weights) in as few launches as the kernel argument space allows.
struct MfmaPackItem {
  MfmaConvArgs a;
  const void* w;
  int64_t s_out, s_red, s_kd, s_kh, s_kw;
  int flip;
  void* packed;
};
int mfma_pack_weight_batch(const MfmaPackItem* items, int n, int dtype, hipStream_t st);
// Bytes of fp32 slices the kernel needs when it cuts the reduction channels to fill the chip (0 when it does not).
size_t mfma_conv_partial_bytes(const MfmaConvArgs& a);
// `gn` (optional): also leave GroupNorm partials of the rounded output (gn_stats.hpp), gn->records per sample as
// mfma_conv_gn_records says for gn->groups groups.
// `in2` / `out2` (optional, where mfma_conv_pair_ok says so): x / y given as a ChannelPair.
int mfma_conv_gather(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y,
                     void* partial, hipStream_t st, const GnPartialOut* gn = nullptr, const ChannelPair* in2 = nullptr,
                     const ChannelPair* out2 = nullptr);
// Same contract, wide-tile kernel (64 or more reduction channels, rows of more than 16 voxels): `applies` is a pure
// function of the shape; mfma_conv_gather routes to it (it needs no partial workspace).
bool mfma_conv_wide_applies(const MfmaConvArgs& a);
int mfma_conv_wide(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                   const GnPartialOut* gn = nullptr, const ChannelPair* in2 = nullptr);
// Same contract, the kernel for the small volumes of the deep levels: 64-voxel bricks, the reduction cut over the four
// wavefronts of a workgroup and summed in LDS (conv_split.hip). `applies` is a pure function of the shape; mfma_conv_gather
// routes to it (it needs no partial workspace). Input or output may be a ChannelPair cut at a multiple of 32.
bool mfma_conv_split_applies(const MfmaConvArgs& a);
int mfma_conv_split(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                    const GnPartialOut* gn = nullptr, const ChannelPair* in2 = nullptr, const ChannelPair* out2 = nullptr);
int mfma_conv_split_gn_records(const MfmaConvArgs& a, int groups);
bool mfma_conv_split_pair_ok(const MfmaConvArgs& a, int first, bool as_output);
// Same contract, persistent one-workgroup-per-CU kernel with register-resident weights.
int mfma_conv_persist(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y,
                      void* partial, hipStream_t st, const GnPartialOut* gn = nullptr, const ChannelPair* in2 = nullptr,
                      const ChannelPair* out2 = nullptr);
// The persistent kernel's form for rows of more than 16 voxels: columns walked along depth with a ring of input planes in
// LDS (conv_ring.hip). `applies` is a pure function of the shape; mfma_conv_persist routes to it. gn.cg must be set.
bool mfma_conv_ring_applies(const MfmaConvArgs& a);
int mfma_conv_ring_workgroups_per_block(const MfmaConvArgs& a);
int mfma_conv_ring(const MfmaConvArgs& a, int dtype, const void* x, const void* packed, const void* bias, void* y, hipStream_t st,
                   const GnPartialOut& gn, const ChannelPair& out2);
// Records of GroupNorm partials per sample that mfma_conv_persist leaves for `groups` groups: a pure function of the
// shape; 0 when the kernel that serves the problem does not offer them (the caller then runs the statistics pass).
int mfma_conv_gn_records(const MfmaConvArgs& a, int groups);
int mfma_conv_gather_gn_records(const MfmaConvArgs& a, int groups);
bool mfma_conv_gather_pair_ok(const MfmaConvArgs& a, int first, bool as_output);
bool mfma_conv_wide_pair_ok(const MfmaConvArgs& a, int first);  // input pairs only, cut in the middle
int mfma_conv_wide_gn_records(const MfmaConvArgs& a, int groups);

// Which of the three kernels mfma_conv_persist ends up launching for a problem, and with what geometry: a pure function of
// the shape. `voxels` is the output tile of a workgroup step, `blocks` the 32-channel output blocks a workgroup produces
// from one staged brick, `slices` the cuts of the reduction channels (1: none, no partial workspace).
enum MfmaConvKernel { kKernelPersist = 1, kKernelBrick = 2, kKernelWide = 3, kKernelSplit = 6 };
struct MfmaConvGeometry { int kernel, voxels, blocks, slices; };
MfmaConvGeometry mfma_conv_geometry(const MfmaConvArgs& a);
bool mfma_conv_persist_applies(const MfmaConvArgs& a);
MfmaConvGeometry mfma_conv_gather_geometry(const MfmaConvArgs& a);
MfmaConvGeometry mfma_conv_wide_geometry(const MfmaConvArgs& a);
MfmaConvGeometry mfma_conv_split_geometry(const MfmaConvArgs& a);

}  // namespace sfh
