// Host-side interface of the MFMA weight-gradient kernel (3x3x3, stride 1, bf16 / fp16).
#pragma once
#include "common.hpp"

namespace sfh {

struct WgradArgs {
  int n, cin, id, ih, iw;
  int cout, od, oh, ow;
  int pd, ph, pw;
};

bool mfma_wgrad_supported(const WgradArgs& a, int dtype);
// Number of fp32 partial slices [Cout][27][Cin]; a pure function of the shape.
int mfma_wgrad_splits(const WgradArgs& a);
size_t mfma_wgrad_workspace_bytes(const WgradArgs& a);
// gw is written in gw_dtype (the operands' dtype, or SFH_FP32 for a full-precision gradient).
// `x2` (optional, where mfma_wgrad_pair_ok says so): x given as two tensors whose channels follow each other (the
// first x2->first in x, the rest in x2->second); the gradient is the one of their concatenation, bit for bit.
bool mfma_wgrad_pair_ok(const WgradArgs& a, int first);
int mfma_wgrad(const WgradArgs& a, int dtype, const void* x, const void* gy, void* gw, int gw_dtype, void* workspace,
               hipStream_t st, const ChannelPair* x2 = nullptr);

// The same gradient for rows of more than 16 voxels (wgrad_ring.hip): columns walked along depth, operands staged as
// they lie in memory and transposed by the LDS reads. `applies` and the slice count are pure functions of the shape;
// the kernel writes `splits` fp32 slices [Cout][27][Cin] into ws. mfma_wgrad routes to it.
bool mfma_wgrad_ring_applies(const WgradArgs& a);
int mfma_wgrad_ring_splits(const WgradArgs& a);
int mfma_wgrad_ring(const WgradArgs& a, int dtype, const void* x, const void* gy, float* ws, hipStream_t st, const ChannelPair& x2);

// Several weight gradients from as few launches as possible: the ring-served problems of a list (rows of more than 16
// voxels) in one launch and one sum pass (wgrad_ring.hip), its small-volume problems (rows of 16 or 8 voxels, at most 32
// tiles under a block) in one launch that writes the gradients directly (wgrad_mfma.hip). The cost every launch pays
// -- the first fetch of all workgroups, the slices written and read back, launch gaps -- is paid once per family. All
// problems share dtype and the gradient's dtype; how the work is cut over the workgroups is a pure function of the
// list of problems, every sum has a fixed order (not that of the one-problem launch: the cuts differ).
constexpr int kWgradBatchMax = 16;
struct WgradBatchItem {
  WgradArgs a;
  const void* x;
  const void* x1;  // with c_first: the input as two tensors (mfma_wgrad_pair_ok), or null
  int c_first;
  const void* gy;
  void* gw;
};
bool mfma_wgrad_batch_applies(const WgradArgs& a, int dtype);
// max_wgs > 0: the ring-served launch takes at most that many workgroups (it is meant to run beside other work)
size_t mfma_wgrad_batch_workspace_bytes(const WgradBatchItem* items, int count, int max_wgs);  // 0: the list cannot share a launch
int mfma_wgrad_batch(const WgradBatchItem* items, int count, int dtype, int gw_dtype, void* workspace, size_t workspace_bytes,
                     hipStream_t st, int max_wgs);
// the ring-served family alone (every item must be ring-served)
size_t mfma_wgrad_ring_batch_workspace_bytes(const WgradBatchItem* items, int count, int max_wgs);
int mfma_wgrad_ring_batch(const WgradBatchItem* items, int count, int dtype, int gw_dtype, void* workspace, size_t workspace_bytes,
                          hipStream_t st, int max_wgs);

}  // namespace sfh
