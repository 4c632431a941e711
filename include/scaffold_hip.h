/*
 * scaffold_hip.h -- C ABI of libscaffold_hip.so: the MI355X (gfx950) kernels behind the
 * ScaFFold 3D U-Net compute hot path (channels-last conv3d forward / data-gradient /
 * weight-gradient, kernel==stride transposed conv3d, channels-last GroupNorm fwd/bwd).
 *
 * Conventions (all entry points):
 *   - every tensor pointer is a DEVICE pointer on the current HIP device; nothing is
 *     allocated, freed or synchronised by the library; `stream` is a hipStream_t (NULL =
 *     the default stream) and all work is enqueued on it;
 *   - activations are dense NDHWC ("channels_last_3d"): element (n,c,d,h,w) lives at
 *     (((n*D + d)*H + h)*W + w)*C + c;
 *   - weights are read where they lie: `w_stride[5]` are ELEMENT strides of the logical
 *     (Cout, Cin, kd, kh, kw) tensor (for the transposed conv: (Cin, Cout, kd, kh, kw));
 *   - return value 0 = success, otherwise one of SFH_ERR_*; sfh_last_error() returns a
 *     thread-local human-readable message for the last failure on this thread;
 *   - launch geometry (tiles, split counts) is a pure function of the descriptor and dtype,
 *     and no floating-point atomics are used: the same call gives the same bits.
 *
 * Each declaration cites the reference interface (LBANN/ScaFFold) that it stands in for.
 */
#ifndef SCAFFOLD_HIP_H
#define SCAFFOLD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SFH_OK 0
#define SFH_ERR_INVALID 1     /* contract violation (null pointer, bad enum, inconsistent sizes) */
#define SFH_ERR_UNSUPPORTED 2 /* a problem this library does not serve (e.g. dgrad at stride != 1) */
#define SFH_ERR_WORKSPACE 3   /* workspace missing or smaller than *_workspace_bytes() */
#define SFH_ERR_LAUNCH 4      /* the HIP runtime refused a launch */

/* Element type of activations and weights; accumulation is always fp32. */
#define SFH_BF16 0
#define SFH_FP16 1
#define SFH_FP32 2

/* Flags for the convolution entry points. */
#define SFH_FLAG_FORCE_GENERIC 1u /* use the direct (non-MFMA) kernels whatever the shape */
#define SFH_FLAG_WEIGHT_PACKED 4u /* sfh_conv3d_fwd / _dgrad: `w` is the weight already packed for that direction by
                                     sfh_conv3d_pack_weights (same descriptor and dtype); w_stride is ignored and
                                     the workspace only needs the bytes beyond sfh_conv3d_packed_weight_bytes. */
#define SFH_FLAG_GRAD_FP32 2u     /* sfh_conv3d_wgrad: write grad_w as fp32 (the master weight's dtype under
                                     autocast) instead of the operands' dtype: the fp32 sum of the slices is
                                     stored as it is, saving the rounding and the caller's up-cast. Served by
                                     the tiled kernels; SFH_ERR_UNSUPPORTED where only the untiled one applies. */
#define SFH_FLAG_SHARE_DEVICE 8u  /* sfh_conv3d_wgrad_batch (and its workspace query: the workspace depends on it):
                                     the launch of the problems with rows of more than 16 voxels takes half of the
                                     compute units, for a batch issued on a stream of its own beside other work (a
                                     workgroup of that kernel fills a CU's LDS; on the CUs it leaves alone the other
                                     stream's kernels run undisturbed). Same bits on every run; within summation-order
                                     rounding of the full-width call's. */

/* A convolution problem as torch.nn.functional.conv3d names it (groups == 1). */
typedef struct sfh_conv3d_desc {
  int32_t n, cin, in_d, in_h, in_w;
  int32_t cout, kd, kh, kw;
  int32_t sd, sh, sw; /* stride   */
  int32_t pd, ph, pw; /* padding  */
  int32_t dd, dh, dw; /* dilation */
} sfh_conv3d_desc;

/* A kernel==stride, padding 0 transposed convolution (the U-Net up-convolution). */
typedef struct sfh_convT3d_desc {
  int32_t n, cin, in_d, in_h, in_w;
  int32_t cout, kd, kh, kw; /* stride == kernel */
} sfh_convT3d_desc;

/* A GroupNorm problem over a dense (N, S, C) channels-last tensor, S = D*H*W. */
typedef struct sfh_groupnorm_desc {
  int32_t n, c, groups;
  int32_t relu;    /* 1: fuse y = relu(y) into the store / gate the backward on the pre-activation */
  int64_t spatial; /* S */
  float eps;
} sfh_groupnorm_desc;

/* ---- library ------------------------------------------------------------------------ */
/* 100: the first published set of entry points. 101: sfh_conv3d_launch_geometry, sfh_conv3d_fwd_gn_records,
 * sfh_conv3d_fwd_gn, sfh_groupnorm_fwd_from_partials, sfh_tuned_compute_units added; nothing removed or changed.
 * 102: sfh_conv3d_pair_supported, sfh_conv3d_fwd_pair, sfh_conv3d_dgrad_pair, sfh_conv3d_wgrad_pair,
 * sfh_maxpool2_fwd_slab, sfh_convT3d_fwd_slab, sfh_convT3d_wgrad_bias(_workspace_bytes),
 * sfh_conv3d_wgrad_bias(_workspace_bytes) added.
 * 103: the GroupNorm statistics a convolution leaves are self-contained Welford records: sfh_conv3d_fwd_gn,
 * sfh_conv3d_fwd_pair and sfh_groupnorm_fwd_from_partials lost their shift arguments (CHANGED signatures, and the record
 * is 4 floats per group instead of 2), sfh_groupnorm_fwd_from_partials takes the byte size of the records;
 * sfh_groupnorm_fwd_noalloc_prepare, sfh_mfma_ceiling_probe added. fp32 problems of the tiled shape have needed a
 * workspace since 102 (sfh_conv3d_{fwd,dgrad,wgrad}_workspace_bytes are non-zero for them; callers that sized their
 * workspace with those functions are unaffected).
 * 104: sfh_conv3d_wgrad_batch, sfh_conv3d_wgrad_batch_supported, sfh_conv3d_wgrad_batch_workspace_bytes added;
 * SFH_KERNEL_SPLIT (6) is a value sfh_conv3d_launch_geometry may report. Nothing removed or changed.
 * 105: SFH_FLAG_SHARE_DEVICE; sfh_conv3d_wgrad_batch_workspace_bytes takes the call's flags (changed: one more argument). */
int sfh_version(void);
const char* sfh_last_error(void);
/* Fills name (<= name_len bytes), compute-unit count, LDS bytes per workgroup. */
int sfh_device_info(char* name, size_t name_len, int32_t* compute_units, int32_t* lds_bytes);
/* The compute-unit count the launch geometry (persistent grids, split counts) is written for: 256, MI355X. Split
 * counts -- and with them the summation order of split results -- are functions of the problem shape and of this
 * constant alone, never of the device the call runs on, so results are the same bits on every device; on a device
 * with another count the geometry is merely not the best one (compare with sfh_device_info). No counterpart in
 * the reference (its split counts are functions of shape and a compiled-in target as well,
 * triton_conv3d/reduce_gemm.py:71-96). */
int sfh_tuned_compute_units(void);
/* Output spatial extents of a conv3d problem; SFH_ERR_INVALID if the output would be empty. */
int sfh_conv3d_out_shape(const sfh_conv3d_desc* p, int32_t out_dhw[3]);
/* 1 if the MFMA implicit-GEMM kernels (rather than the direct kernels) serve this problem
 * in the given direction: 0 = forward, 1 = data-gradient, 2 = weight-gradient. SFH_BF16 / SFH_FP16
 * problems run on the 16-bit matrix pipe with fp32 accumulation; SFH_FP32 problems of the tiled shape
 * (3x3x3, stride 1, channel counts multiples of 16 / 32) on the fp32 matrix pipe with fp32 operands and
 * products, the precision the reference asks of its fp32 path (gather_gemm.py:1334, "ieee"). */
int sfh_conv3d_uses_mfma(const sfh_conv3d_desc* p, int dtype, int direction);
/* Which kernel serves a problem in a direction (0 forward, 1 data-gradient, 2 weight-gradient) and with what launch
 * geometry: geometry[0] = SFH_KERNEL_*, [1] = output voxels per workgroup step, [2] = 32-channel output blocks a
 * workgroup produces from one staged brick, [3] = slices of the reduction (channels for forward / data-gradient,
 * voxels for the weight gradient) whose fp32 partials are summed in fixed order. A pure function of the problem and
 * the compute-unit count the library is written for -- the property the reference's plan machinery exists to
 * guarantee (triton_conv3d/_rungs.py, reduce_gemm.py:71-96: the split count must not depend on the device or the
 * run). [1] and [2] are 0 for SFH_KERNEL_DIRECT (the direct and the thin-channel kernels: whatever
 * sfh_conv3d_uses_mfma answers 0 for) and SFH_KERNEL_OTHER_MATRIX (2x2x2 family, fp32 tiles). */
#define SFH_KERNEL_DIRECT 0
#define SFH_KERNEL_PERSIST 1
#define SFH_KERNEL_BRICK 2
#define SFH_KERNEL_WIDE 3
#define SFH_KERNEL_WGRAD 4
#define SFH_KERNEL_OTHER_MATRIX 5
#define SFH_KERNEL_SPLIT 6 /* 64-voxel bricks, the reduction cut over the wavefronts of a workgroup: one slice in memory */
int sfh_conv3d_launch_geometry(const sfh_conv3d_desc* p, int dtype, int direction, int32_t geometry[4]);

/* ---- measurement: what the matrix pipe sustains ----------------------------------------
 * No counterpart in the reference's operator interface; its bench measures its ceiling with a vendor GEMM
 * (triton_conv3d/bench/baseline.py). One launch of `workgroups` 4-wavefront workgroups (one per CU at 256), each
 * wavefront running `tiles` x 216 v_mfma_f32_32x32x16_bf16 on four accumulators, under one of three instruction mixes:
 *   0  nothing but the MFMAs;   1  plus one 16-byte LDS read per two MFMAs (the persistent 3x3x3 convolution's
 *      operand rate): the ceiling for that kernel's instruction mix without any global memory traffic;
 *   2  plus, per tile and workgroup, 48 KiB of direct-to-LDS loads streaming through src and 32 KiB of stores
 *      streaming through sink, and a barrier per tile (the convolution's traffic per 512-voxel step, all of it from
 *      and to HBM: a reference point, not a bound -- the convolution finds its halo rows in L2).
 * operands: 64 KiB of bf16 bits the MFMAs multiply (the sustained clock depends on them: Gaussian values and zeros are
 * the two cases worth timing); src / sink: 1 MiB .. 2 GiB each, multiples of 1 KiB, only read / written by mix 2 (may be
 * NULL otherwise); out: workgroups * 256 floats. The caller times the launch; sfh_mfma_ceiling_probe_flops gives its
 * FLOP count. */
double sfh_mfma_ceiling_probe_flops(int32_t workgroups, int32_t tiles);
int sfh_mfma_ceiling_probe(int32_t mix, int32_t workgroups, int32_t tiles, const void* operands, const void* src,
                           size_t src_bytes, void* sink, size_t sink_bytes, float* out, void* stream);

/* ---- conv3d forward ------------------------------------------------------------------
 * Stands in for triton_conv3d.conv3d_forward (triton_conv3d/gather_gemm.py:1187) and its
 * kernel _conv3d_fwd_kernel (gather_gemm.py:112).
 * y[n,co,od,oh,ow] = bias[co] + sum_{ci,kd,kh,kw} x[n,ci,od*sd+kd*dd-pd,...] * w[co,ci,kd,kh,kw]
 * bias may be NULL; when given it has Cout elements of the activation dtype.
 * The workspace holds the weight repacked into MFMA fragment order (16-bit and fp32 tiled problems). */
size_t sfh_conv3d_fwd_workspace_bytes(const sfh_conv3d_desc* p, int dtype);
int sfh_conv3d_fwd(const sfh_conv3d_desc* p, int dtype, const void* x, const void* w,
                   const int64_t w_stride[5], const void* bias, void* y, void* workspace,
                   size_t workspace_bytes, uint32_t flags, void* stream);
/* The forward that also leaves the GroupNorm statistics of its output, so that the normalisation after it
 * (unet_parts.py:123-160: every convolution of a DoubleConv is followed by GroupNorm + ReLU) does not read the tensor
 * a first time to find them: the reference's traffic model of GroupNorm (triton_group_norm.py:116, x read twice, y
 * written once) becomes one read and one write. Every workgroup of the convolution leaves, per group, the Welford
 * record { count, mean, M2, 0 } of the ROUNDED values it stored, gn_partials[N][records][groups][4] in fp32 -- every slot
 * written by exactly one workgroup, no atomics, the same bits on every run -- and sfh_groupnorm_fwd_from_partials
 * merges the records in a fixed order with the pairwise rule of the reference's tile statistics
 * (triton_group_norm.py:148-165,594-607). A record is a function of the values it covers alone: inside a workgroup the
 * sums are taken about one of its own outputs, so the variance does not cancel however large the mean is against the
 * spread, nothing is carried from call to call and nothing comes from the caller.
 * sfh_conv3d_fwd_gn_records gives `records` for a problem and group count, a pure function of both; 0 means
 * the kernel that serves the problem does not offer it (direct / fp32 / 2x2x2 kernels, thin-channel ones other than
 * the one-channel 3x3x3 stem, several samples on the persistent kernel, groups of fewer than 4 or a non-multiple-of-4
 * channels) and the caller uses sfh_conv3d_fwd and
 * the ordinary GroupNorm. 16-bit dtypes only. gn_partials must be 16-byte aligned. */
int32_t sfh_conv3d_fwd_gn_records(const sfh_conv3d_desc* p, int dtype, int groups);
int sfh_conv3d_fwd_gn(const sfh_conv3d_desc* p, int dtype, const void* x, const void* w,
                      const int64_t w_stride[5], const void* bias, void* y, void* workspace,
                      size_t workspace_bytes, uint32_t flags, int groups, float* gn_partials,
                      size_t gn_partials_bytes, void* stream);

/* ---- conv3d data gradient ------------------------------------------------------------
 * Stands in for triton_conv3d.conv3d_backward_data (triton_conv3d/bwd_data.py:275).
 * `p` describes the FORWARD problem; gy has its output shape, gx its input shape.
 * Served for stride 1 and padding <= dilation*(k-1) only (bwd_data.py:250-253). */
size_t sfh_conv3d_dgrad_workspace_bytes(const sfh_conv3d_desc* p, int dtype);
int sfh_conv3d_dgrad(const sfh_conv3d_desc* p, int dtype, const void* gy, const void* w,
                     const int64_t w_stride[5], void* gx, void* workspace,
                     size_t workspace_bytes, uint32_t flags, void* stream);

/* ---- packing a weight once for both directions ------------------------------------------
 * The MFMA kernels read the weight in fragment order; sfh_conv3d_fwd / _dgrad repack it on every
 * call (the reference transforms nothing, gather_gemm.py:894-942, and this keeps that contract by
 * default). A caller that runs forward and data gradient with one weight (every training step)
 * can pack both forms in ONE launch here and pass them with SFH_FLAG_WEIGHT_PACKED.
 * sfh_conv3d_packed_weight_bytes: bytes of the packed form for direction 0 (forward) or
 * 1 (data gradient), 0 when that direction of this problem does not read a packed weight.
 * Either output of sfh_conv3d_pack_weights may be NULL. For a 2x2x2 stride-2 problem the forward
 * form is what sfh_conv3d_fwd reads, and the data-gradient form is what sfh_convT3d_fwd -- the
 * transposed convolution, which IS that data gradient -- reads under SFH_FLAG_WEIGHT_PACKED
 * (describe the up-convolution's weight (Cin_T, Cout_T, 2,2,2) as the stride-2 convolution with
 * cout = Cin_T, cin = Cout_T over the up-convolution's output extents). No counterpart in the
 * reference. */
size_t sfh_conv3d_packed_weight_bytes(const sfh_conv3d_desc* p, int dtype, int direction);
int sfh_conv3d_pack_weights(const sfh_conv3d_desc* p, int dtype, const void* w,
                            const int64_t w_stride[5], void* packed_fwd, void* packed_dgrad,
                            void* stream);

/* The packings of many weights in as few launches as possible (a training loop repacks every
 * convolution weight once per optimizer step). Each item is one sfh_conv3d_pack_weights call;
 * all weights share `dtype`. No counterpart in the reference. */
typedef struct sfh_pack_item {
  sfh_conv3d_desc desc;
  const void* w;
  int64_t w_stride[5];
  void* packed_fwd;   /* may be NULL */
  void* packed_dgrad; /* may be NULL */
} sfh_pack_item;
int sfh_conv3d_pack_weights_batch(const sfh_pack_item* items, int32_t nitems, int dtype,
                                  void* stream);

/* ---- conv3d weight gradient ----------------------------------------------------------
 * Stands in for triton_conv3d.conv3d_backward_weight (triton_conv3d/reduce_gemm.py:1177),
 * _conv3d_bwd_weight_kernel (:137) and _reduce_partials_kernel (:396).
 * gw is written dense as [Cout][kd][kh][kw][Cin] (channels_last_3d for a weight) in the
 * activation dtype, from fp32 split partials summed in a fixed order.
 * sfh_conv3d_wgrad_splits() reports the number of partial slices (1 = no workspace pass). */
int sfh_conv3d_wgrad_splits(const sfh_conv3d_desc* p, int dtype);
size_t sfh_conv3d_wgrad_workspace_bytes(const sfh_conv3d_desc* p, int dtype);
int sfh_conv3d_wgrad(const sfh_conv3d_desc* p, int dtype, const void* x, const void* gy, void* gw,
                     void* workspace, size_t workspace_bytes, uint32_t flags, void* stream);

/* ---- conv3d over a skip connection that is never concatenated -----------------------------
 * The decoder's first convolution reads torch.cat([skip, upsampled], dim=1) (unet_parts.py:107-120 writes that tensor,
 * unet_parts.py:123-160 convolves it). Here the convolution takes the two tensors themselves: x_first holds the first
 * cin_first input channels of every voxel, x_second the other p->cin - cin_first, both dense channels-last over the
 * same (N, in_d, in_h, in_w) voxels; `p`, the weight and every other argument are those of the convolution over the
 * concatenation. The forward stages each 32-channel chunk of its reduction from the tensor that holds it; the data
 * gradient stores each 32-channel block of its result into gx_first or gx_second (what the concatenation's backward
 * would have split); the weight gradient reads each 32-channel input block from its tensor. Every result is, bit for
 * bit, that of the ordinary entry point on the concatenated tensor -- the same kernels, launch geometry and summation
 * order -- while the concatenated activation and its gradient are neither written nor read (4 bytes x voxels x Cin of
 * HBM traffic per direction pair, and the memory of both tensors).
 * sfh_conv3d_pair_supported: 1 when `direction` (0 forward, 1 data gradient, 2 weight gradient) of the problem takes
 * the cut, a pure function of problem, dtype and cut: 16-bit MFMA problems with cin_first a multiple of 32; the forward
 * of a 64-channel output over 128 or more input channels at rows of more than 16 voxels (SFH_KERNEL_WIDE) only when
 * the two tensors have the same channel count (a data gradient whose reduction is sliced, geometry[3] > 1, writes the
 * two tensors from the sum of its slices). A caller asks for all three before it drops its concatenation, and
 * concatenates otherwise.
 * sfh_conv3d_fwd_pair with groups > 0 also leaves the GroupNorm partials of sfh_conv3d_fwd_gn (same records, same
 * arguments); groups = 0 and NULL / 0 for the two gn arguments is the plain forward. Workspaces are those of the
 * ordinary entry points. SFH_FLAG_FORCE_GENERIC is refused. */
int sfh_conv3d_pair_supported(const sfh_conv3d_desc* p, int dtype, int32_t cin_first, int direction);
int sfh_conv3d_fwd_pair(const sfh_conv3d_desc* p, int dtype, const void* x_first, const void* x_second,
                        int32_t cin_first, const void* w, const int64_t w_stride[5], const void* bias, void* y,
                        void* workspace, size_t workspace_bytes, uint32_t flags, int groups,
                        float* gn_partials, size_t gn_partials_bytes, void* stream);
int sfh_conv3d_dgrad_pair(const sfh_conv3d_desc* p, int dtype, const void* gy, const void* w,
                          const int64_t w_stride[5], void* gx_first, void* gx_second, int32_t cin_first,
                          void* workspace, size_t workspace_bytes, uint32_t flags, void* stream);
int sfh_conv3d_wgrad_pair(const sfh_conv3d_desc* p, int dtype, const void* x_first, const void* x_second,
                          int32_t cin_first, const void* gy, void* gw, void* workspace, size_t workspace_bytes,
                          uint32_t flags, void* stream);

/* ---- several conv3d weight gradients in one launch ------------------------------------------
 * The weight gradients of a training step (triton_conv3d.conv3d_backward_weight once per convolution,
 * triton_conv3d/reduce_gemm.py:1177; nothing reads them before the optimizer, ScaFFold/utils/trainer.py:678-694) as ONE
 * few launches instead of one kernel launch and one sum pass per convolution: what a launch of sfh_conv3d_wgrad costs
 * whatever the problem -- all workgroups fetching their first operands at once, all writing their partial slice at once,
 * the sum pass reading the slices back, two launch gaps: 15-20 us on MI355X -- is paid once for up to
 * SFH_WGRAD_BATCH_MAX problems. Problems with output rows of more than 16 voxels share one launch and one sum pass: the
 * work of all of them is laid on one line and cut evenly over the workgroups; a workgroup that covers parts of several
 * 32 x 32 channel blocks writes a slice for each. Small-volume problems (rows of 16 or 8 voxels, at most 32 tiles of
 * 256 voxels) share a second launch in which every 32 x 32 block is walked from its first tile to its last by one
 * workgroup and stored straight into the gradient: no slices, no sum pass. Each item is one sfh_conv3d_wgrad
 * (x_second NULL) or sfh_conv3d_wgrad_pair call; all share `dtype` and the gradient dtype (SFH_FLAG_GRAD_FP32).
 * Results: every gradient is the sum of fp32 partials in a fixed order that is a pure function of the LIST of problems
 * (their shapes, in order) -- the same bits on every run, and within fp32 summation-order rounding of
 * sfh_conv3d_wgrad's (whose cuts differ).
 * Served: the problems sfh_conv3d_wgrad_batch_supported answers 1 for -- 3 x 3 x 3, unit stride and dilation, SFH_BF16 /
 * SFH_FP16, channel counts multiples of 32, and either rows of more than 16 voxels or a small volume as above; anything
 * else in the list fails the call with SFH_ERR_UNSUPPORTED before any launch (the caller runs those through
 * sfh_conv3d_wgrad). The workspace query answers 0 for a refused list and is never 0 for a served one.
 * The batching itself has no counterpart in the reference. */
#define SFH_WGRAD_BATCH_MAX 16
typedef struct sfh_conv3d_wgrad_item {
  sfh_conv3d_desc desc;
  const void* x;        /* the input, or its first cin_first channels when x_second is given */
  const void* x_second; /* NULL: one tensor */
  int32_t cin_first;
  const void* gy;
  void* gw;             /* [Cout][3][3][3][Cin] dense */
} sfh_conv3d_wgrad_item;
/* 0: not served in a batch; 1: served, in the launch of the problems with rows of more than 16 voxels; 2: served, in the
 * launch of the small-volume problems (a caller with more than SFH_WGRAD_BATCH_MAX problems fills its calls by family). */
int sfh_conv3d_wgrad_batch_supported(const sfh_conv3d_desc* p, int dtype);
size_t sfh_conv3d_wgrad_batch_workspace_bytes(const sfh_conv3d_wgrad_item* items, int32_t count, int dtype,
                                              uint32_t flags); /* pointers unused; flags as in the call; 0: refused */
int sfh_conv3d_wgrad_batch(const sfh_conv3d_wgrad_item* items, int32_t count, int dtype, void* workspace,
                           size_t workspace_bytes, uint32_t flags, void* stream);

/* Weight gradient and bias gradient from one pass over gy, where the kernel that serves the problem reads gy tile by tile
 * anyway: the 1x1x1 convolutions with at most 32 output channels over 32 / 64 / 128 input channels (the U-Net's head),
 * 16-bit dtypes. gb: Cout elements in gw's dtype (the operands', or fp32 with SFH_FLAG_GRAD_FP32) =
 * gy.sum over voxels (ScaFFold/unet/conv3d.py:1231), fp32 slices summed in a fixed order. The workspace query returns 0
 * and the call SFH_ERR_UNSUPPORTED for every other problem: the caller then uses sfh_conv3d_wgrad and sfh_bias_grad. */
size_t sfh_conv3d_wgrad_bias_workspace_bytes(const sfh_conv3d_desc* p, int dtype);
int sfh_conv3d_wgrad_bias(const sfh_conv3d_desc* p, int dtype, const void* x, const void* gy, void* gw, void* gb,
                          void* workspace, size_t workspace_bytes, uint32_t flags, void* stream);

/* ---- bias gradient --------------------------------------------------------------------
 * Stands in for `grad_output.sum((0, 2, 3, 4))` in the reference's autograd functions
 * (ScaFFold/unet/conv3d.py:1231 for conv3d, :1786 for the transposed conv).
 * g: dense (rows, channels) of `dtype` (rows = N*D*H*W of a channels-last gradient);
 * gb: `channels` elements of `out_dtype`; fp32 accumulation in a fixed order. */
size_t sfh_bias_grad_workspace_bytes(int64_t rows, int32_t channels);
int sfh_bias_grad(int dtype, int out_dtype, const void* g, int64_t rows, int32_t channels, void* gb,
                  void* workspace, size_t workspace_bytes, void* stream);

/* ---- transposed conv3d (kernel == stride) forward ------------------------------------
 * Stands in for triton_conv3d.conv_transpose3d_forward (triton_conv3d/transposed.py:941)
 * and _convT3d_fwd_kernel (:135).
 * y[n,oc,d*kd+a,h*kh+b,w*kw+c] = bias[oc] + sum_ic x[n,ic,d,h,w] * w[ic,oc,a,b,c].
 * Its data gradient is sfh_conv3d_fwd at stride k (transposed.py:1073) and its weight
 * gradient sfh_conv3d_wgrad at stride k with the operands swapped (transposed.py:1113). */
size_t sfh_convT3d_fwd_workspace_bytes(const sfh_convT3d_desc* p, int dtype);
int sfh_convT3d_fwd(const sfh_convT3d_desc* p, int dtype, const void* x, const void* w,
                    const int64_t w_stride[5], const void* bias, void* y, void* workspace,
                    size_t workspace_bytes, uint32_t flags, void* stream);
/* The same with y written into the interior of a depth slab: y_slab holds halo_elems elements of face, the result, and
 * halo_elems elements of face again; the launch zeroes both faces. One sample, the 2x2x2 matrix-core kernel only
 * (16-bit dtypes, channel counts multiples of 32), faces and tensor multiples of 16 bytes: SFH_ERR_UNSUPPORTED otherwise.
 * With halo_elems = 0 it is sfh_convT3d_fwd. The decoder's up-convolution feeds a convolution whose halo exchange
 * (ScaFFold/unet/conv3d.py:769-776) assembles exactly this buffer; here its producer writes it in place. */
int sfh_convT3d_fwd_slab(const sfh_convT3d_desc* p, int dtype, const void* x, const void* w,
                         const int64_t w_stride[5], const void* bias, void* y_slab, int64_t halo_elems,
                         void* workspace, size_t workspace_bytes, uint32_t flags, void* stream);

/* Weight gradient AND bias gradient of the transposed convolution from one pass over its output gradient gy
 * (the reference computes them apart: transposed.py:1113 and `grad_output.sum((0, 2, 3, 4))`, ScaFFold/unet/conv3d.py:1786).
 * gw: [Cin][kd][kh][kw][Cout] dense, as sfh_conv3d_wgrad writes it for the swapped problem; gb: Cout elements; both in the
 * operands' dtype, or fp32 with SFH_FLAG_GRAD_FP32; fp32 partial slices summed in a fixed order, no atomics. 2x2x2
 * problems on the matrix cores only (16-bit dtypes, Cin a multiple of 64, Cout of 32): SFH_ERR_UNSUPPORTED otherwise, and
 * the workspace query returns 0. */
size_t sfh_convT3d_wgrad_bias_workspace_bytes(const sfh_convT3d_desc* p, int dtype);
int sfh_convT3d_wgrad_bias(const sfh_convT3d_desc* p, int dtype, const void* x, const void* gy, void* gw, void* gb,
                           void* workspace, size_t workspace_bytes, uint32_t flags, void* stream);

/* ---- GroupNorm forward ---------------------------------------------------------------
 * Stands in for torch.ops.scaffold_gn.group_norm (ScaFFold/unet/triton_group_norm.py:1339)
 * and its kernels _stats_partial_kernel (:609) and _normalize_kernel (:697).
 * x: (N,S,C) of x_dtype; gamma/beta: C elements of param_dtype or NULL; y: (N,S,C) of
 * y_dtype; mean, rstd: (N, groups) fp32. Statistics and the normalisation are fp32. */
size_t sfh_groupnorm_fwd_workspace_bytes(const sfh_groupnorm_desc* p, int x_dtype);
int sfh_groupnorm_fwd(const sfh_groupnorm_desc* p, int x_dtype, int y_dtype, int param_dtype,
                      const void* x, const void* gamma, const void* beta, void* y, float* mean,
                      float* rstd, void* workspace, size_t workspace_bytes, void* stream);
/* The same with the result written into the interior of a slab: y_slab is
 * (N, halo_rows + S + halo_rows, C) and its two faces of halo_rows rows per sample are set to
 * zero. With S = D*H*W and halo_rows = h*H*W that is the input a depth shard's convolution reads
 * after the halo exchange (ScaFFold/unet/conv3d.py:648-677), produced without a copy of the
 * interior; a neighbour's planes, where there is one, overwrite the zero faces. The output must
 * have the input's element width. Same workspace as sfh_groupnorm_fwd. */
int sfh_groupnorm_fwd_slab(const sfh_groupnorm_desc* p, int x_dtype, int y_dtype, int param_dtype,
                           const void* x, const void* gamma, const void* beta, void* y_slab,
                           int64_t halo_rows, float* mean, float* rstd, void* workspace,
                           size_t workspace_bytes, void* stream);
/* The same again with the statistics merged from the Welford records the producer of x left (sfh_conv3d_fwd_gn):
 * partials[N][records][groups][4] = { count, mean, M2, - } in fp32, 16-byte aligned, partials_bytes of them
 * (SFH_ERR_WORKSPACE when that is less than N * records * groups * 16). The merge is the reference's
 * (triton_group_norm.py:594-607) in fixed order; the result depends on the records alone.
 * No statistics pass and no workspace; halo_rows may be 0 (y_slab is then a plain output). Needs the vector path
 * (16-byte aligned tensors, channel counts the 16-byte vectors divide): SFH_ERR_UNSUPPORTED otherwise. */
int sfh_groupnorm_fwd_from_partials(const sfh_groupnorm_desc* p, int x_dtype, int y_dtype, int param_dtype,
                                    const void* x, const void* gamma, const void* beta, void* y_slab,
                                    int64_t halo_rows, float* mean, float* rstd, const float* partials,
                                    size_t partials_bytes, int32_t records, void* stream);

/* The forward for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc. It has no counterpart in the reference. Same kernels and results as sfh_groupnorm_fwd, but the
 * scratch for the partial statistics is a device array inside the library (sfh_groupnorm_fwd_noalloc_max_bytes() =
 * 256 KiB, held by every GPU the library runs on until the process ends) instead of a workspace argument; neither this
 * call nor anything it calls allocates or frees memory. A problem whose scratch exceeds the built-in buffer returns
 * SFH_ERR_WORKSPACE (compare sfh_groupnorm_fwd_workspace_bytes with the maximum).
 * Device: the scratch used is the CURRENT device's copy of the array, not the copy of the device the pointers live
 * on -- the call does not look at its pointers' device. The caller must therefore have made the tensors' device current
 * (hipSetDevice / a device guard) before the call, exactly as for a kernel launch of its own; a call with another
 * device current would hand the kernels a scratch address of the wrong GPU.
 * Capture: the first call on a device looks the array's address up (once per device); that lookup must not run on a
 * capturing stream, so a first call that finds `stream` capturing is refused with SFH_ERR_INVALID. Call
 * sfh_groupnorm_fwd_noalloc_prepare() once per device, with that device current and before any capture, to do the lookup
 * ahead of time (idempotent, allocates nothing). At most 64 devices (SFH_ERR_UNSUPPORTED beyond).
 * All calls on one GPU share the buffer: calls that overlap in time on one GPU (two streams, or two captured graphs
 * replayed on different streams) race. */
size_t sfh_groupnorm_fwd_noalloc_max_bytes(void);
int sfh_groupnorm_fwd_noalloc_prepare(void);
int sfh_groupnorm_fwd_noalloc(const sfh_groupnorm_desc* p, int x_dtype, int y_dtype, int param_dtype,
                              const void* x, const void* gamma, const void* beta, void* y, float* mean,
                              float* rstd, void* stream);

/* ---- GroupNorm backward --------------------------------------------------------------
 * Stands in for torch.ops.scaffold_gn.group_norm_backward (triton_group_norm.py:1394) and
 * its kernels _bwd_partial_kernel (:813) and _dx_kernel (:908).
 * x, dx: (N,S,C) of x_dtype; dy: (N,S,C) of dy_dtype (x_dtype, or fp32 when the forward
 * produced an fp32 output from a 16-bit input); dgamma, dbeta: C fp32 elements each (either
 * may be NULL).
 * With p->relu the incoming gradient is gated on the recomputed pre-activation. */
size_t sfh_groupnorm_bwd_workspace_bytes(const sfh_groupnorm_desc* p, int x_dtype);
int sfh_groupnorm_bwd(const sfh_groupnorm_desc* p, int x_dtype, int dy_dtype, int param_dtype,
                      const void* dy, const void* x, const void* gamma, const void* beta, const float* mean,
                      const float* rstd, void* dx, float* dgamma, float* dbeta, void* workspace,
                      size_t workspace_bytes, void* stream);

/* ---- loss head ------------------------------------------------------------------------
 * Stands in for the loss block of the reference's train step (ScaFFold/utils/trainer.py:634-663):
 * fp32 log-softmax of the class logits, cross entropy summed and divided by its normaliser
 * (ScaFFold/utils/losses.py:119-214; the voxel count, or the sum of the target weights when class
 * weights are given), soft Dice per (sample, class) (ScaFFold/utils/dice_score.py:101-136) and
 *   loss = CE + 1 - mean over samples and classes >= 1 of (2 I + eps) / (P + T + eps).
 * logits: dense (N, S, classes) of `dtype` (a channels-last (N, classes, D, H, W) tensor);
 * labels: (N, S) int64, values outside [0, classes) contribute nothing; class_weight: `classes`
 * floats or NULL; loss: one float; stats: N*3*classes + 2 floats kept for the backward.
 * The backward writes d loss / d logits * grad_loss[0] in `dtype`. 2 <= classes <= 32. */
typedef struct sfh_loss_desc {
  int32_t n, classes;
  int64_t spatial;
  float eps;
} sfh_loss_desc;
size_t sfh_ce_dice_workspace_bytes(const sfh_loss_desc* p);
int sfh_ce_dice_fwd(const sfh_loss_desc* p, int dtype, const void* logits, const int64_t* labels,
                    const float* class_weight, float* loss, float* stats, void* workspace,
                    size_t workspace_bytes, void* stream);
int sfh_ce_dice_bwd(const sfh_loss_desc* p, int dtype, const void* logits, const int64_t* labels,
                    const float* class_weight, const float* stats, const float* grad_loss,
                    void* dlogits, void* stream);

/* ---- 2x2x2 max pooling --------------------------------------------------------------------
 * The down-sampling step between U-Net levels, nn.MaxPool3d(2) in the reference
 * (ScaFFold/unet/unet_parts.py:165), on dense channels-last tensors: x (N, D, H, W, C),
 * y (N, D/2, H/2, W/2, C) of `dtype`. Stock semantics: odd trailing planes are dropped, ties go to
 * the first voxel of the cell in depth-major order, a NaN wins over any number. `idx` gets one
 * byte per output element (which of the eight voxels, kd*4 + kh*2 + kw) and is what the backward
 * needs besides grad_y; the backward writes every element of grad_x. */
typedef struct sfh_pool_desc {
  int32_t n, c, in_d, in_h, in_w;
} sfh_pool_desc;
int sfh_maxpool2_fwd(const sfh_pool_desc* p, int dtype, const void* x, void* y, uint8_t* idx,
                     void* stream);
/* The same with y written into the interior of a depth slab: y_slab holds halo_elems elements of face, the pooled
 * tensor, and halo_elems elements of face again; the launch zeroes both faces (one sample; faces and tensor multiples of
 * 16 bytes, else SFH_ERR_UNSUPPORTED). It is the [recv_minus | x | recv_plus] buffer of the halo exchange
 * (ScaFFold/unet/conv3d.py:769-776) for the convolution that follows the pooling, produced without a copy. */
int sfh_maxpool2_fwd_slab(const sfh_pool_desc* p, int dtype, const void* x, void* y_slab, int64_t halo_elems,
                          uint8_t* idx, void* stream);
int sfh_maxpool2_bwd(const sfh_pool_desc* p, int dtype, const void* grad_y, const uint8_t* idx,
                     void* grad_x, void* stream);
/* grad_x = (the pooling gradient) + add, summed in fp32 and rounded once; `add` has the input's
 * shape. In the U-Net the pooled tensor is also the skip connection (unet_model.py:141-155): its
 * two gradients meet here instead of in a separate addition. */
int sfh_maxpool2_bwd_add(const sfh_pool_desc* p, int dtype, const void* grad_y, const uint8_t* idx,
                         const void* add, void* grad_x, void* stream);

/* ---- halo slab assembly ------------------------------------------------------------------
 * The local step of a depth shard's forward halo exchange: out = [lo | x | hi] along depth, where
 * lo / hi are the `halo` boundary planes received from the lower / upper neighbour, or NULL for
 * zeros (no neighbour) -- what ScaFFold/unet/conv3d.py:769-776 builds with three strided copies
 * after its receives. x (N, D, H, W, C), lo / hi (N, halo, H, W, C), out (N, D + 2*halo, H, W, C),
 * all dense channels-last of `dtype`. The convolution then runs on `out` at depth padding 0. */
typedef struct sfh_halo_desc {
  int32_t n, c, d, h, w, halo;
} sfh_halo_desc;
int sfh_halo_assemble(const sfh_halo_desc* p, int dtype, const void* x, const void* lo,
                      const void* hi, void* out, void* stream);
/* The sending side of the same exchange, and its backward. sfh_halo_pack gathers the boundary planes a
 * shard sends into plain dense buffers (the wire format of ScaFFold/unet/conv3d.py:710-731,757-768):
 * lo_out (N, halo, H, W, C) = x[:, :halo] for the lower neighbour, hi_out = x[:, D - halo:] for the
 * upper one; either may be NULL (no such neighbour). In the backward exchange (conv3d.py:795-841) the
 * same call on the slab's gradient (depth D + 2*halo) packs the outer planes that go back to their
 * owners, and sfh_halo_accumulate adds what came back into the shard's own boundary planes, in place:
 * g[:, :halo] += lo_in, g[:, D - halo:] += hi_in (fp32 sum, one rounding; NULL = nothing received),
 * g (N, D, H, W, C) being the interior of that gradient. D >= 2*halo is required so the two ranges
 * stay disjoint (the reference requires a shard at least two voxels thick, conv3d.py:669). */
int sfh_halo_pack(const sfh_halo_desc* p, int dtype, const void* x, void* lo_out, void* hi_out,
                  void* stream);
int sfh_halo_accumulate(const sfh_halo_desc* p, int dtype, void* g, const void* lo_in,
                        const void* hi_in, void* stream);

/* ---- skip connection concat ---------------------------------------------------------------
 * torch.cat([skip, upsampled], dim=1) of the decoder (ScaFFold/unet/unet_parts.py:107-120) on
 * channels-last tensors, one streaming pass: out (N, halo_rows + rows + halo_rows, c_a + c_b) gets
 * [a (N, rows, c_a) | b (N, rows, c_b)] in its interior and zeros in its faces. With rows = D*H*W
 * and halo_rows = h*H*W the result is the slab a depth shard's convolution reads (see
 * sfh_halo_assemble); halo_rows = 0 is the plain concatenation. The backward copies the two channel
 * ranges of the interior of g (laid out like out) into ga and gb. Both channel counts must fill
 * whole 16-byte pieces of `dtype`; pointers 16-byte aligned. */
typedef struct sfh_concat_desc {
  int32_t n, c_a, c_b;
  int64_t rows, halo_rows;
} sfh_concat_desc;
int sfh_skip_concat_fwd(const sfh_concat_desc* p, int dtype, const void* a, const void* b, void* out,
                        void* stream);
int sfh_skip_concat_bwd(const sfh_concat_desc* p, int dtype, const void* g, void* ga, void* gb,
                        void* stream);

/* ---- shard ingest ---------------------------------------------------------------------------
 * From a dataset shard as stored on disk to the tensors the step reads. The generator writes a
 * volume as float32 (C, D, H, W) and its mask as uint16 (D, H, W), one pair of .npy files per
 * physical shard (ScaFFold/datagen/volumegen.py:259-292; file names `{id}_shard{k:06d}.npy` and
 * `{id}_shard{k:06d}_mask.npy`, ScaFFold/utils/spatial_sharding.py:130-133,
 * ScaFFold/utils/data_loading.py:308-317). The trainer then does, on the device,
 * images.to(float32, memory_format=channels_last_3d) and masks.to(torch.long)
 * (ScaFFold/utils/trainer.py:572-589), and autocast rounds the volume to the compute type before the
 * first convolution. This entry point is those three steps in one pass over a batch already in
 * device memory: x (N, halo_rows + rows + halo_rows, c) of `dtype` gets the channels-last volume in
 * its interior (bit copy for SFH_FP32, one round-to-nearest-even otherwise) and zeros in its faces;
 * labels (N, rows) int64 gets the widened mask. rows = D*H*W; halo_rows = h*H*W makes x the slab a
 * depth shard's first convolution reads (see sfh_halo_assemble), 0 the plain tensor. `mask` holds
 * 16-bit integers: unsigned as in the file (mask_signed = 0) or the loader's signed carrier
 * (mask_signed = 1; ScaFFold/utils/data_loading.py:540-545); mask and labels may both be NULL.
 * c is 1..4. Any alignment is accepted; 16-byte aligned pointers with rows % 4 == 0 take the
 * vector path. */
typedef struct sfh_ingest_desc {
  int32_t n, c, mask_signed;
  int64_t rows, halo_rows;
} sfh_ingest_desc;
int sfh_shard_ingest(const sfh_ingest_desc* p, int dtype, const void* volume, const void* mask, void* x,
                     void* labels, void* stream);

/* ---- gradient clipping + Adam -----------------------------------------------------------
 * The optimizer step of the trainer: torch.nn.utils.clip_grad_norm_(parameters, max_norm) followed by
 * torch.optim.Adam.step() (ScaFFold/utils/trainer.py:678-694, optimizer built at trainer.py:268-274),
 * over `ntensors` dense fp32 tensors given as HOST arrays of device pointers and element counts
 * (every count >= 1). Pass 1 writes one fp32 slot per 8192-element chunk (sfh_adam_slots of them) and
 * adds 1 to the device float `step`; pass 2 (which may cover a subset of the tensors, e.g. one
 * hyperparameter group) folds all `nslots` slots in a fixed order, scales each gradient
 * by min(1, max_norm / (norm + 1e-6)) on the fly (gradients are not modified; max_norm <= 0: no
 * clipping) and applies Adam with torch's formulas (lerp first moment, bias corrections from
 * `step`, denom = sqrt(v)/sqrt(1-beta2^step) + eps, weight_decay added to the gradient). `shadow`
 * (NULL, or an array whose entries may be NULL) receives each updated parameter rounded to
 * shadow_dtype (SFH_BF16 / SFH_FP16): the copy autocast would otherwise make in the next step.
 * `grad_norm` (may be NULL) receives the unclipped total norm. Nothing synchronises; the pointers
 * are passed to the kernels by value, so the two calls can be captured in a graph. */
typedef struct sfh_adam_desc {
  float lr, beta1, beta2, eps, weight_decay, max_norm;
  int32_t shadow_dtype; /* SFH_BF16, SFH_FP16, or -1 for none */
} sfh_adam_desc;
int64_t sfh_adam_slots(int32_t ntensors, const int64_t* numel);
int sfh_adam_grad_sumsq(int32_t ntensors, const float* const* grads, const int64_t* numel,
                        float* slots, float* step, void* stream);
int sfh_adam_clip_step(const sfh_adam_desc* d, int32_t ntensors, float* const* params,
                       const float* const* grads, float* const* exp_avg, float* const* exp_avg_sq,
                       void* const* shadow, const int64_t* numel, const float* slots,
                       int64_t nslots, const float* step, float* grad_norm, void* stream);

/* ---- measurement helper --------------------------------------------------------------
 * A plain streaming copy of `bytes` bytes (multiple of 16) used to calibrate achieved HBM
 * bandwidth and the scale of the FETCH_SIZE / WRITE_SIZE counters. Has no counterpart in the
 * reference (its bench harness times torch copies, triton_conv3d/bench/harness.py:62). */
int sfh_stream_copy(const void* src, void* dst, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SCAFFOLD_HIP_H */
