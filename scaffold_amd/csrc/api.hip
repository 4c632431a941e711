// extern "C" entry points of libscaffold_hip.so: argument checking, kernel selection (a pure
// function of descriptor and dtype), workspace carving. No allocation, no synchronisation.
#include <string.h>

#include "common.hpp"
#include "concat.hpp"
#include "ingest.hpp"
#include "conv_direct.hpp"
#include "conv_mfma.hpp"
#include "conv_f32.hpp"
#include "conv_patch.hpp"
#include "conv_thin.hpp"
#include "halo.hpp"
#include "loss.hpp"
#include "reduce.hpp"
#include "optim.hpp"
#include "pool.hpp"
#include "wgrad_mfma.hpp"

namespace sfh {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return SFH_OK;
  return fail(SFH_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
}

namespace {

int check_conv(const sfh_conv3d_desc* p, int dtype, int32_t out[3]) {
  if (p == nullptr) return fail(SFH_ERR_INVALID, "conv3d: null descriptor");
  if (!dtype_ok(dtype)) return fail(SFH_ERR_INVALID, "conv3d: bad dtype %d", dtype);
  if (p->n < 0 || p->cin < 1 || p->cout < 1 || p->in_d < 1 || p->in_h < 1 || p->in_w < 1)
    return fail(SFH_ERR_INVALID, "conv3d: bad extents n=%d cin=%d cout=%d in=%dx%dx%d", p->n, p->cin, p->cout, p->in_d, p->in_h,
                p->in_w);
  if (p->kd < 1 || p->kh < 1 || p->kw < 1 || p->sd < 1 || p->sh < 1 || p->sw < 1 || p->dd < 1 || p->dh < 1 || p->dw < 1 ||
      p->pd < 0 || p->ph < 0 || p->pw < 0)
    return fail(SFH_ERR_INVALID, "conv3d: kernel/stride/dilation must be >= 1 and padding >= 0");
  const int in[3] = {p->in_d, p->in_h, p->in_w}, k[3] = {p->kd, p->kh, p->kw}, s[3] = {p->sd, p->sh, p->sw},
            pad[3] = {p->pd, p->ph, p->pw}, dil[3] = {p->dd, p->dh, p->dw};
  for (int i = 0; i < 3; ++i) {
    const int64_t eff = (int64_t)dil[i] * (k[i] - 1) + 1;
    if ((int64_t)in[i] + 2 * pad[i] < eff) return fail(SFH_ERR_INVALID, "conv3d: kernel wider than the padded input on axis %d", i);
    out[i] = (int32_t)(((int64_t)in[i] + 2 * pad[i] - eff) / s[i] + 1);
  }
  return SFH_OK;
}

bool is_unit(const sfh_conv3d_desc& p) {
  return p.sd == 1 && p.sh == 1 && p.sw == 1 && p.dd == 1 && p.dh == 1 && p.dw == 1;
}

MfmaConvArgs fwd_mfma_args(const sfh_conv3d_desc& p, const int32_t out[3]) {
  MfmaConvArgs a{};
  a.n = p.n; a.cred = p.cin; a.id = p.in_d; a.ih = p.in_h; a.iw = p.in_w;
  a.cout = p.cout; a.od = out[0]; a.oh = out[1]; a.ow = out[2];
  a.kd = p.kd; a.kh = p.kh; a.kw = p.kw; a.pd = p.pd; a.ph = p.ph; a.pw = p.pw;
  return a;
}

// The data gradient as a gather over gy: reduction channels = Cout, produced = Cin,
// padding dil*(k-1) - p, output extents = the forward's input extents.
MfmaConvArgs dgrad_mfma_args(const sfh_conv3d_desc& p, const int32_t out[3]) {
  MfmaConvArgs a{};
  a.n = p.n; a.cred = p.cout; a.id = out[0]; a.ih = out[1]; a.iw = out[2];
  a.cout = p.cin; a.od = p.in_d; a.oh = p.in_h; a.ow = p.in_w;
  a.kd = p.kd; a.kh = p.kh; a.kw = p.kw;
  a.pd = (p.kd - 1) - p.pd; a.ph = (p.kh - 1) - p.ph; a.pw = (p.kw - 1) - p.pw;
  return a;
}

bool fwd_uses_mfma(const sfh_conv3d_desc& p, int dtype, const int32_t out[3]) {
  return is_unit(p) && mfma_conv_supported(fwd_mfma_args(p, out), dtype);
}
// fp32 problems of the tiled shape run on the fp32 matrix pipe (the weight is packed per call into the workspace)
bool on_16_bytes(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }  // null counts as aligned

bool fwd_uses_f32_tiles(const sfh_conv3d_desc& p, int dtype, const int32_t out[3]) {
  return dtype == SFH_FP32 && is_unit(p) && f32_conv_supported(fwd_mfma_args(p, out));
}

int check_dgrad(const sfh_conv3d_desc& p) {
  if (p.sd != 1 || p.sh != 1 || p.sw != 1)
    return fail(SFH_ERR_UNSUPPORTED, "conv3d dgrad: served at stride 1 only (got %d,%d,%d)", p.sd, p.sh, p.sw);
  if (p.pd > p.dd * (p.kd - 1) || p.ph > p.dh * (p.kh - 1) || p.pw > p.dw * (p.kw - 1))
    return fail(SFH_ERR_UNSUPPORTED, "conv3d dgrad: padding must not exceed dilation*(k-1)");
  if (p.n < 1) return fail(SFH_ERR_UNSUPPORTED, "conv3d dgrad: empty batch");
  return SFH_OK;
}

bool dgrad_uses_mfma(const sfh_conv3d_desc& p, int dtype, const int32_t out[3]) {
  return is_unit(p) && mfma_conv_supported(dgrad_mfma_args(p, out), dtype);
}
bool dgrad_uses_f32_tiles(const sfh_conv3d_desc& p, int dtype, const int32_t out[3]) {
  return dtype == SFH_FP32 && is_unit(p) && f32_conv_supported(dgrad_mfma_args(p, out));
}

WgradArgs wgrad_args(const sfh_conv3d_desc& p, const int32_t out[3]) {
  WgradArgs a{};
  a.n = p.n; a.cin = p.cin; a.id = p.in_d; a.ih = p.in_h; a.iw = p.in_w;
  a.cout = p.cout; a.od = out[0]; a.oh = out[1]; a.ow = out[2];
  a.pd = p.pd; a.ph = p.ph; a.pw = p.pw;
  return a;
}

bool wgrad_uses_mfma(const sfh_conv3d_desc& p, int dtype, const int32_t out[3]) {
  return is_unit(p) && p.kd == 3 && p.kh == 3 && p.kw == 3 && p.n >= 1 && mfma_wgrad_supported(wgrad_args(p, out), dtype);
}

bool wgrad_uses_f32_tiles(const sfh_conv3d_desc& p, int dtype, const int32_t out[3]) {
  return dtype == SFH_FP32 && is_unit(p) && p.kd == 3 && p.kh == 3 && p.kw == 3 && p.n >= 1 && f32_wgrad_supported(wgrad_args(p, out));
}

// ---- 2x2x2, stride-2, unpadded problems (the up-convolution family) ------------------------------
bool is_patch(const sfh_conv3d_desc& p) {
  return p.kd == 2 && p.kh == 2 && p.kw == 2 && p.sd == 2 && p.sh == 2 && p.sw == 2 && p.pd == 0 && p.ph == 0 && p.pw == 0 &&
         p.dd == 1 && p.dh == 1 && p.dw == 1;
}

// The strided convolution's input is the big volume, its output the small one.
PatchArgs patch_args(const sfh_conv3d_desc& p, const int32_t out[3]) {
  PatchArgs a{};
  a.n = p.n;
  a.cbig = p.cin; a.bd = p.in_d; a.bh = p.in_h; a.bw = p.in_w;
  a.csmall = p.cout; a.sd = out[0]; a.sh = out[1]; a.sw = out[2];
  return a;
}

bool fwd_uses_patch(const sfh_conv3d_desc& p, int dtype, const int32_t out[3]) {
  return is_patch(p) && patch_supported(patch_args(p, out), dtype);
}

bool wgrad_uses_patch(const sfh_conv3d_desc& p, int dtype, const int32_t out[3]) {
  return is_patch(p) && patch_reduce_supported(patch_args(p, out), dtype);
}

// Weight of the strided convolution in fragment order: produced = Cout, reduced = Cin.
MfmaConvArgs patch_pack_args(int produced, int reduced) {
  MfmaConvArgs a{};
  a.cout = produced; a.cred = reduced; a.kd = 2; a.kh = 2; a.kw = 2;
  return a;
}

PatchArgs convT_patch_args(const sfh_convT3d_desc& p) {
  PatchArgs a{};
  a.n = p.n;
  a.cbig = p.cout; a.bd = 2 * p.in_d; a.bh = 2 * p.in_h; a.bw = 2 * p.in_w;
  a.csmall = p.cin; a.sd = p.in_d; a.sh = p.in_h; a.sw = p.in_w;
  return a;
}

bool convT_uses_patch(const sfh_convT3d_desc& p, int dtype) {
  return p.kd == 2 && p.kh == 2 && p.kw == 2 && p.n >= 1 && patch_supported(convT_patch_args(p), dtype);
}

// The transposed convolution that is the data gradient of the kernel == stride convolution `p` (its input is p's output).
sfh_convT3d_desc transposed_of(const sfh_conv3d_desc& p, const int32_t out[3]) {
  sfh_convT3d_desc t{};
  t.n = p.n; t.cin = p.cout; t.in_d = out[0]; t.in_h = out[1]; t.in_w = out[2];
  t.cout = p.cin; t.kd = p.kd; t.kh = p.kh; t.kw = p.kw;
  return t;
}

// One packing job of a weight (Cout, Cin, k, k, k) with element strides ws[5].
struct PackSpec {
  bool any;
  MfmaConvArgs a;
  int64_t s_out, s_red;
  int flip;
};

// What the forward of `p` reads: the tiled 3x3x3 kernels' form, or the 2x2x2 stride-2 gather's.
PackSpec fwd_pack_spec(const sfh_conv3d_desc& p, int dtype, const int32_t out[3], const int64_t ws[5]) {
  if (fwd_uses_mfma(p, dtype, out)) return {true, fwd_mfma_args(p, out), ws[0], ws[1], 0};
  if (fwd_uses_patch(p, dtype, out)) return {true, patch_pack_args(p.cout, p.cin), ws[0], ws[1], 0};
  return {false, MfmaConvArgs{}, 0, 0, 0};
}

// What the data gradient of `p` reads: the tiled kernels' transposed, tap-flipped form, or -- for a 2x2x2 stride-2
// problem, whose data gradient is the transposed convolution -- the scatter's (produced = Cin, reduced = Cout).
PackSpec dgrad_pack_spec(const sfh_conv3d_desc& p, int dtype, const int32_t out[3], const int64_t ws[5]) {
  if (check_dgrad(p) == SFH_OK && dgrad_uses_mfma(p, dtype, out)) return {true, dgrad_mfma_args(p, out), ws[1], ws[0], 1};
  if (is_patch(p) && convT_uses_patch(transposed_of(p, out), dtype)) return {true, patch_pack_args(p.cin, p.cout), ws[1], ws[0], 0};
  return {false, MfmaConvArgs{}, 0, 0, 0};
}

// ---- thin-channel problems (Cin == 1 stems, 1x1x1 heads) ---------------------------------------
bool is_pointwise(const sfh_conv3d_desc& p) {
  return p.kd == 1 && p.kh == 1 && p.kw == 1 && p.sd == 1 && p.sh == 1 && p.sw == 1 && p.pd == 0 && p.ph == 0 && p.pw == 0;
}

bool is_one_channel_cube(const sfh_conv3d_desc& p) {
  return p.cin == 1 && p.kd == p.kh && p.kh == p.kw && (p.kd == 2 || p.kd == 3);
}

ThinArgs thin_base(const sfh_conv3d_desc& p, const int32_t out[3]) {
  ThinArgs a{};
  a.n = p.n; a.od = out[0]; a.oh = out[1]; a.ow = out[2];
  a.td = p.in_d; a.th = p.in_h; a.tw = p.in_w;
  a.sd = p.sd; a.sh = p.sh; a.sw = p.sw; a.pd = p.pd; a.ph = p.ph; a.pw = p.pw; a.dd = p.dd; a.dh = p.dh; a.dw = p.dw;
  return a;
}

enum ThinKind { kThinNone = 0, kThinWideOut, kThinOut, kThinReduce };

// Forward: y[v][co]. Returns the kernel family and fills `a` (weight strides left to the caller).
ThinKind thin_fwd_plan(const sfh_conv3d_desc& p, int dtype, const int32_t out[3], ThinArgs& a) {
  a = thin_base(p, out);
  if (is_one_channel_cube(p)) {
    a.K = p.kd; a.J = p.kd * p.kh * p.kw; a.ct = 1; a.cw = p.cout;
    return thin_supported(a, dtype) ? kThinWideOut : kThinNone;
  }
  if (!is_pointwise(p)) return kThinNone;
  a.K = 0;
  a.J = p.cin; a.ct = p.cin; a.cw = p.cout;
  if (p.cin <= 32 && thin_supported(a, dtype)) return kThinWideOut;
  a.J = p.cout; a.ct = p.cout; a.cw = p.cin;
  if (p.cout <= 32 && thin_supported(a, dtype)) return kThinOut;
  return kThinNone;
}

// Data gradient of a pointwise conv: gx[v][ci] = sum_co gy[v][co] * w[co][ci].
ThinKind thin_dgrad_plan(const sfh_conv3d_desc& p, int dtype, const int32_t out[3], ThinArgs& a) {
  a = thin_base(p, out);
  if (!is_pointwise(p)) return kThinNone;
  a.K = 0;
  a.J = p.cout; a.ct = p.cout; a.cw = p.cin;
  if (p.cout <= 32 && thin_supported(a, dtype)) return kThinWideOut;
  a.J = p.cin; a.ct = p.cin; a.cw = p.cout;
  if (p.cin <= 32 && thin_supported(a, dtype)) return kThinOut;
  return kThinNone;
}

// Weight gradient, dense [Cout][taps][Cin]. `thin_is_x` tells which operand is the thin one.
ThinKind thin_wgrad_plan(const sfh_conv3d_desc& p, int dtype, const int32_t out[3], ThinArgs& a, bool& thin_is_x) {
  a = thin_base(p, out);
  if (p.n < 1) return kThinNone;
  if (is_one_channel_cube(p)) {
    a.K = p.kd; a.J = p.kd * p.kh * p.kw; a.ct = 1; a.cw = p.cout;
    a.so_wide = a.J; a.so_thin = 1;
    thin_is_x = true;
    return thin_supported(a, dtype) ? kThinReduce : kThinNone;
  }
  if (!is_pointwise(p)) return kThinNone;
  a.K = 0;
  a.J = p.cout; a.ct = p.cout; a.cw = p.cin; a.so_wide = 1; a.so_thin = p.cin;
  thin_is_x = false;
  if (p.cout <= 32 && thin_supported(a, dtype)) return kThinReduce;
  a.J = p.cin; a.ct = p.cin; a.cw = p.cout; a.so_wide = p.cin; a.so_thin = 1;
  thin_is_x = true;
  if (p.cin <= 32 && thin_supported(a, dtype)) return kThinReduce;
  return kThinNone;
}

__global__ void __launch_bounds__(256) stream_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  for (; i < n; i += stride) dst[i] = src[i];
}

}  // namespace
}  // namespace sfh

using namespace sfh;

extern "C" int sfh_version(void) { return 105; }

extern "C" const char* sfh_last_error(void) { return g_error; }

extern "C" int sfh_device_info(char* name, size_t name_len, int32_t* compute_units, int32_t* lds_bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(SFH_ERR_LAUNCH, "no HIP device");
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return fail(SFH_ERR_LAUNCH, "hipGetDeviceProperties failed");
  if (name != nullptr && name_len > 0) {
    strncpy(name, prop.gcnArchName, name_len - 1);
    name[name_len - 1] = 0;
  }
  if (compute_units != nullptr) *compute_units = prop.multiProcessorCount;
  if (lds_bytes != nullptr) *lds_bytes = (int32_t)prop.sharedMemPerBlock;
  return SFH_OK;
}

extern "C" int sfh_tuned_compute_units(void) { return kComputeUnits; }

extern "C" int sfh_conv3d_out_shape(const sfh_conv3d_desc* p, int32_t out_dhw[3]) {
  if (out_dhw == nullptr) return fail(SFH_ERR_INVALID, "conv3d: null output");
  return check_conv(p, SFH_FP32, out_dhw);
}

extern "C" int sfh_conv3d_uses_mfma(const sfh_conv3d_desc* p, int dtype, int direction) {
  int32_t out[3];
  if (check_conv(p, dtype, out) != SFH_OK) return 0;
  if (direction == 0) return (fwd_uses_mfma(*p, dtype, out) || fwd_uses_patch(*p, dtype, out) || fwd_uses_f32_tiles(*p, dtype, out)) ? 1 : 0;
  if (direction == 1)
    return (check_dgrad(*p) == SFH_OK && (dgrad_uses_mfma(*p, dtype, out) || dgrad_uses_f32_tiles(*p, dtype, out))) ? 1 : 0;
  return (wgrad_uses_mfma(*p, dtype, out) || wgrad_uses_patch(*p, dtype, out) || wgrad_uses_f32_tiles(*p, dtype, out)) ? 1 : 0;
}

extern "C" int sfh_conv3d_launch_geometry(const sfh_conv3d_desc* p, int dtype, int direction, int32_t geometry[4]) {
  if (geometry == nullptr) return fail(SFH_ERR_INVALID, "conv3d geometry: null output");
  geometry[0] = SFH_KERNEL_DIRECT; geometry[1] = geometry[2] = 0; geometry[3] = 1;
  int32_t out[3];
  if (int rc = check_conv(p, dtype, out)) return rc;
  if (direction < 0 || direction > 2) return fail(SFH_ERR_INVALID, "conv3d geometry: direction %d", direction);
  if (!sfh_conv3d_uses_mfma(p, dtype, direction)) return SFH_OK;
  geometry[0] = SFH_KERNEL_OTHER_MATRIX;
  if (direction == 2) {
    if (!wgrad_uses_mfma(*p, dtype, out)) return SFH_OK;
    geometry[0] = SFH_KERNEL_WGRAD; geometry[1] = 256; geometry[2] = 1;
    geometry[3] = mfma_wgrad_splits(wgrad_args(*p, out));
    return SFH_OK;
  }
  if (direction == 0 ? !fwd_uses_mfma(*p, dtype, out) : !dgrad_uses_mfma(*p, dtype, out)) return SFH_OK;
  const MfmaConvGeometry g = mfma_conv_geometry(direction == 0 ? fwd_mfma_args(*p, out) : dgrad_mfma_args(*p, out));
  geometry[0] = g.kernel; geometry[1] = g.voxels; geometry[2] = g.blocks; geometry[3] = g.slices;
  return SFH_OK;
}

// ---- forward ---------------------------------------------------------------------------
extern "C" size_t sfh_conv3d_fwd_workspace_bytes(const sfh_conv3d_desc* p, int dtype) {
  int32_t out[3];
  if (check_conv(p, dtype, out) != SFH_OK) return 0;
  if (fwd_uses_patch(*p, dtype, out)) return mfma_conv_packed_weight_bytes(patch_pack_args(p->cout, p->cin));
  if (fwd_uses_f32_tiles(*p, dtype, out)) return f32_conv_packed_weight_bytes(fwd_mfma_args(*p, out));
  if (!fwd_uses_mfma(*p, dtype, out)) return 0;
  return mfma_conv_packed_weight_bytes(fwd_mfma_args(*p, out)) + mfma_conv_partial_bytes(fwd_mfma_args(*p, out));
}

static int conv3d_fwd_any(const sfh_conv3d_desc* p, int dtype, const void* x, const void* w, const int64_t w_stride[5],
                          const void* bias, void* y, void* workspace, size_t workspace_bytes, uint32_t flags, void* stream,
                          const GnPartialOut* gn, const ChannelPair* in2 = nullptr) {
  int32_t out[3];
  if (int rc = check_conv(p, dtype, out)) return rc;
  if (x == nullptr || w == nullptr || y == nullptr || (w_stride == nullptr && !(flags & SFH_FLAG_WEIGHT_PACKED)))
    return fail(SFH_ERR_INVALID, "conv3d fwd: null tensor");
  if (p->n == 0) return SFH_OK;
  hipStream_t st = (hipStream_t)stream;
  if (!(flags & SFH_FLAG_FORCE_GENERIC) && fwd_uses_mfma(*p, dtype, out)) {
    const MfmaConvArgs a = fwd_mfma_args(*p, out);
    const size_t packed_bytes = mfma_conv_packed_weight_bytes(a), partial_bytes = mfma_conv_partial_bytes(a);
    if (flags & SFH_FLAG_WEIGHT_PACKED) {  // w is the packed weight; the workspace only holds the partial slices
      if (partial_bytes && (workspace == nullptr || workspace_bytes < partial_bytes))
        return fail(SFH_ERR_WORKSPACE, "conv3d fwd: workspace of %zu bytes needed, got %zu", partial_bytes, workspace_bytes);
      return mfma_conv_persist(a, dtype, x, w, bias, y, partial_bytes ? workspace : nullptr, st, gn, in2);
    }
    const size_t need = packed_bytes + partial_bytes;
    if (workspace == nullptr || workspace_bytes < need)
      return fail(SFH_ERR_WORKSPACE, "conv3d fwd: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    if (int rc = mfma_pack_weight(a, dtype, w, w_stride[0], w_stride[1], w_stride[2], w_stride[3], w_stride[4], 0, workspace, st))
      return rc;
    void* partial = partial_bytes ? (char*)workspace + packed_bytes : nullptr;
    return mfma_conv_persist(a, dtype, x, workspace, bias, y, partial, st, gn, in2);
  }
  if (in2 != nullptr) return fail(SFH_ERR_UNSUPPORTED, "conv3d fwd: this problem does not take its input as two tensors");
  if (gn != nullptr) {  // the one-channel stem is the only other kernel that leaves them
    ThinArgs t;
    if ((flags & SFH_FLAG_WEIGHT_PACKED) || thin_fwd_plan(*p, dtype, out, t) != kThinWideOut || thin_wide_out_gn_records(t, dtype, gn->groups) == 0)
      return fail(SFH_ERR_UNSUPPORTED, "conv3d fwd: GroupNorm partials are not offered for this problem");
    t.ws_kd = w_stride[2]; t.ws_kh = w_stride[3]; t.ws_kw = w_stride[4];
    t.ws_wide = w_stride[0]; t.ws_thin = w_stride[1];
    return thin_wide_out(t, dtype, x, w, bias, y, st, gn);
  }
  // the fp32 tiles move 16-byte pieces of x, bias and y: a view 4 bytes off that grid runs the direct kernel instead
  if (!(flags & (SFH_FLAG_FORCE_GENERIC | SFH_FLAG_WEIGHT_PACKED)) && fwd_uses_f32_tiles(*p, dtype, out) && on_16_bytes(x) &&
      on_16_bytes(y) && on_16_bytes(bias)) {
    const MfmaConvArgs a = fwd_mfma_args(*p, out);
    const size_t need = f32_conv_packed_weight_bytes(a);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(SFH_ERR_WORKSPACE, "conv3d fwd: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    if (int rc = f32_pack_weight(a, w, w_stride[0], w_stride[1], w_stride[2], w_stride[3], w_stride[4], 0, workspace, st)) return rc;
    return f32_conv(a, x, workspace, bias, y, st);
  }
  if (!(flags & SFH_FLAG_FORCE_GENERIC) && (flags & SFH_FLAG_WEIGHT_PACKED) && fwd_uses_patch(*p, dtype, out))
    return patch_gather(patch_args(*p, out), dtype, x, w, bias, y, st);
  if (flags & SFH_FLAG_WEIGHT_PACKED) return fail(SFH_ERR_INVALID, "conv3d fwd: this problem does not read a packed weight");
  if (!(flags & SFH_FLAG_FORCE_GENERIC) && fwd_uses_patch(*p, dtype, out)) {
    const MfmaConvArgs pk = patch_pack_args(p->cout, p->cin);
    const size_t need = mfma_conv_packed_weight_bytes(pk);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(SFH_ERR_WORKSPACE, "conv3d fwd: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    if (int rc = mfma_pack_weight(pk, dtype, w, w_stride[0], w_stride[1], w_stride[2], w_stride[3], w_stride[4], 0, workspace, st))
      return rc;
    return patch_gather(patch_args(*p, out), dtype, x, workspace, bias, y, st);
  }
  if (!(flags & SFH_FLAG_FORCE_GENERIC)) {
    ThinArgs t;
    const ThinKind kind = thin_fwd_plan(*p, dtype, out, t);
    t.ws_kd = w_stride[2]; t.ws_kh = w_stride[3]; t.ws_kw = w_stride[4];
    if (kind == kThinWideOut) {
      t.ws_wide = w_stride[0]; t.ws_thin = w_stride[1];
      return thin_wide_out(t, dtype, x, w, bias, y, st);
    }
    if (kind == kThinOut) {
      t.ws_wide = w_stride[1]; t.ws_thin = w_stride[0];
      return thin_out(t, dtype, x, w, bias, y, st);
    }
  }
  DirectConvArgs a{};
  a.n = p->n; a.cin = p->cin; a.id = p->in_d; a.ih = p->in_h; a.iw = p->in_w;
  a.cout = p->cout; a.od = out[0]; a.oh = out[1]; a.ow = out[2];
  a.kd = p->kd; a.kh = p->kh; a.kw = p->kw; a.sd = p->sd; a.sh = p->sh; a.sw = p->sw;
  a.pd = p->pd; a.ph = p->ph; a.pw = p->pw; a.dd = p->dd; a.dh = p->dh; a.dw = p->dw;
  a.flip = 0;
  a.ws_co = w_stride[0]; a.ws_ci = w_stride[1]; a.ws_kd = w_stride[2]; a.ws_kh = w_stride[3]; a.ws_kw = w_stride[4];
  return direct_conv_gather(a, dtype, x, w, bias, y, st);
}

extern "C" int sfh_conv3d_fwd(const sfh_conv3d_desc* p, int dtype, const void* x, const void* w, const int64_t w_stride[5],
                              const void* bias, void* y, void* workspace, size_t workspace_bytes, uint32_t flags, void* stream) {
  return conv3d_fwd_any(p, dtype, x, w, w_stride, bias, y, workspace, workspace_bytes, flags, stream, nullptr);
}

extern "C" int32_t sfh_conv3d_fwd_gn_records(const sfh_conv3d_desc* p, int dtype, int groups) {
  int32_t out[3];
  if (check_conv(p, dtype, out) != SFH_OK || groups < 1 || p->n == 0) return 0;
  if (fwd_uses_mfma(*p, dtype, out)) return mfma_conv_gn_records(fwd_mfma_args(*p, out), groups);
  if (fwd_uses_f32_tiles(*p, dtype, out) || fwd_uses_patch(*p, dtype, out)) return 0;
  ThinArgs t;
  if (thin_fwd_plan(*p, dtype, out, t) == kThinWideOut) return thin_wide_out_gn_records(t, dtype, groups);
  return 0;
}

extern "C" int sfh_conv3d_fwd_gn(const sfh_conv3d_desc* p, int dtype, const void* x, const void* w, const int64_t w_stride[5],
                                 const void* bias, void* y, void* workspace, size_t workspace_bytes, uint32_t flags, int groups,
                                 float* gn_partials, size_t gn_partials_bytes, void* stream) {
  if (flags & SFH_FLAG_FORCE_GENERIC) return fail(SFH_ERR_INVALID, "conv3d fwd: the direct kernels leave no GroupNorm partials");
  const int32_t records = sfh_conv3d_fwd_gn_records(p, dtype, groups);
  if (records == 0) return fail(SFH_ERR_UNSUPPORTED, "conv3d fwd: GroupNorm partials are not offered for this problem");
  const size_t need = (size_t)p->n * records * groups * kGnRecordFloats * sizeof(float);
  if (gn_partials == nullptr || gn_partials_bytes < need || (reinterpret_cast<uintptr_t>(gn_partials) & 15u) != 0)
    return fail(SFH_ERR_WORKSPACE, "conv3d fwd: GroupNorm partials need %zu bytes at a 16-byte boundary, got %zu", need, gn_partials_bytes);
  const GnPartialOut gn{gn_partials, groups, p->cout / groups, records};
  return conv3d_fwd_any(p, dtype, x, w, w_stride, bias, y, workspace, workspace_bytes, flags, stream, &gn);
}

// ---- packing a weight once for both directions ------------------------------------------------
extern "C" size_t sfh_conv3d_packed_weight_bytes(const sfh_conv3d_desc* p, int dtype, int direction) {
  int32_t out[3];
  if (check_conv(p, dtype, out) != SFH_OK) return 0;
  const int64_t unit[5] = {1, 1, 1, 1, 1};
  const PackSpec spec = direction == 0 ? fwd_pack_spec(*p, dtype, out, unit)
                                       : direction == 1 ? dgrad_pack_spec(*p, dtype, out, unit) : PackSpec{false, MfmaConvArgs{}, 0, 0, 0};
  return spec.any ? mfma_conv_packed_weight_bytes(spec.a) : 0;
}

// Appends the packings one weight asks for (its forward form and / or its data-gradient form) to jobs[njobs...]; the
// caller leaves room for two.
static int collect_pack_jobs(const sfh_conv3d_desc* p, int dtype, const void* w, const int64_t* w_stride, void* packed_fwd,
                             void* packed_dgrad, MfmaPackItem* jobs, int* njobs) {
  int32_t out[3];
  if (int rc = check_conv(p, dtype, out)) return rc;
  if (w == nullptr || w_stride == nullptr) return fail(SFH_ERR_INVALID, "conv3d pack: null weight");
  if (packed_fwd != nullptr) {
    const PackSpec spec = fwd_pack_spec(*p, dtype, out, w_stride);
    if (!spec.any) return fail(SFH_ERR_UNSUPPORTED, "conv3d pack: the forward of this problem does not read a packed weight");
    jobs[(*njobs)++] = MfmaPackItem{spec.a, w, spec.s_out, spec.s_red, w_stride[2], w_stride[3], w_stride[4], spec.flip, packed_fwd};
  }
  if (packed_dgrad != nullptr) {
    const PackSpec spec = dgrad_pack_spec(*p, dtype, out, w_stride);
    if (!spec.any) return fail(SFH_ERR_UNSUPPORTED, "conv3d pack: the data gradient of this problem does not read a packed weight");
    jobs[(*njobs)++] = MfmaPackItem{spec.a, w, spec.s_out, spec.s_red, w_stride[2], w_stride[3], w_stride[4], spec.flip, packed_dgrad};
  }
  return SFH_OK;
}

extern "C" int sfh_conv3d_pack_weights(const sfh_conv3d_desc* p, int dtype, const void* w, const int64_t w_stride[5], void* packed_fwd,
                                       void* packed_dgrad, void* stream) {
  MfmaPackItem jobs[2];
  int njobs = 0;
  if (int rc = collect_pack_jobs(p, dtype, w, w_stride, packed_fwd, packed_dgrad, jobs, &njobs)) return rc;
  if (njobs == 0) return SFH_OK;
  return mfma_pack_weight_batch(jobs, njobs, dtype, (hipStream_t)stream);
}

extern "C" int sfh_conv3d_pack_weights_batch(const sfh_pack_item* items, int32_t nitems, int dtype, void* stream) {
  if (nitems < 0 || (nitems > 0 && items == nullptr)) return fail(SFH_ERR_INVALID, "conv3d pack batch: bad item list");
  // Every item is validated before the first launch (a bad item must leave nothing half done), then the jobs go out in
  // groups of a fixed-size array on the stack: nothing on this path touches the heap.
  {
    MfmaPackItem probe[2];
    for (int i = 0; i < nitems; ++i) {
      int n = 0;
      if (int rc = collect_pack_jobs(&items[i].desc, dtype, items[i].w, items[i].w_stride, items[i].packed_fwd, items[i].packed_dgrad,
                                     probe, &n))
        return rc;
    }
  }
  constexpr int kGroup = 46;  // (an item adds up to two jobs; 48 jobs are one launch)
  MfmaPackItem jobs[kGroup + 2];
  int njobs = 0;
  for (int i = 0; i < nitems; ++i) {
    collect_pack_jobs(&items[i].desc, dtype, items[i].w, items[i].w_stride, items[i].packed_fwd, items[i].packed_dgrad, jobs, &njobs);
    if (njobs >= kGroup || i + 1 == nitems) {
      if (njobs > 0)
        if (int rc = mfma_pack_weight_batch(jobs, njobs, dtype, (hipStream_t)stream)) return rc;
      njobs = 0;
    }
  }
  return SFH_OK;
}

// ---- data gradient ---------------------------------------------------------------------
extern "C" size_t sfh_conv3d_dgrad_workspace_bytes(const sfh_conv3d_desc* p, int dtype) {
  int32_t out[3];
  if (check_conv(p, dtype, out) != SFH_OK) return 0;
  if (check_dgrad(*p) != SFH_OK) return 0;
  if (dgrad_uses_f32_tiles(*p, dtype, out)) return f32_conv_packed_weight_bytes(dgrad_mfma_args(*p, out));
  if (!dgrad_uses_mfma(*p, dtype, out)) return 0;
  return mfma_conv_packed_weight_bytes(dgrad_mfma_args(*p, out)) + mfma_conv_partial_bytes(dgrad_mfma_args(*p, out));
}

static int conv3d_dgrad_any(const sfh_conv3d_desc* p, int dtype, const void* gy, const void* w, const int64_t w_stride[5],
                            void* gx, void* workspace, size_t workspace_bytes, uint32_t flags, void* stream, const ChannelPair* out2) {
  int32_t out[3];
  if (int rc = check_conv(p, dtype, out)) return rc;
  if (int rc = check_dgrad(*p)) return rc;
  if (gy == nullptr || w == nullptr || gx == nullptr || (w_stride == nullptr && !(flags & SFH_FLAG_WEIGHT_PACKED)))
    return fail(SFH_ERR_INVALID, "conv3d dgrad: null tensor");
  hipStream_t st = (hipStream_t)stream;
  if (!(flags & SFH_FLAG_FORCE_GENERIC) && dgrad_uses_mfma(*p, dtype, out)) {
    const MfmaConvArgs a = dgrad_mfma_args(*p, out);
    const size_t packed_bytes = mfma_conv_packed_weight_bytes(a), partial_bytes = mfma_conv_partial_bytes(a);
    if (flags & SFH_FLAG_WEIGHT_PACKED) {
      if (partial_bytes && (workspace == nullptr || workspace_bytes < partial_bytes))
        return fail(SFH_ERR_WORKSPACE, "conv3d dgrad: workspace of %zu bytes needed, got %zu", partial_bytes, workspace_bytes);
      return mfma_conv_persist(a, dtype, gy, w, nullptr, gx, partial_bytes ? workspace : nullptr, st, nullptr, nullptr, out2);
    }
    const size_t need = packed_bytes + partial_bytes;
    if (workspace == nullptr || workspace_bytes < need)
      return fail(SFH_ERR_WORKSPACE, "conv3d dgrad: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    // produced channel = Cin (stride w_stride[1]), reduction channel = Cout (w_stride[0]), taps flipped
    if (int rc = mfma_pack_weight(a, dtype, w, w_stride[1], w_stride[0], w_stride[2], w_stride[3], w_stride[4], 1, workspace, st))
      return rc;
    void* partial = partial_bytes ? (char*)workspace + packed_bytes : nullptr;
    return mfma_conv_persist(a, dtype, gy, workspace, nullptr, gx, partial, st, nullptr, nullptr, out2);
  }
  if (out2 != nullptr) return fail(SFH_ERR_UNSUPPORTED, "conv3d dgrad: this problem does not write its result as two tensors");
  if (!(flags & (SFH_FLAG_FORCE_GENERIC | SFH_FLAG_WEIGHT_PACKED)) && dgrad_uses_f32_tiles(*p, dtype, out) && on_16_bytes(gy) &&
      on_16_bytes(gx)) {
    const MfmaConvArgs a = dgrad_mfma_args(*p, out);
    const size_t need = f32_conv_packed_weight_bytes(a);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(SFH_ERR_WORKSPACE, "conv3d dgrad: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    // produced channel = Cin (stride w_stride[1]), reduction channel = Cout (w_stride[0]), taps flipped
    if (int rc = f32_pack_weight(a, w, w_stride[1], w_stride[0], w_stride[2], w_stride[3], w_stride[4], 1, workspace, st)) return rc;
    return f32_conv(a, gy, workspace, nullptr, gx, st);
  }
  if (flags & SFH_FLAG_WEIGHT_PACKED) return fail(SFH_ERR_INVALID, "conv3d dgrad: this problem does not read a packed weight");
  if (!(flags & SFH_FLAG_FORCE_GENERIC)) {
    ThinArgs t;
    const ThinKind kind = thin_dgrad_plan(*p, dtype, out, t);
    if (kind == kThinWideOut) {
      t.ws_wide = w_stride[1]; t.ws_thin = w_stride[0];
      return thin_wide_out(t, dtype, gy, w, nullptr, gx, st);
    }
    if (kind == kThinOut) {
      t.ws_wide = w_stride[0]; t.ws_thin = w_stride[1];
      return thin_out(t, dtype, gy, w, nullptr, gx, st);
    }
  }
  DirectConvArgs a{};
  a.n = p->n; a.cin = p->cout; a.id = out[0]; a.ih = out[1]; a.iw = out[2];
  a.cout = p->cin; a.od = p->in_d; a.oh = p->in_h; a.ow = p->in_w;
  a.kd = p->kd; a.kh = p->kh; a.kw = p->kw; a.sd = 1; a.sh = 1; a.sw = 1;
  a.pd = p->dd * (p->kd - 1) - p->pd; a.ph = p->dh * (p->kh - 1) - p->ph; a.pw = p->dw * (p->kw - 1) - p->pw;
  a.dd = p->dd; a.dh = p->dh; a.dw = p->dw;
  a.flip = 1;
  a.ws_co = w_stride[1]; a.ws_ci = w_stride[0]; a.ws_kd = w_stride[2]; a.ws_kh = w_stride[3]; a.ws_kw = w_stride[4];
  return direct_conv_gather(a, dtype, gy, w, nullptr, gx, st);
}

extern "C" int sfh_conv3d_dgrad(const sfh_conv3d_desc* p, int dtype, const void* gy, const void* w, const int64_t w_stride[5],
                                void* gx, void* workspace, size_t workspace_bytes, uint32_t flags, void* stream) {
  return conv3d_dgrad_any(p, dtype, gy, w, w_stride, gx, workspace, workspace_bytes, flags, stream, nullptr);
}

// ---- weight gradient -------------------------------------------------------------------
extern "C" int sfh_conv3d_wgrad_splits(const sfh_conv3d_desc* p, int dtype) {
  int32_t out[3];
  if (check_conv(p, dtype, out) != SFH_OK) return 0;
  if (wgrad_uses_mfma(*p, dtype, out)) return mfma_wgrad_splits(wgrad_args(*p, out));
  if (wgrad_uses_f32_tiles(*p, dtype, out)) return f32_wgrad_splits(wgrad_args(*p, out));
  if (wgrad_uses_patch(*p, dtype, out)) return patch_reduce_splits(patch_args(*p, out));
  ThinArgs t;
  bool thin_is_x;
  if (thin_wgrad_plan(*p, dtype, out, t, thin_is_x) == kThinReduce) return thin_reduce_splits(t);
  return 1;
}

extern "C" size_t sfh_conv3d_wgrad_workspace_bytes(const sfh_conv3d_desc* p, int dtype) {
  int32_t out[3];
  if (check_conv(p, dtype, out) != SFH_OK) return 0;
  if (wgrad_uses_mfma(*p, dtype, out)) return mfma_wgrad_workspace_bytes(wgrad_args(*p, out));
  if (wgrad_uses_f32_tiles(*p, dtype, out)) return f32_wgrad_workspace_bytes(wgrad_args(*p, out));
  if (wgrad_uses_patch(*p, dtype, out)) return patch_reduce_workspace_bytes(patch_args(*p, out));
  ThinArgs t;
  bool thin_is_x;
  if (thin_wgrad_plan(*p, dtype, out, t, thin_is_x) == kThinReduce) return thin_reduce_workspace_bytes(t);
  return 0;
}

static int conv3d_wgrad_any(const sfh_conv3d_desc* p, int dtype, const void* x, const void* gy, void* gw, void* workspace,
                            size_t workspace_bytes, uint32_t flags, void* stream, const ChannelPair* x2) {
  int32_t out[3];
  if (int rc = check_conv(p, dtype, out)) return rc;
  if (x == nullptr || gy == nullptr || gw == nullptr) return fail(SFH_ERR_INVALID, "conv3d wgrad: null tensor");
  hipStream_t st = (hipStream_t)stream;
  const int gw_dtype = (flags & SFH_FLAG_GRAD_FP32) ? SFH_FP32 : dtype;
  if (!(flags & SFH_FLAG_FORCE_GENERIC) && wgrad_uses_mfma(*p, dtype, out)) {
    const WgradArgs a = wgrad_args(*p, out);
    const size_t need = mfma_wgrad_workspace_bytes(a);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(SFH_ERR_WORKSPACE, "conv3d wgrad: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    return mfma_wgrad(a, dtype, x, gy, gw, gw_dtype, workspace, st, x2);
  }
  if (x2 != nullptr) return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad: this problem does not take its input as two tensors");
  if (!(flags & SFH_FLAG_FORCE_GENERIC) && wgrad_uses_f32_tiles(*p, dtype, out)) {
    const WgradArgs a = wgrad_args(*p, out);
    const size_t need = f32_wgrad_workspace_bytes(a);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(SFH_ERR_WORKSPACE, "conv3d wgrad: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    return f32_wgrad(a, x, gy, gw, workspace, st);
  }
  if (!(flags & SFH_FLAG_FORCE_GENERIC) && wgrad_uses_patch(*p, dtype, out)) {
    const PatchArgs a = patch_args(*p, out);
    const size_t need = patch_reduce_workspace_bytes(a);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(SFH_ERR_WORKSPACE, "conv3d wgrad: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    return patch_reduce(a, dtype, gy, x, gw, gw_dtype, workspace, st);
  }
  if (!(flags & SFH_FLAG_FORCE_GENERIC)) {
    ThinArgs t;
    bool thin_is_x = false;
    if (thin_wgrad_plan(*p, dtype, out, t, thin_is_x) == kThinReduce) {
      const size_t need = thin_reduce_workspace_bytes(t);
      if (workspace == nullptr || workspace_bytes < need)
        return fail(SFH_ERR_WORKSPACE, "conv3d wgrad: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
      return thin_is_x ? thin_reduce(t, dtype, x, gy, gw, gw_dtype, workspace, st)
                       : thin_reduce(t, dtype, gy, x, gw, gw_dtype, workspace, st);
    }
  }
  if (gw_dtype != dtype)
    return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad: the untiled kernel writes the gradient in the operands' dtype only");
  DirectConvArgs a{};
  a.n = p->n; a.cin = p->cin; a.id = p->in_d; a.ih = p->in_h; a.iw = p->in_w;
  a.cout = p->cout; a.od = out[0]; a.oh = out[1]; a.ow = out[2];
  a.kd = p->kd; a.kh = p->kh; a.kw = p->kw; a.sd = p->sd; a.sh = p->sh; a.sw = p->sw;
  a.pd = p->pd; a.ph = p->ph; a.pw = p->pw; a.dd = p->dd; a.dh = p->dh; a.dw = p->dw;
  return direct_conv_wgrad(a, dtype, x, gy, gw, st);
}

extern "C" int sfh_conv3d_wgrad(const sfh_conv3d_desc* p, int dtype, const void* x, const void* gy, void* gw, void* workspace,
                                size_t workspace_bytes, uint32_t flags, void* stream) {
  return conv3d_wgrad_any(p, dtype, x, gy, gw, workspace, workspace_bytes, flags, stream, nullptr);
}

// ---- weight gradient with the bias gradient from the same pass (the 1x1x1 head) ------------------------------------
static bool wgrad_bias_plan(const sfh_conv3d_desc& p, int dtype, const int32_t out[3], ThinArgs& t) {
  bool thin_is_x = false;
  // the output gradient must be the thin operand: its sums over the voxels are the bias gradient
  return thin_wgrad_plan(p, dtype, out, t, thin_is_x) == kThinReduce && !thin_is_x && thin_reduce_offers_thin_sums(t, dtype);
}

extern "C" size_t sfh_conv3d_wgrad_bias_workspace_bytes(const sfh_conv3d_desc* p, int dtype) {
  int32_t out[3];
  ThinArgs t;
  if (check_conv(p, dtype, out) != SFH_OK || wgrad_uses_mfma(*p, dtype, out) || wgrad_uses_f32_tiles(*p, dtype, out) ||
      wgrad_uses_patch(*p, dtype, out) || !wgrad_bias_plan(*p, dtype, out, t))
    return 0;
  return thin_reduce_workspace_bytes(t, true);
}

extern "C" int sfh_conv3d_wgrad_bias(const sfh_conv3d_desc* p, int dtype, const void* x, const void* gy, void* gw, void* gb,
                                     void* workspace, size_t workspace_bytes, uint32_t flags, void* stream) {
  int32_t out[3];
  if (int rc = check_conv(p, dtype, out)) return rc;
  if (x == nullptr || gy == nullptr || gw == nullptr || gb == nullptr) return fail(SFH_ERR_INVALID, "conv3d wgrad: null tensor");
  const size_t need = sfh_conv3d_wgrad_bias_workspace_bytes(p, dtype);
  if ((flags & SFH_FLAG_FORCE_GENERIC) || need == 0)
    return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad with bias gradient: the 1x1x1 thin-output problems on the matrix cores only");
  if (workspace == nullptr || workspace_bytes < need)
    return fail(SFH_ERR_WORKSPACE, "conv3d wgrad: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
  ThinArgs t;
  wgrad_bias_plan(*p, dtype, out, t);
  const int g_dtype = (flags & SFH_FLAG_GRAD_FP32) ? SFH_FP32 : dtype;
  return thin_reduce(t, dtype, gy, x, gw, g_dtype, workspace, (hipStream_t)stream, gb);
}

// ---- a convolution over two tensors whose channels follow each other (the skip connection, never concatenated) ------
extern "C" int sfh_conv3d_pair_supported(const sfh_conv3d_desc* p, int dtype, int32_t cin_first, int direction) {
  int32_t out[3];
  if (check_conv(p, dtype, out) != SFH_OK || p->n == 0) return 0;
  if (direction == 0) return (fwd_uses_mfma(*p, dtype, out) && mfma_conv_pair_ok(fwd_mfma_args(*p, out), cin_first, false)) ? 1 : 0;
  if (direction == 1)
    return (check_dgrad(*p) == SFH_OK && dgrad_uses_mfma(*p, dtype, out) && mfma_conv_pair_ok(dgrad_mfma_args(*p, out), cin_first, true)) ? 1 : 0;
  if (direction == 2) return (wgrad_uses_mfma(*p, dtype, out) && mfma_wgrad_pair_ok(wgrad_args(*p, out), cin_first)) ? 1 : 0;
  return 0;
}

extern "C" int sfh_conv3d_fwd_pair(const sfh_conv3d_desc* p, int dtype, const void* x_first, const void* x_second, int32_t cin_first,
                                   const void* w, const int64_t w_stride[5], const void* bias, void* y, void* workspace,
                                   size_t workspace_bytes, uint32_t flags, int groups, float* gn_partials,
                                   size_t gn_partials_bytes, void* stream) {
  if (x_second == nullptr) return fail(SFH_ERR_INVALID, "conv3d fwd pair: null tensor");
  if (flags & SFH_FLAG_FORCE_GENERIC) return fail(SFH_ERR_INVALID, "conv3d fwd pair: the direct kernels read one tensor");
  if (!sfh_conv3d_pair_supported(p, dtype, cin_first, 0))
    return fail(SFH_ERR_UNSUPPORTED, "conv3d fwd pair: not offered for this problem cut at channel %d", (int)cin_first);
  const ChannelPair in2{const_cast<void*>(x_second), cin_first};
  if (groups <= 0) return conv3d_fwd_any(p, dtype, x_first, w, w_stride, bias, y, workspace, workspace_bytes, flags, stream, nullptr, &in2);
  const int32_t records = sfh_conv3d_fwd_gn_records(p, dtype, groups);
  if (records == 0) return fail(SFH_ERR_UNSUPPORTED, "conv3d fwd pair: GroupNorm partials are not offered for this problem");
  const size_t need = (size_t)p->n * records * groups * kGnRecordFloats * sizeof(float);
  if (gn_partials == nullptr || gn_partials_bytes < need || (reinterpret_cast<uintptr_t>(gn_partials) & 15u) != 0)
    return fail(SFH_ERR_WORKSPACE, "conv3d fwd pair: GroupNorm partials need %zu bytes at a 16-byte boundary, got %zu", need,
                gn_partials_bytes);
  const GnPartialOut gn{gn_partials, groups, p->cout / groups, records};
  return conv3d_fwd_any(p, dtype, x_first, w, w_stride, bias, y, workspace, workspace_bytes, flags, stream, &gn, &in2);
}

extern "C" int sfh_conv3d_dgrad_pair(const sfh_conv3d_desc* p, int dtype, const void* gy, const void* w, const int64_t w_stride[5],
                                     void* gx_first, void* gx_second, int32_t cin_first, void* workspace, size_t workspace_bytes,
                                     uint32_t flags, void* stream) {
  if (gx_second == nullptr) return fail(SFH_ERR_INVALID, "conv3d dgrad pair: null tensor");
  if (flags & SFH_FLAG_FORCE_GENERIC) return fail(SFH_ERR_INVALID, "conv3d dgrad pair: the direct kernels write one tensor");
  if (!sfh_conv3d_pair_supported(p, dtype, cin_first, 1))
    return fail(SFH_ERR_UNSUPPORTED, "conv3d dgrad pair: not offered for this problem cut at channel %d", (int)cin_first);
  const ChannelPair out2{gx_second, cin_first};
  return conv3d_dgrad_any(p, dtype, gy, w, w_stride, gx_first, workspace, workspace_bytes, flags, stream, &out2);
}

extern "C" int sfh_conv3d_wgrad_pair(const sfh_conv3d_desc* p, int dtype, const void* x_first, const void* x_second, int32_t cin_first,
                                     const void* gy, void* gw, void* workspace, size_t workspace_bytes, uint32_t flags, void* stream) {
  if (x_second == nullptr) return fail(SFH_ERR_INVALID, "conv3d wgrad pair: null tensor");
  if (flags & SFH_FLAG_FORCE_GENERIC) return fail(SFH_ERR_INVALID, "conv3d wgrad pair: the direct kernels read one tensor");
  if (!sfh_conv3d_pair_supported(p, dtype, cin_first, 2))
    return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad pair: not offered for this problem cut at channel %d", (int)cin_first);
  const ChannelPair x2{const_cast<void*>(x_second), cin_first};
  return conv3d_wgrad_any(p, dtype, x_first, gy, gw, workspace, workspace_bytes, flags, stream, &x2);
}

// ---- several weight gradients in one launch ----------------------------------------------
static_assert(kWgradBatchMax == SFH_WGRAD_BATCH_MAX, "the header's limit is the kernel table's");
static int wgrad_batch_items(const sfh_conv3d_wgrad_item* items, int32_t count, int dtype, WgradBatchItem* out_items) {
  if (items == nullptr || count < 1) return fail(SFH_ERR_INVALID, "conv3d wgrad batch: no problems");
  if (count > SFH_WGRAD_BATCH_MAX) return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad batch: at most %d problems a call", SFH_WGRAD_BATCH_MAX);
  for (int32_t i = 0; i < count; ++i) {
    int32_t out[3];
    if (int rc = check_conv(&items[i].desc, dtype, out)) return rc;
    const sfh_conv3d_desc& d = items[i].desc;
    if (!wgrad_uses_mfma(d, dtype, out) || !mfma_wgrad_batch_applies(wgrad_args(d, out), dtype))
      return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad batch: problem %d is served only by a launch of its own (sfh_conv3d_wgrad_batch_supported)", (int)i);
    WgradBatchItem& o = out_items[i];
    o.a = wgrad_args(d, out);
    o.x = items[i].x; o.x1 = items[i].x_second; o.c_first = items[i].cin_first; o.gy = items[i].gy; o.gw = items[i].gw;
    if (o.x1 != nullptr && !mfma_wgrad_pair_ok(o.a, o.c_first))
      return fail(SFH_ERR_UNSUPPORTED, "conv3d wgrad batch: problem %d cannot be cut at channel %d", (int)i, (int)o.c_first);
  }
  return SFH_OK;
}

extern "C" int sfh_conv3d_wgrad_batch_supported(const sfh_conv3d_desc* p, int dtype) {
  int32_t out[3];
  if (p == nullptr || sfh_conv3d_out_shape(p, out) != SFH_OK || !dtype_ok(dtype)) return 0;
  if (!wgrad_uses_mfma(*p, dtype, out) || !mfma_wgrad_batch_applies(wgrad_args(*p, out), dtype)) return 0;
  return mfma_wgrad_ring_applies(wgrad_args(*p, out)) ? 1 : 2;
}

// SFH_FLAG_SHARE_DEVICE: the launch of the large-row family takes half of the compute units
static int wgrad_batch_max_wgs(uint32_t flags) { return (flags & SFH_FLAG_SHARE_DEVICE) ? kComputeUnits / 2 : 0; }

extern "C" size_t sfh_conv3d_wgrad_batch_workspace_bytes(const sfh_conv3d_wgrad_item* items, int32_t count, int dtype, uint32_t flags) {
  WgradBatchItem list[SFH_WGRAD_BATCH_MAX];
  if (wgrad_batch_items(items, count, dtype, list) != SFH_OK) return 0;
  return mfma_wgrad_batch_workspace_bytes(list, count, wgrad_batch_max_wgs(flags));
}

extern "C" int sfh_conv3d_wgrad_batch(const sfh_conv3d_wgrad_item* items, int32_t count, int dtype, void* workspace, size_t workspace_bytes,
                                      uint32_t flags, void* stream) {
  WgradBatchItem list[SFH_WGRAD_BATCH_MAX];
  if (int rc = wgrad_batch_items(items, count, dtype, list)) return rc;
  for (int32_t i = 0; i < count; ++i)
    if (list[i].x == nullptr || list[i].gy == nullptr || list[i].gw == nullptr) return fail(SFH_ERR_INVALID, "conv3d wgrad batch: null tensor");
  if (flags & SFH_FLAG_FORCE_GENERIC) return fail(SFH_ERR_INVALID, "conv3d wgrad batch: the direct kernels take one problem a call");
  const int gw_dtype = (flags & SFH_FLAG_GRAD_FP32) ? SFH_FP32 : dtype;
  return mfma_wgrad_batch(list, count, dtype, gw_dtype, workspace, workspace_bytes, (hipStream_t)stream, wgrad_batch_max_wgs(flags));
}

// ---- bias gradient ---------------------------------------------------------------------
extern "C" size_t sfh_bias_grad_workspace_bytes(int64_t rows, int32_t channels) {
  if (rows < 1 || channels < 1) return 0;
  return bias_grad_workspace_bytes(rows, channels);
}

extern "C" int sfh_bias_grad(int dtype, int out_dtype, const void* g, int64_t rows, int32_t channels, void* gb, void* workspace,
                             size_t workspace_bytes, void* stream) {
  if (!dtype_ok(dtype) || !dtype_ok(out_dtype)) return fail(SFH_ERR_INVALID, "bias grad: bad dtype %d / %d", dtype, out_dtype);
  if (rows < 1 || channels < 1) return fail(SFH_ERR_INVALID, "bias grad: bad extents rows=%lld channels=%d", (long long)rows, channels);
  if (g == nullptr || gb == nullptr) return fail(SFH_ERR_INVALID, "bias grad: null tensor");
  const size_t need = bias_grad_workspace_bytes(rows, channels);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(SFH_ERR_WORKSPACE, "bias grad: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
  return bias_grad(dtype, out_dtype, g, rows, channels, gb, workspace, (hipStream_t)stream);
}

// ---- 2x2x2 max pooling -----------------------------------------------------------------
static int check_pool(const sfh_pool_desc* p, int dtype, const char* what) {
  if (p == nullptr) return fail(SFH_ERR_INVALID, "%s: null descriptor", what);
  if (!dtype_ok(dtype)) return fail(SFH_ERR_INVALID, "%s: bad dtype %d", what, dtype);
  if (p->n < 0 || p->c < 1 || p->in_d < 1 || p->in_h < 1 || p->in_w < 1)
    return fail(SFH_ERR_INVALID, "%s: bad extents n=%d c=%d in=(%d,%d,%d)", what, p->n, p->c, p->in_d, p->in_h, p->in_w);
  return SFH_OK;
}

extern "C" int sfh_maxpool2_fwd(const sfh_pool_desc* p, int dtype, const void* x, void* y, uint8_t* idx, void* stream) {
  if (int rc = check_pool(p, dtype, "maxpool fwd")) return rc;
  if (p->n == 0 || p->in_d < 2 || p->in_h < 2 || p->in_w < 2) return SFH_OK;  // empty output
  if (x == nullptr || y == nullptr || idx == nullptr) return fail(SFH_ERR_INVALID, "maxpool fwd: null tensor");
  return maxpool2_fwd(*p, dtype, x, y, idx, (hipStream_t)stream);
}

extern "C" int sfh_maxpool2_fwd_slab(const sfh_pool_desc* p, int dtype, const void* x, void* y_slab, int64_t halo_elems, uint8_t* idx,
                                     void* stream) {
  if (int rc = check_pool(p, dtype, "maxpool fwd")) return rc;
  if (halo_elems < 0) return fail(SFH_ERR_INVALID, "maxpool fwd: negative halo");
  if (p->n == 0 || p->in_d < 2 || p->in_h < 2 || p->in_w < 2) return fail(SFH_ERR_UNSUPPORTED, "maxpool fwd: no slab around an empty output");
  if (x == nullptr || y_slab == nullptr || idx == nullptr) return fail(SFH_ERR_INVALID, "maxpool fwd: null tensor");
  const size_t elem = dtype == SFH_FP32 ? 4 : 2;
  return maxpool2_fwd(*p, dtype, x, static_cast<char*>(y_slab) + (size_t)halo_elems * elem, idx, (hipStream_t)stream, halo_elems);
}

extern "C" int sfh_maxpool2_bwd(const sfh_pool_desc* p, int dtype, const void* grad_y, const uint8_t* idx, void* grad_x,
                                void* stream) {
  if (int rc = check_pool(p, dtype, "maxpool bwd")) return rc;
  if (p->n == 0) return SFH_OK;
  const bool empty_out = p->in_d < 2 || p->in_h < 2 || p->in_w < 2;
  if (grad_x == nullptr || (!empty_out && (grad_y == nullptr || idx == nullptr)))
    return fail(SFH_ERR_INVALID, "maxpool bwd: null tensor");
  return maxpool2_bwd(*p, dtype, grad_y, idx, nullptr, grad_x, (hipStream_t)stream);
}

extern "C" int sfh_maxpool2_bwd_add(const sfh_pool_desc* p, int dtype, const void* grad_y, const uint8_t* idx, const void* add,
                                    void* grad_x, void* stream) {
  if (int rc = check_pool(p, dtype, "maxpool bwd")) return rc;
  if (p->n == 0) return SFH_OK;
  const bool empty_out = p->in_d < 2 || p->in_h < 2 || p->in_w < 2;
  if (grad_x == nullptr || add == nullptr || (!empty_out && (grad_y == nullptr || idx == nullptr)))
    return fail(SFH_ERR_INVALID, "maxpool bwd: null tensor");
  return maxpool2_bwd(*p, dtype, grad_y, idx, add, grad_x, (hipStream_t)stream);
}

// ---- transposed convolution ------------------------------------------------------------
static int check_convT(const sfh_convT3d_desc* p, int dtype) {
  if (p == nullptr) return fail(SFH_ERR_INVALID, "convT3d: null descriptor");
  if (!dtype_ok(dtype)) return fail(SFH_ERR_INVALID, "convT3d: bad dtype %d", dtype);
  if (p->n < 0 || p->cin < 1 || p->cout < 1 || p->in_d < 1 || p->in_h < 1 || p->in_w < 1 || p->kd < 1 || p->kh < 1 || p->kw < 1)
    return fail(SFH_ERR_INVALID, "convT3d: bad extents");
  return SFH_OK;
}

extern "C" size_t sfh_convT3d_fwd_workspace_bytes(const sfh_convT3d_desc* p, int dtype) {
  if (check_convT(p, dtype) != SFH_OK) return 0;
  if (convT_uses_patch(*p, dtype)) return mfma_conv_packed_weight_bytes(patch_pack_args(p->cout, p->cin));
  return 0;
}

static int convT3d_fwd_any(const sfh_convT3d_desc* p, int dtype, const void* x, const void* w, const int64_t w_stride[5],
                           const void* bias, void* y, void* workspace, size_t workspace_bytes, uint32_t flags, void* stream,
                           int64_t halo_elems) {
  if (int rc = check_convT(p, dtype)) return rc;
  if (x == nullptr || w == nullptr || y == nullptr || (w_stride == nullptr && !(flags & SFH_FLAG_WEIGHT_PACKED)))
    return fail(SFH_ERR_INVALID, "convT3d fwd: null tensor");
  if (p->n == 0) return SFH_OK;
  if (flags & SFH_FLAG_WEIGHT_PACKED) {
    // w is the packed form: the data-gradient packing of the kernel == stride convolution this one transposes
    if ((flags & SFH_FLAG_FORCE_GENERIC) || !convT_uses_patch(*p, dtype))
      return fail(SFH_ERR_INVALID, "convT3d fwd: this problem does not read a packed weight");
    return patch_scatter(convT_patch_args(*p), dtype, x, w, bias, y, (hipStream_t)stream, halo_elems);
  }
  if (!(flags & SFH_FLAG_FORCE_GENERIC) && convT_uses_patch(*p, dtype)) {
    // produced channel = Cout (w_stride[1]), reduced channel = Cin (w_stride[0])
    const MfmaConvArgs pk = patch_pack_args(p->cout, p->cin);
    const size_t need = mfma_conv_packed_weight_bytes(pk);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(SFH_ERR_WORKSPACE, "convT3d fwd: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
    hipStream_t st = (hipStream_t)stream;
    if (int rc = mfma_pack_weight(pk, dtype, w, w_stride[1], w_stride[0], w_stride[2], w_stride[3], w_stride[4], 0, workspace, st))
      return rc;
    return patch_scatter(convT_patch_args(*p), dtype, x, workspace, bias, y, st, halo_elems);
  }
  if (halo_elems > 0) return fail(SFH_ERR_UNSUPPORTED, "convT3d fwd: only the 2x2x2 matrix-core kernel writes into a slab");
  return direct_convT(*p, dtype, w_stride, x, w, bias, y, (hipStream_t)stream);
}

extern "C" int sfh_convT3d_fwd(const sfh_convT3d_desc* p, int dtype, const void* x, const void* w, const int64_t w_stride[5],
                               const void* bias, void* y, void* workspace, size_t workspace_bytes, uint32_t flags, void* stream) {
  return convT3d_fwd_any(p, dtype, x, w, w_stride, bias, y, workspace, workspace_bytes, flags, stream, 0);
}

extern "C" int sfh_convT3d_fwd_slab(const sfh_convT3d_desc* p, int dtype, const void* x, const void* w, const int64_t w_stride[5],
                                    const void* bias, void* y_slab, int64_t halo_elems, void* workspace, size_t workspace_bytes,
                                    uint32_t flags, void* stream) {
  if (halo_elems < 0) return fail(SFH_ERR_INVALID, "convT3d fwd: negative halo");
  if (y_slab == nullptr) return fail(SFH_ERR_INVALID, "convT3d fwd: null tensor");
  if (p != nullptr && p->n == 0) return fail(SFH_ERR_UNSUPPORTED, "convT3d fwd: no slab around an empty output");
  const size_t elem = dtype == SFH_FP32 ? 4 : 2;
  return convT3d_fwd_any(p, dtype, x, w, w_stride, bias, static_cast<char*>(y_slab) + (size_t)halo_elems * elem, workspace, workspace_bytes,
                         flags, stream, halo_elems);
}

// Weight and bias gradient of the transposed convolution in one pass over its output gradient (2x2x2 matrix-core
// problems): the weight gradient is the stride-2 convolution's with the operands swapped, the bias gradient the column
// sums of the same tiles.
static bool convT_wgrad_bias_ok(const sfh_convT3d_desc& p, int dtype) {
  return p.kd == 2 && p.kh == 2 && p.kw == 2 && p.n >= 1 && patch_reduce_supported(convT_patch_args(p), dtype);
}

extern "C" size_t sfh_convT3d_wgrad_bias_workspace_bytes(const sfh_convT3d_desc* p, int dtype) {
  if (check_convT(p, dtype) != SFH_OK || !convT_wgrad_bias_ok(*p, dtype)) return 0;
  return patch_reduce_workspace_bytes(convT_patch_args(*p), true);
}

extern "C" int sfh_convT3d_wgrad_bias(const sfh_convT3d_desc* p, int dtype, const void* x, const void* gy, void* gw, void* gb,
                                      void* workspace, size_t workspace_bytes, uint32_t flags, void* stream) {
  if (int rc = check_convT(p, dtype)) return rc;
  if (x == nullptr || gy == nullptr || gw == nullptr || gb == nullptr) return fail(SFH_ERR_INVALID, "convT3d wgrad: null tensor");
  if ((flags & SFH_FLAG_FORCE_GENERIC) || !convT_wgrad_bias_ok(*p, dtype))
    return fail(SFH_ERR_UNSUPPORTED, "convT3d wgrad with bias gradient: 2x2x2 matrix-core problems only");
  const PatchArgs a = convT_patch_args(*p);
  const size_t need = patch_reduce_workspace_bytes(a, true);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(SFH_ERR_WORKSPACE, "convT3d wgrad: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
  const int g_dtype = (flags & SFH_FLAG_GRAD_FP32) ? SFH_FP32 : dtype;
  // small = the transposed convolution's input, big = its output gradient
  return patch_reduce(a, dtype, x, gy, gw, g_dtype, workspace, (hipStream_t)stream, gb);
}

// ---- loss head -------------------------------------------------------------------------
static int check_loss(const sfh_loss_desc* p, int dtype) {
  if (p == nullptr) return fail(SFH_ERR_INVALID, "ce_dice: null descriptor");
  if (!dtype_ok(dtype)) return fail(SFH_ERR_INVALID, "ce_dice: bad dtype %d", dtype);
  if (!loss_supported(*p))
    return fail(SFH_ERR_UNSUPPORTED, "ce_dice: n=%d classes=%d spatial=%lld (2..32 classes, non-empty)", p->n, p->classes,
                (long long)p->spatial);
  return SFH_OK;
}

extern "C" size_t sfh_ce_dice_workspace_bytes(const sfh_loss_desc* p) {
  if (p == nullptr || !loss_supported(*p)) return 0;
  return loss_workspace_bytes(*p);
}

extern "C" int sfh_ce_dice_fwd(const sfh_loss_desc* p, int dtype, const void* logits, const int64_t* labels, const float* class_weight,
                               float* loss, float* stats, void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_loss(p, dtype)) return rc;
  if (logits == nullptr || labels == nullptr || loss == nullptr || stats == nullptr) return fail(SFH_ERR_INVALID, "ce_dice: null tensor");
  const size_t need = loss_workspace_bytes(*p);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(SFH_ERR_WORKSPACE, "ce_dice fwd: workspace of %zu bytes needed, got %zu", need, workspace_bytes);
  return loss_forward(*p, dtype, logits, labels, class_weight, loss, stats, workspace, (hipStream_t)stream);
}

extern "C" int sfh_ce_dice_bwd(const sfh_loss_desc* p, int dtype, const void* logits, const int64_t* labels, const float* class_weight,
                               const float* stats, const float* grad_loss, void* dlogits, void* stream) {
  if (int rc = check_loss(p, dtype)) return rc;
  if (logits == nullptr || labels == nullptr || stats == nullptr || grad_loss == nullptr || dlogits == nullptr)
    return fail(SFH_ERR_INVALID, "ce_dice: null tensor");
  return loss_backward(*p, dtype, logits, labels, class_weight, stats, grad_loss, dlogits, (hipStream_t)stream);
}

// ---- halo slab assembly ------------------------------------------------------------------
extern "C" int sfh_halo_assemble(const sfh_halo_desc* p, int dtype, const void* x, const void* lo, const void* hi, void* out,
                                 void* stream) {
  if (p == nullptr) return fail(SFH_ERR_INVALID, "halo assemble: null descriptor");
  if (!dtype_ok(dtype)) return fail(SFH_ERR_INVALID, "halo assemble: bad dtype %d", dtype);
  if (p->n < 0 || p->c < 1 || p->d < 1 || p->h < 1 || p->w < 1 || p->halo < 0)
    return fail(SFH_ERR_INVALID, "halo assemble: bad extents n=%d c=%d (%d,%d,%d) halo=%d", p->n, p->c, p->d, p->h, p->w, p->halo);
  if (p->n == 0) return SFH_OK;
  if (x == nullptr || out == nullptr) return fail(SFH_ERR_INVALID, "halo assemble: null tensor");
  return halo_assemble(*p, dtype, x, lo, hi, out, (hipStream_t)stream);
}

static int check_halo_faces(const sfh_halo_desc* p, int dtype, const char* what) {
  if (p == nullptr) return fail(SFH_ERR_INVALID, "%s: null descriptor", what);
  if (!dtype_ok(dtype)) return fail(SFH_ERR_INVALID, "%s: bad dtype %d", what, dtype);
  if (p->n < 0 || p->c < 1 || p->d < 1 || p->h < 1 || p->w < 1 || p->halo < 0)
    return fail(SFH_ERR_INVALID, "%s: bad extents n=%d c=%d (%d,%d,%d) halo=%d", what, p->n, p->c, p->d, p->h, p->w, p->halo);
  return SFH_OK;
}

extern "C" int sfh_halo_pack(const sfh_halo_desc* p, int dtype, const void* x, void* lo_out, void* hi_out, void* stream) {
  if (int rc = check_halo_faces(p, dtype, "halo pack")) return rc;
  if (p->halo > p->d) return fail(SFH_ERR_INVALID, "halo pack: halo %d exceeds the depth %d", p->halo, p->d);
  if (p->n == 0 || p->halo == 0) return SFH_OK;
  if (x == nullptr) return fail(SFH_ERR_INVALID, "halo pack: null tensor");
  return halo_pack(*p, dtype, x, lo_out, hi_out, (hipStream_t)stream);
}

extern "C" int sfh_halo_accumulate(const sfh_halo_desc* p, int dtype, void* g, const void* lo_in, const void* hi_in, void* stream) {
  if (int rc = check_halo_faces(p, dtype, "halo accumulate")) return rc;
  if (2 * (int64_t)p->halo > p->d)
    return fail(SFH_ERR_UNSUPPORTED, "halo accumulate: depth %d is thinner than two halos of %d (the faces would overlap)", p->d, p->halo);
  if (p->n == 0 || p->halo == 0) return SFH_OK;
  if (g == nullptr) return fail(SFH_ERR_INVALID, "halo accumulate: null tensor");
  return halo_accumulate(*p, dtype, g, lo_in, hi_in, (hipStream_t)stream);
}

// ---- skip connection concat ------------------------------------------------------------------
static int check_concat(const sfh_concat_desc* p, int dtype) {
  if (p == nullptr) return fail(SFH_ERR_INVALID, "skip concat: null descriptor");
  if (!dtype_ok(dtype)) return fail(SFH_ERR_INVALID, "skip concat: bad dtype %d", dtype);
  if (p->n < 0 || p->c_a < 1 || p->c_b < 1 || p->rows < 1 || p->halo_rows < 0)
    return fail(SFH_ERR_INVALID, "skip concat: bad extents n=%d channels=(%d, %d) rows=%lld halo_rows=%lld", p->n, p->c_a, p->c_b,
                (long long)p->rows, (long long)p->halo_rows);
  if (p->n > 0 && !concat_supported(*p, dtype))
    return fail(SFH_ERR_UNSUPPORTED, "skip concat: channel counts (%d, %d) do not fill 16-byte pieces", p->c_a, p->c_b);
  return SFH_OK;
}

extern "C" int sfh_skip_concat_fwd(const sfh_concat_desc* p, int dtype, const void* a, const void* b, void* out, void* stream) {
  if (int rc = check_concat(p, dtype)) return rc;
  if (p->n == 0) return SFH_OK;
  if (a == nullptr || b == nullptr || out == nullptr) return fail(SFH_ERR_INVALID, "skip concat: null tensor");
  return concat_forward(*p, dtype, a, b, out, (hipStream_t)stream);
}

extern "C" int sfh_skip_concat_bwd(const sfh_concat_desc* p, int dtype, const void* g, void* ga, void* gb, void* stream) {
  if (int rc = check_concat(p, dtype)) return rc;
  if (p->n == 0) return SFH_OK;
  if (g == nullptr || ga == nullptr || gb == nullptr) return fail(SFH_ERR_INVALID, "skip concat: null tensor");
  return concat_backward(*p, dtype, g, ga, gb, (hipStream_t)stream);
}

// ---- shard ingest -----------------------------------------------------------------------------
extern "C" int sfh_shard_ingest(const sfh_ingest_desc* p, int dtype, const void* volume, const void* mask, void* x, void* labels,
                                void* stream) {
  if (p == nullptr) return fail(SFH_ERR_INVALID, "shard ingest: null descriptor");
  if (!dtype_ok(dtype)) return fail(SFH_ERR_INVALID, "shard ingest: bad dtype %d", dtype);
  if (p->n < 0 || p->c < 1 || p->rows < 1 || p->halo_rows < 0)
    return fail(SFH_ERR_INVALID, "shard ingest: bad extents n=%d c=%d rows=%lld halo_rows=%lld", p->n, p->c, (long long)p->rows,
                (long long)p->halo_rows);
  if (p->c > kIngestMaxChannels) return fail(SFH_ERR_UNSUPPORTED, "shard ingest: %d channels (1..%d supported)", p->c, kIngestMaxChannels);
  if ((mask == nullptr) != (labels == nullptr)) return fail(SFH_ERR_INVALID, "shard ingest: mask and labels go together");
  if (p->n == 0) return SFH_OK;
  if (volume == nullptr || x == nullptr) return fail(SFH_ERR_INVALID, "shard ingest: null tensor");
  if ((reinterpret_cast<uintptr_t>(volume) & 3) || (reinterpret_cast<uintptr_t>(mask) & 1) || (reinterpret_cast<uintptr_t>(labels) & 7) ||
      (reinterpret_cast<uintptr_t>(x) & (dtype_size(dtype) - 1)))
    return fail(SFH_ERR_INVALID, "shard ingest: a pointer is not aligned to its element size");
  return shard_ingest(*p, dtype, (const float*)volume, mask, x, (int64_t*)labels, (hipStream_t)stream);
}

// ---- gradient clipping + Adam ------------------------------------------------------------
static int check_tensor_list(int32_t ntensors, const int64_t* numel, const char* what) {
  if (ntensors < 1 || numel == nullptr) return fail(SFH_ERR_INVALID, "%s: need at least one tensor", what);
  for (int i = 0; i < ntensors; ++i)
    if (numel[i] < 1) return fail(SFH_ERR_INVALID, "%s: tensor %d has %lld elements", what, i, (long long)numel[i]);
  return SFH_OK;
}

extern "C" int64_t sfh_adam_slots(int32_t ntensors, const int64_t* numel) {
  if (ntensors < 1 || numel == nullptr) return 0;
  return optim_chunks(ntensors, numel);
}

extern "C" int sfh_adam_grad_sumsq(int32_t ntensors, const float* const* grads, const int64_t* numel, float* slots, float* step,
                                   void* stream) {
  if (int rc = check_tensor_list(ntensors, numel, "adam sumsq")) return rc;
  if (grads == nullptr || slots == nullptr || step == nullptr) return fail(SFH_ERR_INVALID, "adam sumsq: null argument");
  for (int i = 0; i < ntensors; ++i)
    if (grads[i] == nullptr) return fail(SFH_ERR_INVALID, "adam sumsq: gradient %d is null", i);
  return optim_grad_sumsq(ntensors, grads, numel, slots, step, (hipStream_t)stream);
}

extern "C" int sfh_adam_clip_step(const sfh_adam_desc* d, int32_t ntensors, float* const* params, const float* const* grads,
                                  float* const* exp_avg, float* const* exp_avg_sq, void* const* shadow, const int64_t* numel,
                                  const float* slots, int64_t nslots, const float* step, float* grad_norm, void* stream) {
  if (d == nullptr) return fail(SFH_ERR_INVALID, "adam: null descriptor");
  if (nslots < 1 || nslots > 0x7fffffff) return fail(SFH_ERR_INVALID, "adam: bad slot count %lld", (long long)nslots);
  if (int rc = check_tensor_list(ntensors, numel, "adam")) return rc;
  if (params == nullptr || grads == nullptr || exp_avg == nullptr || exp_avg_sq == nullptr || slots == nullptr || step == nullptr)
    return fail(SFH_ERR_INVALID, "adam: null argument");
  if (!(d->lr >= 0.f) || !(d->beta1 >= 0.f && d->beta1 < 1.f) || !(d->beta2 >= 0.f && d->beta2 < 1.f) || !(d->eps >= 0.f) ||
      !(d->weight_decay >= 0.f))
    return fail(SFH_ERR_INVALID, "adam: bad hyperparameters lr=%g betas=(%g, %g) eps=%g weight_decay=%g", d->lr, d->beta1, d->beta2,
                d->eps, d->weight_decay);
  if (shadow != nullptr && d->shadow_dtype != SFH_BF16 && d->shadow_dtype != SFH_FP16)
    return fail(SFH_ERR_INVALID, "adam: shadow copies need shadow_dtype bf16 or fp16, got %d", d->shadow_dtype);
  for (int i = 0; i < ntensors; ++i)
    if (params[i] == nullptr || grads[i] == nullptr || exp_avg[i] == nullptr || exp_avg_sq[i] == nullptr)
      return fail(SFH_ERR_INVALID, "adam: tensor %d has a null pointer", i);
  return optim_clip_adam(*d, ntensors, params, grads, exp_avg, exp_avg_sq, shadow, numel, slots, (int)nslots, step, grad_norm,
                         (hipStream_t)stream);
}

// ---- measurement helper ----------------------------------------------------------------
extern "C" int sfh_stream_copy(const void* src, void* dst, size_t bytes, void* stream) {
  if (src == nullptr || dst == nullptr || bytes % 16 != 0) return fail(SFH_ERR_INVALID, "stream copy: need 16-byte multiples");
  if (bytes == 0) return SFH_OK;
  hipLaunchKernelGGL(stream_copy_kernel, dim3(kComputeUnits * 4), dim3(256), 0, (hipStream_t)stream, (const uint4*)src,
                     (uint4*)dst, bytes / 16);
  return check_launch("stream_copy_kernel");
}
