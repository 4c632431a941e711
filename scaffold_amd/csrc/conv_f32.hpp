// Host-side interface of the tiled fp32 convolution on the fp32 matrix pipe (3x3x3, stride 1, dilation 1).
#pragma once
#include "conv_mfma.hpp"
#include "wgrad_mfma.hpp"

namespace sfh {

// Roles as in MfmaConvArgs: `cred` reduction channels (a multiple of 16), `cout` produced channels (a multiple of 32).
bool f32_conv_supported(const MfmaConvArgs& a);
size_t f32_conv_packed_weight_bytes(const MfmaConvArgs& a);
// packed[cout/32][cred/16][tap][q(2)][lane(64)][4] with lane = cout % 32 + 32 * kg, channel = 16 cc + 8 kg + 4 q + e;
// strides in elements as for mfma_pack_weight.
int f32_pack_weight(const MfmaConvArgs& a, const void* w, int64_t s_out, int64_t s_red, int64_t s_kd, int64_t s_kh, int64_t s_kw, int flip,
                    void* packed, hipStream_t st);
int f32_conv(const MfmaConvArgs& a, const void* x, const void* packed, const void* bias, void* y, hipStream_t st);

// Weight gradient of the same family (3x3x3, stride 1; both channel counts multiples of 32): split-K over output rows into
// fp32 slices [Cout][27][Cin] in the workspace, summed in fixed order into gw (fp32, [Cout][27][Cin]).
bool f32_wgrad_supported(const WgradArgs& a);
int f32_wgrad_splits(const WgradArgs& a);
size_t f32_wgrad_workspace_bytes(const WgradArgs& a);
int f32_wgrad(const WgradArgs& a, const void* x, const void* gy, void* gw, void* workspace, hipStream_t st);

}  // namespace sfh
