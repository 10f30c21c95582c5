// fp16 convolution (fp32 accumulate) on gfx950 MFMA.
#pragma once
#include "common.h"

#include <type_traits>

namespace dnnrt {

// f(std::integral_constant<int, mode>{}) for the activation mode `act` names: a kernel's epilogue loop is compiled
// once per mode and picked once, instead of asking for the mode per value.
template <typename F>
__device__ __forceinline__ void by_act_mode(int act, F &&f) {
  switch (act) {
    case DNNRT_ACT_RELU: f(std::integral_constant<int, DNNRT_ACT_RELU>{}); break;
    case DNNRT_ACT_CLIPPED_RELU: f(std::integral_constant<int, DNNRT_ACT_CLIPPED_RELU>{}); break;
    case DNNRT_ACT_LEAKY_RELU: f(std::integral_constant<int, DNNRT_ACT_LEAKY_RELU>{}); break;
    case ACT_GELU: f(std::integral_constant<int, ACT_GELU>{}); break;
    default: f(std::integral_constant<int, DNNRT_ACT_IDENTITY>{}); break;
  }
}

struct ConvF16Args {
  const __half *X, *Wt, *bias;
  const __half *Z;  // residual tensor laid out like Y, or null
  __half *Y;
  int N, C, H, W, K, Cg, R, S, P, Q, ph, pw, sh, sw, group;
  int act;     // DNNRT_ACT_{IDENTITY, RELU, CLIPPED_RELU, LEAKY_RELU}
  float act_coef;  // ceiling / slope of the last two
  int format;  // physical layout of X and Y (DNNRT_NCHW / NHWC / NCHW_TO_NHWC)
  int variant;  // the call's own choice of channels-last variant (its `algo` operand), used where it can run the problem; 0: none
  unsigned magic_pq, magic_q;  // filled in by the launcher: ceil(2^32 / (P*Q)), ceil(2^32 / Q)
  unsigned magic_pw, magic_hp;  // (conv_f16_patch.hip) ceil(2^32 / (W + 2)), ceil(2^32 / (H + 2))
  // a second 1x1 convolution onto the same result (launch_conv_f16_dual): input N x H2 x W2 x C2 read with strides
  // sh2, sw2, filter K x C2, bias or null
  const __half *X2, *Wt2, *bias2;
  int C2, H2, W2, sh2, sw2;
};

bool launch_conv_f16(const dnnrtContext *ctx, const ConvF16Args &a);
// Y = act(fp16(conv(X, W) + bias) + fp16(conv(X2, W2) + bias2)), both convolutions 1x1 without padding (a residual
// block's last convolution and its projection shortcut); `a` must satisfy dual_conv_applies.
bool dual_conv_applies(const ConvF16Args &a);
bool launch_conv_f16_dual(const dnnrtContext *ctx, const ConvF16Args &a);
// Channels-last 1x1 stride-1 layers over at most this many output pixels (a fully connected layer at small batch).
constexpr int FEWPIX_MAX_PIXELS = 64;
bool launch_conv_f16_fewpix(const dnnrtContext *ctx, const ConvF16Args &a, bool &launched);
// The 3-channel 7x7 stride-2 first layer (NCHW in, NHWC out); `launched` says whether it took the problem.
bool launch_conv_f16_stem(const dnnrtContext *ctx, const ConvF16Args &a, bool &launched);
// Other first layers (conv_f16_first.hip): N,C,H,W input of at most four channels, a filter of at most 3x3, 16 to 64
// filters, channels-last output; `launched` says whether it took the problem.
bool launch_conv_f16_first(const dnnrtContext *ctx, const ConvF16Args &a, bool &launched);
// The same layer with the 3x3 stride-2 pad-1 max-pool behind it in one kernel: `a` is the convolution (a.Y unused),
// Yp the pooled tensor N x PP x QQ x 64.  Fails with an error on any other shape.
bool launch_conv_f16_stem_pool(const dnnrtContext *ctx, const ConvF16Args &a, __half *Yp, int PP, int QQ);

// Channels-last 1x1 stride-1 layers over a multiple of 8 channels up to 256 (conv_f16_pointwise.hip): one wavefront
// per 32 pixels, operands read from global memory in the MFMA's shape.
bool pointwise_conv_applies(const ConvF16Args &a);
bool launch_conv_f16_pointwise(const dnnrtContext *ctx, const ConvF16Args &a);

// Channels-last convolutions whose operands are loaded straight into LDS (conv_f16_dma.hip): `variant` is one of
// that file's tile ids, `a` must satisfy dma_conv_applies and carry the division constants.
bool dma_conv_applies(const ConvF16Args &a);
bool launch_conv_f16_dma(const dnnrtContext *ctx, const ConvF16Args &a, int variant);
// Y = act(conv(X, W) + bias + conv(X2, W2) + bias2) as one reduction over both convolutions' channels (both 1x1, no
// padding; the sum is formed in fp32 and rounded once); variant: one of the ids dma_dual_variant accepts, else the
// launcher picks.
bool dma_dual_applies(const ConvF16Args &a);
bool dma_dual_variant(int variant);
bool launch_conv_f16_dma_dual(const dnnrtContext *ctx, const ConvF16Args &a, int variant);

// 3x3 stride-1 pad-1 channels-last convolutions over at least 128 channels with the input patch kept in LDS
// (conv_f16_patch.hip): `variant` is one of that file's tile ids, `a` must satisfy patch_conv_applies and carry the
// division constants of P * Q and Q.  patch_conv_capacity: the smallest compiled patch capacity that holds this
// problem's patches at tile width bn, or 0.
bool patch_conv_applies(const ConvF16Args &a);
int patch_conv_capacity(const ConvF16Args &a, int bn);
bool patch_variant_fits(const ConvF16Args &a, int variant);  // the variant's patch capacity holds this problem's patches
bool launch_conv_f16_patch(const dnnrtContext *ctx, const ConvF16Args &a, int variant);

// 3x3 stride-1 pad-1 channels-last convolutions over exactly 64 channels, images up to 62 wide, no residual
// (conv_f16_c64.hip): persistent workgroups, filter in registers, input patch in LDS.
bool c64_conv_applies(const ConvF16Args &a);
bool launch_conv_f16_c64(const dnnrtContext *ctx, const ConvF16Args &a);

}  // namespace dnnrt
