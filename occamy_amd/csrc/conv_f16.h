// fp16 convolution (fp32 accumulate) on gfx950 MFMA.
#pragma once
#include "common.h"

namespace dnnrt {

struct ConvF16Args {
  const __half *X, *Wt, *bias;
  const __half *Z;  // residual tensor laid out like Y, or null
  __half *Y;
  int N, C, H, W, K, Cg, R, S, P, Q, ph, pw, sh, sw, group;
  int act;     // DNNRT_ACT_{IDENTITY, RELU, CLIPPED_RELU, LEAKY_RELU}
  float act_coef;  // ceiling / slope of the last two
  int format;  // physical layout of X and Y (DNNRT_NCHW / NHWC / NCHW_TO_NHWC)
  unsigned magic_pq, magic_q;  // filled in by the launcher: ceil(2^32 / (P*Q)), ceil(2^32 / Q)
};

bool launch_conv_f16(const dnnrtContext *ctx, const ConvF16Args &a);
// Channels-last 1x1 stride-1 layers over at most this many output pixels (a fully connected layer at small batch).
constexpr int FEWPIX_MAX_PIXELS = 64;
bool launch_conv_f16_fewpix(const dnnrtContext *ctx, const ConvF16Args &a, bool &launched);
// The 3-channel 7x7 stride-2 first layer (NCHW in, NHWC out); `launched` says whether it took the problem.
bool launch_conv_f16_stem(const dnnrtContext *ctx, const ConvF16Args &a, bool &launched);

// Channels-last convolutions whose operands are loaded straight into LDS (conv_f16_dma.hip): `variant` is one of
// that file's tile ids, `a` must satisfy dma_conv_applies and carry the division constants.
bool dma_conv_applies(const ConvF16Args &a);
bool launch_conv_f16_dma(const dnnrtContext *ctx, const ConvF16Args &a, int variant);

}  // namespace dnnrt
