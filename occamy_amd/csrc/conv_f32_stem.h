// fp32 N,C,H,W first layer (3 -> 64 channels, 7x7, stride 2, pad 3) with bias and activation, optionally with the
// 3x3 stride-2 pad-1 max pooling behind it in the same kernel (conv_f32_stem.hip).
#pragma once
#include "common.h"

namespace dnnrt {

// X: N x 3 x H x W, filter in the context's layout, Y: N x 64 x P x Q (Z: a residual operand shaped like Y, or null),
// or with `pool` the pooled N x 64 x PP x QQ (activation ReLU or identity, no residual).  P, Q: the convolution's
// output size.
bool launch_conv_f32_stem(const dnnrtContext *ctx, int N, int H, int W, int P, int Q, const float *X, const float *Wt,
                          const float *bias, const float *Z, int act, float *Y, bool pool, int PP, int QQ);

}  // namespace dnnrt
