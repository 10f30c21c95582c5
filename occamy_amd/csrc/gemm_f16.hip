// fp16 matrix product.  Out[M,N] = A[M,K] * B[N,K]^T is exactly a channels-last
// 1x1 convolution (M "pixels" of K channels, N filters), so it runs on the
// fp16 convolution kernels (a bias row is the convolution's bias); other
// operand layouts are not built yet and fail loudly.
#include "gemm_f16.h"

#include "conv_f16.h"

namespace dnnrt {

bool gemm_f16(const dnnrtContext *ctx, const __half *A, const __half *B, const __half *C, __half *Out, int M,
              int N, int K, float alpha, float beta, bool transA, bool transB, int Z, int64_t az, int64_t bz,
              int64_t yz, bool c_is_row) {
  (void)az; (void)bz; (void)yz;
  // C: nothing, or one row of N values with beta 1 (a Gemm's bias), which is the convolution's per-filter bias
  const bool bias_row = C && c_is_row && beta == 1.f;
  if (transA || !transB || Z != 1 || alpha != 1.f || (!bias_row && (beta != 0.f || C))) {
    set_error("matmul(fp16): only Out = A * B^T [+ one row] (transA=0, transB=1, alpha=1, one batch) is built");
    return false;
  }
  ConvF16Args a{};
  a.X = A; a.Wt = B; a.bias = bias_row ? C : nullptr; a.Y = Out;
  a.N = M; a.C = K; a.H = 1; a.W = 1; a.K = N; a.Cg = K; a.R = 1; a.S = 1; a.P = 1; a.Q = 1;
  a.ph = 0; a.pw = 0; a.sh = 1; a.sw = 1; a.group = 1;
  a.act = DNNRT_ACT_IDENTITY;
  a.format = DNNRT_NHWC;
  return launch_conv_f16(ctx, a);
}

}  // namespace dnnrt
