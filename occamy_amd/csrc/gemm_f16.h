// fp16 matrix product (fp32 accumulate) on gfx950 MFMA.
#pragma once
#include "common.h"

namespace dnnrt {

// Out[z][M,N] = alpha * op(A[z]) op(B[z]) + beta * C[z]; strides in elements,
// 0 = operand shared by every z.
// bias: one value per column n, added to every row (may be null); act: an activation mode of apply_act applied last;
// C (scaled by beta) is a matrix like Out with the batch stride yz, or with c_is_row one row of N values.
bool gemm_f16(const dnnrtContext *ctx, const __half *A, const __half *B, const __half *C,
              __half *Out, int M, int N, int K, float alpha, float beta, bool transA, bool transB,
              int Z, int64_t az, int64_t bz, int64_t yz, bool c_is_row = false, const __half *bias = nullptr,
              int act = DNNRT_ACT_IDENTITY);

}  // namespace dnnrt
