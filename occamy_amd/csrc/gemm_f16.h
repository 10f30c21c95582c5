// fp16 matrix product (fp32 accumulate) on gfx950 MFMA.
#pragma once
#include "common.h"

namespace dnnrt {

// Out[z][M,N] = alpha * op(A[z]) op(B[z]) + beta * C[z]; strides in elements,
// 0 = operand shared by every z.
bool gemm_f16(const dnnrtContext *ctx, const __half *A, const __half *B, const __half *C,
              __half *Out, int M, int N, int K, float alpha, float beta, bool transA, bool transB,
              int Z, int64_t az, int64_t bz, int64_t yz, bool c_is_row = false);  // c_is_row: C is one row of N values

}  // namespace dnnrt
