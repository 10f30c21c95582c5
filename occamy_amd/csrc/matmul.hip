// Matrix-product entry points: dnnrtMatmul2d / dnnrtMatmulNd
// (reference: src/Tools/dnn-wrapper/cublas/CUBLASMatmul2dFunc.cu:9-153 and
//  cuda/CUDAMatmulNdFunc.cu:14-173).
//
// A product Out[M,N] = op(A) op(B) is the implicit-GEMM kernel with a 1x1
// "filter": rows of the left matrix are filters, the right matrix is a
// K-channel image of 1 x N pixels.  Products with very few rows and a
// transposed right operand (the classifier layer at batch 1) are bandwidth
// bound on the right matrix and use a wave-per-output dot-product kernel.
#include "common.h"
#include "igemm_f32.h"
#include "gemm_f16.h"

namespace dnnrt {

// Out[m, n] = alpha * dot(A[m, :], B[n, :]) + beta * C[m, n], M <= 8.
// WPO wavefronts share one n, each striding over its own slices of k; B is
// read exactly once.  The partial sums of an n meet in LDS and are added in
// wavefront order, so the result does not depend on timing.  WPO is picked on
// the host so that a narrow N (a few hundred outputs over a long K) still puts
// a few thousand wavefronts on the device.
template <int MMAX, int WPO>
__global__ __launch_bounds__(WPO > 4 ? 64 * WPO : 256) void gemv_f32_kernel(
    const float *__restrict__ A, const float *__restrict__ B, const float *__restrict__ C,
    float *__restrict__ Out, int M, int N, int K, float alpha, float beta, bool vec4, int64_t c_ld) {
  constexpr int WAVES = WPO > 4 ? WPO : 4, NPB = WAVES / WPO;
  __shared__ float part[WAVES][MMAX];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = blockIdx.x * NPB + wave / WPO, slice = wave % WPO;
  float acc[MMAX];
#pragma unroll
  for (int m = 0; m < MMAX; m++) acc[m] = 0.f;
  if (n < N) {
    const float *b = B + (int64_t)n * K;
    if (vec4) {
      for (int k = (slice * 64 + lane) * 4; k < K; k += 256 * WPO) {
        const float4 bv = *reinterpret_cast<const float4 *>(b + k);
#pragma unroll
        for (int m = 0; m < MMAX; m++)
          if (m < M) {
            const float4 av = *reinterpret_cast<const float4 *>(A + (int64_t)m * K + k);
            acc[m] += av.x * bv.x + av.y * bv.y + av.z * bv.z + av.w * bv.w;
          }
      }
    } else {
      for (int k = slice * 64 + lane; k < K; k += 64 * WPO) {
        const float bv = b[k];
#pragma unroll
        for (int m = 0; m < MMAX; m++)
          if (m < M) acc[m] += A[(int64_t)m * K + k] * bv;
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MMAX; m++) {
    float v = acc[m];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    if (lane == 0) part[wave][m] = v;
  }
  __syncthreads();
  if (slice == 0 && n < N && lane < M) {
    float v = part[wave][lane];
#pragma unroll
    for (int w = 1; w < WPO; w++) v += part[wave + w][lane];
    float r = alpha * v;
    if (C) r += beta * C[(int64_t)lane * c_ld + n];
    Out[(int64_t)lane * N + n] = r;
  }
}

template <int WPO>
static void launch_gemv(const dnnrtContext *ctx, const float *A, const float *B, const float *C, float *Out,
                        int M, int N, int K, float alpha, float beta, bool vec4, int64_t c_ld) {
  constexpr int WAVES = WPO > 4 ? WPO : 4, NPB = WAVES / WPO;
  hipLaunchKernelGGL((gemv_f32_kernel<8, WPO>), dim3((unsigned)ceil_div(N, NPB)), dim3(64 * WAVES), 0, ctx->stream,
                     A, B, C, Out, M, N, K, alpha, beta, vec4, c_ld);
}

static bool gemm_f32(const dnnrtContext *ctx, const float *A, const float *B, const float *C,
                     float *Out, int M, int N, int K, float alpha, float beta, bool transA,
                     bool transB, int Z, int64_t az, int64_t bz, int64_t yz, bool c_is_row = false,
                     const float *bias_col = nullptr, int act = DNNRT_ACT_IDENTITY) {
  // c_is_row: C holds one row of N values that is added to every row of every product
  // bias_col, act: Out = act(alpha * A B + bias_col[n] + beta * C)
  if (Z == 1 && M <= 8 && transB && !transA && !bias_col && act == DNNRT_ACT_IDENTITY) {
    const bool vec4 = (K % 4 == 0) && aligned16(A) && aligned16(B);
    // wavefronts per output: the fewest that give 2048 wavefronts, each keeping >= 512 elements of k
    int wpo = 1;
    while (wpo < 16 && (int64_t)N * wpo < 2048 && K / (wpo * 4) >= 512) wpo *= 4;
    if (wpo == 1) launch_gemv<1>(ctx, A, B, C, Out, M, N, K, alpha, beta, vec4, c_is_row ? 0 : N);
    else if (wpo == 4) launch_gemv<4>(ctx, A, B, C, Out, M, N, K, alpha, beta, vec4, c_is_row ? 0 : N);
    else launch_gemv<16>(ctx, A, B, C, Out, M, N, K, alpha, beta, vec4, c_is_row ? 0 : N);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("gemv_f32: launch failed: %s", hipGetErrorString(e)); return false; }
    return true;
  }
  IgemmArgs a{};
  a.A = A; a.X = B; a.Y = Out; a.bias = nullptr; a.Cin = C;
  a.alpha = alpha; a.beta = beta; a.act = act; a.bias_col = bias_col;
  a.M = M; a.Kdim = K; a.Ncols = N;
  a.H = 1; a.W = N; a.R = 1; a.S = 1; a.P = 1; a.Q = N; a.ph = 0; a.pw = 0; a.sh = 1; a.sw = 1;
  a.x_img_stride = 0; a.y_img_stride = 0; a.y_row_stride = N;
  a.Z = Z; a.a_z_stride = az; a.x_z_stride = bz; a.y_z_stride = yz; a.bias_z_stride = 0;
  a.c_row_stride = c_is_row ? 0 : N; a.c_z_stride = c_is_row ? 0 : yz;
  a.b_kcontig = transB; a.a_mcontig = transA; a.a_ld = M;
  a.a_vec4 = !transA && (K % 4 == 0) && aligned16(A) && (az % 4 == 0);
  a.b_vec4 = transB && (K % 4 == 0) && aligned16(B) && (bz % 4 == 0);
  bool launched = false;
  if (!launch_gemm_f32_rows(ctx, a, launched)) return false;
  if (launched) return true;
  return launch_igemm_f32(ctx, a);
}

}  // namespace dnnrt

using namespace dnnrt;

extern "C" {

void *dnnrtMatmul2d(dnnrtHandle_t handle, int64_t rank, const void *A, const int64_t *dimA,
                    const void *B, const int64_t *dimB, const void *C, const int64_t *dimC,
                    void *Out, const int64_t *dimOut, float alpha, float beta, int64_t transA,
                    int64_t transB, int32_t dtype) {
  (void)rank;
  if (!handle) DNNRT_FAIL("dnnrtMatmul2d: null handle");
  if (!A || !B || !Out || !dimA || !dimB || !dimOut) DNNRT_FAIL("dnnrtMatmul2d: null argument");
  const int64_t M = transA ? dimA[1] : dimA[0], K = transA ? dimA[0] : dimA[1];
  const int64_t Kb = transB ? dimB[1] : dimB[0], N = transB ? dimB[0] : dimB[1];
  if (K == Kb && dimOut[0] == M && dimOut[1] == N && M >= 0 && N >= 0 && K > 0 && (M == 0 || N == 0)) return Out;  // empty product: no work
  if (K != Kb || dimOut[0] != M || dimOut[1] != N || M <= 0 || N <= 0 || K <= 0)
    DNNRT_FAIL("dnnrtMatmul2d: shapes [%ld,%ld] x [%ld,%ld] -> [%ld,%ld] do not agree", (long)M,
               (long)K, (long)Kb, (long)N, (long)dimOut[0], (long)dimOut[1]);
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) DNNRT_FAIL("dnnrtMatmul2d: dims exceed 32 bits");
  if (beta != 0.f && !C) DNNRT_FAIL("dnnrtMatmul2d: beta != 0 needs C");
  const void *Cin = beta != 0.f ? C : nullptr;
  // C is [M, N], or one row [1, N] added to every row of the product
  const bool c_is_row = Cin && dimC && dimC[0] == 1 && dimC[1] == N && M > 1;
  if (Cin && dimC && !c_is_row && (dimC[0] != M || dimC[1] != N))
    DNNRT_FAIL("dnnrtMatmul2d: C is [%ld,%ld], neither [M,N] nor [1,N]", (long)dimC[0], (long)dimC[1]);
  if (dtype == DNNRT_F32) {
    if (!gemm_f32(handle, (const float *)A, (const float *)B, (const float *)Cin, (float *)Out, (int)M,
                  (int)N, (int)K, alpha, beta, transA != 0, transB != 0, 1, 0, 0, 0, c_is_row))
      return nullptr;
    return Out;
  }
  if (dtype == DNNRT_F16) {
    if (!gemm_f16(handle, (const __half *)A, (const __half *)B, (const __half *)Cin, (__half *)Out,
                  (int)M, (int)N, (int)K, alpha, beta, transA != 0, transB != 0, 1, 0, 0, 0, c_is_row || (Cin && M == 1)))
      return nullptr;
    return Out;
  }
  DNNRT_FAIL("dnnrtMatmul2d: dtype %d", dtype);
}

static void *matmul_nd(dnnrtHandle_t handle, const void *A, const int64_t *dimA, int32_t rankA,
                       const void *B, const int64_t *dimB, int32_t rankB, const void *bias, const void *Zr, int act,
                       void *Y, const int64_t *dimY, int32_t rankY, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtMatmulNd: null handle");
  if (!A || !B || !Y || !dimA || !dimB || !dimY) DNNRT_FAIL("dnnrtMatmulNd: null argument");
  if (rankA < 2 || rankB < 2 || rankA > 4 || rankB > 4 || rankY != (rankA > rankB ? rankA : rankB))
    DNNRT_FAIL("dnnrtMatmulNd: ranks %d x %d -> %d (2..4 supported)", rankA, rankB, rankY);
  const int64_t M = dimA[rankA - 2], K = dimA[rankA - 1], N = dimB[rankB - 1];
  {
    bool neg = false;
    for (int i = 0; i < rankA; i++) neg = neg || dimA[i] < 0;
    for (int i = 0; i < rankB; i++) neg = neg || dimB[i] < 0;
    for (int i = 0; i < rankY; i++) neg = neg || dimY[i] < 0;
    if (!neg && K > 0 && dimB[rankB - 2] == K && numel(dimY, rankY) == 0) return Y;  // empty product (a zero batch or row count): no work
  }
  if (dimB[rankB - 2] != K || dimY[rankY - 2] != M || dimY[rankY - 1] != N || M <= 0 || N <= 0 || K <= 0)
    DNNRT_FAIL("dnnrtMatmulNd: inner/outer dims do not agree");
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) DNNRT_FAIL("dnnrtMatmulNd: dims exceed 32 bits");
  const int nb = rankY - 2;
  int64_t batchY = 1, batchA = 1, batchB = 1;
  bool a_full = true, b_full = true;
  for (int i = 0; i < nb; i++) {
    batchY *= dimY[i];
    const int ia = i - (rankY - rankA), ib = i - (rankY - rankB);
    const int64_t da = ia >= 0 ? dimA[ia] : 1, db = ib >= 0 ? dimB[ib] : 1;
    if ((da != dimY[i] && da != 1) || (db != dimY[i] && db != 1))
      DNNRT_FAIL("dnnrtMatmulNd: batch dims do not broadcast");
    batchA *= da; batchB *= db;
    if (da != dimY[i]) a_full = false;
    if (db != dimY[i]) b_full = false;
  }
  // Each operand must be either batched over every batch dim or shared by all.
  if ((!a_full && batchA != 1) || (!b_full && batchB != 1))
    DNNRT_FAIL("dnnrtMatmulNd: partial batch broadcast is not supported");
  if (batchY > 65535) DNNRT_FAIL("dnnrtMatmulNd: more than 65535 batches");
  const int64_t az = (a_full && batchY > 1) ? M * K : 0, bz = (b_full && batchY > 1) ? K * N : 0;
  // A shared right matrix under a batched left one is one tall product.
  int64_t Mz = M; int Z = (int)batchY; int64_t azz = az, yz = M * N;
  if (bz == 0 && Z > 1 && az != 0) { Mz = M * batchY; Z = 1; azz = 0; yz = 0; }
  if (Mz > INT32_MAX) DNNRT_FAIL("dnnrtMatmulNd: dims exceed 32 bits");
  if (dtype == DNNRT_F32) {
    // the residual is laid out like Y: one tall product (yz == 0) or one product per batch
    if (!gemm_f32(handle, (const float *)A, (const float *)B, (const float *)Zr, (float *)Y, (int)Mz, (int)N, (int)K,
                  1.f, Zr ? 1.f : 0.f, false, false, Z, azz, bz, yz, false, (const float *)bias, act))
      return nullptr;
    return Y;
  }
  if (dtype == DNNRT_F16) {
    // the residual is laid out like Y (one tall product or one product per batch, as above)
    if (!gemm_f16(handle, (const __half *)A, (const __half *)B, (const __half *)Zr, (__half *)Y, (int)Mz, (int)N,
                  (int)K, 1.f, Zr ? 1.f : 0.f, false, false, Z, azz, bz, yz, false, (const __half *)bias, act))
      return nullptr;
    return Y;
  }
  DNNRT_FAIL("dnnrtMatmulNd: dtype %d", dtype);
}

void *dnnrtMatmulNd(dnnrtHandle_t handle, const void *A, const int64_t *dimA, int32_t rankA,
                    const void *B, const int64_t *dimB, int32_t rankB, void *Y, const int64_t *dimY,
                    int32_t rankY, int32_t dtype) {
  return matmul_nd(handle, A, dimA, rankA, B, dimB, rankB, nullptr, nullptr, DNNRT_ACT_IDENTITY, Y, dimY, rankY, dtype);
}

void *dnnrtMatmulNdBias(dnnrtHandle_t handle, const void *A, const int64_t *dimA, int32_t rankA,
                        const void *B, const int64_t *dimB, int32_t rankB, const void *bias, const void *Z,
                        int32_t gelu, void *Y, const int64_t *dimY, int32_t rankY, int32_t dtype) {
  if (!bias) DNNRT_FAIL("dnnrtMatmulNdBias: null bias");
  if (Z && Z == Y) DNNRT_FAIL("dnnrtMatmulNdBias: the residual must not be the output buffer");
  return matmul_nd(handle, A, dimA, rankA, B, dimB, rankB, bias, Z, gelu ? ACT_GELU : DNNRT_ACT_IDENTITY, Y, dimY, rankY, dtype);
}

}  // extern "C"
