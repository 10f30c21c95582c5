// Reductions and normalisations: dnnrtReduce (mean), dnnrtSoftmax,
// dnnrtLayerNorm.  Wavefront-per-row kernels: a 64-lane wave walks one row
// with coalesced loads and combines with cross-lane shuffles; no LDS, no
// atomics.  Reference wrappers replaced:
// src/Tools/dnn-wrapper/cudnn/CUDNNReduceFunc.cpp:8-142 and
// src/Tools/dnn-wrapper/cuda/CUDASoftmaxFunc.cu:7-128.
#include "common.h"

namespace dnnrt {

__device__ __forceinline__ float ld_f(const float *p) { return *p; }
__device__ __forceinline__ float ld_f(const __half *p) { return __half2float(*p); }
__device__ __forceinline__ void st_f(float *p, float v) { *p = v; }
__device__ __forceinline__ void st_f(__half *p, float v) { *p = __float2half_rn(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// mean over the last (contiguous) L elements of each row
template <typename T>
__global__ __launch_bounds__(256) void mean_rows_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                        int64_t rows, int L) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T *xr = x + row * L;
  float s = 0.f;
  for (int i = lane; i < L; i += 64) s += ld_f(xr + i);
  s = wave_sum(s);
  if (lane == 0) st_f(y + row, s / (float)L);
}

// mean over the middle dim of [outer, red, inner]; one thread per (outer, inner)
template <typename T>
__global__ __launch_bounds__(256) void mean_cols_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                        int64_t outer, int red, int64_t inner) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= outer * inner) return;
  const int64_t o = i / inner, in = i - o * inner;
  const T *xp = x + o * red * inner + in;
  float s = 0.f;
  for (int r = 0; r < red; r++) s += ld_f(xp + (int64_t)r * inner);
  st_f(y + i, s / (float)red);
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_rows_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                           int64_t rows, int L) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T *xr = x + row * L;
  T *yr = y + row * L;
  float m = -INFINITY;
  for (int i = lane; i < L; i += 64) m = fmaxf(m, ld_f(xr + i));
  m = wave_max(m);
  float s = 0.f;
  for (int i = lane; i < L; i += 64) s += expf(ld_f(xr + i) - m);
  s = wave_sum(s);
  for (int i = lane; i < L; i += 64) st_f(yr + i, expf(ld_f(xr + i) - m) / s);
}

// softmax over the middle dim of [outer, L, inner], inner > 1
template <typename T>
__global__ __launch_bounds__(256) void softmax_cols_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                           int64_t outer, int L, int64_t inner) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= outer * inner) return;
  const int64_t o = i / inner, in = i - o * inner;
  const T *xp = x + o * L * inner + in;
  T *yp = y + o * L * inner + in;
  float m = -INFINITY;
  for (int l = 0; l < L; l++) m = fmaxf(m, ld_f(xp + (int64_t)l * inner));
  float s = 0.f;
  for (int l = 0; l < L; l++) s += expf(ld_f(xp + (int64_t)l * inner) - m);
  for (int l = 0; l < L; l++) st_f(yp + (int64_t)l * inner, expf(ld_f(xp + (int64_t)l * inner) - m) / s);
}

template <typename T>
__global__ __launch_bounds__(256) void layernorm_kernel(const T *__restrict__ x, const T *__restrict__ g,
                                                        const T *__restrict__ b, T *__restrict__ y,
                                                        int64_t rows, int L, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T *xr = x + row * L;
  T *yr = y + row * L;
  float s = 0.f;
  for (int i = lane; i < L; i += 64) s += ld_f(xr + i);
  const float mu = wave_sum(s) / (float)L;
  float v = 0.f;
  for (int i = lane; i < L; i += 64) { const float d = ld_f(xr + i) - mu; v += d * d; }
  const float inv = 1.0f / sqrtf(wave_sum(v) / (float)L + eps);
  for (int i = lane; i < L; i += 64)
    st_f(yr + i, (ld_f(xr + i) - mu) * inv * ld_f(g + i) + ld_f(b + i));
}

template <typename T>
static bool run_reduce(const dnnrtContext *ctx, const void *X, void *Y, int64_t outer, int64_t red,
                       int64_t inner) {
  if (red > INT32_MAX) { set_error("reduce: reduced extent too large"); return false; }
  if (inner == 1) {
    const int64_t blocks = ceil_div(outer, 4);
    if (blocks > INT32_MAX) { set_error("reduce: too many rows"); return false; }
    hipLaunchKernelGGL((mean_rows_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                       (const T *)X, (T *)Y, outer, (int)red);
  } else {
    const int64_t blocks = ceil_div(outer * inner, 256);
    if (blocks > INT32_MAX) { set_error("reduce: tensor too large"); return false; }
    hipLaunchKernelGGL((mean_cols_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                       (const T *)X, (T *)Y, outer, (int)red, inner);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("reduce: launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

}  // namespace dnnrt

using namespace dnnrt;

extern "C" {

void *dnnrtReduce(dnnrtHandle_t handle, int32_t rank, const void *X, const int64_t *dimX, void *Y,
                  const int64_t *dimY, int32_t mode, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtReduce: null handle");
  if (!X || !Y || !dimX || !dimY) DNNRT_FAIL("dnnrtReduce: null argument");
  if (mode != DNNRT_REDUCE_AVG) DNNRT_FAIL("dnnrtReduce: mode %d (only 5 = AVG)", mode);
  if (rank < 1 || rank > 8) DNNRT_FAIL("dnnrtReduce: rank %d", rank);
  int64_t dx[8], dy[8];
  for (int i = 0; i < rank; i++) { dx[i] = dimX[i]; dy[i] = dimY[i]; }
  if (handle->format != DNNRT_NCHW && rank == 4) {  // channels-last: dense [N,H,W,C]
    dx[1] = dimX[2]; dx[2] = dimX[3]; dx[3] = dimX[1];
    dy[1] = dimY[2]; dy[2] = dimY[3]; dy[3] = dimY[1];
  }
  // reduced dims must form one contiguous run: [outer, red, inner]
  int64_t outer = 1, red = 1, inner = 1;
  int state = 0;  // 0 before the run, 1 inside, 2 after
  for (int i = 0; i < rank; i++) {
    if (dx[i] <= 0) DNNRT_FAIL("dnnrtReduce: non-positive dim");
    if (dy[i] != dx[i] && dy[i] != 1) DNNRT_FAIL("dnnrtReduce: dimY[%d] must be dimX[%d] or 1", i, i);
    const bool r = dy[i] == 1 && dx[i] != 1;
    if (dx[i] == 1) continue;
    if (r) {
      if (state == 2) DNNRT_FAIL("dnnrtReduce: reduced dims must be adjacent");
      state = 1; red *= dx[i];
    } else {
      if (state == 0) outer *= dx[i];
      else { state = 2; inner *= dx[i]; }
    }
  }
  bool ok;
  if (dtype == DNNRT_F32) ok = run_reduce<float>(handle, X, Y, outer, red, inner);
  else if (dtype == DNNRT_F16) ok = run_reduce<__half>(handle, X, Y, outer, red, inner);
  else DNNRT_FAIL("dnnrtReduce: dtype %d", dtype);
  return ok ? Y : nullptr;
}

void *dnnrtSoftmax(dnnrtHandle_t handle, const void *X, const int64_t *dimX, void *Y,
                   const int64_t *dimY, int64_t axis, int64_t rank, int32_t dtype) {
  (void)dimY;
  if (!handle) DNNRT_FAIL("dnnrtSoftmax: null handle");
  if (!X || !Y || !dimX) DNNRT_FAIL("dnnrtSoftmax: null argument");
  if (rank < 1 || rank > 8) DNNRT_FAIL("dnnrtSoftmax: rank %ld", (long)rank);
  if (axis < 0) axis += rank;
  if (axis < 0 || axis >= rank) DNNRT_FAIL("dnnrtSoftmax: axis out of range");
  if (handle->format != DNNRT_NCHW && rank == 4) DNNRT_FAIL("dnnrtSoftmax: channels-last tensors are not supported");
  int64_t outer = 1, inner = 1;
  const int64_t L = dimX[axis];
  for (int64_t i = 0; i < axis; i++) outer *= dimX[i];
  for (int64_t i = axis + 1; i < rank; i++) inner *= dimX[i];
  if (L <= 0 || L > INT32_MAX || outer <= 0 || inner <= 0) DNNRT_FAIL("dnnrtSoftmax: bad dims");
#define SOFTMAX_LAUNCH(T)                                                                           \
  do {                                                                                              \
    if (inner == 1) {                                                                               \
      const int64_t blocks = ceil_div(outer, 4);                                                    \
      if (blocks > INT32_MAX) DNNRT_FAIL("dnnrtSoftmax: too many rows");                            \
      hipLaunchKernelGGL((softmax_rows_kernel<T>), dim3((unsigned)blocks), dim3(256), 0,            \
                         handle->stream, (const T *)X, (T *)Y, outer, (int)L);                      \
    } else {                                                                                        \
      const int64_t blocks = ceil_div(outer * inner, 256);                                          \
      if (blocks > INT32_MAX) DNNRT_FAIL("dnnrtSoftmax: tensor too large");                         \
      hipLaunchKernelGGL((softmax_cols_kernel<T>), dim3((unsigned)blocks), dim3(256), 0,            \
                         handle->stream, (const T *)X, (T *)Y, outer, (int)L, inner);               \
    }                                                                                               \
  } while (0)
  if (dtype == DNNRT_F32) SOFTMAX_LAUNCH(float);
  else if (dtype == DNNRT_F16) SOFTMAX_LAUNCH(__half);
  else DNNRT_FAIL("dnnrtSoftmax: dtype %d", dtype);
#undef SOFTMAX_LAUNCH
  DNNRT_CHECK_LAUNCH("dnnrtSoftmax");
  return Y;
}

void *dnnrtLayerNorm(dnnrtHandle_t handle, const void *X, const int64_t *dimX, int64_t rank,
                     const void *gamma, const void *beta, float eps, void *Y, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtLayerNorm: null handle");
  if (!X || !Y || !dimX || !gamma || !beta) DNNRT_FAIL("dnnrtLayerNorm: null argument");
  if (rank < 1 || rank > 8) DNNRT_FAIL("dnnrtLayerNorm: rank %ld", (long)rank);
  const int64_t L = dimX[rank - 1], rows = numel(dimX, rank - 1);
  if (L <= 0 || L > INT32_MAX || rows <= 0) DNNRT_FAIL("dnnrtLayerNorm: bad dims");
  const int64_t blocks = ceil_div(rows, 4);
  if (blocks > INT32_MAX) DNNRT_FAIL("dnnrtLayerNorm: too many rows");
  if (dtype == DNNRT_F32)
    hipLaunchKernelGGL((layernorm_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, handle->stream,
                       (const float *)X, (const float *)gamma, (const float *)beta, (float *)Y, rows,
                       (int)L, eps);
  else if (dtype == DNNRT_F16)
    hipLaunchKernelGGL((layernorm_kernel<__half>), dim3((unsigned)blocks), dim3(256), 0, handle->stream,
                       (const __half *)X, (const __half *)gamma, (const __half *)beta, (__half *)Y,
                       rows, (int)L, eps);
  else DNNRT_FAIL("dnnrtLayerNorm: dtype %d", dtype);
  DNNRT_CHECK_LAUNCH("dnnrtLayerNorm");
  return Y;
}

}  // extern "C"
