// Elementwise and broadcast entry points.  All of them are HBM-bound: one
// 128-bit load and one 128-bit store per lane where the pointers allow it,
// consecutive lanes on consecutive 16-byte words.
//
// Reference wrappers replaced here:
//   cudnn/CUDNNActiveFunc.cpp, cudnn/CUDNNTensorOpFunc.cpp,
//   cuda/CUDAClipFunc.cu, CUDAErfFunc.cu, CUDANegativeFunc.cu,
//   CUDAReciprocalFunc.cu, CUDAPowFunc.cu, CUDACastI64toFloatFunc.cu,
//   CUDALeakyReluFunc.cu, CUDAPReluFunc.cu
// (all under src/Tools/dnn-wrapper/).
#include "common.h"

namespace dnnrt {

__device__ __forceinline__ float to_f(float v) { return v; }
__device__ __forceinline__ float to_f(__half v) { return __half2float(v); }
template <typename T> __device__ __forceinline__ T from_f(float v);
template <> __device__ __forceinline__ float from_f<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_f<__half>(float v) { return __float2half_rn(v); }

template <typename T> struct Pack {  // 16 bytes of T
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

// y[i] = f(x[i])
template <typename T, bool VEC, typename F>
__global__ __launch_bounds__(256) void unary_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                    int64_t n, F f) {
  constexpr int V = VEC ? Pack<T>::N : 1;
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
  if (i >= n) return;
  if (VEC && i + V <= n) {
    Pack<T> p = *reinterpret_cast<const Pack<T> *>(x + i);
#pragma unroll
    for (int j = 0; j < V; j++) p.v[j] = from_f<T>(f(to_f(p.v[j])));
    *reinterpret_cast<Pack<T> *>(y + i) = p;
  } else {
    for (int64_t j = i; j < n && j < i + V; j++) y[j] = from_f<T>(f(to_f(x[j])));
  }
}

// o[i] = f(a[i], b[i])
template <typename T, bool VEC, typename F>
__global__ __launch_bounds__(256) void binary_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                     T *__restrict__ o, int64_t n, F f) {
  constexpr int V = VEC ? Pack<T>::N : 1;
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
  if (i >= n) return;
  if (VEC && i + V <= n) {
    Pack<T> pa = *reinterpret_cast<const Pack<T> *>(a + i);
    const Pack<T> pb = *reinterpret_cast<const Pack<T> *>(b + i);
#pragma unroll
    for (int j = 0; j < V; j++) pa.v[j] = from_f<T>(f(to_f(pa.v[j]), to_f(pb.v[j])));
    *reinterpret_cast<Pack<T> *>(o + i) = pa;
  } else {
    for (int64_t j = i; j < n && j < i + V; j++) o[j] = from_f<T>(f(to_f(a[j]), to_f(b[j])));
  }
}

// Broadcast of b over a: dims collapsed on the host to at most 4, each with
// the element stride of b (0 where b is broadcast).
struct BcastDims {
  int64_t d[4];
  int64_t sb[4];
};
template <typename T, typename F>
__global__ __launch_bounds__(256) void bcast_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                    T *__restrict__ o, int64_t n, BcastDims g, F f) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  int64_t rem = i, ib = 0;
#pragma unroll
  for (int k = 3; k >= 0; k--) {
    const int64_t q = rem / g.d[k];
    ib += (rem - q * g.d[k]) * g.sb[k];
    rem = q;
  }
  o[i] = from_f<T>(f(to_f(a[i]), to_f(b[ib])));
}

// The same below 2^31 elements when the innermost run is a multiple of 16
// bytes and everything is 16-byte aligned: a thread owns 16 bytes of a, which
// lie inside one innermost run, so b is either one value for all of them
// (INNER_BC: the innermost run is a broadcast one) or 16 consecutive bytes.
struct BcastDims32 {
  unsigned d[4];
  unsigned sb[4];
};
template <typename T, bool INNER_BC, typename F>
__global__ __launch_bounds__(256) void bcast_vec_kernel(const T *__restrict__ a, const T *__restrict__ b,
                                                        T *__restrict__ o, unsigned n, BcastDims32 g, F f) {
  constexpr int V = Pack<T>::N;
  const unsigned i = (blockIdx.x * 256u + threadIdx.x) * (unsigned)V;
  if (i >= n) return;
  unsigned rem = i, ib = 0;
#pragma unroll
  for (int k = 3; k >= 0; k--) {
    if (g.d[k] == 1u) continue;  // the same for every thread
    const unsigned q = rem / g.d[k];
    ib += (rem - q * g.d[k]) * g.sb[k];
    rem = q;
  }
  Pack<T> pa = *reinterpret_cast<const Pack<T> *>(a + i);
  if (INNER_BC) {
    const float bv = to_f(b[ib]);
#pragma unroll
    for (int j = 0; j < V; j++) pa.v[j] = from_f<T>(f(to_f(pa.v[j]), bv));
  } else {
    const Pack<T> pb = *reinterpret_cast<const Pack<T> *>(b + ib);
#pragma unroll
    for (int j = 0; j < V; j++) pa.v[j] = from_f<T>(f(to_f(pa.v[j]), to_f(pb.v[j])));
  }
  *reinterpret_cast<Pack<T> *>(o + i) = pa;
}

template <typename T, typename F>
static bool run_unary(const dnnrtContext *ctx, const void *x, void *y, int64_t n, F f) {
  if (n == 0) return true;
  const bool vec = aligned16(x) && aligned16(y);
  const int V = vec ? Pack<T>::N : 1;
  const int64_t blocks = ceil_div(ceil_div(n, V), 256);
  if (blocks > INT32_MAX) { set_error("elementwise: tensor too large"); return false; }
  if (vec)
    hipLaunchKernelGGL((unary_kernel<T, true, F>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                       (const T *)x, (T *)y, n, f);
  else
    hipLaunchKernelGGL((unary_kernel<T, false, F>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                       (const T *)x, (T *)y, n, f);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("elementwise: launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

template <typename F>
static void *unary_entry(const char *who, dnnrtHandle_t h, const void *X, void *Y, const int64_t *d,
                         int64_t rank, int32_t dtype, F f) {
  if (!h) DNNRT_FAIL("%s: null handle", who);
  if (!X || !Y || !d || rank < 0) DNNRT_FAIL("%s: null argument", who);
  const int64_t n = numel(d, rank);
  if (n < 0) DNNRT_FAIL("%s: negative dim", who);
  bool ok;
  if (dtype == DNNRT_F32) ok = run_unary<float>(h, X, Y, n, f);
  else if (dtype == DNNRT_F16) ok = run_unary<__half>(h, X, Y, n, f);
  else DNNRT_FAIL("%s: dtype %d", who, dtype);
  return ok ? Y : nullptr;
}

struct FRelu { __device__ float operator()(float v) const { return v < 0.f ? 0.f : v; } };
struct FSigmoid { __device__ float operator()(float v) const { return 1.0f / (1.0f + expf(-v)); } };
struct FTanh { __device__ float operator()(float v) const { return tanhf(v); } };
struct FErf { __device__ float operator()(float v) const { return erff(v); } };
struct FNeg { __device__ float operator()(float v) const { return -v; } };
struct FRcp { __device__ float operator()(float v) const { return 1.0f / v; } };
struct FSqrt { __device__ float operator()(float v) const { return sqrtf(v); } };
struct FSquare { __device__ float operator()(float v) const { return __fmul_rn(v, v); } };
struct FGelu {
  __device__ float operator()(float v) const { return 0.5f * v * (1.0f + erff(v * 0.70710678118654752f)); }
};
struct FClip {
  float lo, hi;
  __device__ float operator()(float v) const {
    v = v < lo ? lo : v;
    return v > hi ? hi : v;
  }
};
struct FLeaky {
  float alpha;
  __device__ float operator()(float v) const { return v < 0.f ? __fmul_rn(alpha, v) : v; }
};
struct FPRelu {
  __device__ float operator()(float v, float slope) const { return v < 0.f ? __fmul_rn(slope, v) : v; }
};
struct FPow {
  float e;
  __device__ float operator()(float v) const { return powf(v, e); }
};
// a + coef*b and a * (coef*b) with each operation rounded separately, so that
// the result does not depend on FMA contraction.
struct FAdd {
  float coef;
  __device__ float operator()(float a, float b) const { return __fadd_rn(a, __fmul_rn(coef, b)); }
};
struct FMul {
  float coef;
  __device__ float operator()(float a, float b) const { return __fmul_rn(a, __fmul_rn(coef, b)); }
};

template <typename T, typename F>
static bool run_binary(const dnnrtContext *ctx, const void *A, const void *B, void *O,
                       const int64_t *dA, const int64_t *dB, int rank, F f) {
  const int64_t n = numel(dA, rank);
  if (n == 0) return true;
  bool same = true;
  for (int i = 0; i < rank; i++) same = same && dA[i] == dB[i];
  hipError_t e;
  if (same) {
    const bool vec = aligned16(A) && aligned16(B) && aligned16(O);
    const int V = vec ? Pack<T>::N : 1;
    const int64_t blocks = ceil_div(ceil_div(n, V), 256);
    if (blocks > INT32_MAX) { set_error("tensorOp: tensor too large"); return false; }
    if (vec)
      hipLaunchKernelGGL((binary_kernel<T, true, F>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                         (const T *)A, (const T *)B, (T *)O, n, f);
    else
      hipLaunchKernelGGL((binary_kernel<T, false, F>), dim3((unsigned)blocks), dim3(256), 0,
                         ctx->stream, (const T *)A, (const T *)B, (T *)O, n, f);
  } else {
    // Collapse runs of dims that are all broadcast or all not.
    int64_t cd[8], cs[8];
    int nc = 0;
    int64_t sb = 1;
    int64_t strideB[8];
    for (int i = rank - 1; i >= 0; i--) { strideB[i] = dB[i] == 1 ? 0 : sb; sb *= dB[i]; }
    for (int i = 0; i < rank; i++) {
      if (dA[i] == 1) continue;
      const bool bc = strideB[i] == 0;
      if (nc > 0 && ((cs[nc - 1] == 0) == bc)) {
        cd[nc - 1] *= dA[i];
        if (!bc) cs[nc - 1] = strideB[i];  // innermost stride of the run
      } else {
        cd[nc] = dA[i];
        cs[nc] = strideB[i];
        nc++;
      }
    }
    if (nc > 4) { set_error("tensorOp: broadcast pattern with more than 4 runs"); return false; }
    BcastDims g;
    for (int k = 0; k < 4; k++) { g.d[k] = 1; g.sb[k] = 0; }
    for (int k = 0; k < nc; k++) { g.d[4 - nc + k] = cd[k]; g.sb[4 - nc + k] = cs[k]; }
    const int64_t blocks = ceil_div(n, 256);
    if (blocks > INT32_MAX) { set_error("tensorOp: tensor too large"); return false; }
    constexpr int V = Pack<T>::N;
    const bool inner_bc = g.sb[3] == 0;
    if (n < (1ll << 31) && nc >= 1 && g.d[3] % V == 0 && (inner_bc || g.sb[3] == 1) && aligned16(A) && aligned16(O) &&
        (inner_bc || aligned16(B))) {
      // b's strides for the outer runs are multiples of its innermost run's length, itself a multiple of V
      BcastDims32 h;
      for (int k = 0; k < 4; k++) { h.d[k] = (unsigned)g.d[k]; h.sb[k] = (unsigned)g.sb[k]; }
      const unsigned vblocks = (unsigned)ceil_div(n / V, 256);
      if (inner_bc)
        hipLaunchKernelGGL((bcast_vec_kernel<T, true, F>), dim3(vblocks), dim3(256), 0, ctx->stream,
                           (const T *)A, (const T *)B, (T *)O, (unsigned)n, h, f);
      else
        hipLaunchKernelGGL((bcast_vec_kernel<T, false, F>), dim3(vblocks), dim3(256), 0, ctx->stream,
                           (const T *)A, (const T *)B, (T *)O, (unsigned)n, h, f);
    } else {
      hipLaunchKernelGGL((bcast_kernel<T, F>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                         (const T *)A, (const T *)B, (T *)O, n, g, f);
    }
  }
  e = hipGetLastError();
  if (e != hipSuccess) { set_error("tensorOp: launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

__global__ __launch_bounds__(256) void cast_i64_f32_kernel(const int64_t *__restrict__ x,
                                                           float *__restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) y[i] = (float)x[i];
}
__global__ __launch_bounds__(256) void cast_i64_f16_kernel(const int64_t *__restrict__ x,
                                                           __half *__restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) y[i] = __float2half_rn((float)x[i]);
}

// y = pow(x, e[0]) with the exponent on the device; e == 2 squares, as the
// reference kernel does (cuda/CUDAPowFunc.cu:4-32).
template <typename T>
__global__ __launch_bounds__(256) void pow_kernel(const T *__restrict__ x, const T *__restrict__ e,
                                                  T *__restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float ex = to_f(e[0]), v = to_f(x[i]);
  y[i] = from_f<T>(ex == 2.0f ? __fmul_rn(v, v) : powf(v, ex));
}

}  // namespace dnnrt

using namespace dnnrt;

extern "C" {

void *dnnrtActive(dnnrtHandle_t handle, const void *X, const int64_t *dimX, int32_t mode, void *Y,
                  int32_t dtype) {
  switch (mode) {
    case DNNRT_ACT_RELU: return unary_entry("dnnrtActive", handle, X, Y, dimX, 4, dtype, FRelu{});
    case DNNRT_ACT_SIGMOID: return unary_entry("dnnrtActive", handle, X, Y, dimX, 4, dtype, FSigmoid{});
    case DNNRT_ACT_TANH: return unary_entry("dnnrtActive", handle, X, Y, dimX, 4, dtype, FTanh{});
    case DNNRT_ACT_CLIPPED_RELU:
      if (!handle) DNNRT_FAIL("dnnrtActive: null handle");
      return unary_entry("dnnrtActive", handle, X, Y, dimX, 4, dtype, FClip{0.f, handle->act_coef});
    case DNNRT_ACT_LEAKY_RELU:
      if (!handle) DNNRT_FAIL("dnnrtActive: null handle");
      return unary_entry("dnnrtActive", handle, X, Y, dimX, 4, dtype, FLeaky{handle->act_coef});
    default: DNNRT_FAIL("dnnrtActive: mode %d (0 sigmoid, 1 relu, 2 tanh, 3 clipped relu, 6 leaky relu)", mode);
  }
}

void *dnnrtClip(dnnrtHandle_t handle, const void *X, void *Y, const int64_t *dimY, float lo, float hi,
                int64_t rank, int32_t dtype) {
  return unary_entry("dnnrtClip", handle, X, Y, dimY, rank, dtype, FClip{lo, hi});
}
void *dnnrtErf(dnnrtHandle_t handle, const void *X, void *Y, const int64_t *dim, int64_t rank,
               int32_t dtype) {
  return unary_entry("dnnrtErf", handle, X, Y, dim, rank, dtype, FErf{});
}
void *dnnrtNegative(dnnrtHandle_t handle, const void *X, void *Y, const int64_t *dim, int64_t rank,
                    int32_t dtype) {
  return unary_entry("dnnrtNegative", handle, X, Y, dim, rank, dtype, FNeg{});
}
void *dnnrtReciprocal(dnnrtHandle_t handle, const void *X, void *Y, const int64_t *dim, int64_t rank,
                      int32_t dtype) {
  return unary_entry("dnnrtReciprocal", handle, X, Y, dim, rank, dtype, FRcp{});
}
void *dnnrtGelu(dnnrtHandle_t handle, const void *X, void *Y, const int64_t *dim, int64_t rank,
                int32_t dtype) {
  return unary_entry("dnnrtGelu", handle, X, Y, dim, rank, dtype, FGelu{});
}

void *dnnrtLeakyRelu(dnnrtHandle_t handle, const void *X, void *Y, const int64_t *dimY, float alpha,
                     int64_t rank, int32_t dtype) {
  return unary_entry("dnnrtLeakyRelu", handle, X, Y, dimY, rank, dtype, FLeaky{alpha});
}

void *dnnrtPRelu(dnnrtHandle_t handle, const void *X, void *Y, const int64_t *dimY, const void *slope,
                 const int64_t *dimSlope, int64_t rank, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtPRelu: null handle");
  if (!X || !Y || !dimY || !slope || !dimSlope) DNNRT_FAIL("dnnrtPRelu: null argument");
  if (rank < 1 || rank > 8) DNNRT_FAIL("dnnrtPRelu: rank %ld (1..8)", (long)rank);
  for (int i = 0; i < rank; i++) {
    if (dimY[i] < 0) DNNRT_FAIL("dnnrtPRelu: negative dim");
    if (dimSlope[i] != dimY[i] && dimSlope[i] != 1)
      DNNRT_FAIL("dnnrtPRelu: dimSlope[%d]=%ld cannot broadcast to %ld", i, (long)dimSlope[i], (long)dimY[i]);
  }
  int64_t dy[8], ds[8];
  for (int i = 0; i < rank; i++) { dy[i] = dimY[i]; ds[i] = dimSlope[i]; }
  if (handle->format != DNNRT_NCHW && rank == 4) {  // dense [N,H,W,C] arrays
    dy[1] = dimY[2]; dy[2] = dimY[3]; dy[3] = dimY[1];
    ds[1] = dimSlope[2]; ds[2] = dimSlope[3]; ds[3] = dimSlope[1];
  }
  bool ok;
  if (dtype == DNNRT_F32) ok = run_binary<float>(handle, X, slope, Y, dy, ds, (int)rank, FPRelu{});
  else if (dtype == DNNRT_F16) ok = run_binary<__half>(handle, X, slope, Y, dy, ds, (int)rank, FPRelu{});
  else DNNRT_FAIL("dnnrtPRelu: dtype %d", dtype);
  return ok ? Y : nullptr;
}

void *dnnrtPow(dnnrtHandle_t handle, const void *X, const void *exponent, void *Y, const int64_t *dimY,
               int64_t rank, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtPow: null handle");
  if (!X || !exponent || !Y || !dimY) DNNRT_FAIL("dnnrtPow: null argument");
  const int64_t n = numel(dimY, rank);
  if (n == 0) return Y;
  const int64_t blocks = ceil_div(n, 256);
  if (blocks > INT32_MAX) DNNRT_FAIL("dnnrtPow: tensor too large");
  if (dtype == DNNRT_F32)
    hipLaunchKernelGGL((pow_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, handle->stream,
                       (const float *)X, (const float *)exponent, (float *)Y, n);
  else if (dtype == DNNRT_F16)
    hipLaunchKernelGGL((pow_kernel<__half>), dim3((unsigned)blocks), dim3(256), 0, handle->stream,
                       (const __half *)X, (const __half *)exponent, (__half *)Y, n);
  else DNNRT_FAIL("dnnrtPow: dtype %d", dtype);
  DNNRT_CHECK_LAUNCH("dnnrtPow");
  return Y;
}

void *dnnrtCastI64toFloat(dnnrtHandle_t handle, const int64_t *X, void *Y, const int64_t *dimY,
                          int64_t rank, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtCastI64toFloat: null handle");
  if (!X || !Y || !dimY) DNNRT_FAIL("dnnrtCastI64toFloat: null argument");
  const int64_t n = numel(dimY, rank);
  if (n == 0) return Y;
  const int64_t blocks = ceil_div(n, 256);
  if (blocks > INT32_MAX) DNNRT_FAIL("dnnrtCastI64toFloat: tensor too large");
  if (dtype == DNNRT_F32)
    hipLaunchKernelGGL(cast_i64_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, handle->stream, X,
                       (float *)Y, n);
  else if (dtype == DNNRT_F16)
    hipLaunchKernelGGL(cast_i64_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, handle->stream, X,
                       (__half *)Y, n);
  else DNNRT_FAIL("dnnrtCastI64toFloat: dtype %d", dtype);
  DNNRT_CHECK_LAUNCH("dnnrtCastI64toFloat");
  return Y;
}

void *dnnrtTensorOp(dnnrtHandle_t handle, int64_t op, const void *A, const int64_t *dimA, int32_t rankA,
                    const void *B, const int64_t *dimB, int32_t rankB, void *O, const int64_t *dimO,
                    int32_t rankO, float coefB, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtTensorOp: null handle");
  if (!A || !O || !dimA || !dimO) DNNRT_FAIL("dnnrtTensorOp: null argument");
  if (rankA != rankO || rankA < 1 || rankA > 8) DNNRT_FAIL("dnnrtTensorOp: ranks %d/%d", rankA, rankO);
  for (int i = 0; i < rankA; i++)
    if (dimA[i] != dimO[i] || dimA[i] < 0) DNNRT_FAIL("dnnrtTensorOp: dimA and dimO differ");
  if (op == DNNRT_OP_SQRT) return unary_entry("dnnrtTensorOp", handle, A, O, dimA, rankA, dtype, FSqrt{});
  if (op != DNNRT_OP_ADD && op != DNNRT_OP_MUL) DNNRT_FAIL("dnnrtTensorOp: op %ld (0 add, 1 mul, 4 sqrt)", (long)op);
  if (!B || !dimB || rankB != rankA) DNNRT_FAIL("dnnrtTensorOp: B must have the rank of A");
  for (int i = 0; i < rankA; i++)
    if (dimB[i] != dimA[i] && dimB[i] != 1)
      DNNRT_FAIL("dnnrtTensorOp: dimB[%d]=%ld cannot broadcast to %ld", i, (long)dimB[i], (long)dimA[i]);
  if (handle->format != DNNRT_NCHW && rankA == 4) {
    // A channels-last [N,C,H,W] tensor is a dense [N,H,W,C] array: permute
    // the dims of both operands accordingly before collapsing.
    const int64_t pa[4] = {dimA[0], dimA[2], dimA[3], dimA[1]}, pb[4] = {dimB[0], dimB[2], dimB[3], dimB[1]};
    bool ok;
    if (dtype == DNNRT_F16)
      ok = op == DNNRT_OP_ADD ? run_binary<__half>(handle, A, B, O, pa, pb, 4, FAdd{coefB})
                              : run_binary<__half>(handle, A, B, O, pa, pb, 4, FMul{coefB});
    else if (dtype == DNNRT_F32)
      ok = op == DNNRT_OP_ADD ? run_binary<float>(handle, A, B, O, pa, pb, 4, FAdd{coefB})
                              : run_binary<float>(handle, A, B, O, pa, pb, 4, FMul{coefB});
    else DNNRT_FAIL("dnnrtTensorOp: dtype %d", dtype);
    return ok ? O : nullptr;
  }
  bool ok;
  if (dtype == DNNRT_F32)
    ok = op == DNNRT_OP_ADD ? run_binary<float>(handle, A, B, O, dimA, dimB, rankA, FAdd{coefB})
                            : run_binary<float>(handle, A, B, O, dimA, dimB, rankA, FMul{coefB});
  else if (dtype == DNNRT_F16)
    ok = op == DNNRT_OP_ADD ? run_binary<__half>(handle, A, B, O, dimA, dimB, rankA, FAdd{coefB})
                            : run_binary<__half>(handle, A, B, O, dimA, dimB, rankA, FMul{coefB});
  else DNNRT_FAIL("dnnrtTensorOp: dtype %d", dtype);
  return ok ? O : nullptr;
}

}  // extern "C"
