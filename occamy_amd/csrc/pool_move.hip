// Pooling and pure data-movement entry points (all HBM-bound).
// Reference wrappers replaced (under src/Tools/dnn-wrapper/):
//   cudnn/CUDNNMaxPoolFunc.cpp, cudnn/CUDNNAveragePoolFunc.cpp,
//   cuda/CUDAFlattenFunc.cpp, CUDAReshapeFunc.cpp,
//   CUDATranspose{2,3,4,6}D{Float,Int64}Func.cu, CUDAGatherFloatFunc.cu,
//   CUDAConcat{Float,Int64}Func.cu, CUDA{Squeeze,Unsqueeze}{Float,Int64}Func.cpp.
#include "common.h"

namespace dnnrt {

__device__ __forceinline__ float pl_ld(const float *p) { return *p; }
__device__ __forceinline__ float pl_ld(const __half *p) { return __half2float(*p); }
__device__ __forceinline__ void pl_st(float *p, float v) { *p = v; }
__device__ __forceinline__ void pl_st(__half *p, float v) { *p = __float2half_rn(v); }

// One thread per output element.  Element strides of the input / output are
// passed in, so the same kernel serves NCHW (w fastest) and NHWC (c fastest);
// the thread index runs over the output in its memory order.
struct PoolGeom {
  int N, C, H, W, P, Q, R, S, ph, pw, sh, sw;
  int nhwc;
};
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(256) void pool_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                   PoolGeom g, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  int n, c, p, q;
  int64_t t = i;
  if (g.nhwc) {
    c = (int)(t % g.C); t /= g.C; q = (int)(t % g.Q); t /= g.Q; p = (int)(t % g.P); n = (int)(t / g.P);
  } else {
    q = (int)(t % g.Q); t /= g.Q; p = (int)(t % g.P); t /= g.P; c = (int)(t % g.C); n = (int)(t / g.C);
  }
  const int64_t sx_w = g.nhwc ? g.C : 1, sx_h = sx_w * g.W;
  const T *xb = g.nhwc ? x + (int64_t)n * g.H * g.W * g.C + c : x + ((int64_t)n * g.C + c) * g.H * g.W;
  const int ih0 = p * g.sh - g.ph, iw0 = q * g.sw - g.pw;
  float m = -INFINITY, s = 0.f;
  bool nan = false;
  for (int r = 0; r < g.R; r++) {
    const int ih = ih0 + r;
    if ((unsigned)ih >= (unsigned)g.H) continue;
    for (int ss = 0; ss < g.S; ss++) {
      const int iw = iw0 + ss;
      if ((unsigned)iw >= (unsigned)g.W) continue;
      const float v = pl_ld(xb + ih * sx_h + iw * sx_w);
      nan = nan || (v != v);
      m = v > m ? v : m;
      s += v;
    }
  }
  const float out = IS_MAX ? (nan ? __builtin_nanf("") : m) : s / (float)(g.R * g.S);
  pl_st(y + i, out);
}

// Channels-last fp16, C % 8 == 0: one thread per output pixel and group of
// eight channels, 16-byte loads and stores (the scalar kernel above reads two
// bytes per lane).  Same arithmetic: fp32 max / sum, NaN propagates.
typedef _Float16 pl_half8 __attribute__((ext_vector_type(8)));
template <bool IS_MAX>
__global__ __launch_bounds__(256) void pool_nhwc_f16x8_kernel(const _Float16 *__restrict__ x, _Float16 *__restrict__ y,
                                                              PoolGeom g, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int c8 = g.C >> 3;
  int64_t t = i;
  const int cg = (int)(t % c8); t /= c8;
  const int q = (int)(t % g.Q); t /= g.Q;
  const int p = (int)(t % g.P);
  const int n = (int)(t / g.P);
  const _Float16 *xb = x + (int64_t)n * g.H * g.W * g.C + cg * 8;
  const int ih0 = p * g.sh - g.ph, iw0 = q * g.sw - g.pw;
  float m[8], s[8];
  bool nan[8];
#pragma unroll
  for (int e = 0; e < 8; e++) { m[e] = -INFINITY; s[e] = 0.f; nan[e] = false; }
  for (int r = 0; r < g.R; r++) {
    const int ih = ih0 + r;
    if ((unsigned)ih >= (unsigned)g.H) continue;
    for (int ss = 0; ss < g.S; ss++) {
      const int iw = iw0 + ss;
      if ((unsigned)iw >= (unsigned)g.W) continue;
      const pl_half8 v8 = *reinterpret_cast<const pl_half8 *>(xb + ((int64_t)ih * g.W + iw) * g.C);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float v = (float)v8[e];
        nan[e] = nan[e] || (v != v);
        m[e] = v > m[e] ? v : m[e];
        s[e] += v;
      }
    }
  }
  pl_half8 o;
#pragma unroll
  for (int e = 0; e < 8; e++)
    o[e] = (_Float16)(IS_MAX ? (nan[e] ? __builtin_nanf("") : m[e]) : s[e] / (float)(g.R * g.S));
  *reinterpret_cast<pl_half8 *>(y + i * 8) = o;
}

// The same for a window size known at compile time: every tap is loaded
// unconditionally from an address clamped into the image (all R * S loads in
// flight at once) and a tap outside the image is replaced by -inf / 0 with a
// select.  With the loads under the bounds checks of the loops above each tap
// was a memory round trip of its own.
//
// TILED (C % 64 == 0): a workgroup is 64 channels of a 4 x 8 patch of output
// pixels instead of 256 consecutive (channel group, pixel) pairs of one row,
// so that overlapping windows (3x3, stride 2) meet in the workgroup's own
// cache: its input patch is 1.2 times its share of the image instead of 2.25.
template <bool IS_MAX, int R, int S, bool TILED>
__global__ __launch_bounds__(256) void pool_nhwc_f16x8_fixed_kernel(const _Float16 *__restrict__ x, _Float16 *__restrict__ y,
                                                                    PoolGeom g, int64_t total) {
  const int c8 = g.C >> 3;
  int cg, q, p, n;
  int64_t i;
  if (TILED) {
    const int tq = (g.Q + 7) >> 3, tp = (g.P + 3) >> 2, cb = c8 >> 3;
    unsigned b = blockIdx.x;
    const unsigned bc = b % (unsigned)cb; b /= (unsigned)cb;
    const unsigned bq = b % (unsigned)tq; b /= (unsigned)tq;
    const unsigned bp = b % (unsigned)tp;
    n = (int)(b / (unsigned)tp);
    cg = (int)bc * 8 + (threadIdx.x & 7);
    q = (int)bq * 8 + ((threadIdx.x >> 3) & 7);
    p = (int)bp * 4 + (threadIdx.x >> 6);
    if (p >= g.P || q >= g.Q) return;
    i = (((int64_t)n * g.P + p) * g.Q + q) * c8 + cg;
  } else {
    i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    int64_t t = i;
    cg = (int)(t % c8); t /= c8;
    q = (int)(t % g.Q); t /= g.Q;
    p = (int)(t % g.P);
    n = (int)(t / g.P);
  }
  const _Float16 *xb = x + (int64_t)n * g.H * g.W * g.C + cg * 8;
  const int ih0 = p * g.sh - g.ph, iw0 = q * g.sw - g.pw;
  pl_half8 v8[R][S];
  bool ok[R][S];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int ss = 0; ss < S; ss++) {
      const int ih = ih0 + r, iw = iw0 + ss;
      ok[r][ss] = (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
      const int ihc = min(max(ih, 0), g.H - 1), iwc = min(max(iw, 0), g.W - 1);
      v8[r][ss] = *reinterpret_cast<const pl_half8 *>(xb + ((int64_t)ihc * g.W + iwc) * g.C);
    }
  float m[8], sum[8];
  bool nan[8];
#pragma unroll
  for (int e = 0; e < 8; e++) { m[e] = -INFINITY; sum[e] = 0.f; nan[e] = false; }
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int ss = 0; ss < S; ss++)
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float raw = (float)v8[r][ss][e];
        const float v = ok[r][ss] ? raw : (IS_MAX ? -INFINITY : 0.f);
        nan[e] = nan[e] || (v != v);
        m[e] = v > m[e] ? v : m[e];
        sum[e] += v;
      }
  pl_half8 o;
#pragma unroll
  for (int e = 0; e < 8; e++)
    o[e] = (_Float16)(IS_MAX ? (nan[e] ? __builtin_nanf("") : m[e]) : sum[e] / (float)(R * S));
  *reinterpret_cast<pl_half8 *>(y + i * 8) = o;
}

static void *pool_entry(const char *who, dnnrtHandle_t h, const void *X, const int64_t *dX, void *Y,
                        const int64_t *dY, const int64_t *kr, const int64_t *pads, const int64_t *st,
                        bool is_max, int32_t dtype) {
  if (!h) DNNRT_FAIL("%s: null handle", who);
  if (!X || !Y || !dX || !dY || !kr || !pads || !st) DNNRT_FAIL("%s: null argument", who);
  if (dY[0] != dX[0] || dY[1] != dX[1]) DNNRT_FAIL("%s: N and C of X and Y differ", who);
  // an empty batch is no work: nothing is launched and Y is left as it is (the reference's zero-block launches do nothing either)
  if (dX[0] == 0 || dX[1] == 0) return Y;
  for (int i = 0; i < 4; i++)
    if (dX[i] <= 0 || dY[i] <= 0 || dX[i] > INT32_MAX) DNNRT_FAIL("%s: bad dims", who);
  if (kr[0] < 1 || kr[1] < 1 || st[0] < 1 || st[1] < 1 || pads[0] < 0 || pads[1] < 0)
    DNNRT_FAIL("%s: bad kernel/strides/pads", who);
  PoolGeom g;
  g.N = (int)dX[0]; g.C = (int)dX[1]; g.H = (int)dX[2]; g.W = (int)dX[3];
  g.P = (int)dY[2]; g.Q = (int)dY[3]; g.R = (int)kr[0]; g.S = (int)kr[1];
  g.ph = (int)pads[0]; g.pw = (int)pads[1]; g.sh = (int)st[0]; g.sw = (int)st[1];
  g.nhwc = h->format != DNNRT_NCHW;
  // every window must touch the input, or max would be -inf / avg 0 silently
  if ((int64_t)(g.P - 1) * g.sh - g.ph >= g.H || (int64_t)(g.Q - 1) * g.sw - g.pw >= g.W ||
      g.ph >= g.R || g.pw >= g.S)
    DNNRT_FAIL("%s: a pooling window lies outside the input", who);
  const int64_t total = numel(dY, 4), blocks = ceil_div(total, 256);
  if (blocks > INT32_MAX) DNNRT_FAIL("%s: tensor too large", who);
  if (dtype == DNNRT_F16 && g.nhwc && g.C % 8 == 0 && aligned16(X) && aligned16(Y)) {
    const int64_t tot8 = total / 8, blocks8 = ceil_div(tot8, 256);
    const int64_t tiled_blocks = (int64_t)g.N * ((g.P + 3) / 4) * ((g.Q + 7) / 8) * (g.C / 64);
    const bool tiled = g.C % 64 == 0 && tiled_blocks <= INT32_MAX;
#define POOL_FIXED_T(MX_, R_, S_)                                                                                          \
  do {                                                                                                                      \
    if (tiled) hipLaunchKernelGGL((pool_nhwc_f16x8_fixed_kernel<MX_, R_, S_, true>), dim3((unsigned)tiled_blocks), dim3(256), 0, \
                                  h->stream, (const _Float16 *)X, (_Float16 *)Y, g, tot8);                                  \
    else hipLaunchKernelGGL((pool_nhwc_f16x8_fixed_kernel<MX_, R_, S_, false>), dim3((unsigned)blocks8), dim3(256), 0,      \
                            h->stream, (const _Float16 *)X, (_Float16 *)Y, g, tot8);                                        \
  } while (0)
#define POOL_FIXED(R_, S_)                                                                                                  \
  do {                                                                                                                      \
    if (is_max) POOL_FIXED_T(true, R_, S_); else POOL_FIXED_T(false, R_, S_);                                               \
    DNNRT_CHECK_LAUNCH(who);                                                                                                \
    return Y;                                                                                                               \
  } while (0)
    if (g.R == 3 && g.S == 3) POOL_FIXED(3, 3);
    if (g.R == 2 && g.S == 2) POOL_FIXED(2, 2);
#undef POOL_FIXED
#undef POOL_FIXED_T
    if (is_max)
      hipLaunchKernelGGL((pool_nhwc_f16x8_kernel<true>), dim3((unsigned)blocks8), dim3(256), 0, h->stream,
                         (const _Float16 *)X, (_Float16 *)Y, g, tot8);
    else
      hipLaunchKernelGGL((pool_nhwc_f16x8_kernel<false>), dim3((unsigned)blocks8), dim3(256), 0, h->stream,
                         (const _Float16 *)X, (_Float16 *)Y, g, tot8);
    DNNRT_CHECK_LAUNCH(who);
    return Y;
  }
#define POOL_LAUNCH(T, MX)                                                                       \
  hipLaunchKernelGGL((pool_kernel<T, MX>), dim3((unsigned)blocks), dim3(256), 0, h->stream,      \
                     (const T *)X, (T *)Y, g, total)
  if (dtype == DNNRT_F32) { if (is_max) POOL_LAUNCH(float, true); else POOL_LAUNCH(float, false); }
  else if (dtype == DNNRT_F16) { if (is_max) POOL_LAUNCH(__half, true); else POOL_LAUNCH(__half, false); }
  else DNNRT_FAIL("%s: dtype %d", who, dtype);
#undef POOL_LAUNCH
  DNNRT_CHECK_LAUNCH(who);
  return Y;
}

struct PermGeom {
  int64_t dy[6];  // output dims
  int64_t sx[6];  // input stride of the dim each output dim comes from
};
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                        PermGeom g, int rank, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  int64_t rem = i, ix = 0;
  for (int d = rank - 1; d >= 0; d--) {
    const int64_t q = rem / g.dy[d];
    ix += (rem - q * g.dy[d]) * g.sx[d];
    rem = q;
  }
  y[i] = x[ix];
}

// The same for tensors below 2^31 elements, V consecutive output elements
// per thread (V divides the last output dim): 32-bit index arithmetic, one
// V-element store, and one V-element load too when the last output dim is
// the input's last dim as well (CONTIG).  Dims arrive merged where a run of
// output dims is a run of input dims, and without size-1 dims.
struct PermGeom32 {
  unsigned dy[6];  // output dims, the last one divided by V
  unsigned sx[6];  // input strides in elements
};
template <typename U, int V> struct alignas(sizeof(U) * V) VecOf { U v[V]; };
template <typename U, int V, bool CONTIG>
__global__ __launch_bounds__(256) void transpose_vec_kernel(const U *__restrict__ x, U *__restrict__ y,
                                                            PermGeom32 g, int rank, unsigned units) {
  const unsigned i = blockIdx.x * 256u + threadIdx.x;
  if (i >= units) return;
  unsigned rem = i, ix = 0;
#pragma unroll 1
  for (int d = rank - 1; d >= 0; d--) {
    const unsigned q = rem / g.dy[d];
    ix += (rem - q * g.dy[d]) * g.sx[d] * (d == rank - 1 ? (unsigned)V : 1u);
    rem = q;
  }
  VecOf<U, V> out;
  if (CONTIG) {
    out = *reinterpret_cast<const VecOf<U, V> *>(x + ix);
  } else {
    const unsigned step = g.sx[rank - 1];
#pragma unroll
    for (int j = 0; j < V; j++) out.v[j] = x[ix + (unsigned)j * step];
  }
  reinterpret_cast<VecOf<U, V> *>(y)[i] = out;
}

// Y[o, j, in] = X[o, idx[j], in]; out-of-range indices produce zeros.
template <typename T>
__global__ __launch_bounds__(256) void gather_kernel(const T *__restrict__ x, const int64_t *__restrict__ idx,
                                                     T *__restrict__ y, int64_t ni, int64_t L,
                                                     int64_t inner, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t in = i % inner, t = i / inner, j = t % ni, o = t / ni;
  int64_t k = idx[j];
  if (k < 0) k += L;
  T v = T(0);
  if (k >= 0 && k < L) v = x[(o * L + k) * inner + in];
  y[i] = v;
}

static int64_t esize(int32_t dtype) {
  return dtype == DNNRT_F32 ? 4 : dtype == DNNRT_F16 ? 2 : dtype == DNNRT_I64 ? 8 : 0;
}

// Plain copy, 16 bytes per lane where both pointers allow it.  A kernel rather
// than a memcpy call so that a captured graph holds kernel nodes only.
__global__ __launch_bounds__(256) void copy16_kernel(const uint4 *__restrict__ x, uint4 *__restrict__ y, int64_t n16) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) y[i] = x[i];
}
__global__ __launch_bounds__(256) void copy1_kernel(const uint8_t *__restrict__ x, uint8_t *__restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) y[i] = x[i];
}

static void *copy_entry(const char *who, dnnrtHandle_t h, const void *X, const int64_t *dX, int64_t rank,
                        void *Y, int32_t dtype) {
  if (!h) DNNRT_FAIL("%s: null handle", who);
  if (!X || !Y || !dX) DNNRT_FAIL("%s: null argument", who);
  const int64_t es = esize(dtype);
  if (!es) DNNRT_FAIL("%s: dtype %d", who, dtype);
  if (h->format != DNNRT_NCHW && rank == 4 && dX[1] > 1 && dX[2] * dX[3] > 1)
    DNNRT_FAIL("%s: a channels-last tensor with spatial extent cannot be re-viewed by a copy", who);
  const int64_t bytes = numel(dX, rank) * es;
  if (bytes > 0 && X != Y) {
    const int64_t n16 = (aligned16(X) && aligned16(Y)) ? bytes / 16 : 0, tail = bytes - n16 * 16;
    if (ceil_div(bytes, 256) > INT32_MAX) DNNRT_FAIL("%s: tensor too large", who);
    if (n16 > 0)
      hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)ceil_div(n16, 256)), dim3(256), 0, h->stream,
                         (const uint4 *)X, (uint4 *)Y, n16);
    if (tail > 0)
      hipLaunchKernelGGL(copy1_kernel, dim3((unsigned)ceil_div(tail, 256)), dim3(256), 0, h->stream,
                         (const uint8_t *)X + n16 * 16, (uint8_t *)Y + n16 * 16, tail);
    DNNRT_CHECK_LAUNCH(who);
  }
  return Y;
}

// Concatenation along one axis.  Every tensor is seen as [outer][row] with
// row = dim[axis] * inner; output row j comes from the input whose span of
// the output row holds j.  U is the copy unit: 16 bytes when every row length
// and pointer allows it, else one element.
constexpr int CONCAT_MAX_INPUTS = 16;
struct ConcatGeom {
  const void *x[CONCAT_MAX_INPUTS];
  int64_t begin[CONCAT_MAX_INPUTS + 1];  // prefix sums of the input rows, in units
  int n;
};
template <typename U>
__global__ __launch_bounds__(256) void concat_kernel(ConcatGeom g, U *__restrict__ y, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t row = g.begin[g.n], o = i / row, j = i - o * row;
  int s = 0;
#pragma unroll 1
  for (int k = 1; k < g.n; k++) s += j >= g.begin[k] ? 1 : 0;
  const int64_t len = g.begin[s + 1] - g.begin[s];
  y[i] = static_cast<const U *>(g.x[s])[o * len + (j - g.begin[s])];
}


// Expand: output element i reads the input element whose index along every
// broadcast axis is 0 (input stride 0 there).  U is the element as an
// unsigned integer of the same width: the values are only moved.
constexpr int EXPAND_MAX_RANK = 8;
struct ExpandGeom {
  int64_t out_dim[EXPAND_MAX_RANK], in_stride[EXPAND_MAX_RANK];
  int rank;
};
template <typename U>
__global__ __launch_bounds__(256) void expand_kernel(ExpandGeom g, const U *__restrict__ x, U *__restrict__ y, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  int64_t rest = i, src = 0;
#pragma unroll 1
  for (int d = g.rank - 1; d >= 0; d--) {
    const int64_t q = rest / g.out_dim[d];
    src += (rest - q * g.out_dim[d]) * g.in_stride[d];
    rest = q;
  }
  y[i] = x[src];
}

// NonZero, in the reference's sense: the flat indices of the elements that are
// not zero, in ascending order, converted to the tensor's own element type and
// written to the front of Y; the rest of Y is left as it is.  One workgroup
// walks the tensor 1024 elements at a time: a ballot gives every wavefront its
// count and every lane its rank inside the wavefront, the 16 wavefront counts
// are summed in LDS, and the running total stays in a register.
template <typename T> __device__ __forceinline__ bool is_nonzero(T v) { return v != T(0); }
template <> __device__ __forceinline__ bool is_nonzero<__half>(__half v) { return __half2float(v) != 0.f; }
template <typename T> __device__ __forceinline__ T from_index(int64_t j) { return (T)j; }
template <> __device__ __forceinline__ __half from_index<__half>(int64_t j) { return __float2half((float)j); }
template <typename T>
__global__ __launch_bounds__(1024) void nonzero_kernel(const T *__restrict__ x, T *__restrict__ y, int64_t n, int64_t cap) {
  __shared__ int wave_count[2][16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int64_t base = 0;
  int flip = 0;
  for (int64_t start = 0; start < n; start += 1024, flip ^= 1) {
    const int64_t j = start + threadIdx.x;
    const bool hit = j < n && is_nonzero<T>(x[j]);
    const unsigned long long votes = __ballot(hit);
    if (lane == 0) wave_count[flip][wave] = __popcll(votes);
    __syncthreads();  // the other half of wave_count is what the previous chunk used
    int before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < 16; w++) {
      const int c = wave_count[flip][w];
      before += w < wave ? c : 0;
      all += c;
    }
    if (hit) {
      const int64_t slot = base + before + __popcll(votes & ((1ull << lane) - 1ull));
      if (slot < cap) y[slot] = from_index<T>(j);
    }
    base += all;
  }
}

}  // namespace dnnrt

using namespace dnnrt;

extern "C" {

void *dnnrtMaxPool(dnnrtHandle_t handle, const void *X, const int64_t *dimX, void *Y, const int64_t *dimY,
                   const int64_t *kernel, const int64_t *pads, const int64_t *strides, int32_t dtype) {
  return pool_entry("dnnrtMaxPool", handle, X, dimX, Y, dimY, kernel, pads, strides, true, dtype);
}
void *dnnrtAveragePool(dnnrtHandle_t handle, const void *X, const int64_t *dimX, void *Y,
                       const int64_t *dimY, const int64_t *kernel, const int64_t *pads,
                       const int64_t *strides, int32_t dtype) {
  return pool_entry("dnnrtAveragePool", handle, X, dimX, Y, dimY, kernel, pads, strides, false, dtype);
}

void *dnnrtFlatten(dnnrtHandle_t handle, const void *X, const int64_t *dimX, void *Y, const int64_t *dimY,
                   int32_t axis, int64_t rank, int32_t dtype) {
  (void)dimY; (void)axis;
  return copy_entry("dnnrtFlatten", handle, X, dimX, rank, Y, dtype);
}
void *dnnrtReshape(dnnrtHandle_t handle, const void *X, const int64_t *dimX, int64_t rankX, void *Y,
                   int32_t dtype) {
  return copy_entry("dnnrtReshape", handle, X, dimX, rankX, Y, dtype);
}

// Squeeze / Unsqueeze move no data around: dimY must be dimX with size-1 dims
// removed or inserted.
static void *same_order_copy(const char *who, dnnrtHandle_t h, const void *X, const int64_t *dX, int64_t rX,
                             void *Y, const int64_t *dY, int64_t rY, int32_t dtype) {
  if (!h) DNNRT_FAIL("%s: null handle", who);
  if (!X || !Y || !dX || !dY || rX < 0 || rY < 0) DNNRT_FAIL("%s: null argument", who);
  int64_t i = 0, j = 0;
  while (true) {
    while (i < rX && dX[i] == 1) i++;
    while (j < rY && dY[j] == 1) j++;
    if (i == rX || j == rY) break;
    if (dX[i] != dY[j]) DNNRT_FAIL("%s: dims differ beyond size-1 axes (%ld vs %ld)", who, (long)dX[i], (long)dY[j]);
    i++; j++;
  }
  if (i != rX || j != rY) DNNRT_FAIL("%s: dims differ beyond size-1 axes", who);
  if (h->format != DNNRT_NCHW && (rX == 4 || rY == 4)) DNNRT_FAIL("%s: channels-last tensors are not supported", who);
  return copy_entry(who, h, X, dX, rX, Y, dtype);
}

void *dnnrtSqueeze(dnnrtHandle_t handle, const void *X, const int64_t *dimX, int64_t rankX, void *Y,
                   const int64_t *dimY, int64_t rankY, int32_t dtype) {
  return same_order_copy("dnnrtSqueeze", handle, X, dimX, rankX, Y, dimY, rankY, dtype);
}
void *dnnrtUnsqueeze(dnnrtHandle_t handle, const void *X, const int64_t *dimX, int64_t rankX, void *Y,
                     const int64_t *dimY, int64_t rankY, int32_t dtype) {
  return same_order_copy("dnnrtUnsqueeze", handle, X, dimX, rankX, Y, dimY, rankY, dtype);
}

void *dnnrtExpand(dnnrtHandle_t handle, const void *X, const int64_t *dimX, int64_t rankX, void *Y,
                  const int64_t *dimY, int64_t rankY, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtExpand: null handle");
  if (!X || !Y || !dimX || !dimY) DNNRT_FAIL("dnnrtExpand: null argument");
  if (rankY < 1 || rankY > EXPAND_MAX_RANK || rankX < 0 || rankX > rankY)
    DNNRT_FAIL("dnnrtExpand: ranks %ld -> %ld (input rank <= output rank <= %d)", (long)rankX, (long)rankY, EXPAND_MAX_RANK);
  const int64_t es = esize(dtype);
  if (!es) DNNRT_FAIL("dnnrtExpand: dtype %d", dtype);
  if (handle->format != DNNRT_NCHW && (rankX == 4 || rankY == 4)) DNNRT_FAIL("dnnrtExpand: channels-last tensors are not supported");
  ExpandGeom g{};
  g.rank = (int)rankY;
  int64_t stride = 1;
  for (int64_t d = rankY - 1; d >= 0; d--) {
    const int64_t dx = d - (rankY - rankX);  // dimX is aligned with the trailing dims of dimY
    const int64_t in = dx >= 0 ? dimX[dx] : 1;
    if (dimY[d] < 0 || in < 0) DNNRT_FAIL("dnnrtExpand: negative dim");
    if (in != dimY[d] && in != 1) DNNRT_FAIL("dnnrtExpand: input dim %ld cannot be broadcast to %ld", (long)in, (long)dimY[d]);
    g.out_dim[d] = dimY[d];
    g.in_stride[d] = in == 1 ? 0 : stride;
    stride *= in;
  }
  const int64_t total = numel(dimY, rankY);
  if (total == 0) return Y;
  if (ceil_div(total, 256) > INT32_MAX) DNNRT_FAIL("dnnrtExpand: tensor too large");
  const dim3 grid((unsigned)ceil_div(total, 256)), block(256);
  if (es == 8) hipLaunchKernelGGL(expand_kernel<uint64_t>, grid, block, 0, handle->stream, g, (const uint64_t *)X, (uint64_t *)Y, total);
  else if (es == 4) hipLaunchKernelGGL(expand_kernel<uint32_t>, grid, block, 0, handle->stream, g, (const uint32_t *)X, (uint32_t *)Y, total);
  else hipLaunchKernelGGL(expand_kernel<uint16_t>, grid, block, 0, handle->stream, g, (const uint16_t *)X, (uint16_t *)Y, total);
  DNNRT_CHECK_LAUNCH("dnnrtExpand");
  return Y;
}

void *dnnrtNonZero(dnnrtHandle_t handle, const void *X, const int64_t *dimX, int64_t rankX, void *Y,
                   const int64_t *dimY, int64_t rankY, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtNonZero: null handle");
  if (!X || !Y || !dimX || !dimY || rankX < 0 || rankY < 0) DNNRT_FAIL("dnnrtNonZero: null argument");
  if (handle->format != DNNRT_NCHW && rankX == 4) DNNRT_FAIL("dnnrtNonZero: channels-last tensors are not supported");
  const int64_t n = numel(dimX, rankX), cap = numel(dimY, rankY);
  if (n == 0) return Y;
  if (dtype == DNNRT_F32) hipLaunchKernelGGL(nonzero_kernel<float>, dim3(1), dim3(1024), 0, handle->stream, (const float *)X, (float *)Y, n, cap);
  else if (dtype == DNNRT_F16) hipLaunchKernelGGL(nonzero_kernel<__half>, dim3(1), dim3(1024), 0, handle->stream, (const __half *)X, (__half *)Y, n, cap);
  else if (dtype == DNNRT_I64) hipLaunchKernelGGL(nonzero_kernel<int64_t>, dim3(1), dim3(1024), 0, handle->stream, (const int64_t *)X, (int64_t *)Y, n, cap);
  else DNNRT_FAIL("dnnrtNonZero: dtype %d", dtype);
  DNNRT_CHECK_LAUNCH("dnnrtNonZero");
  return Y;
}

void *dnnrtConcat(dnnrtHandle_t handle, const void *const *X, const int64_t *const *dimX, void *Y,
                  const int64_t *dimY, int64_t axis, int64_t numInputs, int32_t rank, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtConcat: null handle");
  if (!X || !dimX || !Y || !dimY) DNNRT_FAIL("dnnrtConcat: null argument");
  if (rank < 1 || rank > 8) DNNRT_FAIL("dnnrtConcat: rank %d (1..8)", rank);
  if (numInputs < 1 || numInputs > CONCAT_MAX_INPUTS) DNNRT_FAIL("dnnrtConcat: %ld inputs (1..%d)", (long)numInputs, CONCAT_MAX_INPUTS);
  if (axis < 0) axis += rank;
  if (axis < 0 || axis >= rank) DNNRT_FAIL("dnnrtConcat: axis out of range");
  const int64_t es = esize(dtype);
  if (!es) DNNRT_FAIL("dnnrtConcat: dtype %d", dtype);
  int64_t along = 0;
  for (int64_t k = 0; k < numInputs; k++) {
    if (!X[k] || !dimX[k]) DNNRT_FAIL("dnnrtConcat: null input %ld", (long)k);
    for (int i = 0; i < rank; i++)
      if (dimX[k][i] < 0 || (i != axis && dimX[k][i] != dimY[i])) DNNRT_FAIL("dnnrtConcat: input %ld dim %d differs from the output's", (long)k, i);
    along += dimX[k][axis];
  }
  if (along != dimY[axis]) DNNRT_FAIL("dnnrtConcat: the inputs' dims along the axis sum to %ld, dimY has %ld", (long)along, (long)dimY[axis]);
  // memory order of the dims: a channels-last [N,C,H,W] tensor is a dense [N,H,W,C] array
  int order[8];
  for (int i = 0; i < rank; i++) order[i] = i;
  if (handle->format != DNNRT_NCHW && rank == 4) { order[1] = 2; order[2] = 3; order[3] = 1; }
  int64_t outer = 1, inner = 1;
  bool before = true;
  for (int i = 0; i < rank; i++) {
    if (order[i] == axis) { before = false; continue; }
    (before ? outer : inner) *= dimY[order[i]];
  }
  ConcatGeom g;
  g.n = (int)numInputs;
  bool vec = aligned16(Y);
  for (int64_t k = 0; k < numInputs; k++) {
    vec = vec && aligned16(X[k]) && (dimX[k][axis] * inner * es) % 16 == 0;
    g.x[k] = X[k];
  }
  const int64_t unit = vec ? 16 : es;
  g.begin[0] = 0;
  for (int64_t k = 0; k < numInputs; k++) g.begin[k + 1] = g.begin[k] + dimX[k][axis] * inner * es / unit;
  const int64_t total = outer * g.begin[numInputs];
  if (total == 0) return Y;
  const int64_t blocks = ceil_div(total, 256);
  if (blocks > INT32_MAX) DNNRT_FAIL("dnnrtConcat: tensor too large");
  const dim3 grid((unsigned)blocks), block(256);
  if (unit == 16) hipLaunchKernelGGL((concat_kernel<uint4>), grid, block, 0, handle->stream, g, (uint4 *)Y, total);
  else if (unit == 8) hipLaunchKernelGGL((concat_kernel<uint64_t>), grid, block, 0, handle->stream, g, (uint64_t *)Y, total);
  else if (unit == 4) hipLaunchKernelGGL((concat_kernel<uint32_t>), grid, block, 0, handle->stream, g, (uint32_t *)Y, total);
  else hipLaunchKernelGGL((concat_kernel<uint16_t>), grid, block, 0, handle->stream, g, (uint16_t *)Y, total);
  DNNRT_CHECK_LAUNCH("dnnrtConcat");
  return Y;
}

void *dnnrtTranspose(dnnrtHandle_t handle, const void *X, const int64_t *dimX, void *Y,
                     const int64_t *dimY, const int64_t *perm, int64_t rank, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtTranspose: null handle");
  if (!X || !Y || !dimX || !dimY || !perm) DNNRT_FAIL("dnnrtTranspose: null argument");
  if (rank < 1 || rank > 6) DNNRT_FAIL("dnnrtTranspose: rank %ld (1..6)", (long)rank);
  if (handle->format != DNNRT_NCHW && rank == 4) DNNRT_FAIL("dnnrtTranspose: channels-last tensors are not supported");
  int64_t sx[6], s = 1;
  bool seen[6] = {false, false, false, false, false, false};
  for (int i = (int)rank - 1; i >= 0; i--) { sx[i] = s; s *= dimX[i]; }
  PermGeom g;
  for (int i = 0; i < rank; i++) {
    if (perm[i] < 0 || perm[i] >= rank || seen[perm[i]]) DNNRT_FAIL("dnnrtTranspose: perm is not a permutation");
    seen[perm[i]] = true;
    if (dimY[i] != dimX[perm[i]] || dimY[i] < 0) DNNRT_FAIL("dnnrtTranspose: dimY[%d] != dimX[perm[%d]]", i, i);
    g.dy[i] = dimY[i];
    g.sx[i] = sx[perm[i]];
  }
  const int64_t es = esize(dtype);
  if (!es) DNNRT_FAIL("dnnrtTranspose: dtype %d", dtype);
  if (s == 0) return Y;  // an empty tensor: nothing to move
  if (s > 0 && s < (1ll << 31)) {
    // size-1 dims dropped, runs of dims that stay together merged
    int64_t my[6], ms[6];
    int n = 0;
    for (int i = 0; i < rank; i++) {
      if (g.dy[i] == 1) continue;
      if (n > 0 && ms[n - 1] == g.sx[i] * g.dy[i]) { my[n - 1] *= g.dy[i]; ms[n - 1] = g.sx[i]; }
      else { my[n] = g.dy[i]; ms[n] = g.sx[i]; n++; }
    }
    if (n == 0) { my[0] = 1; ms[0] = 1; n = 1; }
    const bool contig = ms[n - 1] == 1;
    int v = (int)(16 / es);
    auto fits = [&](int w) {
      if (my[n - 1] % w || (reinterpret_cast<uintptr_t>(Y) % (uintptr_t)(w * es))) return false;
      if (!contig) return true;
      if (reinterpret_cast<uintptr_t>(X) % (uintptr_t)(w * es)) return false;
      for (int i = 0; i < n - 1; i++) if (ms[i] % w) return false;
      return true;
    };
    while (v > 1 && !fits(v)) v >>= 1;
    PermGeom32 h{};
    for (int i = 0; i < n; i++) { h.dy[i] = (unsigned)my[i]; h.sx[i] = (unsigned)ms[i]; }
    h.dy[n - 1] = (unsigned)(my[n - 1] / v);
    const unsigned units = (unsigned)(s / v), blocks32 = (units + 255u) / 256u;
#define LAUNCH_T(U, V_)                                                                                          \
  do {                                                                                                           \
    if (contig) hipLaunchKernelGGL((transpose_vec_kernel<U, V_, true>), dim3(blocks32), dim3(256), 0, handle->stream, (const U *)X, (U *)Y, h, n, units); \
    else hipLaunchKernelGGL((transpose_vec_kernel<U, V_, false>), dim3(blocks32), dim3(256), 0, handle->stream, (const U *)X, (U *)Y, h, n, units);      \
  } while (0)
    if (es == 4) { if (v == 4) LAUNCH_T(uint32_t, 4); else if (v == 2) LAUNCH_T(uint32_t, 2); else LAUNCH_T(uint32_t, 1); }
    else if (es == 2) { if (v == 8) LAUNCH_T(uint16_t, 8); else if (v == 4) LAUNCH_T(uint16_t, 4); else if (v == 2) LAUNCH_T(uint16_t, 2); else LAUNCH_T(uint16_t, 1); }
    else { if (v == 2) LAUNCH_T(uint64_t, 2); else LAUNCH_T(uint64_t, 1); }
#undef LAUNCH_T
    DNNRT_CHECK_LAUNCH("dnnrtTranspose");
    return Y;
  }
  const int64_t total = s, blocks = ceil_div(total, 256);
  if (blocks > INT32_MAX) DNNRT_FAIL("dnnrtTranspose: tensor too large");
  if (dtype == DNNRT_F32)
    hipLaunchKernelGGL((transpose_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, handle->stream,
                       (const float *)X, (float *)Y, g, (int)rank, total);
  else if (dtype == DNNRT_F16)
    hipLaunchKernelGGL((transpose_kernel<uint16_t>), dim3((unsigned)blocks), dim3(256), 0, handle->stream,
                       (const uint16_t *)X, (uint16_t *)Y, g, (int)rank, total);
  else if (dtype == DNNRT_I64)
    hipLaunchKernelGGL((transpose_kernel<int64_t>), dim3((unsigned)blocks), dim3(256), 0, handle->stream,
                       (const int64_t *)X, (int64_t *)Y, g, (int)rank, total);
  else DNNRT_FAIL("dnnrtTranspose: dtype %d", dtype);
  DNNRT_CHECK_LAUNCH("dnnrtTranspose");
  return Y;
}

void *dnnrtGather(dnnrtHandle_t handle, const void *X, const int64_t *dimX, int64_t rankX, void *Y,
                  const int64_t *dimY, int64_t rankY, const int64_t *indices, const int64_t *dimIndices,
                  int64_t rankIndices, int64_t axis, int32_t dtype) {
  (void)dimY; (void)rankY;
  if (!handle) DNNRT_FAIL("dnnrtGather: null handle");
  if (!X || !Y || !dimX || !indices || (rankIndices > 0 && !dimIndices)) DNNRT_FAIL("dnnrtGather: null argument");
  if (rankX < 1 || rankX > 8) DNNRT_FAIL("dnnrtGather: rank %ld", (long)rankX);
  if (axis < 0) axis += rankX;
  if (axis < 0 || axis >= rankX) DNNRT_FAIL("dnnrtGather: axis out of range");
  int64_t outer = 1, inner = 1;
  const int64_t ni = numel(dimIndices, rankIndices), L = dimX[axis];
  for (int64_t i = 0; i < axis; i++) outer *= dimX[i];
  for (int64_t i = axis + 1; i < rankX; i++) inner *= dimX[i];
  const int64_t total = outer * ni * inner;
  if (total == 0) return Y;
  const int64_t blocks = ceil_div(total, 256);
  if (blocks > INT32_MAX) DNNRT_FAIL("dnnrtGather: tensor too large");
  if (dtype == DNNRT_F32)
    hipLaunchKernelGGL((gather_kernel<float>), dim3((unsigned)blocks), dim3(256), 0, handle->stream,
                       (const float *)X, indices, (float *)Y, ni, L, inner, total);
  else if (dtype == DNNRT_F16)
    hipLaunchKernelGGL((gather_kernel<uint16_t>), dim3((unsigned)blocks), dim3(256), 0, handle->stream,
                       (const uint16_t *)X, indices, (uint16_t *)Y, ni, L, inner, total);
  else if (dtype == DNNRT_I64)
    hipLaunchKernelGGL((gather_kernel<int64_t>), dim3((unsigned)blocks), dim3(256), 0, handle->stream,
                       (const int64_t *)X, indices, (int64_t *)Y, ni, L, inner, total);
  else DNNRT_FAIL("dnnrtGather: dtype %d", dtype);
  DNNRT_CHECK_LAUNCH("dnnrtGather");
  return Y;
}

}  // extern "C"
