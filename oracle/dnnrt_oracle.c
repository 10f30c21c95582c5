/* dnnrt_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT.
 *
 * A CPU restatement, in plain C, of what each call of the reference's runtime
 * wrapper library (src/Tools/dnn-wrapper/ in the reference tree) computes,
 * exported under the same C ABI as the GPU library (include/dnnrt.h) so that
 * one DNN program can be executed against either.  Only tests, the smoke
 * check and the CPU-baseline leg of the benchmark may load this file's shared
 * object; nothing in the product package links or opens it.
 *
 * The reference's arithmetic for these calls lives in closed-source cuDNN
 * 8.9.0 / cuBLASLt (CUDA 11.8) and in its own CUDA kernels; neither can be
 * built or run here, and the reference's tests hold no golden vectors for
 * them.  Each function below therefore states the published definition of the
 * operator at the reference's call site (cited), and is pinned by the tests
 * against closed forms, brute force on tiny shapes and an independent library
 * (torch CPU) -- see tests/test_oracle_ops.py.  Nothing here was checked
 * against reference OUTPUT: parity with the reference's numbers is unpinned.
 *
 * Arithmetic: tensors are fp32 or fp16 in memory; fp16 tensors are widened to
 * fp32 on load and rounded to nearest-even on store.  Reductions (convolution,
 * matrix products, means, softmax sums) accumulate in double and round once,
 * so the oracle sits closer to the exact value than any fp32 summation order.
 * Layout is dense NCHW / row-major, as in the reference
 * (src/Tools/dnn-wrapper/cudnn/CUDNNConvFunc.cpp:48-60).
 */
#define _POSIX_C_SOURCE 200809L
#include "../include/dnnrt.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static __thread char g_err[256];
static int g_threads = 0; /* 0 = OpenMP default */

#define FAIL(...)                                                              \
  do {                                                                         \
    snprintf(g_err, sizeof g_err, __VA_ARGS__);                                \
    return NULL;                                                               \
  } while (0)

const char *dnnrtLastError(void) { return g_err; }
int32_t dnnrtIsHostBackend(void) { return 1; }

/* Oracle-only: number of OpenMP threads used by the heavy loops. */
int32_t dnnrtOracleSetThreads(int32_t n) {
  g_threads = n;
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#endif
  return 0;
}
int32_t dnnrtOracleGetThreads(void) {
#ifdef _OPENMP
  return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---- fp16 <-> fp32 (IEEE binary16, round to nearest even) -------------- */

static float h2f(uint16_t h) {
  uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1fu,
           m = h & 0x3ffu, u;
  if (e == 0) {
    if (m == 0) u = s;
    else {
      int sh = 0;
      while (!(m & 0x400u)) { m <<= 1; sh++; }
      u = s | ((uint32_t)(113 - sh) << 23) | ((m & 0x3ffu) << 13);
    }
  } else if (e == 31) u = s | 0x7f800000u | (m << 13);
  else u = s | ((e + 112) << 23) | (m << 13);
  float f; memcpy(&f, &u, 4); return f;
}
static uint16_t f2h(float f) {
  uint32_t u; memcpy(&u, &f, 4);
  uint32_t s = (u >> 16) & 0x8000u; int32_t e = (int32_t)((u >> 23) & 0xff);
  uint32_t m = u & 0x7fffffu;
  if (e == 255) return (uint16_t)(s | 0x7c00u | (m ? 0x200u | (m >> 13) : 0));
  e -= 112;
  if (e >= 31) return (uint16_t)(s | 0x7c00u);
  if (e <= 0) {
    if (e < -10) return (uint16_t)s;
    m |= 0x800000u;
    uint32_t shift = (uint32_t)(14 - e), r = m >> shift,
             rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (r & 1))) r++;
    return (uint16_t)(s | r);
  }
  uint32_t r = ((uint32_t)e << 10) | (m >> 13), rem = m & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) r++;
  return (uint16_t)(s | r);
}

static int64_t numel(const int64_t *d, int64_t rank) {
  int64_t n = 1;
  for (int64_t i = 0; i < rank; i++) n *= d[i];
  return n;
}
/* widen a tensor to a fresh float buffer (fp32: plain copy of the pointer) */
static const float *widen(const void *p, int64_t n, int32_t dtype, float **tmp) {
  *tmp = NULL;
  if (dtype == DNNRT_F32) return (const float *)p;
  float *t = (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
  const uint16_t *h = (const uint16_t *)p;
  for (int64_t i = 0; i < n; i++) t[i] = h2f(h[i]);
  *tmp = t;
  return t;
}
static float *outbuf(void *p, int64_t n, int32_t dtype, float **tmp) {
  *tmp = NULL;
  if (dtype == DNNRT_F32) return (float *)p;
  *tmp = (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
  return *tmp;
}
static void narrow(void *p, float *tmp, int64_t n, int32_t dtype) {
  if (dtype == DNNRT_F32 || !tmp) return;
  uint16_t *h = (uint16_t *)p;
  for (int64_t i = 0; i < n; i++) h[i] = f2h(tmp[i]);
  free(tmp);
}
static int bad_dtype(int32_t dtype) { return dtype != DNNRT_F32 && dtype != DNNRT_F16; }

/* ---- handle / stream / memory: host stand-ins -------------------------- */

struct dnnrtContext { int format; float act_coef; };

int32_t dnnrtCreate(dnnrtHandle_t *h) {
  *h = (dnnrtHandle_t)calloc(1, sizeof(struct dnnrtContext));
  return *h ? 0 : 1;
}
int32_t dnnrtDestroy(dnnrtHandle_t h) { free(h); return 0; }
int32_t dnnrtStreamCreate(dnnrtStream_t *s) { *s = NULL; return 0; }
int32_t dnnrtStreamDestroy(dnnrtStream_t s) { (void)s; return 0; }
int32_t dnnrtSetStream(dnnrtHandle_t h, dnnrtStream_t s) { (void)h; (void)s; return 0; }
int32_t dnnrtSetTensorFormat(dnnrtHandle_t h, int32_t format) {
  if (format != DNNRT_NCHW) {
    snprintf(g_err, sizeof g_err, "oracle: only NCHW is implemented");
    return 1;
  }
  h->format = format;
  return 0;
}
int32_t dnnrtSetFilterLayout(dnnrtHandle_t h, int32_t layout) {
  (void)h;
  if (layout != DNNRT_FILTER_KCRS) {
    snprintf(g_err, sizeof g_err, "oracle: only K,C,R,S filters are implemented");
    return 1;
  }
  return 0;
}
/* The oracle has one convolution (the 7-loop definition): no variants to list, only "automatic" to select. */
int32_t dnnrtListConvTiles(int32_t *ids, int32_t capacity) { (void)ids; (void)capacity; return 0; }
int32_t dnnrtSetConvTile(dnnrtHandle_t h, int32_t tile) {
  (void)h;
  if (tile != 0) { snprintf(g_err, sizeof g_err, "oracle: no convolution variants"); return 1; }
  return 0;
}
int32_t dnnrtSetActivationCoef(dnnrtHandle_t h, float coef) {
  if (!h || coef != coef) { snprintf(g_err, sizeof g_err, "setActivationCoef: bad argument"); return 1; }
  h->act_coef = coef;
  return 0;
}
int32_t dnnrtSync(dnnrtHandle_t h) { (void)h; return 0; }
static int32_t no_graph(void) { snprintf(g_err, sizeof g_err, "oracle: no stream capture on the host"); return 1; }
int32_t dnnrtGraphBegin(dnnrtHandle_t h) { (void)h; return no_graph(); }
int32_t dnnrtGraphEnd(dnnrtHandle_t h, void **g) { (void)h; (void)g; return no_graph(); }
int32_t dnnrtGraphLaunch(dnnrtHandle_t h, void *g) { (void)h; (void)g; return no_graph(); }
int32_t dnnrtGraphDestroy(void *g) { (void)g; return 0; }

/* host stand-in for stream timestamps: the wall clock at record time */
#include <time.h>
int32_t dnnrtEventCreate(void **e) { *e = calloc(1, sizeof(double)); return *e ? 0 : 1; }
int32_t dnnrtEventRecord(void *e, dnnrtStream_t s) {
  (void)s;
  struct timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  *(double *)e = (double)t.tv_sec * 1e3 + (double)t.tv_nsec * 1e-6;
  return 0;
}
int32_t dnnrtEventElapsedMs(void *a, void *b, float *ms) { *ms = (float)(*(double *)b - *(double *)a); return 0; }
int32_t dnnrtEventDestroy(void *e) { free(e); return 0; }

/* wrapDNNMemPoolInit.cpp:19-29 / wrapDNNMalloc.cpp: one allocation. */
/* "Device" memory of the host build is heap memory behind a 64-byte header that holds the block's size, so that
 * the same accounting call exists here (dnnrtDeviceMemoryStats): bytes taken and not yet returned, and their peak. */
static int64_t g_mem_now = 0, g_mem_peak = 0;
int32_t dnnrtMemPoolInit(void **pool, int64_t bytes) {
  const int64_t n = bytes > 0 ? bytes : 1;
  void *base = NULL;
  if (posix_memalign(&base, 64, (size_t)n + 64)) { *pool = NULL; return 1; }
  *(int64_t *)base = n;
  *pool = (char *)base + 64;
#pragma omp critical(dnnrt_mem)
  {
    g_mem_now += n;
    if (g_mem_now > g_mem_peak) g_mem_peak = g_mem_now;
  }
  return 0;
}
int32_t dnnrtMalloc(void **p, int64_t bytes) { return dnnrtMemPoolInit(p, bytes); }
int32_t dnnrtDealloc(void *p) {
  if (!p) return 0;
  void *base = (char *)p - 64;
#pragma omp critical(dnnrt_mem)
  g_mem_now -= *(int64_t *)base;
  free(base);
  return 0;
}
int32_t dnnrtDeviceMemoryStats(int64_t *allocated_now, int64_t *allocated_peak, int64_t *static_bytes, int32_t reset_peak) {
  if (allocated_now) *allocated_now = g_mem_now;
  if (allocated_peak) *allocated_peak = g_mem_peak;
  if (static_bytes) *static_bytes = 0;
  if (reset_peak) g_mem_peak = g_mem_now;
  return 0;
}
int32_t dnnrtHostAlloc(void **p, int64_t bytes) {
  *p = malloc((size_t)(bytes > 0 ? bytes : 1));
  return *p ? 0 : 1;
}
int32_t dnnrtHostFree(void *p) { free(p); return 0; }
/* wrapDNNMemOffset.cpp:26: *p = base + offset. */
int32_t dnnrtMemOffset(void **p, void *base, int64_t off, int64_t bytes) {
  (void)bytes;
  *p = (char *)base + off;
  return 0;
}
/* wrapDNNMemcpy.cpp:17-61. */
int32_t dnnrtMemFill(void *ptr, int32_t byte, int64_t bytes, dnnrtStream_t stream) {
  (void)stream;
  if (bytes > 0) memset(ptr, byte, (size_t)bytes);
  return 0;
}
int32_t dnnrtMemcpy(void *dst, void *src, int64_t bytes, int32_t kind, dnnrtStream_t s) {
  (void)kind; (void)s;
  if (bytes > 0) memmove(dst, src, (size_t)bytes);
  return 0;
}

/* ---- convolution -------------------------------------------------------
 * CUDNNConvFunc.cpp:9-105 calls cudnnConvolutionForward with
 * CUDNN_CROSS_CORRELATION, dilation 1, alpha 1, beta 0, `group` groups; the
 * published definition is
 *   Y[n,k,p,q] = sum_{c,r,s} X[n, g*Cg + c, p*sh - ph + r, q*sw - pw + s]
 *                            * W[k, c, r, s],        g = k / (K/group)
 * with out-of-range taps contributing 0.  CUDNNConvBiasReluFunc.cpp:8-140
 * adds B[k] and applies ReLU (mode 1) or identity (mode 5). */
static float act_apply(float v, int64_t mode, float coef) {
  switch (mode) {
  case DNNRT_ACT_RELU: return v < 0.0f ? 0.0f : v; /* NaN passes through */
  case DNNRT_ACT_CLIPPED_RELU: v = v < 0.0f ? 0.0f : v; return v > coef ? coef : v;
  case DNNRT_ACT_LEAKY_RELU: return v < 0.0f ? coef * v : v;
  case DNNRT_ACT_SIGMOID: return 1.0f / (1.0f + expf(-v));
  case DNNRT_ACT_TANH: return tanhf(v);
  default: return v;
  }
}

static void conv_core(const float *X, const int64_t *dX, const float *Wt,
                      const int64_t *dW, const float *B, int64_t group,
                      const int64_t *pads, const int64_t *strides, int64_t act,
                      float *Y) {
  const int64_t N = dX[0], C = dX[1], H = dX[2], Wd = dX[3];
  const int64_t K = dW[0], Cg = dW[1], R = dW[2], S = dW[3];
  const int64_t ph = pads[0], pw = pads[1], sh = strides[0], sw = strides[1];
  const int64_t P = (H + 2 * ph - R) / sh + 1, Q = (Wd + 2 * pw - S) / sw + 1;
  const int64_t Kg = K / group;
  (void)C;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (int64_t n = 0; n < N; n++)
    for (int64_t k = 0; k < K; k++) {
      double *acc = (double *)calloc((size_t)(P * Q), sizeof(double));
      const int64_t g = k / Kg;
      for (int64_t c = 0; c < Cg; c++) {
        const float *xc = X + ((n * dX[1] + g * Cg + c) * H) * Wd;
        for (int64_t r = 0; r < R; r++)
          for (int64_t s = 0; s < S; s++) {
            const double w = Wt[((k * Cg + c) * R + r) * S + s];
            for (int64_t p = 0; p < P; p++) {
              const int64_t ih = p * sh - ph + r;
              if (ih < 0 || ih >= H) continue;
              /* q range with 0 <= q*sw - pw + s < W */
              int64_t q0 = 0, q1 = Q;
              while (q0 < Q && q0 * sw - pw + s < 0) q0++;
              while (q1 > q0 && (q1 - 1) * sw - pw + s >= Wd) q1--;
              const float *xr = xc + ih * Wd - pw + s;
              double *ar = acc + p * Q;
              for (int64_t q = q0; q < q1; q++) ar[q] += w * (double)xr[q * sw];
            }
          }
      }
      float *y = Y + (n * K + k) * P * Q;
      const double b = B ? (double)B[k] : 0.0;
      for (int64_t i = 0; i < P * Q; i++) y[i] = act_apply((float)(acc[i] + b), act, 0.0f);
      free(acc);
    }
}

static void *conv_entry(const void *X, const int64_t *dX, const void *W,
                        const int64_t *dW, const void *B, int64_t group,
                        const int64_t *pads, const int64_t *strides,
                        int64_t act, void *Y, int32_t dtype) {
  if (bad_dtype(dtype)) FAIL("conv: bad dtype %d", dtype);
  if (group < 1 || dX[1] != dW[1] * group || dW[0] % group)
    FAIL("conv: C=%ld, W has C/g=%ld, group=%ld, K=%ld do not agree",
         (long)dX[1], (long)dW[1], (long)group, (long)dW[0]);
  const int64_t P = (dX[2] + 2 * pads[0] - dW[2]) / strides[0] + 1,
                Q = (dX[3] + 2 * pads[1] - dW[3]) / strides[1] + 1;
  if (P < 1 || Q < 1) FAIL("conv: empty output");
  float *tx, *tw, *tb = NULL, *ty;
  const float *x = widen(X, numel(dX, 4), dtype, &tx);
  const float *w = widen(W, numel(dW, 4), dtype, &tw);
  const float *b = B ? widen(B, dW[0], dtype, &tb) : NULL;
  const int64_t ny = dX[0] * dW[0] * P * Q;
  float *y = outbuf(Y, ny, dtype, &ty);
  conv_core(x, dX, w, dW, b, group, pads, strides, act, y);
  narrow(Y, ty, ny, dtype);
  free(tx); free(tw); free(tb);
  return Y;
}

void *dnnrtConv(dnnrtHandle_t h, const void *X, const int64_t *dX, const void *W,
                const int64_t *dW, void *ws, int64_t wsBytes, int64_t algo,
                int64_t group, const int64_t *pads, const int64_t *strides,
                void *Y, int32_t dtype) {
  (void)h; (void)ws; (void)wsBytes; (void)algo;
  return conv_entry(X, dX, W, dW, NULL, group, pads, strides, DNNRT_ACT_IDENTITY, Y, dtype);
}
void *dnnrtConvBiasActiv(dnnrtHandle_t h, const void *X, const int64_t *dX,
                         const void *W, const int64_t *dW, const void *B,
                         const int64_t *dB, void *ws, int64_t wsBytes,
                         int64_t algo, int64_t group, const int64_t *pads,
                         const int64_t *strides, int64_t act, void *Y,
                         int32_t dtype) {
  (void)ws; (void)wsBytes; (void)algo;
  if (numel(dB, 4) != dW[0]) FAIL("convBiasActiv: bias must hold K values");
  if (act == DNNRT_ACT_CLIPPED_RELU || act == DNNRT_ACT_LEAKY_RELU) {
    /* the reference has no such fused call: it runs conv+bias (identity) and
     * then CUDAClipFunc.cu / CUDALeakyReluFunc.cu on the stored tensor */
    if (!conv_entry(X, dX, W, dW, B, group, pads, strides, DNNRT_ACT_IDENTITY, Y, dtype)) return NULL;
    const int64_t P = (dX[2] + 2 * pads[0] - dW[2]) / strides[0] + 1,
                  Q = (dX[3] + 2 * pads[1] - dW[3]) / strides[1] + 1;
    const int64_t dY[4] = {dX[0], dW[0], P, Q};
    return act == DNNRT_ACT_CLIPPED_RELU ? dnnrtClip(h, Y, Y, dY, 0.f, h->act_coef, 4, dtype)
                                         : dnnrtLeakyRelu(h, Y, Y, dY, h->act_coef, 4, dtype);
  }
  if (act != DNNRT_ACT_RELU && act != DNNRT_ACT_IDENTITY)
    FAIL("convBiasActiv: activMode %ld", (long)act);
  return conv_entry(X, dX, W, dW, B, group, pads, strides, act, Y, dtype);
}
/* No reference counterpart: dnnrtConvBiasActiv on the defaults of a fresh
 * handle (the GPU library's variant differs only in where its scratch lives). */
void *dnnrtConvBiasActivNoAlloc(dnnrtStream_t stream, const void *X, const int64_t *dX,
                                const void *W, const int64_t *dW, const void *B,
                                const int64_t *dB, int64_t group, const int64_t *pads,
                                const int64_t *strides, int64_t act, void *Y, int32_t dtype) {
  (void)stream;
  struct dnnrtContext fresh = {DNNRT_NCHW, 0.f};
  return dnnrtConvBiasActiv(&fresh, X, dX, W, dW, B, dB, NULL, 0, 0, group, pads, strides, act, Y, dtype);
}
/* No reference wrapper of its own: the reference runs this as three calls,
 * conv+bias (CUDNNConvBiasReluFunc.cpp, identity), cudnnAddTensor
 * (CUDNNAddFunc.cpp) and cudnnActivationForward (CUDNNActiveFunc.cpp), each
 * storing its result in the tensor's type.  Restated as exactly that chain. */
void *dnnrtConvBiasAddActiv(dnnrtHandle_t h, const void *X, const int64_t *dX,
                            const void *W, const int64_t *dW, const void *B,
                            const int64_t *dB, const void *Z, void *ws,
                            int64_t wsBytes, int64_t algo, int64_t group,
                            const int64_t *pads, const int64_t *strides,
                            int64_t act, void *Y, int32_t dtype) {
  (void)ws; (void)wsBytes; (void)algo;
  if (act != DNNRT_ACT_RELU && act != DNNRT_ACT_IDENTITY && act != DNNRT_ACT_CLIPPED_RELU && act != DNNRT_ACT_LEAKY_RELU)
    FAIL("convBiasAddActiv: activMode %ld", (long)act);
  if (numel(dB, 4) != dW[0]) FAIL("convBiasAddActiv: bias must hold K values");
  if (!Z) FAIL("convBiasAddActiv: null residual tensor");
  const int64_t P = (dX[2] + 2 * pads[0] - dW[2]) / strides[0] + 1,
                Q = (dX[3] + 2 * pads[1] - dW[3]) / strides[1] + 1;
  const int64_t ny = dX[0] * dW[0] * P * Q;
  /* Z may be Y itself (cudnnConvolutionBiasActivationForward allows zData == yData;
   * the GPU library's in-place residual relies on it): the chain below stores the
   * convolution in Y first, so the residual is set aside. */
  void *z_copy = NULL;
  if (Z == Y && ny > 0) {
    const size_t bytes = (size_t)ny * (dtype == DNNRT_F16 ? 2 : 4);
    z_copy = malloc(bytes);
    if (!z_copy) FAIL("convBiasAddActiv: out of memory");
    memcpy(z_copy, Z, bytes);
    Z = z_copy;
  }
  if (!conv_entry(X, dX, W, dW, B, group, pads, strides, DNNRT_ACT_IDENTITY, Y, dtype)) {
    free(z_copy);
    return NULL;
  }
  float *ty, *tz, *to;
  const float *y = widen(Y, ny, dtype, &ty);
  const float *z = widen(Z, ny, dtype, &tz);
  float *o = outbuf(Y, ny, dtype, &to);
  /* rounding to the tensor's type commutes with ReLU, so one narrow() at the
   * end stands for the add's and the activation's stores */
  for (int64_t i = 0; i < ny; i++) o[i] = act_apply(y[i] + z[i], act, h->act_coef);
  narrow(Y, to, ny, dtype);
  free(ty); free(tz); free(z_copy);
  return Y;
}

/* ---- elementwise -------------------------------------------------------- */

/* CUDNNActiveFunc.cpp:8-91: cudnnActivationForward, alpha 1 beta 0. */
void *dnnrtActive(dnnrtHandle_t h, const void *X, const int64_t *dX, int32_t mode,
                  void *Y, int32_t dtype) {
  if (bad_dtype(dtype)) FAIL("active: bad dtype");
  if (mode != DNNRT_ACT_RELU && mode != DNNRT_ACT_SIGMOID && mode != DNNRT_ACT_TANH &&
      mode != DNNRT_ACT_CLIPPED_RELU && mode != DNNRT_ACT_LEAKY_RELU)
    FAIL("active: mode %d", mode);
  const int64_t n = numel(dX, 4);
  float *tx, *ty;
  const float *x = widen(X, n, dtype, &tx);
  float *y = outbuf(Y, n, dtype, &ty);
  for (int64_t i = 0; i < n; i++) y[i] = act_apply(x[i], mode, h->act_coef);
  narrow(Y, ty, n, dtype); free(tx);
  return Y;
}

/* CUDNNTensorOpFunc.cpp:8-149: cudnnOpTensor, C = op(1*A, coefB*B) + 0*C,
 * B broadcast where its dim is 1. */
void *dnnrtTensorOp(dnnrtHandle_t h, int64_t op, const void *A, const int64_t *dA,
                    int32_t rA, const void *B, const int64_t *dB, int32_t rB,
                    void *O, const int64_t *dO, int32_t rO, float coefB,
                    int32_t dtype) {
  (void)h;
  if (bad_dtype(dtype)) FAIL("tensorOp: bad dtype");
  if (op != DNNRT_OP_ADD && op != DNNRT_OP_MUL && op != DNNRT_OP_SQRT)
    FAIL("tensorOp: op %ld", (long)op);
  if (rA != rO || (op != DNNRT_OP_SQRT && rB != rA) || rA < 1 || rA > 8)
    FAIL("tensorOp: ranks %d %d %d", rA, rB, rO);
  for (int i = 0; i < rA; i++) {
    if (dA[i] != dO[i]) FAIL("tensorOp: dimA != dimO");
    if (op != DNNRT_OP_SQRT && dB[i] != dA[i] && dB[i] != 1)
      FAIL("tensorOp: dimB[%d]=%ld cannot broadcast to %ld", i, (long)dB[i], (long)dA[i]);
  }
  const int64_t n = numel(dA, rA);
  float *ta, *tb = NULL, *to;
  const float *a = widen(A, n, dtype, &ta);
  float *o = outbuf(O, n, dtype, &to);
  if (op == DNNRT_OP_SQRT) {
    for (int64_t i = 0; i < n; i++) o[i] = sqrtf(a[i]);
  } else {
    const float *b = widen(B, numel(dB, rB), dtype, &tb);
    int64_t sB[8], s = 1;
    for (int i = rA - 1; i >= 0; i--) { sB[i] = dB[i] == 1 ? 0 : s; s *= dB[i]; }
    for (int64_t i = 0; i < n; i++) {
      int64_t rem = i, ib = 0;
      for (int d = rA - 1; d >= 0; d--) { ib += (rem % dA[d]) * sB[d]; rem /= dA[d]; }
      const float bv = coefB * b[ib];
      o[i] = op == DNNRT_OP_ADD ? a[i] + bv : a[i] * bv;
    }
  }
  narrow(O, to, n, dtype); free(ta); free(tb);
  return O;
}

#define UNARY(NAME, EXPR)                                                      \
  void *NAME(dnnrtHandle_t h, const void *X, void *Y, const int64_t *d,        \
             int64_t rank, int32_t dtype) {                                    \
    (void)h;                                                                   \
    if (bad_dtype(dtype)) FAIL(#NAME ": bad dtype");                           \
    const int64_t n = numel(d, rank);                                          \
    float *tx, *ty;                                                            \
    const float *x = widen(X, n, dtype, &tx);                                  \
    float *y = outbuf(Y, n, dtype, &ty);                                       \
    for (int64_t i = 0; i < n; i++) { const float v = x[i]; y[i] = (EXPR); }   \
    narrow(Y, ty, n, dtype); free(tx);                                         \
    return Y;                                                                  \
  }
/* CUDAErfFunc.cu:4-27, CUDANegativeFunc.cu:4-28, CUDAReciprocalFunc.cu:4-28 */
UNARY(dnnrtErf, erff(v))
UNARY(dnnrtNegative, -v)
UNARY(dnnrtReciprocal, 1.0f / v)
/* GELU(erf), the chain the reference lowers to: Div(sqrt 2), Erf, Add 1,
 * Mul x, Mul 0.5 -- evaluated in double, rounded once. */
UNARY(dnnrtGelu, (float)(0.5 * (double)v * (1.0 + erf((double)v / sqrt(2.0)))))

/* CUDAClipFunc.cu:5-28: min(max(x, lo), hi). */
void *dnnrtClip(dnnrtHandle_t h, const void *X, void *Y, const int64_t *d, float lo,
                float hi, int64_t rank, int32_t dtype) {
  (void)h;
  if (bad_dtype(dtype)) FAIL("clip: bad dtype");
  const int64_t n = numel(d, rank);
  float *tx, *ty;
  const float *x = widen(X, n, dtype, &tx);
  float *y = outbuf(Y, n, dtype, &ty);
  for (int64_t i = 0; i < n; i++) {
    float v = x[i];
    v = v < lo ? lo : v;
    v = v > hi ? hi : v;
    y[i] = v;
  }
  narrow(Y, ty, n, dtype); free(tx);
  return Y;
}

/* CUDALeakyReluFunc.cu:4-15: x < 0 ? alpha * x : x. */
void *dnnrtLeakyRelu(dnnrtHandle_t h, const void *X, void *Y, const int64_t *d, float alpha,
                     int64_t rank, int32_t dtype) {
  (void)h;
  if (bad_dtype(dtype)) FAIL("leakyrelu: bad dtype");
  const int64_t n = numel(d, rank);
  float *tx, *ty;
  const float *x = widen(X, n, dtype, &tx);
  float *y = outbuf(Y, n, dtype, &ty);
  for (int64_t i = 0; i < n; i++) y[i] = x[i] < 0.f ? alpha * x[i] : x[i];
  narrow(Y, ty, n, dtype); free(tx);
  return Y;
}

/* CUDAPReluFunc.cu:4-15 applies slope[0] to the whole tensor; ONNX PRelu
 * broadcasts the slope tensor to X (unidirectional, right-aligned), which is
 * what is computed here: with a one-element slope the two agree. */
void *dnnrtPRelu(dnnrtHandle_t h, const void *X, void *Y, const int64_t *d, const void *S,
                 const int64_t *dS, int64_t rank, int32_t dtype) {
  (void)h;
  if (bad_dtype(dtype)) FAIL("prelu: bad dtype");
  if (rank < 1 || rank > 8) FAIL("prelu: rank");
  int64_t ss[8], acc = 1;
  for (int i = (int)rank - 1; i >= 0; i--) {
    if (dS[i] != d[i] && dS[i] != 1) FAIL("prelu: slope does not broadcast");
    ss[i] = dS[i] == 1 ? 0 : acc;
    acc *= dS[i];
  }
  const int64_t n = numel(d, rank), ns = numel(dS, rank);
  float *tx, *ts, *ty;
  const float *x = widen(X, n, dtype, &tx);
  const float *sl = widen(S, ns, dtype, &ts);
  float *y = outbuf(Y, n, dtype, &ty);
  for (int64_t i = 0; i < n; i++) {
    int64_t rem = i, is = 0;
    for (int k = (int)rank - 1; k >= 0; k--) { is += (rem % d[k]) * ss[k]; rem /= d[k]; }
    y[i] = x[i] < 0.f ? sl[is] * x[i] : x[i];
  }
  narrow(Y, ty, n, dtype); free(tx); free(ts);
  return Y;
}

/* CUDAPowFunc.cu:4-32: exponent from a 1-element tensor; exponent 2 is x*x. */
void *dnnrtPow(dnnrtHandle_t h, const void *X, const void *E, void *Y,
               const int64_t *d, int64_t rank, int32_t dtype) {
  (void)h;
  if (bad_dtype(dtype)) FAIL("pow: bad dtype");
  const int64_t n = numel(d, rank);
  float *tx, *te, *ty;
  const float *x = widen(X, n, dtype, &tx);
  const float *e = widen(E, 1, dtype, &te);
  float *y = outbuf(Y, n, dtype, &ty);
  if (e[0] == 2.0f) for (int64_t i = 0; i < n; i++) y[i] = x[i] * x[i];
  else for (int64_t i = 0; i < n; i++) y[i] = powf(x[i], e[0]);
  narrow(Y, ty, n, dtype); free(tx); free(te);
  return Y;
}

/* CUDACastI64toFloatFunc.cu:4-26. */
void *dnnrtCastI64toFloat(dnnrtHandle_t h, const int64_t *X, void *Y,
                          const int64_t *d, int64_t rank, int32_t dtype) {
  (void)h;
  if (bad_dtype(dtype)) FAIL("cast: bad dtype");
  const int64_t n = numel(d, rank);
  float *ty;
  float *y = outbuf(Y, n, dtype, &ty);
  for (int64_t i = 0; i < n; i++) y[i] = (float)X[i];
  narrow(Y, ty, n, dtype);
  return Y;
}

/* ---- reductions ---------------------------------------------------------
 * CUDNNReduceFunc.cpp:8-142: cudnnReduceTensor AVG over the dims where the
 * output dim is 1. */
void *dnnrtReduce(dnnrtHandle_t h, int32_t rank, const void *X, const int64_t *dX,
                  void *Y, const int64_t *dY, int32_t mode, int32_t dtype) {
  (void)h;
  if (bad_dtype(dtype)) FAIL("reduce: bad dtype");
  if (mode != DNNRT_REDUCE_AVG) FAIL("reduce: mode %d", mode);
  if (rank < 1 || rank > 8) FAIL("reduce: rank %d", rank);
  for (int i = 0; i < rank; i++)
    if (dY[i] != dX[i] && dY[i] != 1) FAIL("reduce: dimY[%d]", i);
  const int64_t nx = numel(dX, rank), ny = numel(dY, rank);
  if (nx == 0 || ny == 0) return Y;  /* nothing to average, nothing to write */
  float *tx, *ty;
  const float *x = widen(X, nx, dtype, &tx);
  float *y = outbuf(Y, ny, dtype, &ty);
  double *acc = (double *)calloc((size_t)ny, sizeof(double));
  int64_t sY[8], s = 1;
  for (int i = rank - 1; i >= 0; i--) { sY[i] = dY[i] == 1 ? 0 : s; s *= dY[i]; }
  for (int64_t i = 0; i < nx; i++) {
    int64_t rem = i, iy = 0;
    for (int d = rank - 1; d >= 0; d--) { iy += (rem % dX[d]) * sY[d]; rem /= dX[d]; }
    acc[iy] += (double)x[i];
  }
  const double cnt = (double)(nx / ny);
  for (int64_t i = 0; i < ny; i++) y[i] = (float)(acc[i] / cnt);
  free(acc);
  narrow(Y, ty, ny, dtype); free(tx);
  return Y;
}

/* CUDASoftmaxFunc.cu:7-128: exp(x - m) / sum exp(x - m) along `axis`.  The
 * reference subtracts the tensor-wide max; any per-row constant gives the
 * same quotient, the row max is used here. */
void *dnnrtSoftmax(dnnrtHandle_t h, const void *X, const int64_t *dX, void *Y,
                   const int64_t *dY, int64_t axis, int64_t rank, int32_t dtype) {
  (void)h; (void)dY;
  if (bad_dtype(dtype)) FAIL("softmax: bad dtype");
  if (axis < 0) axis += rank;
  if (axis < 0 || axis >= rank) FAIL("softmax: axis");
  int64_t outer = 1, inner = 1;
  const int64_t L = dX[axis];
  for (int64_t i = 0; i < axis; i++) outer *= dX[i];
  for (int64_t i = axis + 1; i < rank; i++) inner *= dX[i];
  const int64_t n = outer * L * inner;
  float *tx, *ty;
  const float *x = widen(X, n, dtype, &tx);
  float *y = outbuf(Y, n, dtype, &ty);
  for (int64_t o = 0; o < outer; o++)
    for (int64_t in = 0; in < inner; in++) {
      const float *xr = x + o * L * inner + in;
      float *yr = y + o * L * inner + in;
      float m = xr[0];
      for (int64_t l = 1; l < L; l++) m = xr[l * inner] > m ? xr[l * inner] : m;
      double sum = 0;
      for (int64_t l = 0; l < L; l++) sum += exp((double)xr[l * inner] - (double)m);
      for (int64_t l = 0; l < L; l++)
        yr[l * inner] = (float)(exp((double)xr[l * inner] - (double)m) / sum);
    }
  narrow(Y, ty, n, dtype); free(tx);
  return Y;
}

/* LayerNorm over the last dim, i.e. the chain the reference emits for it:
 * ReduceMean, Sub, Pow 2, ReduceMean, Add eps, Sqrt, Div, Mul gamma, Add beta. */
void *dnnrtLayerNorm(dnnrtHandle_t h, const void *X, const int64_t *dX, int64_t rank,
                     const void *G, const void *Bt, float eps, void *Y, int32_t dtype) {
  (void)h;
  if (bad_dtype(dtype)) FAIL("layernorm: bad dtype");
  const int64_t L = dX[rank - 1], rows = numel(dX, rank - 1), n = rows * L;
  float *tx, *tg, *tb, *ty;
  const float *x = widen(X, n, dtype, &tx);
  const float *g = widen(G, L, dtype, &tg);
  const float *b = widen(Bt, L, dtype, &tb);
  float *y = outbuf(Y, n, dtype, &ty);
  for (int64_t r = 0; r < rows; r++) {
    const float *xr = x + r * L;
    double mu = 0, var = 0;
    for (int64_t i = 0; i < L; i++) mu += xr[i];
    mu /= (double)L;
    for (int64_t i = 0; i < L; i++) { const double d = xr[i] - mu; var += d * d; }
    var /= (double)L;
    const double inv = 1.0 / sqrt(var + (double)eps);
    for (int64_t i = 0; i < L; i++)
      y[r * L + i] = (float)((xr[i] - mu) * inv * (double)g[i] + (double)b[i]);
  }
  narrow(Y, ty, n, dtype); free(tx); free(tg); free(tb);
  return Y;
}

/* ---- pooling -------------------------------------------------------------
 * CUDNNMaxPoolFunc.cpp:8-78 / CUDNNAveragePoolFunc.cpp:8-78:
 * cudnnPoolingForward, window kernel[0] x kernel[1], vertical pad pads[0],
 * horizontal pad pads[1] (the lowering hands over ONNX's 4 pads; begin pads
 * are used for both sides), strides.  Max ignores padding; average divides
 * by the full window (CUDNN_POOLING_AVERAGE_COUNT_INCLUDE_PADDING, :44).
 * The reference's beta = 1 accumulate into a zeroed Y is a plain overwrite. */
static void *pool_entry(const void *X, const int64_t *dX, void *Y, const int64_t *dY,
                        const int64_t *kr, const int64_t *pads, const int64_t *st,
                        int is_max, int32_t dtype) {
  if (bad_dtype(dtype)) FAIL("pool: bad dtype");
  const int64_t N = dX[0], C = dX[1], H = dX[2], W = dX[3], P = dY[2], Q = dY[3];
  const int64_t R = kr[0], S = kr[1], ph = pads[0], pw = pads[1];
  if (dY[0] != N || dY[1] != C) FAIL("pool: dimY");
  if ((P - 1) * st[0] - ph >= H || (Q - 1) * st[1] - pw >= W) FAIL("pool: window outside");
  const int64_t nx = N * C * H * W, ny = N * C * P * Q;
  float *tx, *ty;
  const float *x = widen(X, nx, dtype, &tx);
  float *y = outbuf(Y, ny, dtype, &ty);
#pragma omp parallel for
  for (int64_t nc = 0; nc < N * C; nc++)
    for (int64_t p = 0; p < P; p++)
      for (int64_t q = 0; q < Q; q++) {
        float m = -INFINITY; double sum = 0; int any_nan = 0;
        for (int64_t r = 0; r < R; r++)
          for (int64_t s = 0; s < S; s++) {
            const int64_t ih = p * st[0] - ph + r, iw = q * st[1] - pw + s;
            if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
            const float v = x[(nc * H + ih) * W + iw];
            if (v != v) any_nan = 1;
            m = v > m ? v : m; sum += v;
          }
        y[(nc * P + p) * Q + q] =
            is_max ? (any_nan ? NAN : m) : (float)(sum / (double)(R * S));
      }
  narrow(Y, ty, ny, dtype); free(tx);
  return Y;
}
void *dnnrtMaxPool(dnnrtHandle_t h, const void *X, const int64_t *dX, void *Y,
                   const int64_t *dY, const int64_t *k, const int64_t *p,
                   const int64_t *s, int32_t dtype) {
  (void)h; return pool_entry(X, dX, Y, dY, k, p, s, 1, dtype);
}
void *dnnrtAveragePool(dnnrtHandle_t h, const void *X, const int64_t *dX, void *Y,
                       const int64_t *dY, const int64_t *k, const int64_t *p,
                       const int64_t *s, int32_t dtype) {
  (void)h; return pool_entry(X, dX, Y, dY, k, p, s, 0, dtype);
}

/* No reference wrapper of its own: the reference runs this as two calls,
 * CUDNNConvBiasReluFunc.cpp:8-140 and CUDNNMaxPoolFunc.cpp:8-78, the first
 * storing its result in the tensor's type.  Restated as exactly that chain,
 * for any shape the two calls take (the GPU library's kernel takes one). */
void *dnnrtConvBiasActivMaxPool(dnnrtHandle_t h, const void *X, const int64_t *dX,
                                const void *W, const int64_t *dW, const void *B,
                                const int64_t *dB, int64_t group, const int64_t *pads,
                                const int64_t *strides, int64_t act, const int64_t *pk,
                                const int64_t *pp, const int64_t *ps, void *Y,
                                const int64_t *dY, int32_t dtype) {
  if (bad_dtype(dtype)) FAIL("convBiasActivMaxPool: bad dtype");
  const int64_t P = (dX[2] + 2 * pads[0] - dW[2]) / strides[0] + 1,
                Q = (dX[3] + 2 * pads[1] - dW[3]) / strides[1] + 1;
  if (P < 1 || Q < 1) FAIL("convBiasActivMaxPool: empty convolution output");
  const int64_t dC[4] = {dX[0], dW[0], P, Q};
  const int64_t PP = (P + 2 * pp[0] - pk[0]) / ps[0] + 1, QQ = (Q + 2 * pp[1] - pk[1]) / ps[1] + 1;
  if (dY[0] != dC[0] || dY[1] != dC[1] || dY[2] != PP || dY[3] != QQ) FAIL("convBiasActivMaxPool: dimY");
  void *mid = malloc((size_t)(numel(dC, 4) * (dtype == DNNRT_F16 ? 2 : 4)));
  if (!mid) FAIL("convBiasActivMaxPool: out of memory");
  void *r = dnnrtConvBiasActiv(h, X, dX, W, dW, B, dB, NULL, 0, 0, group, pads, strides, act, mid, dtype);
  if (r) r = dnnrtMaxPool(h, mid, dC, Y, dY, pk, pp, ps, dtype);
  free(mid);
  return r ? Y : NULL;
}

/* No reference wrapper of its own: the reference runs this as dnnrtConvBiasActiv
 * (identity) on the second convolution and then the chain of
 * dnnrtConvBiasAddActiv with that result as Z, every call storing its result
 * in the tensor's type.  Restated as exactly that, for any shapes the two
 * calls take. */
void *dnnrtConvBiasAddConvBiasActiv(dnnrtHandle_t h, const void *X, const int64_t *dX, const void *W,
                                    const int64_t *dW, const void *B, const int64_t *pads,
                                    const int64_t *strides, const void *X2, const int64_t *dX2,
                                    const void *W2, const int64_t *dW2, const void *B2,
                                    const int64_t *pads2, const int64_t *strides2, int64_t act,
                                    int64_t algo, int64_t algo2, void *Y, int32_t dtype) {
  (void)algo; (void)algo2;
  if (bad_dtype(dtype)) FAIL("convBiasAddConvBiasActiv: bad dtype");
  const int64_t P = (dX2[2] + 2 * pads2[0] - dW2[2]) / strides2[0] + 1,
                Q = (dX2[3] + 2 * pads2[1] - dW2[3]) / strides2[1] + 1;
  if (P < 1 || Q < 1) FAIL("convBiasAddConvBiasActiv: empty second convolution");
  const int64_t dZ[4] = {dX2[0], dW2[0], P, Q};
  const int64_t dB[4] = {1, dW[0], 1, 1}, dB2[4] = {1, dW2[0], 1, 1};
  const size_t es = dtype == DNNRT_F16 ? 2 : 4;
  void *z = malloc((size_t)numel(dZ, 4) * es);
  void *zero = calloc((size_t)(dW[0] > dW2[0] ? dW[0] : dW2[0]), es);
  if (!z || !zero) { free(z); free(zero); FAIL("convBiasAddConvBiasActiv: out of memory"); }
  void *r = dnnrtConvBiasActiv(h, X2, dX2, W2, dW2, B2 ? B2 : zero, dB2, NULL, 0, 0, 1, pads2, strides2, DNNRT_ACT_IDENTITY, z, dtype);
  if (r) r = dnnrtConvBiasAddActiv(h, X, dX, W, dW, B ? B : zero, dB, z, NULL, 0, 0, 1, pads, strides, act, Y, dtype);
  free(z); free(zero);
  return r ? Y : NULL;
}

/* ---- matrix products ----------------------------------------------------- */

/* C[M,N] = alpha * sum_k A(m,k) B(k,n) (+ beta * Cin), element strides given */
static void gemm_core(const float *A, int64_t sam, int64_t sak, const float *B,
                      int64_t sbk, int64_t sbn, const float *Cin, float *C,
                      int64_t M, int64_t N, int64_t K, float alpha, float beta) {
#pragma omp parallel for
  for (int64_t m = 0; m < M; m++)
    for (int64_t n = 0; n < N; n++) {
      double acc = 0;
      for (int64_t k = 0; k < K; k++)
        acc += (double)A[m * sam + k * sak] * (double)B[k * sbk + n * sbn];
      double v = (double)alpha * acc;
      if (beta != 0.0f) v += (double)beta * (double)Cin[m * N + n];
      C[m * N + n] = (float)v;
    }
}

/* CUBLASMatmul2dFunc.cu:9-153: cublasLtMatmul, fp32 compute,
 * Out = alpha op(A) op(B) + beta C with row-major operands. */
void *dnnrtMatmul2d(dnnrtHandle_t h, int64_t rank, const void *A, const int64_t *dA,
                    const void *B, const int64_t *dB, const void *C,
                    const int64_t *dC, void *Out, const int64_t *dO, float alpha,
                    float beta, int64_t transA, int64_t transB, int32_t dtype) {
  (void)h; (void)rank;
  if (bad_dtype(dtype)) FAIL("matmul2d: bad dtype");
  const int64_t M = transA ? dA[1] : dA[0], K = transA ? dA[0] : dA[1];
  const int64_t Kb = transB ? dB[1] : dB[0], N = transB ? dB[0] : dB[1];
  if (K != Kb || dO[0] != M || dO[1] != N) FAIL("matmul2d: shapes");
  if (beta != 0.0f && !C) FAIL("matmul2d: beta != 0 needs C");
  float *ta, *tb, *tc = NULL, *to;
  const float *a = widen(A, M * K, dtype, &ta);
  const float *b = widen(B, K * N, dtype, &tb);
  /* C: [M,N] (CUBLASMatmul2dFunc.cu:32 sizes it by dimOutput) or one row [1,N] for every row of the product */
  const int c_row = beta != 0.0f && dC && dC[0] == 1 && dC[1] == N; /* also when M == 1: the chain's two roundings */
  if (beta != 0.0f && dC && !c_row && (dC[0] != M || dC[1] != N)) FAIL("matmul2d: C dims");
  const float *c = (beta != 0.0f) ? widen(C, c_row ? N : M * N, dtype, &tc) : NULL;
  float *o = outbuf(Out, M * N, dtype, &to);
  float *cc = NULL;
  if (c) { /* C may alias Out */
    cc = (float *)malloc(sizeof(float) * (size_t)(c_row ? N : M * N));
    memcpy(cc, c, sizeof(float) * (size_t)(c_row ? N : M * N));
  }
  gemm_core(a, transA ? 1 : K, transA ? M : 1, b, transB ? 1 : N, transB ? K : 1,
            c_row ? NULL : cc, o, M, N, K, alpha, c_row ? 0.0f : beta);
  if (c_row) /* the row case is the reference's Gemm chain (Ops/cublas/Gemm.cpp:60-81): product, then the broadcast add */
    for (int64_t m = 0; m < M; m++)
      for (int64_t n = 0; n < N; n++) {
        const float t = beta * cc[n];
        /* fp16: the product is stored (rounded) before the add reads it */
        const float prod = dtype == DNNRT_F16 ? h2f(f2h(o[m * N + n])) : o[m * N + n];
        o[m * N + n] = prod + t;
      }
  free(cc);
  narrow(Out, to, M * N, dtype); free(ta); free(tb); free(tc);
  return Out;
}

/* CUDAMatmulNdFunc.cu:14-173: numpy.matmul, ranks 2..4; batch dims of the
 * lower-rank (or size-1) operand are broadcast. */
void *dnnrtMatmulNd(dnnrtHandle_t h, const void *A, const int64_t *dA, int32_t rA,
                    const void *B, const int64_t *dB, int32_t rB, void *Y,
                    const int64_t *dY, int32_t rY, int32_t dtype) {
  (void)h;
  if (bad_dtype(dtype)) FAIL("matmulNd: bad dtype");
  if (rA < 2 || rB < 2 || rY < 2 || rA > 4 || rB > 4 || rY > 4 ||
      rY != (rA > rB ? rA : rB))
    FAIL("matmulNd: ranks %d %d %d", rA, rB, rY);
  const int64_t M = dA[rA - 2], K = dA[rA - 1], N = dB[rB - 1];
  if (dB[rB - 2] != K || dY[rY - 2] != M || dY[rY - 1] != N) FAIL("matmulNd: shapes");
  const int nb = rY - 2;
  int64_t bY[2] = {1, 1}, bA[2] = {1, 1}, bB[2] = {1, 1};
  for (int i = 0; i < nb; i++) {
    bY[2 - nb + i] = dY[i];
    const int ia = i - (rY - rA), ib = i - (rY - rB);
    if (ia >= 0) bA[2 - nb + i] = dA[ia];
    if (ib >= 0) bB[2 - nb + i] = dB[ib];
  }
  for (int i = 0; i < 2; i++)
    if ((bA[i] != bY[i] && bA[i] != 1) || (bB[i] != bY[i] && bB[i] != 1))
      FAIL("matmulNd: batch dims do not broadcast");
  const int64_t na = bA[0] * bA[1] * M * K, nbB = bB[0] * bB[1] * K * N,
                ny = bY[0] * bY[1] * M * N;
  float *ta, *tb, *ty;
  const float *a = widen(A, na, dtype, &ta);
  const float *b = widen(B, nbB, dtype, &tb);
  float *y = outbuf(Y, ny, dtype, &ty);
  for (int64_t i0 = 0; i0 < bY[0]; i0++)
    for (int64_t i1 = 0; i1 < bY[1]; i1++) {
      const int64_t a0 = bA[0] == 1 ? 0 : i0, a1 = bA[1] == 1 ? 0 : i1;
      const int64_t b0 = bB[0] == 1 ? 0 : i0, b1 = bB[1] == 1 ? 0 : i1;
      gemm_core(a + (a0 * bA[1] + a1) * M * K, K, 1, b + (b0 * bB[1] + b1) * K * N,
                N, 1, NULL, y + (i0 * bY[1] + i1) * M * N, M, N, K, 1.0f, 0.0f);
    }
  narrow(Y, ty, ny, dtype); free(ta); free(tb);
  return Y;
}
/* No reference wrapper of its own: CUDAMatmulNdFunc.cu, then the broadcast
 * add of CUDNNTensorOpFunc.cpp on the stored product, then the residual add
 * and Gelu (CUDAErfFunc.cu and friends) -- restated as that chain. */
void *dnnrtMatmulNdBias(dnnrtHandle_t h, const void *A, const int64_t *dA, int32_t rA,
                        const void *B, const int64_t *dB, int32_t rB, const void *bias,
                        const void *Z, int32_t gelu, void *Y, const int64_t *dY, int32_t rY,
                        int32_t dtype) {
  if (!bias) FAIL("matmulNdBias: null bias");
  if (!dnnrtMatmulNd(h, A, dA, rA, B, dB, rB, Y, dY, rY, dtype)) return NULL;
  int64_t db[8];
  for (int i = 0; i < rY; i++) db[i] = 1;
  db[rY - 1] = dY[rY - 1];
  if (!dnnrtTensorOp(h, DNNRT_OP_ADD, Y, dY, rY, bias, db, rY, Y, dY, rY, 1.0f, dtype)) return NULL;
  if (Z && !dnnrtTensorOp(h, DNNRT_OP_ADD, Y, dY, rY, Z, dY, rY, Y, dY, rY, 1.0f, dtype)) return NULL;
  if (gelu && !dnnrtGelu(h, Y, Y, dY, rY, dtype)) return NULL;
  return Y;
}
/* No reference wrapper of its own: per head, the reference's chain of
 * CUDAMatmulNdFunc.cu (scores), the scaling multiply, CUDASoftmaxFunc.cu (over
 * the keys, maximum subtracted) and CUDAMatmulNdFunc.cu again; the Reshape /
 * Transpose calls around them only move data.  Each stage is stored in fp32
 * as the chain would store it. */
void *dnnrtAttention(dnnrtHandle_t h, const void *Q, const void *K, const void *V, void *Y,
                     int64_t B, int64_t Sq, int64_t Sk, int64_t H, int64_t D, int64_t ldIn, float scale,
                     int32_t dtype) {
  (void)h;
  if (dtype != DNNRT_F32 && dtype != DNNRT_F16) FAIL("attention: fp32 and fp16 only");
  if (B < 0 || Sq < 0) FAIL("attention: bad dims");
  if (B == 0 || Sq == 0) return Y;  /* no queries */
  if (Sk <= 0 || H <= 0 || D <= 0) FAIL("attention: bad dims");
  const int64_t ldy = H * D, ld = ldIn ? ldIn : ldy;
  if (ld < ldy) FAIL("attention: ldIn");
  /* fp16 tensors: widened here, one rounding of the result at the end (packed
   * operands are three views of one buffer: each is widened over its own rows) */
  float *tq, *tk, *tv, *to;
  const int64_t nq = (B * Sq - 1) * ld + ldy, nk = (B * Sk - 1) * ld + ldy;
  const float *q = widen(Q, nq, dtype, &tq), *k = widen(K, nk, dtype, &tk), *v = widen(V, nk, dtype, &tv);
  float *y = outbuf(Y, B * Sq * ldy, dtype, &to);
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t b = 0; b < B; b++)
    for (int64_t hd = 0; hd < H; hd++) {
      float *p = (float *)malloc((size_t)Sk * sizeof(float));
      for (int64_t i = 0; i < Sq; i++) {
        const float *qi = q + (b * Sq + i) * ld + hd * D;
        float mx = -INFINITY;
        for (int64_t j = 0; j < Sk; j++) {
          const float *kj = k + (b * Sk + j) * ld + hd * D;
          double acc = 0.0;
          for (int64_t d = 0; d < D; d++) acc += (double)qi[d] * (double)kj[d];
          p[j] = (float)acc * scale;
          mx = p[j] > mx ? p[j] : mx;
        }
        double sum = 0.0;
        for (int64_t j = 0; j < Sk; j++) { p[j] = expf(p[j] - mx); sum += p[j]; }
        for (int64_t j = 0; j < Sk; j++) p[j] = (float)(p[j] / sum);
        for (int64_t d = 0; d < D; d++) {
          double acc = 0.0;
          for (int64_t j = 0; j < Sk; j++) acc += (double)p[j] * (double)v[(b * Sk + j) * ld + hd * D + d];
          y[(b * Sq + i) * ldy + hd * D + d] = (float)acc;
        }
      }
      free(p);
    }
  narrow(Y, to, B * Sq * ldy, dtype);
  free(tq); free(tk); free(tv);
  return Y;
}

/* ---- data movement -------------------------------------------------------- */

static int64_t esize(int32_t dtype) {
  return dtype == DNNRT_F32 ? 4 : dtype == DNNRT_F16 ? 2 : dtype == DNNRT_I64 ? 8 : 0;
}
/* CUDAFlattenFunc.cpp:32 / CUDAReshapeFunc.cpp:30: device-to-device copy. */
void *dnnrtFlatten(dnnrtHandle_t h, const void *X, const int64_t *dX, void *Y,
                   const int64_t *dY, int32_t axis, int64_t rank, int32_t dtype) {
  (void)h; (void)dY; (void)axis;
  if (!esize(dtype)) FAIL("flatten: bad dtype");
  memmove(Y, X, (size_t)(numel(dX, rank) * esize(dtype)));
  return Y;
}
void *dnnrtReshape(dnnrtHandle_t h, const void *X, const int64_t *dX, int64_t rank,
                   void *Y, int32_t dtype) {
  (void)h;
  if (!esize(dtype)) FAIL("reshape: bad dtype");
  memmove(Y, X, (size_t)(numel(dX, rank) * esize(dtype)));
  return Y;
}
/* CUDASqueezeFloatFunc.cpp:25-31 / CUDAUnsqueezeFloatFunc.cpp: device-to-device copy. */
static int same_but_ones(const int64_t *dX, int64_t rX, const int64_t *dY, int64_t rY) {
  int64_t i = 0, j = 0;
  for (;;) {
    while (i < rX && dX[i] == 1) i++;
    while (j < rY && dY[j] == 1) j++;
    if (i == rX || j == rY) return i == rX && j == rY;
    if (dX[i++] != dY[j++]) return 0;
  }
}
void *dnnrtSqueeze(dnnrtHandle_t h, const void *X, const int64_t *dX, int64_t rX, void *Y,
                   const int64_t *dY, int64_t rY, int32_t dtype) {
  (void)h;
  if (!esize(dtype)) FAIL("squeeze: bad dtype");
  if (!same_but_ones(dX, rX, dY, rY)) FAIL("squeeze: dims differ beyond size-1 axes");
  memmove(Y, X, (size_t)(numel(dX, rX) * esize(dtype)));
  return Y;
}
void *dnnrtUnsqueeze(dnnrtHandle_t h, const void *X, const int64_t *dX, int64_t rX, void *Y,
                     const int64_t *dY, int64_t rY, int32_t dtype) {
  (void)h;
  if (!esize(dtype)) FAIL("unsqueeze: bad dtype");
  if (!same_but_ones(dX, rX, dY, rY)) FAIL("unsqueeze: dims differ beyond size-1 axes");
  memmove(Y, X, (size_t)(numel(dX, rX) * esize(dtype)));
  return Y;
}
/* CUDAExpandInt64Func.cu:10-15 copies prod(dimX) elements, which is the whole
 * answer only when dimY == dimX.  Restated as the ONNX operator the lowering
 * stands for (Ops/cuda/Expand.cpp:30-47: output sized by the broadcast shape):
 * per output element, the multi-index with every broadcast coordinate set to
 * 0 addresses the input.  With dimY == dimX this is the reference's copy. */
void *dnnrtExpand(dnnrtHandle_t h, const void *X, const int64_t *dX, int64_t rX, void *Y,
                  const int64_t *dY, int64_t rY, int32_t dtype) {
  (void)h;
  const int64_t es = esize(dtype);
  if (!es) FAIL("expand: bad dtype");
  if (rY < 1 || rY > 8 || rX < 0 || rX > rY) FAIL("expand: ranks");
  int64_t in_dim[8];
  for (int64_t d = 0; d < rY; d++) {
    const int64_t dx = d - (rY - rX);
    in_dim[d] = dx >= 0 ? dX[dx] : 1;
    if (in_dim[d] != dY[d] && in_dim[d] != 1) FAIL("expand: dims cannot be broadcast");
  }
  const int64_t total = numel(dY, rY);
  for (int64_t i = 0; i < total; i++) {
    int64_t idx[8], rest = i, src = 0;
    for (int64_t d = rY - 1; d >= 0; d--) { idx[d] = rest % dY[d]; rest /= dY[d]; }
    for (int64_t d = 0; d < rY; d++) src = src * in_dim[d] + (in_dim[d] == 1 ? 0 : idx[d]);
    memcpy((char *)Y + i * es, (const char *)X + src * es, (size_t)es);
  }
  return Y;
}
/* CUDANonZeroFloatFunc.cu:4-17 / CUDANonZeroInt64Func.cu: one sequential walk;
 * the index of every element != 0 goes to the next output slot, converted to
 * the element type.  Slots past prod(dimY) are not written (the reference
 * does not check). */
void *dnnrtNonZero(dnnrtHandle_t h, const void *X, const int64_t *dX, int64_t rX, void *Y,
                   const int64_t *dY, int64_t rY, int32_t dtype) {
  (void)h;
  if (!esize(dtype)) FAIL("nonzero: bad dtype");
  const int64_t n = numel(dX, rX), cap = numel(dY, rY);
  int64_t cur = 0;
  for (int64_t j = 0; j < n; j++) {
    int hit;
    if (dtype == DNNRT_F32) hit = ((const float *)X)[j] != 0.f;
    else if (dtype == DNNRT_F16) hit = h2f(((const uint16_t *)X)[j]) != 0.f;
    else hit = ((const int64_t *)X)[j] != 0;
    if (!hit) continue;
    if (cur < cap) {
      if (dtype == DNNRT_F32) ((float *)Y)[cur] = (float)j;
      else if (dtype == DNNRT_F16) ((uint16_t *)Y)[cur] = f2h((float)j);
      else ((int64_t *)Y)[cur] = j;
    }
    cur++;
  }
  return Y;
}
/* CUDAConcatFloatFunc.cu:7-62, per output element: split the flat index into
 * a multi-index, find the input whose span along the axis holds it, rebase
 * that coordinate and gather from that input. */
void *dnnrtConcat(dnnrtHandle_t h, const void *const *X, const int64_t *const *dX, void *Y,
                  const int64_t *dY, int64_t axis, int64_t n_in, int32_t rank, int32_t dtype) {
  (void)h;
  const int64_t es = esize(dtype);
  if (!es) FAIL("concat: bad dtype");
  if (rank < 1 || rank > 8 || n_in < 1 || n_in > 16) FAIL("concat: rank or input count");
  if (axis < 0) axis += rank;
  if (axis < 0 || axis >= rank) FAIL("concat: axis");
  int64_t acc[17];
  acc[0] = 0;
  for (int64_t k = 0; k < n_in; k++) {
    for (int i = 0; i < rank; i++)
      if (i != axis && dX[k][i] != dY[i]) FAIL("concat: input dims");
    acc[k + 1] = acc[k] + dX[k][axis];
  }
  if (acc[n_in] != dY[axis]) FAIL("concat: axis dims do not add up");
  const int64_t n = numel(dY, rank);
  for (int64_t i = 0; i < n; i++) {
    int64_t idx[8], rem = i;
    for (int k = rank - 1; k >= 0; k--) { idx[k] = rem % dY[k]; rem /= dY[k]; }
    int64_t src = 0;
    while (!(idx[axis] >= acc[src] && idx[axis] < acc[src + 1])) src++;
    idx[axis] -= acc[src];
    int64_t off = 0;
    for (int k = 0; k < rank; k++) off = off * dX[src][k] + idx[k];
    memcpy((char *)Y + i * es, (const char *)X[src] + off * es, (size_t)es);
  }
  return Y;
}
/* CUDATranspose4DFloatFunc.cu: Y[i_perm] = X[i]; dimY[j] = dimX[perm[j]]. */
void *dnnrtTranspose(dnnrtHandle_t h, const void *X, const int64_t *dX, void *Y,
                     const int64_t *dY, const int64_t *perm, int64_t rank,
                     int32_t dtype) {
  (void)h;
  const int64_t es = esize(dtype);
  if (!es) FAIL("transpose: bad dtype");
  if (rank < 1 || rank > 6) FAIL("transpose: rank");
  int64_t sX[6], s = 1;
  for (int i = (int)rank - 1; i >= 0; i--) { sX[i] = s; s *= dX[i]; }
  for (int i = 0; i < rank; i++)
    if (perm[i] < 0 || perm[i] >= rank || dY[i] != dX[perm[i]]) FAIL("transpose: perm/dimY");
  const int64_t n = numel(dX, rank);
  for (int64_t i = 0; i < n; i++) {
    int64_t rem = i, ix = 0;
    for (int d = (int)rank - 1; d >= 0; d--) { ix += (rem % dY[d]) * sX[perm[d]]; rem /= dY[d]; }
    memcpy((char *)Y + i * es, (const char *)X + ix * es, (size_t)es);
  }
  return Y;
}
/* CUDAGatherFloatFunc.cu:7-82: numpy.take(X, indices, axis). */
void *dnnrtGather(dnnrtHandle_t h, const void *X, const int64_t *dX, int64_t rX,
                  void *Y, const int64_t *dY, int64_t rY, const int64_t *idx,
                  const int64_t *dI, int64_t rI, int64_t axis, int32_t dtype) {
  (void)h; (void)dY; (void)rY;
  const int64_t es = esize(dtype);
  if (!es) FAIL("gather: bad dtype");
  if (axis < 0) axis += rX;
  if (axis < 0 || axis >= rX) FAIL("gather: axis");
  int64_t outer = 1, inner = 1;
  const int64_t ni = numel(dI, rI), L = dX[axis];
  for (int64_t i = 0; i < axis; i++) outer *= dX[i];
  for (int64_t i = axis + 1; i < rX; i++) inner *= dX[i];
  for (int64_t j = 0; j < ni; j++) {
    int64_t t = idx[j];
    if (t < 0) t += L;
    if (t < 0 || t >= L) FAIL("gather: index %ld out of range", (long)idx[j]);
  }
  for (int64_t o = 0; o < outer; o++)
    for (int64_t j = 0; j < ni; j++) {
      int64_t t = idx[j] < 0 ? idx[j] + L : idx[j];
      memcpy((char *)Y + ((o * ni + j) * inner) * es,
             (const char *)X + ((o * L + t) * inner) * es, (size_t)(inner * es));
    }
  return Y;
}
