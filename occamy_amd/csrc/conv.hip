// Convolution entry points: dnnrtConv / dnnrtConvBiasActiv
// (reference: src/Tools/dnn-wrapper/cudnn/CUDNNConvFunc.cpp:9-105 and
//  cudnn/fusedOp/CUDNNConvBiasReluFunc.cpp:8-140).
//
// Dispatch: depthwise (one input channel per group) goes to a memory-bound
// direct kernel; everything else is implicit GEMM on MFMA (igemm_f32.hip for
// fp32 NCHW, conv_f16.hip for fp16).
#include "common.h"
#include "igemm_f32.h"
#include "conv_f16.h"
#include "conv_f32_stem.h"

#include <string.h>

#include <mutex>

namespace dnnrt {

// ---- depthwise, fp32, NCHW ------------------------------------------------
// One thread per output element, q fastest so that a wavefront reads
// contiguous input rows.  The R*S filter taps of a channel are wave-uniform
// most of the time and come from the scalar/L1 path.
template <int R, int S>
__global__ __launch_bounds__(256) void dwconv_f32_nchw_kernel(
    const float *__restrict__ X, const float *__restrict__ Wt, const float *__restrict__ bias,
    const float *__restrict__ Zr, float *__restrict__ Y, int C, int H, int W, int K, int Kg, int P, int Q, int ph, int pw,
    int sh, int sw, int rr, int ss, int act, float act_coef, int64_t total, int w_k_stride, int w_tap_stride) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int q = (int)(i % Q);
  int64_t t = i / Q;
  const int p = (int)(t % P);
  t /= P;
  const int k = (int)(t % K);
  const int n = (int)(t / K);
  const int c = k / Kg;
  const int Rr = R ? R : rr, Ss = S ? S : ss;
  const float *x = X + ((int64_t)n * C + c) * H * W;
  const float *w = Wt + (int64_t)k * w_k_stride;  // tap (r, s) at w[(r * S + s) * w_tap_stride]
  const int ih0 = p * sh - ph, iw0 = q * sw - pw;
  float acc = 0.f;
#pragma unroll 3
  for (int r = 0; r < Rr; r++) {
    const int ih = ih0 + r;
    if ((unsigned)ih >= (unsigned)H) continue;
#pragma unroll 3
    for (int s = 0; s < Ss; s++) {
      const int iw = iw0 + s;
      if ((unsigned)iw < (unsigned)W) acc = fmaf(x[(int64_t)ih * W + iw], w[(r * Ss + s) * w_tap_stride], acc);
    }
  }
  if (bias) acc += bias[k];
  if (Zr) acc += Zr[i];
  acc = apply_act(acc, act, act_coef);
  Y[i] = acc;
}

// The 3x3 case on outputs of fewer than 2^31 elements (every depthwise layer of a MobileNetV2).  At batch 1 such a
// layer is one short wave of threads and what it costs is its chain of dependent steps: here the nine input and
// nine filter values are requested together, from clamped addresses (a load under a divergent branch is waited
// for before the next one is issued: nine memory round trips one after the other), a tap in the padding has its
// value replaced by zero, and the index is taken apart with multiply-high divisions instead of 64-bit ones.
// Taps are summed in the order of the kernel above.
__global__ __launch_bounds__(256) void dwconv3x3_f32_nchw_kernel(
    const float *__restrict__ X, const float *__restrict__ Wt, const float *__restrict__ bias, const float *Zr, float *Y, int C,
    int H, int W, int K, int Kg, int P, int Q, int ph, int pw, int sh, int sw, int act, float act_coef, int total, int w_k_stride,
    int w_tap_stride, unsigned magic_q, unsigned magic_p, unsigned magic_k, unsigned magic_kg) {
  const int i = (int)(blockIdx.x * 256 + threadIdx.x);
  if (i >= total) return;
  int t = div_magic(i, Q, magic_q);
  const int q = i - t * Q;
  const int t2 = div_magic(t, P, magic_p), p = t - t2 * P;
  const int n = div_magic(t2, K, magic_k), k = t2 - n * K;
  const int c = div_magic(k, Kg, magic_kg);
  const float *__restrict__ x = X + ((int64_t)n * C + c) * H * W;
  const float *__restrict__ w = Wt + (int64_t)k * w_k_stride;
  const int ih0 = p * sh - ph, iw0 = q * sw - pw;
  float xv[9], wv[9];
#pragma unroll
  for (int r = 0; r < 3; r++)
#pragma unroll
    for (int s = 0; s < 3; s++) {
      const int ih = ih0 + r, iw = iw0 + s;
      const bool ok = (unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W;
      const float v = x[min(max(ih, 0), H - 1) * W + min(max(iw, 0), W - 1)];
      xv[3 * r + s] = ok ? v : 0.f;
      wv[3 * r + s] = w[(3 * r + s) * w_tap_stride];
    }
  const float b = bias ? bias[k] : 0.f, z = Zr ? Zr[i] : 0.f;
  float acc = 0.f;
#pragma unroll
  for (int j = 0; j < 9; j++) acc = fmaf(xv[j], wv[j], acc);
  if (bias) acc += b;
  if (Zr) acc += z;
  Y[i] = apply_act(acc, act, act_coef);
}

struct ConvShape {
  int N, C, H, W, K, Cg, R, S, P, Q, ph, pw, sh, sw, group;
};

static bool parse_conv(const char *who, const int64_t *dX, const int64_t *dW, int64_t group,
                       const int64_t *pads, const int64_t *strides, ConvShape &s) {
  if (!dX || !dW || !pads || !strides) { set_error("%s: null dims", who); return false; }
  for (int i = 0; i < 4; i++)
    if (dX[i] <= 0 || dW[i] <= 0 || dX[i] > INT32_MAX || dW[i] > INT32_MAX) {
      set_error("%s: dims must be positive 32-bit values", who);
      return false;
    }
  if (group < 1 || dW[0] % group || dX[1] != dW[1] * group) {
    set_error("%s: C=%ld, W holds C/group=%ld, group=%ld, K=%ld do not agree", who, (long)dX[1],
              (long)dW[1], (long)group, (long)dW[0]);
    return false;
  }
  if (pads[0] < 0 || pads[1] < 0 || strides[0] < 1 || strides[1] < 1) {
    set_error("%s: bad pads/strides", who);
    return false;
  }
  s.N = (int)dX[0]; s.C = (int)dX[1]; s.H = (int)dX[2]; s.W = (int)dX[3];
  s.K = (int)dW[0]; s.Cg = (int)dW[1]; s.R = (int)dW[2]; s.S = (int)dW[3];
  s.ph = (int)pads[0]; s.pw = (int)pads[1]; s.sh = (int)strides[0]; s.sw = (int)strides[1];
  s.group = (int)group;
  const int64_t P = (s.H + 2 * (int64_t)s.ph - s.R) / s.sh + 1, Q = (s.W + 2 * (int64_t)s.pw - s.S) / s.sw + 1;
  if (s.H + 2 * s.ph < s.R || s.W + 2 * s.pw < s.S || P < 1 || Q < 1) { set_error("%s: empty output", who); return false; }
  s.P = (int)P; s.Q = (int)Q;
  if ((int64_t)s.N * P * Q > INT32_MAX || (int64_t)s.Cg * s.R * s.S > INT32_MAX ||
      (int64_t)s.C * s.H * s.W > INT32_MAX) {
    set_error("%s: problem too large for 32-bit tile indices", who);
    return false;
  }
  return true;
}

// Dense convolution with at most four output channels (an image-producing
// last layer: 64 -> 3).  A 32-wide MFMA tile would idle 29 of its 32 rows, so
// this is plain FMA code: one thread per output pixel computes all K outputs.
// A workgroup owns a 16 x 16 patch of pixels, so the rows a tap above or
// below reads are rows the same workgroup reads anyway (L1 hits; with a
// workgroup per image row segment every input row came from L2 three times).
// The filter is copied to LDS once per workgroup as [c][tap][KMAX] (zeros
// for k >= K): every lane reads the same address, one broadcast 16-byte LDS
// read per tap instead of K scalar loads.
// Weight element (k, c, r, s) sits at w[k * w_k + ((c * R + r) * S + s) * w_tap].
template <int KMAX, int R, int S>
__global__ __launch_bounds__(256) void conv_f32_narrow_kernel(
    const float *__restrict__ X, const float *__restrict__ Wt, const float *__restrict__ bias,
    const float *__restrict__ Zr, float *__restrict__ Y, int C, int H, int W, int K, int P, int Q, int ph, int pw,
    int sh, int sw, int act, float act_coef, int w_k, int w_tap) {
  extern __shared__ float wl[];
  static_assert(KMAX == 4, "one float4 of filter values per tap");
  for (int i = threadIdx.x; i < C * R * S * KMAX; i += 256) {
    const int k = i % KMAX, ct = i / KMAX;  // ct = c * R * S + tap
    wl[i] = k < K ? Wt[(int64_t)k * w_k + (int64_t)ct * w_tap] : 0.f;
  }
  __syncthreads();
  const int tiles_q = (Q + 15) >> 4, tiles_p = (P + 15) >> 4;
  const int tq = (int)(blockIdx.x % tiles_q), tp = (int)((blockIdx.x / tiles_q) % tiles_p), n = (int)(blockIdx.x / (tiles_q * tiles_p));
  const int p_raw = tp * 16 + (threadIdx.x >> 4), q_raw = tq * 16 + (threadIdx.x & 15);
  const bool live = p_raw < P && q_raw < Q;
  const int p = min(p_raw, P - 1), q = min(q_raw, Q - 1);
  const int ih0 = p * sh - ph, iw0 = q * sw - pw;
  // clamped tap offsets and masks, once
  int off[R][S];
  unsigned msk[R][S];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int s = 0; s < S; s++) {
      const int ih = ih0 + r, iw = iw0 + s;
      const bool ok = (unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W;
      off[r][s] = ok ? ih * W + iw : 0;
      msk[r][s] = ok ? 0xffffffffu : 0u;
    }
  float acc[KMAX];
#pragma unroll
  for (int k = 0; k < KMAX; k++) acc[k] = 0.f;
  const int HW = H * W;
  const float *x = X + (int64_t)n * C * HW;
  // The reads of one channel are a page apart from the next channel's and
  // come back after about a microsecond; four channels' taps are kept in
  // flight in four named register sets (loads of channels past the end
  // re-read the last one and are not used).
  struct Taps { float v[R][S]; };
  auto fetch = [&](int c) {
    Taps t;
    const float *xc = x + (int64_t)min(c, C - 1) * HW;
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
      for (int s = 0; s < S; s++) t.v[r][s] = xc[off[r][s]];
    return t;
  };
  auto use = [&](const Taps &t, int c) {
    const float4 *w = reinterpret_cast<const float4 *>(wl) + c * R * S;
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
      for (int s = 0; s < S; s++) {
        const float v = __uint_as_float(__float_as_uint(t.v[r][s]) & msk[r][s]);
        const float4 f = w[r * S + s];
        acc[0] = fmaf(v, f.x, acc[0]);
        acc[1] = fmaf(v, f.y, acc[1]);
        acc[2] = fmaf(v, f.z, acc[2]);
        acc[3] = fmaf(v, f.w, acc[3]);
      }
  };
  Taps t0 = fetch(0), t1 = fetch(1), t2 = fetch(2), t3 = fetch(3);
  for (int c = 0; c < C; c += 4) {
    use(t0, c);
    t0 = fetch(c + 4);
    if (c + 1 < C) use(t1, c + 1);
    t1 = fetch(c + 5);
    if (c + 2 < C) use(t2, c + 2);
    t2 = fetch(c + 6);
    if (c + 3 < C) use(t3, c + 3);
    t3 = fetch(c + 7);
  }
  if (!live) return;
  const int64_t PQ = (int64_t)P * Q, pix = (int64_t)p * Q + q;
#pragma unroll
  for (int k = 0; k < KMAX; k++)
    if (k < K) {
      const int64_t o = ((int64_t)n * K + k) * PQ + pix;
      float r = acc[k];
      if (bias) r += bias[k];
      if (Zr) r += Zr[o];
      Y[o] = apply_act(r, act, act_coef);
    }
}

// 3 -> 64 channels, 7x7, stride 2, pad 3: the shape conv_f32_stem.hip is written for.
static bool stem_f32_shape(const ConvShape &s) {
  return s.group == 1 && s.C == 3 && s.K == 64 && s.R == 7 && s.S == 7 && s.sh == 2 && s.sw == 2 && s.ph == 3 && s.pw == 3;
}

static void *conv_f32_nchw(const dnnrtContext *ctx, const ConvShape &s, const float *X,
                           const float *Wt, const float *bias, const float *Z, int act, float *Y) {
  // Filter storage: K,C,R,S (the reference's) or C,R,S,K (k_out contiguous),
  // which lets 32 lanes that own 32 consecutive output channels read one
  // contiguous 128-byte line per reduction element.
  const bool crsk = ctx->filter_layout == DNNRT_FILTER_CRSK;
  if (s.Cg == 1 && s.group > 1) {  // depthwise
    const int64_t total = (int64_t)s.N * s.K * s.P * s.Q;
    const int Kg = s.K / s.group;
    dim3 grid((unsigned)ceil_div(total, 256)), block(256);
    if (ceil_div(total, 256) > INT32_MAX) DNNRT_FAIL("conv: depthwise output too large");
    const int w_k = crsk ? 1 : s.R * s.S, w_tap = crsk ? s.K : 1;
    if (s.R == 3 && s.S == 3 && total + 256 < (1ll << 31) && (int64_t)s.H * s.W < (1ll << 31))
      hipLaunchKernelGGL(dwconv3x3_f32_nchw_kernel, grid, block, 0, ctx->stream, X, Wt, bias, Z, Y, s.C, s.H, s.W, s.K, Kg, s.P,
                         s.Q, s.ph, s.pw, s.sh, s.sw, act, ctx->act_coef, (int)total, w_k, w_tap, magic_of(s.Q), magic_of(s.P),
                         magic_of(s.K), magic_of(Kg));
    else if (s.R == 3 && s.S == 3)
      hipLaunchKernelGGL((dwconv_f32_nchw_kernel<3, 3>), grid, block, 0, ctx->stream, X, Wt, bias, Z, Y,
                         s.C, s.H, s.W, s.K, Kg, s.P, s.Q, s.ph, s.pw, s.sh, s.sw, 3, 3, act, ctx->act_coef, total, w_k, w_tap);
    else
      hipLaunchKernelGGL((dwconv_f32_nchw_kernel<0, 0>), grid, block, 0, ctx->stream, X, Wt, bias, Z, Y,
                         s.C, s.H, s.W, s.K, Kg, s.P, s.Q, s.ph, s.pw, s.sh, s.sw, s.R, s.S, act, ctx->act_coef, total, w_k, w_tap);
    DNNRT_CHECK_LAUNCH("conv(depthwise)");
    return Y;
  }
  if (s.group == 1 && s.K <= 4 && ((s.R == 3 && s.S == 3) || (s.R == 1 && s.S == 1)) && (int64_t)s.C * s.H * s.W < (1ll << 31) &&
      (int64_t)s.C * s.R * s.S * 16 <= 48 * 1024) {  // the filter copy fits the default LDS limit
    const int64_t blocks = (int64_t)s.N * ceil_div(s.P, 16) * ceil_div(s.Q, 16);
    if (blocks > INT32_MAX) DNNRT_FAIL("conv: output too large");
    dim3 grid((unsigned)blocks), block(256);
    const size_t lds = (size_t)s.C * s.R * s.S * 4 * sizeof(float);
    const int w_k = crsk ? 1 : s.C * s.R * s.S, w_tap = crsk ? s.K : 1;
    if (s.R == 3)
      hipLaunchKernelGGL((conv_f32_narrow_kernel<4, 3, 3>), grid, block, lds, ctx->stream, X, Wt, bias, Z, Y, s.C, s.H, s.W, s.K,
                         s.P, s.Q, s.ph, s.pw, s.sh, s.sw, act, ctx->act_coef, w_k, w_tap);
    else
      hipLaunchKernelGGL((conv_f32_narrow_kernel<4, 1, 1>), grid, block, lds, ctx->stream, X, Wt, bias, Z, Y, s.C, s.H, s.W, s.K,
                         s.P, s.Q, s.ph, s.pw, s.sh, s.sw, act, ctx->act_coef, w_k, w_tap);
    DNNRT_CHECK_LAUNCH("conv(narrow)");
    return Y;
  }
  if (stem_f32_shape(s) && bias && (int64_t)s.N * ceil_div(s.P, 5) * ceil_div(s.Q, 16) <= 4 * (int64_t)ctx->num_cu) {
    // the first layer of the ImageNet networks at small batches: one workgroup per 5 x 16 pixels, patch in LDS
    if (!launch_conv_f32_stem(ctx, s.N, s.H, s.W, s.P, s.Q, X, Wt, bias, Z, act, Y, false, 0, 0)) return nullptr;
    return Y;
  }
  IgemmArgs a{};
  const int Kg = s.K / s.group;
  a.A = Wt; a.X = X; a.Y = Y; a.bias = bias; a.Cin = Z;  // residual: (acc + bias) + Z
  a.alpha = 1.f; a.beta = Z ? 1.f : 0.f; a.act = act; a.act_coef = ctx->act_coef;
  a.M = Kg; a.Kdim = s.Cg * s.R * s.S; a.Ncols = s.N * s.P * s.Q;
  a.H = s.H; a.W = s.W; a.R = s.R; a.S = s.S; a.P = s.P; a.Q = s.Q;
  a.ph = s.ph; a.pw = s.pw; a.sh = s.sh; a.sw = s.sw;
  a.x_img_stride = (int64_t)s.C * s.H * s.W;
  a.y_img_stride = (int64_t)s.K * s.P * s.Q;
  a.y_row_stride = (int64_t)s.P * s.Q;
  a.Z = s.group;
  // K,C,R,S: group g owns rows [g*Kg, (g+1)*Kg) of Kdim words each;
  // C,R,S,K: element (m, k) of group g sits at k * K + g * Kg + m.
  a.a_z_stride = crsk ? Kg : (int64_t)Kg * a.Kdim;
  a.a_ld = s.K;
  a.x_z_stride = (int64_t)s.Cg * s.H * s.W;
  a.y_z_stride = (int64_t)Kg * s.P * s.Q;
  a.c_row_stride = a.y_row_stride; a.c_z_stride = a.y_z_stride;  // the residual is laid out like Y
  a.bias_z_stride = Kg;
  a.b_kcontig = false; a.a_mcontig = crsk;
  a.a_vec4 = !crsk && (a.Kdim % 4 == 0) && aligned16(Wt);
  a.b_vec4 = false;
  if (!launch_igemm_f32(ctx, a)) return nullptr;
  return Y;
}

// The `algo` operand of the convolution calls: DNNRT_CONV_ALGO_BASE + id asks for the fp16 channels-last variant
// `id` of dnnrtListConvTiles where that variant can run the problem (else, and for every other value, the
// automatic choice).  Values below the base are cuDNN's algorithm numbers, which name nothing here.
static int variant_of_algo(int64_t algo) {
  if (algo <= DNNRT_CONV_ALGO_BASE || algo >= DNNRT_CONV_ALGO_BASE + 1000) return 0;
  const int id = (int)(algo - DNNRT_CONV_ALGO_BASE);
  for (const int *t = F16_TILE_IDS; *t; t++)
    if (*t == id) return id;
  return 0;
}

static void *conv_dispatch(const char *who, dnnrtHandle_t h, const void *X, const int64_t *dX,
                           const void *W, const int64_t *dW, const void *B, const void *Z, int64_t group,
                           const int64_t *pads, const int64_t *strides, int act, void *Y,
                           int32_t dtype, int64_t algo = 0) {
  if (!h) DNNRT_FAIL("%s: null handle", who);
  if (!X || !W || !Y) DNNRT_FAIL("%s: null tensor", who);
  // an empty batch is no work: nothing is launched and Y is left as it is
  if (dX && dX[0] == 0 && dX[1] > 0 && dX[2] > 0 && dX[3] > 0) return Y;
  ConvShape s;
  if (!parse_conv(who, dX, dW, group, pads, strides, s)) return nullptr;
  if (dtype == DNNRT_F32) {
    if (h->format != DNNRT_NCHW) DNNRT_FAIL("%s: fp32 tensors are NCHW only", who);
    return conv_f32_nchw(h, s, (const float *)X, (const float *)W, (const float *)B, (const float *)Z, act, (float *)Y);
  }
  if (dtype == DNNRT_F16) {
    ConvF16Args a{};
    a.X = (const __half *)X; a.Wt = (const __half *)W; a.bias = (const __half *)B; a.Z = (const __half *)Z; a.Y = (__half *)Y;
    a.N = s.N; a.C = s.C; a.H = s.H; a.W = s.W; a.K = s.K; a.Cg = s.Cg; a.R = s.R; a.S = s.S;
    a.P = s.P; a.Q = s.Q; a.ph = s.ph; a.pw = s.pw; a.sh = s.sh; a.sw = s.sw; a.group = s.group;
    a.act = act; a.act_coef = h->act_coef; a.format = h->format;
    a.variant = variant_of_algo(algo);
    if (!launch_conv_f16(h, a)) return nullptr;
    return Y;
  }
  DNNRT_FAIL("%s: dtype %d", who, dtype);
}

// ---- the process-wide scratch of dnnrtConvBiasActivNoAlloc -----------------
// Partial tiles, then arrival counters, in one file-scope device array: every
// GPU the library runs on holds its own copy from the moment the code object
// is loaded until the process ends.  Host code never uses the array's name as
// an address (on the host it is a stand-in, not device memory): the per-device
// address comes from hipGetSymbolAddress, once, with that device current.
constexpr int64_t NOALLOC_SCRATCH_BYTES = NOALLOC_PARTIAL_BYTES + (int64_t)NOALLOC_MAX_TILES * sizeof(unsigned);
static __device__ __align__(256) unsigned char noalloc_scratch[NOALLOC_SCRATCH_BYTES];

constexpr int NOALLOC_MAX_DEVICES = 64;
struct NoAllocDevice {
  bool ready;
  unsigned char *scratch;  // this device's copy of noalloc_scratch
  int num_cu;
};
static NoAllocDevice noalloc_devices[NOALLOC_MAX_DEVICES];
static std::mutex noalloc_mutex;

// The current device's entry, set up on first use (no allocation: the array is part of the loaded code object).
static const NoAllocDevice *noalloc_device(int &dev) {
  if (hipGetDevice(&dev) != hipSuccess) { set_error("dnnrtConvBiasActivNoAlloc: hipGetDevice failed"); return nullptr; }
  if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) { set_error("dnnrtConvBiasActivNoAlloc: device ordinal %d", dev); return nullptr; }
  std::lock_guard<std::mutex> lock(noalloc_mutex);
  NoAllocDevice &d = noalloc_devices[dev];
  if (d.ready) return &d;
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) { set_error("dnnrtConvBiasActivNoAlloc: hipGetDeviceProperties: %s", hipGetErrorString(e)); return nullptr; }
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    set_error("dnnrtConvBiasActivNoAlloc: this library holds gfx950 code only, device is %s", prop.gcnArchName);
    return nullptr;
  }
  void *ptr = nullptr;
  e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(noalloc_scratch));
  if (e != hipSuccess || !ptr) {
    set_error("dnnrtConvBiasActivNoAlloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
    return nullptr;
  }
  d.scratch = static_cast<unsigned char *>(ptr);
  d.num_cu = prop.multiProcessorCount;
  d.ready = true;
  return &d;
}

}  // namespace dnnrt

extern "C" {

void *dnnrtConvBiasActivNoAlloc(dnnrtStream_t stream, const void *X, const int64_t *dimX, const void *W,
                                const int64_t *dimW, const void *B, const int64_t *dimB, int64_t group,
                                const int64_t *pads, const int64_t *strides, int64_t activMode, void *Y,
                                int32_t dtype) {
  if (!dnnrt::fusable_act(activMode))
    DNNRT_FAIL("dnnrtConvBiasActivNoAlloc: activMode %ld (1 ReLU, 3 clipped ReLU, 5 identity, 6 leaky ReLU)", (long)activMode);
  if (!B || !dimB || !dimW || dnnrt::numel(dimB, 4) != dimW[0])
    DNNRT_FAIL("dnnrtConvBiasActivNoAlloc: bias must hold K values");
  int dev = 0;
  const dnnrt::NoAllocDevice *d = dnnrt::noalloc_device(dev);
  if (!d) return nullptr;
  // A handle on the stack: the defaults of dnnrtCreate, and the static scratch where a handle has its own.
  dnnrtContext ctx{};
  ctx.stream = (hipStream_t)stream;
  ctx.format = DNNRT_NCHW;
  ctx.filter_layout = DNNRT_FILTER_KCRS;
  ctx.act_coef = 0.f;
  ctx.device = dev;
  ctx.num_cu = d->num_cu;
  ctx.splitk_partials = reinterpret_cast<float *>(d->scratch);
  ctx.splitk_counters = reinterpret_cast<unsigned *>(d->scratch + dnnrt::NOALLOC_PARTIAL_BYTES);
  ctx.splitk_partial_bytes = dnnrt::NOALLOC_PARTIAL_BYTES;
  ctx.splitk_max_tiles = dnnrt::NOALLOC_MAX_TILES;
  ctx.splitk_shared = true;
  ctx.f16_tile = 0;
  return dnnrt::conv_dispatch("dnnrtConvBiasActivNoAlloc", &ctx, X, dimX, W, dimW, B, nullptr, group, pads, strides,
                              (int)activMode, Y, dtype);
}

void *dnnrtConv(dnnrtHandle_t handle, const void *X, const int64_t *dimX, const void *W,
                const int64_t *dimW, void *workspace, int64_t workspaceBytes, int64_t algo,
                int64_t group, const int64_t *pads, const int64_t *strides, void *Y, int32_t dtype) {
  (void)workspace; (void)workspaceBytes;
  return dnnrt::conv_dispatch("dnnrtConv", handle, X, dimX, W, dimW, nullptr, nullptr, group, pads, strides,
                              DNNRT_ACT_IDENTITY, Y, dtype, algo);
}

void *dnnrtConvBiasActiv(dnnrtHandle_t handle, const void *X, const int64_t *dimX, const void *W,
                         const int64_t *dimW, const void *B, const int64_t *dimB, void *workspace,
                         int64_t workspaceBytes, int64_t algo, int64_t group, const int64_t *pads,
                         const int64_t *strides, int64_t activMode, void *Y, int32_t dtype) {
  (void)workspace; (void)workspaceBytes;
  if (!dnnrt::fusable_act(activMode))
    DNNRT_FAIL("dnnrtConvBiasActiv: activMode %ld (1 ReLU, 3 clipped ReLU, 5 identity, 6 leaky ReLU)", (long)activMode);
  if (!B || !dimB || !dimW || dnnrt::numel(dimB, 4) != dimW[0])
    DNNRT_FAIL("dnnrtConvBiasActiv: bias must hold K values");
  return dnnrt::conv_dispatch("dnnrtConvBiasActiv", handle, X, dimX, W, dimW, B, nullptr, group, pads,
                              strides, (int)activMode, Y, dtype, algo);
}

void *dnnrtConvBiasActivMaxPool(dnnrtHandle_t handle, const void *X, const int64_t *dimX, const void *W,
                                const int64_t *dimW, const void *B, const int64_t *dimB, int64_t group,
                                const int64_t *pads, const int64_t *strides, int64_t activMode,
                                const int64_t *poolKernel, const int64_t *poolPads, const int64_t *poolStrides, void *Y,
                                const int64_t *dimY, int32_t dtype) {
  const char *who = "dnnrtConvBiasActivMaxPool";
  if (!handle) DNNRT_FAIL("%s: null handle", who);
  if (!X || !W || !Y || !dimX || !dimW || !dimY || !pads || !strides || !poolKernel || !poolPads || !poolStrides)
    DNNRT_FAIL("%s: null argument", who);
  if (!B || !dimB || dnnrt::numel(dimB, 4) != dimW[0]) DNNRT_FAIL("%s: bias must hold K values", who);
  if (dtype != DNNRT_F16 && dtype != DNNRT_F32) DNNRT_FAIL("%s: dtype %d", who, dtype);
  if (poolKernel[0] != 3 || poolKernel[1] != 3 || poolStrides[0] != 2 || poolStrides[1] != 2 || poolPads[0] != 1 || poolPads[1] != 1)
    DNNRT_FAIL("%s: the pooling must be 3x3, stride 2, pad 1", who);
  dnnrt::ConvShape s;
  if (!dnnrt::parse_conv(who, dimX, dimW, group, pads, strides, s)) return nullptr;
  const int64_t PP = (s.P + 2 - 3) / 2 + 1, QQ = (s.Q + 2 - 3) / 2 + 1;
  if (dimY[0] != s.N || dimY[1] != s.K || dimY[2] != PP || dimY[3] != QQ)
    DNNRT_FAIL("%s: dimY is [%ld,%ld,%ld,%ld], the pooled convolution is [%d,%d,%ld,%ld]", who, (long)dimY[0], (long)dimY[1],
               (long)dimY[2], (long)dimY[3], s.N, s.K, (long)PP, (long)QQ);
  if (s.N == 0) return Y;
  if (dtype == DNNRT_F32) {
    if (handle->format != DNNRT_NCHW) DNNRT_FAIL("%s: fp32 tensors are NCHW only", who);
    if (!dnnrt::stem_f32_shape(s)) DNNRT_FAIL("%s: the convolution must be 3 -> 64 channels, 7x7, stride 2, pad 3", who);
    if (!dnnrt::launch_conv_f32_stem(handle, s.N, s.H, s.W, s.P, s.Q, (const float *)X, (const float *)W, (const float *)B,
                                     nullptr, (int)activMode, (float *)Y, true, (int)PP, (int)QQ))
      return nullptr;
    return Y;
  }
  dnnrt::ConvF16Args a{};
  a.X = (const __half *)X; a.Wt = (const __half *)W; a.bias = (const __half *)B; a.Z = nullptr; a.Y = nullptr;
  a.N = s.N; a.C = s.C; a.H = s.H; a.W = s.W; a.K = s.K; a.Cg = s.Cg; a.R = s.R; a.S = s.S;
  a.P = s.P; a.Q = s.Q; a.ph = s.ph; a.pw = s.pw; a.sh = s.sh; a.sw = s.sw; a.group = s.group;
  a.act = (int)activMode; a.act_coef = handle->act_coef; a.format = handle->format;
  if (!dnnrt::launch_conv_f16_stem_pool(handle, a, (__half *)Y, (int)PP, (int)QQ)) return nullptr;
  return Y;
}

void *dnnrtConvBiasAddConvBiasActiv(dnnrtHandle_t handle, const void *X, const int64_t *dimX, const void *W, const int64_t *dimW,
                                    const void *B, const int64_t *pads, const int64_t *strides, const void *X2,
                                    const int64_t *dimX2, const void *W2, const int64_t *dimW2, const void *B2,
                                    const int64_t *pads2, const int64_t *strides2, int64_t activMode, int64_t algo,
                                    int64_t algo2, void *Y, int32_t dtype) {
  const char *who = "dnnrtConvBiasAddConvBiasActiv";
  if (!handle) DNNRT_FAIL("%s: null handle", who);
  if (!X || !W || !X2 || !W2 || !Y) DNNRT_FAIL("%s: null tensor", who);
  if (dtype != DNNRT_F16 && dtype != DNNRT_F32) DNNRT_FAIL("%s: dtype %d", who, dtype);
  if (!dnnrt::fusable_act(activMode)) DNNRT_FAIL("%s: activMode %ld (1 ReLU, 3 clipped ReLU, 5 identity, 6 leaky ReLU)", who, (long)activMode);
  dnnrt::ConvShape s1, s2;
  if (!dnnrt::parse_conv(who, dimX, dimW, 1, pads, strides, s1) || !dnnrt::parse_conv(who, dimX2, dimW2, 1, pads2, strides2, s2)) return nullptr;
  if (s1.N != s2.N || s1.K != s2.K || s1.P != s2.P || s1.Q != s2.Q)
    DNNRT_FAIL("%s: the two convolutions give [%d,%d,%d,%d] and [%d,%d,%d,%d]", who, s1.N, s1.K, s1.P, s1.Q, s2.N, s2.K, s2.P, s2.Q);
  const bool both_1x1 = s1.R == 1 && s1.S == 1 && s2.R == 1 && s2.S == 1 && !s1.ph && !s1.pw && !s2.ph && !s2.pw && s1.sh == 1 && s1.sw == 1;
  // one kernel where that is the faster way ...
  if (dtype == DNNRT_F16 && both_1x1) {
    dnnrt::ConvF16Args a{};
    a.X = (const __half *)X; a.Wt = (const __half *)W; a.bias = (const __half *)B; a.Z = nullptr; a.Y = (__half *)Y;
    a.N = s1.N; a.C = s1.C; a.H = s1.H; a.W = s1.W; a.K = s1.K; a.Cg = s1.Cg; a.R = 1; a.S = 1;
    a.P = s1.P; a.Q = s1.Q; a.ph = 0; a.pw = 0; a.sh = 1; a.sw = 1; a.group = 1;
    a.act = (int)activMode; a.act_coef = handle->act_coef; a.format = handle->format;
    a.X2 = (const __half *)X2; a.Wt2 = (const __half *)W2; a.bias2 = (const __half *)B2;
    a.C2 = s2.C; a.H2 = s2.H; a.W2 = s2.W; a.sh2 = s2.sh; a.sw2 = s2.sw;
    // Short reductions (64 + 64 or 128 + 256 channels), where the pair is bound by the bytes of the result: the
    // kernel that gives the two calls' bits.  Longer ones, and the short ones when the call's `algo` names a variant
    // of it: one reduction over both convolutions' channels, rounded once (closer to the exact sum than the
    // chain, not its bits).
    const int asked = dnnrt::variant_of_algo(algo);
    const bool short_pair = (s1.C == 64 && s2.C == 64) || (s1.C == 128 && s2.C == 256);
    if (short_pair && !dnnrt::dma_dual_variant(asked) && dnnrt::dual_conv_applies(a)) {
      if (!dnnrt::launch_conv_f16_dual(handle, a)) return nullptr;
      return Y;
    }
    if (handle->f16_tile == 0 && dnnrt::dma_dual_applies(a)) {
      a.magic_pq = dnnrt::magic_of(a.P * a.Q);
      a.magic_q = dnnrt::magic_of(a.Q);
      if (!dnnrt::launch_conv_f16_dma_dual(handle, a, asked)) return nullptr;
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) DNNRT_FAIL("%s: launch failed: %s", who, hipGetErrorString(e));
      return Y;
    }
    if (short_pair && dnnrt::dual_conv_applies(a)) {
      if (!dnnrt::launch_conv_f16_dual(handle, a)) return nullptr;
      return Y;
    }
  }
  if (dtype == DNNRT_F32 && both_1x1 && handle->format == DNNRT_NCHW) {
    // batch-1 sized problems: the second reduction appended to the first in the small 1x1 kernel (one launch, one
    // rounding of the whole sum instead of the chain's three)
    const bool crsk = handle->filter_layout == DNNRT_FILTER_CRSK;
    dnnrt::IgemmArgs a{};
    a.A = (const float *)W; a.X = (const float *)X; a.Y = (float *)Y; a.bias = (const float *)B; a.Cin = nullptr;
    a.alpha = 1.f; a.beta = 0.f; a.act = (int)activMode; a.act_coef = handle->act_coef;
    a.M = s1.K; a.Kdim = s1.C; a.Ncols = s1.N * s1.P * s1.Q;
    a.H = s1.H; a.W = s1.W; a.R = 1; a.S = 1; a.P = s1.P; a.Q = s1.Q; a.ph = 0; a.pw = 0; a.sh = 1; a.sw = 1;
    a.x_img_stride = (int64_t)s1.C * s1.H * s1.W;
    a.y_img_stride = (int64_t)s1.K * s1.P * s1.Q;
    a.y_row_stride = (int64_t)s1.P * s1.Q;
    a.Z = 1;
    a.a_z_stride = 0; a.a_ld = s1.K; a.x_z_stride = 0; a.y_z_stride = 0;
    a.c_row_stride = a.y_row_stride; a.c_z_stride = 0; a.bias_z_stride = 0;
    a.b_kcontig = false; a.a_mcontig = crsk;
    a.a_vec4 = !crsk && (a.Kdim % 4 == 0) && (s2.C % 4 == 0) && dnnrt::aligned16(W) && dnnrt::aligned16(W2);
    a.b_vec4 = false;
    a.A2 = (const float *)W2; a.X2 = (const float *)X2; a.bias2 = (const float *)B2;
    a.Kdim2 = s2.C; a.H2 = s2.H; a.W2 = s2.W; a.sh2 = s2.sh; a.sw2 = s2.sw; a.x2_img_stride = (int64_t)s2.C * s2.H * s2.W;
    a.magic_rs = dnnrt::magic_of(1); a.magic_s = dnnrt::magic_of(1);
    const auto wgs64 = dnnrt::ceil_div(a.M, 64) * dnnrt::ceil_div(a.Ncols, 64);
    if (wgs64 < handle->num_cu) {  // where a convolution of its own would take the small kernels as well
      bool launched = false;
      if (!dnnrt::launch_igemm_f32_small(handle, a, 1, crsk ? 2 : 0, launched)) return nullptr;
      if (launched) return Y;
    }
  }
  // ... and everywhere else the two calls it stands for, the shortcut's result passing through Y itself: the closing
  // call reads its residual operand and writes its result element by element, each by the thread that read it
  if (!dnnrt::conv_dispatch(who, handle, X2, dimX2, W2, dimW2, B2, nullptr, 1, pads2, strides2, DNNRT_ACT_IDENTITY, Y, dtype, algo2)) return nullptr;
  return dnnrt::conv_dispatch(who, handle, X, dimX, W, dimW, B, Y, 1, pads, strides, (int)activMode, Y, dtype, algo);
}

void *dnnrtConvBiasAddActiv(dnnrtHandle_t handle, const void *X, const int64_t *dimX, const void *W,
                            const int64_t *dimW, const void *B, const int64_t *dimB, const void *Z,
                            void *workspace, int64_t workspaceBytes, int64_t algo, int64_t group,
                            const int64_t *pads, const int64_t *strides, int64_t activMode, void *Y,
                            int32_t dtype) {
  (void)workspace; (void)workspaceBytes;
  if (!dnnrt::fusable_act(activMode))
    DNNRT_FAIL("dnnrtConvBiasAddActiv: activMode %ld (1 ReLU, 3 clipped ReLU, 5 identity, 6 leaky ReLU)", (long)activMode);
  if (!B || !dimB || !dimW || dnnrt::numel(dimB, 4) != dimW[0])
    DNNRT_FAIL("dnnrtConvBiasAddActiv: bias must hold K values");
  if (!Z) DNNRT_FAIL("dnnrtConvBiasAddActiv: null residual tensor");
  return dnnrt::conv_dispatch("dnnrtConvBiasAddActiv", handle, X, dimX, W, dimW, B, Z, group, pads,
                              strides, (int)activMode, Y, dtype, algo);
}

}  // extern "C"
