// fp16 first layers other than the 7x7 one of the ImageNet ResNets: N,C,H,W
// input with at most four channels, a filter of at most 3x3 (any stride and
// padding), 16 to 64 filters, channels-last output (a MobileNetV2's 3 -> 32,
// 3x3, stride 2; a VGG's 3 -> 64, 3x3).
//
// The reduction is at most 36 taps: too short for an MFMA tile to pay for the
// im2col gather, and the layer is bound by the bytes of its result.  A thread
// owns one output pixel and all its filters: it requests its taps (2-byte
// loads, neighbouring lanes neighbouring pixels; a tap in the padding is a
// load from a clamped address whose value is replaced by zero), then walks
// the taps with the tap's K filter values read from an LDS copy of the filter
// transposed to [tap][filter] (the same address in every lane: a broadcast),
// one mixed-precision FMA per tap and filter into fp32 accumulators.  The
// pixel's K results are contiguous in the channels-last tensor and leave as
// 16-byte stores.
#include "conv_f16.h"

namespace dnnrt {

typedef _Float16 fl_half8 __attribute__((ext_vector_type(8)));

constexpr int FIRST_MAX_TAPS = 36;

template <int K8>  // K = 8 * K8 filters
__global__ __launch_bounds__(256) void conv_f16_first_kernel(const ConvF16Args a, const int total, const unsigned magic_pq,
                                                             const unsigned magic_q) {
  constexpr int K = 8 * K8;
  __shared__ __attribute__((aligned(16))) _Float16 wt[FIRST_MAX_TAPS * K];  // [tap][filter], tap = (r S + s) C + c
  const int taps = a.R * a.S * a.C;
  const _Float16 *__restrict__ Wg = reinterpret_cast<const _Float16 *>(a.Wt);  // K x R x S x C
  {  // every value requested before the first one is stored: a load-then-store loop pays a memory round trip per turn
    constexpr int TURNS = (FIRST_MAX_TAPS * K + 255) / 256;
    _Float16 wv[TURNS];
#pragma unroll
    for (int u = 0; u < TURNS; u++) wv[u] = Wg[min((int)threadIdx.x + 256 * u, K * taps - 1)];
#pragma unroll
    for (int u = 0; u < TURNS; u++) {
      const int e = (int)threadIdx.x + 256 * u;
      if (e < K * taps) {
        const int k = e / taps, t = e - k * taps;
        wt[t * K + k] = wv[u];
      }
    }
  }
  __syncthreads();
  const int i = (int)(blockIdx.x * 256 + threadIdx.x);
  if (i >= total) return;
  const int PQ = a.P * a.Q;
  const int n = div_magic(i, PQ, magic_pq), pq = i - n * PQ;
  const int p = div_magic(pq, a.Q, magic_q), q = pq - p * a.Q;
  const int ih0 = p * a.sh - a.ph, iw0 = q * a.sw - a.pw;
  const _Float16 *__restrict__ Xg = reinterpret_cast<const _Float16 *>(a.X) + (int64_t)n * a.C * a.H * a.W;
  _Float16 xv[FIRST_MAX_TAPS];
#pragma unroll
  for (int r = 0; r < 3; r++)
#pragma unroll
    for (int s = 0; s < 3; s++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int t = (r * 3 + s) * 4 + c;  // register slot: fixed at compile time whatever R, S, C are
        const int ih = ih0 + r, iw = iw0 + s;
        const bool wanted = r < a.R && s < a.S && c < a.C;
        const bool ok = wanted && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
        const int ihc = min(max(ih, 0), a.H - 1), iwc = min(max(iw, 0), a.W - 1), cc = min(c, a.C - 1);
        const _Float16 v = Xg[((int64_t)cc * a.H + ihc) * a.W + iwc];
        xv[t] = ok ? v : (_Float16)0.f;
      }
  float acc[K];
#pragma unroll
  for (int k = 0; k < K; k++) acc[k] = 0.f;
#pragma unroll
  for (int r = 0; r < 3; r++)
#pragma unroll
    for (int s = 0; s < 3; s++)
#pragma unroll
      for (int c = 0; c < 4; c++) {
        if (r < a.R && s < a.S && c < a.C) {  // the same for every lane
          const float x = (float)xv[(r * 3 + s) * 4 + c];
          const _Float16 *wrow = wt + ((r * a.S + s) * a.C + c) * K;
#pragma unroll
          for (int g = 0; g < K8; g++) {
            const fl_half8 w8 = *reinterpret_cast<const fl_half8 *>(wrow + 8 * g);
#pragma unroll
            for (int e = 0; e < 8; e++) acc[8 * g + e] = fmaf(x, (float)w8[e], acc[8 * g + e]);
          }
        }
      }
  const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
  const _Float16 *Zg = reinterpret_cast<const _Float16 *>(a.Z);  // may be Y itself: a thread reads an element, then writes it
  _Float16 *Yg = reinterpret_cast<_Float16 *>(a.Y);
  const int64_t off = (int64_t)i * K;
  auto finish = [&](auto mode_c) {  // one copy per activation mode, picked once
    constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
    for (int g = 0; g < K8; g++) {
      fl_half8 z8, o8;
      if (Zg) z8 = *reinterpret_cast<const fl_half8 *>(Zg + off + 8 * g);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float v = acc[8 * g + e];
        if (biasg) v += (float)biasg[8 * g + e];
        if (Zg) v = (float)(_Float16)v + (float)z8[e];
        o8[e] = (_Float16)apply_act(v, MODE, a.act_coef);
      }
      *reinterpret_cast<fl_half8 *>(Yg + off + 8 * g) = o8;
    }
  };
  by_act_mode(a.act, finish);
}

// Launches the kernel if the problem is one of its shapes; `launched` says whether it did.
bool launch_conv_f16_first(const dnnrtContext *ctx, const ConvF16Args &a, bool &launched) {
  launched = false;
  auto aligned = [](const void *p, uintptr_t to) { return (reinterpret_cast<uintptr_t>(p) & (to - 1)) == 0; };
  const int64_t total = (int64_t)a.N * a.P * a.Q;
  if (a.format != DNNRT_NCHW_TO_NHWC || a.group != 1 || a.C > 4 || a.R > 3 || a.S > 3 || a.K % 8 != 0 || !aligned(a.Y, 16) ||
      !aligned(a.Z, 16) || total + 256 >= (1ll << 31) || (int64_t)a.C * a.H * a.W >= (1ll << 31) || total == 0)
    return true;
  const unsigned grid = (unsigned)((total + 255) / 256), m_pq = magic_of(a.P * a.Q), m_q = magic_of(a.Q);
#define FIRST_CASE(K8_)                                                                                                           \
  case K8_: hipLaunchKernelGGL(conv_f16_first_kernel<K8_>, dim3(grid), dim3(256), 0, ctx->stream, a, (int)total, m_pq, m_q); break
  switch (a.K / 8) {
    FIRST_CASE(2); FIRST_CASE(3); FIRST_CASE(4); FIRST_CASE(6); FIRST_CASE(8);
    default: return true;
  }
#undef FIRST_CASE
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("conv(fp16 first layer): launch failed: %s", hipGetErrorString(e)); return false; }
  launched = true;
  return true;
}

}  // namespace dnnrt
