// fp32 N,C,H,W first layer of the ImageNet networks: 3 -> 64 channels, 7x7,
// stride 2, pad 3, with bias and activation, and optionally the 3x3 stride-2
// pad-1 max pooling that follows it, in one kernel.
//
// At batch 1 the layer is 236 MFLOP over 12544 pixels: what matters is how
// few dependent memory round trips a launch has, not its arithmetic rate.  A
// workgroup owns a tile of 5 rows x 16 columns of convolution pixels and all
// 64 filters.  It reads the tile's input patch (3 x 15 x 37 values, each once,
// zeros outside the image) into LDS, each lane reads its 37 filter values
// into registers at the same time, and after one barrier the whole reduction
// (147 taps, 37 steps of v_mfma_f32_16x16x4_f32) runs out of LDS and
// registers: wavefront w owns filters 16w .. 16w+15, an MFMA column block is
// one row of the tile.  The im2col offset of tap k inside the patch comes
// from a 148-entry table in LDS; tap 147 (the reduction padded to a multiple
// of four) multiplies a zero filter value by a word of a zeroed LDS region,
// so that no non-finite input can leak into the sum through it.
//
// With the pooling: the tile is the 5 x 15 convolution pixels under 2 x 7
// pooled ones (neighbouring tiles recompute the shared row and column: 1.34x
// the arithmetic, no carried state, 224 workgroups at 224 x 224).  A lane
// holds one column of all five rows, so the vertical maxima are in registers
// and the horizontal ones two lane shifts away.  The activation is applied
// after the maximum (both supported ones are monotonic); a NaN anywhere in a
// window gives NaN, as the pooling kernel does.
#include "conv_f32_stem.h"

namespace dnnrt {

namespace stem32 {
constexpr int ROWS = 5, COLS = 16;           // convolution pixels per tile
constexpr int PR = 2 * (ROWS - 1) + 7;       // 15 patch rows
constexpr int PW = 2 * (COLS - 1) + 7;       // 37 patch columns
constexpr int PATCH = 3 * PR * PW;           // values
constexpr int ZEROS = 2 * (COLS - 1) + 2 * PW * (ROWS - 1) + 1;  // words the padding tap can reach
constexpr int TAPS = 147, STEPS = 37;
constexpr int PATCH_LOADS = (PATCH + 255) / 256;
}  // namespace stem32

typedef float floatx4 __attribute__((ext_vector_type(4)));

// The larger of two values, NaN if either is one.
__device__ __forceinline__ float nan_max(float a, float b) {
  const float m = a > b ? a : b;
  return (a != a) ? a : ((b != b) ? b : m);
}

template <bool POOL, bool RELU>
__global__ __launch_bounds__(256) void conv_f32_stem_kernel(const float *__restrict__ X, const float *__restrict__ Wt,
                                                            const float *__restrict__ bias, const float *Zr, float *Y,
                                                            const int H, const int W, const int P, const int Q, const int PP,
                                                            const int QQ, const int tiles_r, const int tiles_c,
                                                            const int w_filter_stride, const int w_tap_stride, const int act,
                                                            const float act_coef) {
  using namespace stem32;
  __shared__ float patch[PATCH + ZEROS];
  __shared__ int tap_offset[4 * STEPS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, quad = lane >> 4;
  int b = blockIdx.x;
  const int tc = b % tiles_c; b /= tiles_c;
  const int tr = b % tiles_r;
  const int n = b / tiles_r;
  // first convolution pixel of the tile (may be -1 with the pooling: the pooling's own padding)
  const int cr0 = POOL ? 4 * tr - 1 : ROWS * tr, cc0 = POOL ? 14 * tc - 1 : COLS * tc;
  const int ih0 = 2 * cr0 - 3, iw0 = 2 * cc0 - 3;

  // ---- requests: the patch, the lane's filter values, its bias values ----
  const float *xn = X + (int64_t)n * 3 * H * W;
  float pv[PATCH_LOADS];
#pragma unroll
  for (int i = 0; i < PATCH_LOADS; i++) {
    const int e = tid + 256 * i;
    const int c = e / (PR * PW), rem = e - c * (PR * PW), pr = rem / PW, pc = rem - pr * PW;
    const int ih = ih0 + pr, iw = iw0 + pc;
    const bool ok = e < PATCH && (unsigned)ih < (unsigned)H && (unsigned)iw < (unsigned)W;
    const float v = xn[ok ? ((int64_t)c * H + ih) * W + iw : 0];
    pv[i] = ok ? v : 0.f;
  }
  const int filter = 16 * wave + col;
  float a[STEPS];
#pragma unroll
  for (int t = 0; t < STEPS; t++) {
    const int k = 4 * t + quad;
    const float v = Wt[(int64_t)filter * w_filter_stride + (int64_t)(k < TAPS ? k : TAPS - 1) * w_tap_stride];
    a[t] = k < TAPS ? v : 0.f;
  }
  float bv[4];
#pragma unroll
  for (int i = 0; i < 4; i++) bv[i] = bias[16 * wave + 4 * quad + i];

  // ---- LDS: tap table, patch, the zeroed words behind it ----
  if (tid < 4 * STEPS) {
    const int k = tid;
    const int c = (k * 1338) >> 16, rem = k - 49 * c, r = (rem * 9363) >> 16, s = rem - 7 * r;  // k = (c * 7 + r) * 7 + s
    tap_offset[k] = k < TAPS ? (c * PR + r) * PW + s : PATCH;
  }
  for (int e = tid; e < ZEROS; e += 256) patch[PATCH + e] = 0.f;
#pragma unroll
  for (int i = 0; i < PATCH_LOADS; i++) {
    const int e = tid + 256 * i;
    if (e < PATCH) patch[e] = pv[i];
  }
  __syncthreads();

  int off[STEPS];
#pragma unroll
  for (int t = 0; t < STEPS; t++) off[t] = tap_offset[4 * t + quad] + 2 * col;

  floatx4 acc[ROWS];
#pragma unroll
  for (int j = 0; j < ROWS; j++) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t = 0; t < STEPS; t++) {
    float bj[ROWS];
#pragma unroll
    for (int j = 0; j < ROWS; j++) bj[j] = patch[off[t] + j * 2 * PW];
#pragma unroll
    for (int j = 0; j < ROWS; j++) acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t], bj[j], acc[j], 0, 0, 0);
  }

  // acc[j][i]: filter 16 * wave + 4 * quad + i, tile row j, tile column col
  const int f0 = 16 * wave + 4 * quad;
  if constexpr (POOL) {
    const float ninf = -__builtin_inff();
    const bool col_ok = col < 15 && (unsigned)(cc0 + col) < (unsigned)Q;
    const int pr0 = 2 * tr, pc0 = 7 * tc;
    const int q = col >> 1;
    const bool writer = !(col & 1) && q < 7 && pc0 + q < QQ;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      float v[ROWS];
#pragma unroll
      for (int j = 0; j < ROWS; j++) v[j] = (col_ok && (unsigned)(cr0 + j) < (unsigned)P) ? acc[j][i] + bv[i] : ninf;
#pragma unroll
      for (int p = 0; p < 2; p++) {
        const float m = nan_max(nan_max(v[2 * p], v[2 * p + 1]), v[2 * p + 2]);
        const float m1 = __shfl_down(m, 1, 16), m2 = __shfl_down(m, 2, 16);
        float h = nan_max(nan_max(m, m1), m2);
        if (RELU) h = h < 0.f ? 0.f : h;
        if (h != h) h = __builtin_nanf("");
        if (writer && pr0 + p < PP) Y[(((int64_t)n * 64 + f0 + i) * PP + pr0 + p) * QQ + pc0 + q] = h;
      }
    }
  } else {
    const bool col_ok = cc0 + col < Q;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int j = 0; j < ROWS; j++)
        if (col_ok && cr0 + j < P) {
          const int64_t at = (((int64_t)n * 64 + f0 + i) * P + cr0 + j) * Q + cc0 + col;
          float v = acc[j][i] + bv[i];
          if (Zr) v += Zr[at];  // the residual operand (which may be Y itself: same thread, same element)
          Y[at] = apply_act(v, act, act_coef);
        }
  }
}

bool launch_conv_f32_stem(const dnnrtContext *ctx, int N, int H, int W, int P, int Q, const float *X, const float *Wt,
                          const float *bias, const float *Z, int act, float *Y, bool pool, int PP, int QQ) {
  using namespace stem32;
  if ((int64_t)3 * H * W >= (1ll << 31)) { set_error("first-layer kernel: image too large"); return false; }
  if (!bias) { set_error("first-layer kernel: needs a bias"); return false; }
  if (pool && act != DNNRT_ACT_RELU && act != DNNRT_ACT_IDENTITY) { set_error("conv+maxpool: activation must be ReLU or identity"); return false; }
  if (pool && Z) { set_error("conv+maxpool: no residual operand"); return false; }
  const bool crsk = ctx->filter_layout == DNNRT_FILTER_CRSK;
  const int fs = crsk ? 1 : TAPS, ts = crsk ? 64 : 1;
  const int tiles_r = pool ? (PP + 1) / 2 : (P + ROWS - 1) / ROWS;
  const int tiles_c = pool ? (QQ + 6) / 7 : (Q + COLS - 1) / COLS;
  const int64_t grid = (int64_t)N * tiles_r * tiles_c;
  if (grid > INT32_MAX) { set_error("first-layer kernel: batch too large"); return false; }
  if (grid == 0) return true;
#define STEM32(POOL, RELU)                                                                                                  \
  hipLaunchKernelGGL((conv_f32_stem_kernel<POOL, RELU>), dim3((unsigned)grid), dim3(256), 0, ctx->stream, X, Wt, bias, Z, Y, H,     \
                     W, P, Q, PP, QQ, tiles_r, tiles_c, fs, ts, act, ctx->act_coef)
  if (pool) {
    if (act == DNNRT_ACT_RELU) STEM32(true, true);
    else STEM32(true, false);
  } else {
    STEM32(false, false);
  }
#undef STEM32
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("first-layer kernel: launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

}  // namespace dnnrt
