// fp32 3x3 convolution (any stride and padding) as an LDS-tiled implicit GEMM
// for problems that fill the chip: the 3x3 layers of a detection or
// super-resolution network at hundreds of pixels a side.
//
// Same MFMA core as igemm_f32.hip (BM x BN tile, 2 x 2 wavefronts, 32x32x2
// MFMA, operands staged through LDS as [k][m] / [k][col], the next chunk's
// global loads issued before the current chunk's MFMAs), but the im2col side
// does no index arithmetic in the loop.  The general kernel decodes
// k -> (c, r, s) and checks the image bounds for every element it loads,
// under a branch per element: ~40 vector instructions per loaded word, which
// cost as much issue time as the MFMAs they feed.  Here a thread owns one
// output pixel and, per chunk, ONE input channel: its nine tap offsets and
// nine validity masks are computed once, a chunk is NT / BN channels x 9 taps,
// and its nine loads per chunk are base + tap_off[j] from clamped addresses
// with the mask applied when the word goes to LDS.  No load sits under a
// branch, so the compiler counts the outstanding loads exactly.
#include "igemm_f32.h"

#include <type_traits>

namespace dnnrt {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// A_MC: filter stored C,R,S,K (k rows of K_out contiguous words) instead of K,C,R,S.
template <int BM, int BN, bool A_MC>
__global__ __launch_bounds__(256) void conv3x3_f32_tiled_kernel(const IgemmArgs a) {
  constexpr int NT = 256, WM = 2, WN = 2;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int CH = NT / BN;        // input channels per chunk: one per thread of a column
  constexpr int BKC = 9 * CH;        // reduction elements per chunk
  constexpr int LDA = BM + 4, LDB = BN + 4;
  static_assert(NT / BM == CH, "the A loader gives each filter row's chunk to CH threads as well");
  static_assert(BKC % 2 == 0, "MFMA steps take two k");
  constexpr int A4_TOTAL = BKC * (BM / 4), A4_PER = (A4_TOTAL + NT - 1) / NT;  // float4 loads of a C,R,S,K chunk

  __shared__ float As[2][BKC][LDA];
  __shared__ float Bs[2][BKC][LDB];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);
  const int lrow = lane >> 5, lcol = lane & 31;

  const int tiles_n = (a.Ncols + BN - 1) / BN;
  const int tile_m = blockIdx.x / tiles_n, tile_n = blockIdx.x - tile_m * tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int z = blockIdx.z;
  const float *__restrict__ Ag = a.A + (int64_t)z * a.a_z_stride;
  const float *__restrict__ Xg = a.X + (int64_t)z * a.x_z_stride;
  const int C = a.Kdim / 9, HW = a.H * a.W, PQ = a.P * a.Q;

  // ---- B side: this thread's pixel, its taps, its channel of the chunk ----
  const int bcol = tid % BN, bch = tid / BN;
  const int col = n0 + bcol;
  const bool col_ok = col < a.Ncols;
  unsigned tap_off[9], tap_mask[9];
  unsigned x_pix;
  {
    const int img = col_ok ? col / PQ : 0, pq = col_ok ? col - img * PQ : 0;
    const int p = pq / a.Q, q = pq - p * a.Q;
    const int ih0 = p * a.sh - a.ph, iw0 = q * a.sw - a.pw;
#pragma unroll
    for (int j = 0; j < 9; j++) {
      const int ih = ih0 + j / 3, iw = iw0 + j % 3;
      const bool ok = col_ok && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
      tap_off[j] = ok ? (unsigned)(ih * a.W + iw) : 0u;
      tap_mask[j] = ok ? 0xffffffffu : 0u;
    }
    x_pix = (unsigned)((int64_t)img * a.x_img_stride);
  }
  // ---- A side (K,C,R,S): this thread's filter row and its channel of the chunk ----
  const int arow = tid / CH, ach = tid % CH;
  const unsigned a_row_off = (unsigned)min(m0 + arow, a.M - 1) * (unsigned)a.Kdim;

  float rb[9], ra[9];
  static_assert(A4_PER == 3, "three named registers below");
  float4 ra4_0, ra4_1, ra4_2;  // named, not an array: they must stay in registers
  unsigned cmask_b = 0;
  const int nk = (C + CH - 1) / CH;
  auto load_chunk = [&](int kt) {
    const int c0 = min(kt, nk - 1) * CH;  // past the end: the last chunk again, never stored
    {
      const int c = c0 + bch;
      cmask_b = c < C ? 0xffffffffu : 0u;
      const unsigned base = x_pix + (unsigned)min(c, C - 1) * (unsigned)HW;
#pragma unroll
      for (int j = 0; j < 9; j++) rb[j] = Xg[base + tap_off[j]];
    }
    if (!A_MC) {
      const unsigned base = a_row_off + (unsigned)min(c0 + ach, C - 1) * 9u;
#pragma unroll
      for (int j = 0; j < 9; j++) ra[j] = Ag[base + j];
    } else {
      auto fetch = [&](int i) {
        const int idx = min(tid + i * NT, A4_TOTAL - 1), kk = idx / (BM / 4), m4 = idx - kk * (BM / 4);
        const int k = min(c0 * 9 + kk, a.Kdim - 1), m = min(m0 + m4 * 4, a.M - 4);  // M is a multiple of 4 here
        return *reinterpret_cast<const float4 *>(Ag + (int64_t)k * a.a_ld + m);
      };
      ra4_0 = fetch(0); ra4_1 = fetch(1); ra4_2 = fetch(2);
    }
  };
  auto store_chunk = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 9; j++)
      Bs[buf][bch * 9 + j][bcol] = __uint_as_float(__float_as_uint(rb[j]) & tap_mask[j] & cmask_b);
    if (!A_MC) {
#pragma unroll
      for (int j = 0; j < 9; j++) As[buf][ach * 9 + j][arow] = ra[j];
    } else {
      auto put = [&](int i, const float4 &v) {
        const int idx = tid + i * NT;
        if (idx < A4_TOTAL) {
          const int kk = idx / (BM / 4), m4 = idx - kk * (BM / 4);
          *reinterpret_cast<float4 *>(&As[buf][kk][m4 * 4]) = v;
        }
      };
      put(0, ra4_0); put(1, ra4_1); put(2, ra4_2);
    }
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // bias of the lane's rows, requested before the reduction starts
  auto row_k = [](int r) { return 8 * (r >> 2) + (r & 3); };
  float bias_r[TM][16];
  if (a.bias) {
    const float *__restrict__ biasg = a.bias + (int64_t)z * a.bias_z_stride;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) bias_r[i][r] = biasg[min(m0 + wm0 + i * 32 + 4 * lrow + row_k(r), a.M - 1)];
  } else {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) bias_r[i][r] = 0.f;
  }

  load_chunk(0);
  store_chunk(0);
  __syncthreads();
  for (int kt = 0; kt < nk; kt++) {
    const int buf = kt & 1;
    load_chunk(kt + 1);
#pragma unroll
    for (int ks = 0; ks < BKC; ks += 2) {
      float av[TM], bv[TN];
#pragma unroll
      for (int i = 0; i < TM; i++) av[i] = As[buf][ks + lrow][wm0 + i * 32 + lcol];
#pragma unroll
      for (int j = 0; j < TN; j++) bv[j] = Bs[buf][ks + lrow][wn0 + j * 32 + lcol];
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
    store_chunk(buf ^ 1);  // after the last chunk: rows nobody reads
    __syncthreads();
  }

  // ---- epilogue: register r of lane l in block (i, j) is row 4 * (l / 32) + row_k(r), column l % 32.
  // Residual values come in one batch per block from clamped addresses; a row's
  // address is one per-lane base plus a uniform offset; only stores are predicated.
  float *__restrict__ Yg = a.Y + (int64_t)z * a.y_z_stride;
  auto emit = [&](auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int ecol = n0 + wn0 + j * 32 + lcol;
      const bool ecol_ok = ecol < a.Ncols;
      const int colc = ecol_ok ? ecol : 0;
      const int img = colc / PQ, pq = colc - img * PQ;
      const int64_t ycol = (int64_t)img * a.y_img_stride + pq;
#pragma unroll
      for (int i = 0; i < TM; i++) {
        const int mrow0 = m0 + wm0 + i * 32 + 4 * lrow;
        float res_r[16];
        if (a.Cin) {
          const float *__restrict__ Cg = a.Cin + (int64_t)z * a.c_z_stride;
#pragma unroll
          for (int r = 0; r < 16; r++) res_r[r] = Cg[ycol + (int64_t)min(mrow0 + row_k(r), a.M - 1) * a.c_row_stride];
        } else {
#pragma unroll
          for (int r = 0; r < 16; r++) res_r[r] = 0.f;
        }
        float *__restrict__ y0 = Yg + ycol + (int64_t)mrow0 * a.y_row_stride;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float v = a.alpha * acc[i][j][r] + bias_r[i][r];
          if (a.Cin) v += a.beta * res_r[r];
          v = apply_act(v, MODE, a.act_coef);
          if (ecol_ok && mrow0 + row_k(r) < a.M) y0[(int64_t)row_k(r) * a.y_row_stride] = v;
        }
      }
    }
  };
  switch (a.act) {
    case DNNRT_ACT_RELU: emit(std::integral_constant<int, DNNRT_ACT_RELU>{}); break;
    case DNNRT_ACT_CLIPPED_RELU: emit(std::integral_constant<int, DNNRT_ACT_CLIPPED_RELU>{}); break;
    case DNNRT_ACT_LEAKY_RELU: emit(std::integral_constant<int, DNNRT_ACT_LEAKY_RELU>{}); break;
    default: emit(std::integral_constant<int, DNNRT_ACT_IDENTITY>{}); break;
  }
}

// Takes 3x3 convolutions (reduction a multiple of 9, no per-column bias, every
// operand below 2^31 elements) with the tile sizes the general kernel would
// pick; `launched` says whether it applied.
bool launch_conv3x3_f32_tiled(const dnnrtContext *ctx, const IgemmArgs &a, int layout, bool &launched) {
  launched = false;
  if (a.R != 3 || a.S != 3 || a.Kdim % 9 || a.bias_col || (layout != 0 && layout != 2)) return true;
  if (a.act != DNNRT_ACT_IDENTITY && a.act != DNNRT_ACT_RELU && a.act != DNNRT_ACT_CLIPPED_RELU && a.act != DNNRT_ACT_LEAKY_RELU) return true;
  const bool amc = layout == 2;
  if (amc && (a.M % 4 || a.a_ld % 4 || a.a_z_stride % 4 || !aligned16(a.A))) return true;
  const int64_t a_elems = amc ? (int64_t)a.Kdim * a.a_ld : (int64_t)a.M * a.Kdim;
  const int64_t x_elems = (int64_t)((a.Ncols + a.P * a.Q - 1) / (a.P * a.Q)) * a.x_img_stride + (int64_t)(a.Kdim / 9) * a.H * a.W;
  if (a_elems >= (1ll << 31) || x_elems >= (1ll << 31)) return true;
  auto wgs = [&](int bm, int bn) { return ceil_div(a.M, bm) * ceil_div(a.Ncols, bn) * a.Z; };
#define LAUNCH_T(BM_, BN_)                                                                                         \
  do {                                                                                                             \
    const int64_t tiles = ceil_div(a.M, BM_) * ceil_div(a.Ncols, BN_);                                             \
    if (tiles > INT32_MAX) return true;                                                                            \
    dim3 grid((unsigned)tiles, 1, a.Z), block(256);                                                                \
    if (amc) hipLaunchKernelGGL((conv3x3_f32_tiled_kernel<BM_, BN_, true>), grid, block, 0, ctx->stream, a);       \
    else hipLaunchKernelGGL((conv3x3_f32_tiled_kernel<BM_, BN_, false>), grid, block, 0, ctx->stream, a);          \
  } while (0)
  if (wgs(128, 128) >= ctx->num_cu) LAUNCH_T(128, 128);
  else if (wgs(64, 64) >= ctx->num_cu) LAUNCH_T(64, 64);  // with fewer workgroups than CUs the 32x32-tile kernels win (measured)
  else return true;
#undef LAUNCH_T
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("conv3x3_f32(tiled): launch failed: %s", hipGetErrorString(e)); return false; }
  launched = true;
  return true;
}

}  // namespace dnnrt
