// fp32 implicit-GEMM kernels (v_mfma_f32_32x32x2f32) for gfx950.
//
// Work decomposition: a workgroup of WM x WN wavefronts (64 lanes each) owns a
// BM x BN tile of D; each wavefront owns a (BM/WM) x (BN/WN) sub-tile made of
// 32x32 MFMA blocks whose accumulators stay in registers for the whole
// reduction.  The reduction runs in steps of BK = 16: both operand tiles are
// staged through LDS as [k][m] / [k][col] so that one MFMA operand fetch is a
// conflict-free ds_read_b32 (lane l reads row l/32, column l%32), and the
// next step's global loads are issued before the current step's MFMAs
// (register prefetch + double-buffered LDS, one barrier per step).
//
// The B tile is never materialised in memory: its element (k, col) is
// X[img, c, p*sh - ph + r, q*sw - pw + s] with k -> (c, r, s) and
// col -> (img, p, q) decoded on the fly (im2col fused into the load).
#include "igemm_f32.h"

namespace dnnrt {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BK = 16;

// LAYOUT bit 0: B is k-contiguous ([Ncols][Kdim]); bit 1: A is m-contiguous.
template <int BM, int BN, int WM, int WN, int RSMODE, int LAYOUT>
__global__ __launch_bounds__(64 * WM * WN) void igemm_f32_kernel(const IgemmArgs a) {
  constexpr int NT = 64 * WM * WN;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int LDA = BM + 4, LDB = BN + 4;
  constexpr bool B_KC = (LAYOUT & 1) != 0, A_MC = (LAYOUT & 2) != 0;
  static_assert(TM >= 1 && TN >= 1, "tile too small for the wave grid");
  static_assert((BM * BK / 4) % NT == 0 && (BN * BK / 4) % NT == 0, "loader shape");
  static_assert(NT % BM == 0 || BM % NT == 0, "loader shape");
  static_assert(NT % BN == 0, "each thread must own one B column");

  __shared__ float As[2][BK][LDA];
  __shared__ float Bs[2][BK][LDB];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);

  const int tiles_n = (a.Ncols + BN - 1) / BN;
  const int tile_m = blockIdx.x / tiles_n, tile_n = blockIdx.x - tile_m * tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int z = blockIdx.z;

  const float *__restrict__ Ag = a.A + (int64_t)z * a.a_z_stride;
  const float *__restrict__ Xg = a.X + (int64_t)z * a.x_z_stride;

  // ---- per-thread constants of the B (im2col) loader: one column each ----
  constexpr int B_ROWS_PER_PASS = NT / BN;       // k rows covered by one pass
  constexpr int B_PER = BK / B_ROWS_PER_PASS;    // elements per thread per step
  const int bcol = tid % BN, bkk0 = tid / BN;
  int64_t b_pix_off = 0;
  int ih0 = 0, iw0 = 0;
  bool b_col_ok = false;
  if (!B_KC) {
    const int col = n0 + bcol;
    b_col_ok = col < a.Ncols;
    const int PQ = a.P * a.Q;
    const int img = b_col_ok ? col / PQ : 0;
    const int pq = b_col_ok ? col - img * PQ : 0;
    const int p = pq / a.Q, q = pq - p * a.Q;
    ih0 = p * a.sh - a.ph;
    iw0 = q * a.sw - a.pw;
    b_pix_off = (int64_t)img * a.x_img_stride;
    if (RSMODE == 1) b_pix_off += (int64_t)ih0 * a.W + iw0;
  }
  const int HW = a.H * a.W;

  // ---- k-contiguous loader geometry (A normally, B with transB) ----------
  constexpr int A_PER4 = (BM * BK / 4) / NT;
  constexpr int B_PER4 = (BN * BK / 4) / NT;
  // ---- m-contiguous A loader (transA) -------------------------------------
  constexpr int AM_ROWS_PER_PASS = (NT >= BM) ? NT / BM : 1;
  constexpr int AM_PER = (BM * BK) / NT;

  float4 ra[A_MC ? 1 : A_PER4];
  float ram[A_MC ? AM_PER : 1];
  float rb[B_KC ? 1 : B_PER];
  float4 rb4[B_KC ? B_PER4 : 1];

  auto load_kcontig4 = [&](const float *__restrict__ base, int row, int nrows, int k, bool vec) -> float4 {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row < nrows) {
      const float *p = base + (int64_t)row * a.Kdim + k;
      if (vec) {
        if (k < a.Kdim) v = *reinterpret_cast<const float4 *>(p);
      } else {
        if (k + 0 < a.Kdim) v.x = p[0];
        if (k + 1 < a.Kdim) v.y = p[1];
        if (k + 2 < a.Kdim) v.z = p[2];
        if (k + 3 < a.Kdim) v.w = p[3];
      }
    }
    return v;
  };

  auto load_tiles = [&](int k0) {
    // A
    if (!A_MC) {
#pragma unroll
      for (int i = 0; i < A_PER4; i++) {
        const int idx = tid + i * NT, row = idx >> 2, kq = idx & 3;
        ra[i] = load_kcontig4(Ag, m0 + row, a.M, k0 + kq * 4, a.a_vec4);
      }
    } else {
#pragma unroll
      for (int i = 0; i < AM_PER; i++) {
        const int idx = tid + i * NT, mm = idx % BM, kk = idx / BM;
        const int m = m0 + mm, k = k0 + kk;
        ram[i] = (m < a.M && k < a.Kdim) ? Ag[(int64_t)k * a.a_ld + m] : 0.f;
      }
    }
    // B
    if (B_KC) {
#pragma unroll
      for (int i = 0; i < B_PER4; i++) {
        const int idx = tid + i * NT, row = idx >> 2, kq = idx & 3;
        rb4[i] = load_kcontig4(Xg, n0 + row, a.Ncols, k0 + kq * 4, a.b_vec4);
      }
    } else {
#pragma unroll
      for (int j = 0; j < B_PER; j++) {
        const int k = k0 + bkk0 + j * B_ROWS_PER_PASS;
        float v = 0.f;
        if (RSMODE == 1) {
          if (b_col_ok && k < a.Kdim) v = Xg[b_pix_off + (int64_t)k * HW];
        } else {
          int c, r, s;
          if (RSMODE == 3) { c = k / 9; const int rs = k - c * 9; r = rs / 3; s = rs - r * 3; }
          else if (RSMODE == 7) { c = k / 49; const int rs = k - c * 49; r = rs / 7; s = rs - r * 7; }
          else { const int RS = a.R * a.S; c = div_magic(k, RS, a.magic_rs); const int rs = k - c * RS; r = div_magic(rs, a.S, a.magic_s); s = rs - r * a.S; }
          const int ih = ih0 + r, iw = iw0 + s;
          if (b_col_ok && k < a.Kdim && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W)
            v = Xg[b_pix_off + ((int64_t)c * a.H + ih) * a.W + iw];
        }
        rb[j] = v;
      }
    }
  };

  auto store_tiles = [&](int buf) {
    if (!A_MC) {
#pragma unroll
      for (int i = 0; i < A_PER4; i++) {
        const int idx = tid + i * NT, row = idx >> 2, kq = idx & 3;
        As[buf][kq * 4 + 0][row] = ra[i].x;
        As[buf][kq * 4 + 1][row] = ra[i].y;
        As[buf][kq * 4 + 2][row] = ra[i].z;
        As[buf][kq * 4 + 3][row] = ra[i].w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < AM_PER; i++) {
        const int idx = tid + i * NT, mm = idx % BM, kk = idx / BM;
        As[buf][kk][mm] = ram[i];
      }
    }
    if (B_KC) {
#pragma unroll
      for (int i = 0; i < B_PER4; i++) {
        const int idx = tid + i * NT, row = idx >> 2, kq = idx & 3;
        Bs[buf][kq * 4 + 0][row] = rb4[i].x;
        Bs[buf][kq * 4 + 1][row] = rb4[i].y;
        Bs[buf][kq * 4 + 2][row] = rb4[i].z;
        Bs[buf][kq * 4 + 3][row] = rb4[i].w;
      }
    } else {
#pragma unroll
      for (int j = 0; j < B_PER; j++) Bs[buf][bkk0 + j * B_ROWS_PER_PASS][bcol] = rb[j];
    }
  };
  (void)AM_ROWS_PER_PASS;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const int nk = (a.Kdim + BK - 1) / BK;
  load_tiles(0);
  store_tiles(0);
  __syncthreads();

  const int lrow = lane >> 5, lcol = lane & 31;
  for (int kt = 0; kt < nk; kt++) {
    const int buf = kt & 1;
    if (kt + 1 < nk) load_tiles((kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < BK; ks += 2) {
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
    if (kt + 1 < nk) store_tiles(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: accumulator register r of lane l is
  //      D[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 block --------------
  // Bias and residual values are read in batches from clamped addresses and
  // only the stores are predicated: a load inside a per-row branch would cost
  // a memory round trip per row.
  float *__restrict__ Yg = a.Y + (int64_t)z * a.y_z_stride;
  const int PQ = a.P * a.Q;
  float bias_r[TM][16];
  if (a.bias) {
    const float *__restrict__ biasg = a.bias + (int64_t)z * a.bias_z_stride;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) bias_r[i][r] = biasg[min(m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * lrow + (r & 3), a.M - 1)];
  } else {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) bias_r[i][r] = 0.f;
  }
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int col = n0 + wn0 + j * 32 + lcol;
    const bool col_ok = col < a.Ncols;
    const int colc = col_ok ? col : 0;
    const int img = colc / PQ, pq = colc - img * PQ;
    const int64_t ycol = (int64_t)img * a.y_img_stride + pq;
    const float bias_c = load_bias_col(a, colc);
#pragma unroll
    for (int i = 0; i < TM; i++) {
      float res_r[16];
      if (a.Cin) {
        const float *__restrict__ Cg = a.Cin + (int64_t)z * a.c_z_stride;
#pragma unroll
        for (int r = 0; r < 16; r++)
          res_r[r] = Cg[ycol + (int64_t)min(m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * lrow + (r & 3), a.M - 1) * a.c_row_stride];
      } else {
#pragma unroll
        for (int r = 0; r < 16; r++) res_r[r] = 0.f;
      }
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int m = m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * lrow + (r & 3);
        float v = a.alpha * acc[i][j][r] + bias_r[i][r] + bias_c;
        if (a.Cin) v += a.beta * res_r[r];
        v = apply_act(v, a.act, a.act_coef);
        if (col_ok && m < a.M) Yg[ycol + (int64_t)m * a.y_row_stride] = v;
      }
    }
  }
}

template <int BM, int BN, int WM, int WN>
static bool launch_tile(const dnnrtContext *ctx, const IgemmArgs &a, int rsmode, int layout) {
  const int tiles = (int)(ceil_div(a.M, BM) * ceil_div(a.Ncols, BN));
  dim3 grid(tiles, 1, a.Z), block(64 * WM * WN);
#define LAUNCH(RS, LAY)                                                        \
  hipLaunchKernelGGL((igemm_f32_kernel<BM, BN, WM, WN, RS, LAY>), grid, block, 0, ctx->stream, a)
  if (layout == 0) {
    switch (rsmode) {
      case 1: LAUNCH(1, 0); break;
      case 3: LAUNCH(3, 0); break;
      case 7: LAUNCH(7, 0); break;
      default: LAUNCH(0, 0); break;
    }
  } else if (layout == 1) LAUNCH(1, 1);
  else if (layout == 2) {  // m-contiguous A: transposed left matrix, or filters stored C,R,S,K
    switch (rsmode) {
      case 1: LAUNCH(1, 2); break;
      case 3: LAUNCH(3, 2); break;
      case 7: LAUNCH(7, 2); break;
      default: LAUNCH(0, 2); break;
    }
  } else LAUNCH(1, 3);
#undef LAUNCH
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("igemm_f32: launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

bool launch_igemm_f32(const dnnrtContext *ctx, const IgemmArgs &args) {
  IgemmArgs a = args;
  a.magic_rs = magic_of(a.R * a.S > 0 ? a.R * a.S : 1);
  a.magic_s = magic_of(a.S > 0 ? a.S : 1);
  if (a.M <= 0 || a.Ncols <= 0 || a.Kdim <= 0 || a.Z <= 0) { set_error("igemm_f32: empty problem"); return false; }
  if (a.Z > 65535) { set_error("igemm_f32: more than 65535 groups/batches"); return false; }
  int rsmode = 0;
  if (a.R == 1 && a.S == 1 && a.ph == 0 && a.pw == 0) rsmode = 1;
  else if (a.R == 3 && a.S == 3) rsmode = 3;
  else if (a.R == 7 && a.S == 7) rsmode = 7;
  const int layout = (a.b_kcontig ? 1 : 0) | (a.a_mcontig ? 2 : 0);
  if ((layout & 1) && rsmode != 1) { set_error("igemm_f32: a k-contiguous right operand needs a 1x1 geometry"); return false; }

  if (rsmode == 3) {  // the 3x3 specialisation takes the problems the tiles below would get
    bool launched = false;
    if (!launch_conv3x3_f32_tiled(ctx, a, layout, launched)) return false;
    if (launched) return true;
  }
  // Largest tile that still gives every CU a workgroup; small problems fall
  // through to the one-wave 32x32 tile.
  const int64_t want = ctx->num_cu;
  auto wgs = [&](int bm, int bn) { return ceil_div(a.M, bm) * ceil_div(a.Ncols, bn) * a.Z; };
  if (wgs(128, 128) >= want) return launch_tile<128, 128, 2, 2>(ctx, a, rsmode, layout);
  if (wgs(64, 64) >= want) return launch_tile<64, 64, 2, 2>(ctx, a, rsmode, layout);
  // Too small to fill the chip with LDS-staged tiles: latency-bound territory.
  return launch_igemm_f32_direct(ctx, a, rsmode, layout);
}

}  // namespace dnnrt
