// fp32 implicit GEMM for SMALL problems (batch-1 convolutions, short matrix
// products): latency, not bandwidth, bounds them, so the kernel trades data
// reuse for parallelism.
//
// A workgroup owns one 32x32 tile of D and is made of KS wavefronts that split
// the reduction range between them (split-K inside the workgroup: no
// workspace, no atomics).  Each wavefront streams its slice of both operands
// straight from global memory into MFMA operand registers -- no LDS staging,
// no barrier in the loop -- eight k per iteration:
//   lane l: row/column l % 32, k-offset 4 * (l / 32) .. +3
//   A: one 128-bit load along k of its filter row
//   B: four 32-bit loads, each coalesced over 32 consecutive output pixels
// which feeds four v_mfma_f32_32x32x2f32 (MFMA j pairs k0+j from the lower
// half-wave with k0+4+j from the upper one; any pairing is valid as long as A
// and B agree).  Partial tiles meet in LDS once, at the end; wavefront 0 adds
// bias / residual, applies the activation and stores.
#include "igemm_f32.h"

namespace dnnrt {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// VEC: k-contiguous operands (A unless transposed, B when transposed) are read as aligned float4.
template <int RSMODE, int LAYOUT, int KS, bool VEC>
__global__ __launch_bounds__(64 * KS) void igemm_f32_direct_kernel(const IgemmArgs a, const int k_per_wave) {
  constexpr bool B_KC = (LAYOUT & 1) != 0, A_MC = (LAYOUT & 2) != 0;
  __shared__ float red[KS > 1 ? KS - 1 : 1][16][64];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, half = lane >> 5;
  const int tiles_n = (a.Ncols + 31) / 32;
  const int tile_m = blockIdx.x / tiles_n, tile_n = blockIdx.x - tile_m * tiles_n;
  const int m0 = tile_m * 32, n0 = tile_n * 32;
  const int z = blockIdx.z;
  const float *__restrict__ Ag = a.A + (int64_t)z * a.a_z_stride;
  const float *__restrict__ Xg = a.X + (int64_t)z * a.x_z_stride;

  const int m = m0 + l32;
  const bool m_ok = m < a.M;
  const int col = n0 + l32;
  const bool col_ok = col < a.Ncols;
  const int PQ = a.P * a.Q, HW = a.H * a.W;
  int ih0 = 0, iw0 = 0;
  int64_t pix_off = 0;
  if (!B_KC) {
    const int img = col_ok ? col / PQ : 0;
    const int pq = col_ok ? col - img * PQ : 0;
    const int p = pq / a.Q, q = pq - p * a.Q;
    ih0 = p * a.sh - a.ph;
    iw0 = q * a.sw - a.pw;
    pix_off = (int64_t)img * a.x_img_stride;
    if (RSMODE == 1) pix_off += (int64_t)ih0 * a.W + iw0;
  }

  const int kbeg = wave * k_per_wave;
  const int kend = min(a.Kdim, kbeg + k_per_wave);
  const int mc = m_ok ? m : 0;
  const float *__restrict__ arow = Ag + (int64_t)mc * a.Kdim;
  const float *__restrict__ brow = Xg + (int64_t)(col_ok ? col : 0) * a.Kdim;  // B_KC only

  // Bias of the lane's 16 rows and of its column, requested before the
  // reduction starts: the values are there when the epilogue wants them.
  // Register r holds row m0 + 4 * half + row_k(r).
  auto row_k = [](int r) { return 8 * (r >> 2) + (r & 3); };
  const int mrow0 = m0 + 4 * half;
  const int colc = col_ok ? col : 0;
  const float bias_c = load_bias_col(a, colc);
  float bias_r[16];
  if (a.bias) {
    const float *__restrict__ biasg = a.bias + (int64_t)z * a.bias_z_stride;
#pragma unroll
    for (int r = 0; r < 16; r++) bias_r[r] = biasg[min(mrow0 + row_k(r), a.M - 1)];
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++) bias_r[r] = 0.f;
  }

  // One iteration = eight k: per lane four values of A and four of B.  Every
  // load is unconditional, from an address clamped into the tensor; what must
  // not contribute (k past the wavefront's slice, padding, columns past the
  // end) is zeroed on the B side when it is used.  Rows past the end of A are
  // read from row 0 and never stored.  With no load under a branch the
  // compiler counts the outstanding loads exactly, and a ring of DEPTH
  // iterations keeps several memory round trips in flight.
  constexpr int DEPTH = 4;
  struct It { float av[4], bv[4]; unsigned bm[4]; };
  auto load_it = [&](int k0, It &t) {
    const int ka = k0 + 4 * half;
    // ---- A ----
    if (!A_MC && VEC) {  // Kdim is a multiple of 4 then
      const float4 v = *reinterpret_cast<const float4 *>(arow + min(ka, a.Kdim - 4));
      t.av[0] = v.x; t.av[1] = v.y; t.av[2] = v.z; t.av[3] = v.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int kc = min(ka + j, a.Kdim - 1);
        t.av[j] = A_MC ? Ag[(int64_t)kc * a.a_ld + mc] : arow[kc];
      }
    }
    // ---- B ----
    if (B_KC && VEC) {
      const float4 v = *reinterpret_cast<const float4 *>(brow + min(ka, a.Kdim - 4));
      t.bv[0] = v.x; t.bv[1] = v.y; t.bv[2] = v.z; t.bv[3] = v.w;
#pragma unroll
      for (int j = 0; j < 4; j++) t.bm[j] = (col_ok && ka + j < kend) ? 0xffffffffu : 0u;
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int k = ka + j, kc = min(k, a.Kdim - 1);
        bool ok = col_ok && k < kend;
        if (B_KC) {
          t.bv[j] = brow[kc];
        } else if (RSMODE == 1) {
          t.bv[j] = Xg[pix_off + (int64_t)kc * HW];
        } else {
          int c, r, s;
          if (RSMODE == 3) { c = kc / 9; const int rs = kc - c * 9; r = rs / 3; s = rs - r * 3; }
          else if (RSMODE == 7) { c = kc / 49; const int rs = kc - c * 49; r = rs / 7; s = rs - r * 7; }
          else { const int RS = a.R * a.S; c = div_magic(kc, RS, a.magic_rs); const int rs = kc - c * RS; r = div_magic(rs, a.S, a.magic_s); s = rs - r * a.S; }
          const int ih = ih0 + r, iw = iw0 + s;
          ok = ok && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
          const int64_t off = ok ? ((int64_t)c * a.H + ih) * a.W + iw : 0;
          t.bv[j] = Xg[pix_off + off];
        }
        t.bm[j] = ok ? 0xffffffffu : 0u;
      }
    }
  };

  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  auto mfma_it = [&](const It &t) {
#pragma unroll
    for (int j = 0; j < 4; j++)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(t.av[j], __uint_as_float(__float_as_uint(t.bv[j]) & t.bm[j]), acc, 0, 0, 0);
  };
  const int niter = kend > kbeg ? (kend - kbeg + 7) >> 3 : 0;
  It t0, t1, t2, t3;  // named, not an array: they must stay in registers
  load_it(kbeg, t0); load_it(kbeg + 8, t1); load_it(kbeg + 16, t2); load_it(kbeg + 24, t3);
  // Iteration i lives in slot i % DEPTH and is refilled with iteration
  // i + DEPTH: whole groups that need every refill run without a branch, the
  // last DEPTH iterations refill nothing, the group in between asks per slot.
  int i0 = 0;
  for (; i0 + 2 * DEPTH <= niter; i0 += DEPTH) {
    mfma_it(t0); load_it(kbeg + 8 * (i0 + DEPTH), t0);
    mfma_it(t1); load_it(kbeg + 8 * (i0 + 1 + DEPTH), t1);
    mfma_it(t2); load_it(kbeg + 8 * (i0 + 2 + DEPTH), t2);
    mfma_it(t3); load_it(kbeg + 8 * (i0 + 3 + DEPTH), t3);
  }
  if (i0 < niter) { mfma_it(t0); if (i0 + DEPTH < niter) load_it(kbeg + 8 * (i0 + DEPTH), t0); }
  if (i0 + 1 < niter) { mfma_it(t1); if (i0 + 1 + DEPTH < niter) load_it(kbeg + 8 * (i0 + 1 + DEPTH), t1); }
  if (i0 + 2 < niter) { mfma_it(t2); if (i0 + 2 + DEPTH < niter) load_it(kbeg + 8 * (i0 + 2 + DEPTH), t2); }
  if (i0 + 3 < niter) { mfma_it(t3); if (i0 + 3 + DEPTH < niter) load_it(kbeg + 8 * (i0 + 3 + DEPTH), t3); }
  i0 += DEPTH;
  if (i0 < niter) mfma_it(t0);
  if (i0 + 1 < niter) mfma_it(t1);
  if (i0 + 2 < niter) mfma_it(t2);

  // the residual tensor's 16 values, requested before the partial tiles meet
  const int img = colc / PQ, pq = colc - img * PQ;
  const int64_t ycol = (int64_t)img * a.y_img_stride + pq;
  float res_r[16];
  if (a.Cin && wave == 0) {
    const float *__restrict__ Cg = a.Cin + (int64_t)z * a.c_z_stride;
#pragma unroll
    for (int r = 0; r < 16; r++) res_r[r] = Cg[ycol + (int64_t)min(mrow0 + row_k(r), a.M - 1) * a.c_row_stride];
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++) res_r[r] = 0.f;
  }

  // ---- combine the KS partial tiles ----
  if (KS > 1) {
    if (wave > 0) {
#pragma unroll
      for (int r = 0; r < 16; r++) red[wave - 1][r][lane] = acc[r];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < KS - 1; w++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[r] += red[w][r][lane];
  }

  // ---- epilogue: register r of lane l is D[8*(r/4) + 4*(l/32) + r%4][l%32];
  // a row's address is one per-lane base plus a uniform offset ----
  if (!col_ok) return;
  float *__restrict__ y0 = a.Y + (int64_t)z * a.y_z_stride + ycol + (int64_t)mrow0 * a.y_row_stride;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    if (mrow0 + row_k(r) >= a.M) continue;
    float v = a.alpha * acc[r] + bias_r[r] + bias_c;
    if (a.Cin) v += a.beta * res_r[r];
    y0[(int64_t)row_k(r) * a.y_row_stride] = apply_act(v, a.act, a.act_coef);
  }
}

template <int KS>
static void launch_ks(const dnnrtContext *ctx, const IgemmArgs &a, int rsmode, int layout, int tiles) {
  const int k_per_wave = (int)(ceil_div(ceil_div(a.Kdim, KS), 8) * 8);
  dim3 grid(tiles, 1, a.Z), block(64 * KS);
  // float4 reads only if every k-contiguous operand allows them
  const bool vec = (((layout & 2) != 0) || a.a_vec4) && (((layout & 1) == 0) || a.b_vec4) && (layout != 2);
#define LAUNCH(RS, LAY)                                                                         \
  do {                                                                                          \
    if (vec) hipLaunchKernelGGL((igemm_f32_direct_kernel<RS, LAY, KS, true>), grid, block, 0, ctx->stream, a, k_per_wave);  \
    else hipLaunchKernelGGL((igemm_f32_direct_kernel<RS, LAY, KS, false>), grid, block, 0, ctx->stream, a, k_per_wave);     \
  } while (0)
  if (layout == 0) {
    switch (rsmode) {
      case 1: LAUNCH(1, 0); break;
      case 3: LAUNCH(3, 0); break;
      case 7: LAUNCH(7, 0); break;
      default: LAUNCH(0, 0); break;
    }
  } else if (layout == 1) LAUNCH(1, 1);
  else if (layout == 2) {
    switch (rsmode) {
      case 1: LAUNCH(1, 2); break;
      case 3: LAUNCH(3, 2); break;
      case 7: LAUNCH(7, 2); break;
      default: LAUNCH(0, 2); break;
    }
  } else LAUNCH(1, 3);
#undef LAUNCH
}

bool launch_igemm_f32_direct(const dnnrtContext *ctx, const IgemmArgs &a, int rsmode, int layout) {
  bool launched = false;
  if (!launch_igemm_f32_small(ctx, a, rsmode, layout, launched)) return false;
  if (launched) return true;
  const int64_t tiles64 = ceil_div(a.M, 32) * ceil_div(a.Ncols, 32);
  if (tiles64 > INT32_MAX) { set_error("igemm_f32: too many tiles"); return false; }
  const int tiles = (int)tiles64;
  // Enough wavefronts to give every SIMD a few (4 SIMDs per CU), as long as
  // each keeps a reduction slice worth starting a wavefront for.
  const int64_t want_waves = (int64_t)ctx->num_cu * 8;
  int ks = 1;
  while (ks < 8 && (int64_t)tiles * a.Z * ks < want_waves && ceil_div(a.Kdim, ks * 2) >= 32) ks *= 2;
  switch (ks) {
    case 1: launch_ks<1>(ctx, a, rsmode, layout, tiles); break;
    case 2: launch_ks<2>(ctx, a, rsmode, layout, tiles); break;
    case 4: launch_ks<4>(ctx, a, rsmode, layout, tiles); break;
    default: launch_ks<8>(ctx, a, rsmode, layout, tiles); break;
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("igemm_f32(direct): launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

}  // namespace dnnrt
