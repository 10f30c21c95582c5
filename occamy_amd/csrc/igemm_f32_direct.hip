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

template <int RSMODE, int LAYOUT, int KS>
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
  const float *__restrict__ arow = Ag + (int64_t)(m_ok ? m : 0) * a.Kdim;
  const float *__restrict__ brow = Xg + (int64_t)(col_ok ? col : 0) * a.Kdim;  // B_KC only

  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;


  for (int k0 = kbeg; k0 < kend; k0 += 8) {
    const int ka = k0 + 4 * half;
    float av[4], bv[4];
    // ---- A ----
    if (!A_MC) {
      if (a.a_vec4) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (m_ok && ka < kend) v = *reinterpret_cast<const float4 *>(arow + ka);
        av[0] = v.x; av[1] = v.y; av[2] = v.z; av[3] = v.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; j++) av[j] = (m_ok && ka + j < kend) ? arow[ka + j] : 0.f;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) av[j] = (m_ok && ka + j < kend) ? Ag[(int64_t)(ka + j) * a.a_ld + m] : 0.f;
    }
    // ---- B ----
    if (B_KC) {
      if (a.b_vec4) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (col_ok && ka < kend) v = *reinterpret_cast<const float4 *>(brow + ka);
        bv[0] = v.x; bv[1] = v.y; bv[2] = v.z; bv[3] = v.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; j++) bv[j] = (col_ok && ka + j < kend) ? brow[ka + j] : 0.f;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int k = ka + j;
        float v = 0.f;
        if (RSMODE == 1) {
          if (col_ok && k < kend) v = Xg[pix_off + (int64_t)k * HW];
        } else {
          int c, r, s;
          if (RSMODE == 3) { c = k / 9; const int rs = k - c * 9; r = rs / 3; s = rs - r * 3; }
          else if (RSMODE == 7) { c = k / 49; const int rs = k - c * 49; r = rs / 7; s = rs - r * 7; }
          else { const int RS = a.R * a.S; c = k / RS; const int rs = k - c * RS; r = rs / a.S; s = rs - r * a.S; }
          const int ih = ih0 + r, iw = iw0 + s;
          if (col_ok && k < kend && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W)
            v = Xg[pix_off + ((int64_t)c * a.H + ih) * a.W + iw];
        }
        bv[j] = v;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; j++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j], bv[j], acc, 0, 0, 0);
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

  // ---- epilogue: register r of lane l is D[8*(r/4) + 4*(l/32) + r%4][l%32] ----
  // Bias and residual values are read in one batch from clamped addresses and
  // only the stores are predicated: a load inside a per-row branch would cost
  // a memory round trip per row.
  float *__restrict__ Yg = a.Y + (int64_t)z * a.y_z_stride;
  const int colc = col_ok ? col : 0;
  const int img = colc / PQ, pq = colc - img * PQ;
  const int64_t ycol = (int64_t)img * a.y_img_stride + pq;
  float bias_r[16], res_r[16];
  const float bias_c = load_bias_col(a, colc);
  if (a.bias) {
    const float *__restrict__ biasg = a.bias + (int64_t)z * a.bias_z_stride;
#pragma unroll
    for (int r = 0; r < 16; r++) bias_r[r] = biasg[min(m0 + 8 * (r >> 2) + 4 * half + (r & 3), a.M - 1)];
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++) bias_r[r] = 0.f;
  }
  if (a.Cin) {
    const float *__restrict__ Cg = a.Cin + (int64_t)z * a.c_z_stride;
#pragma unroll
    for (int r = 0; r < 16; r++) res_r[r] = Cg[ycol + (int64_t)min(m0 + 8 * (r >> 2) + 4 * half + (r & 3), a.M - 1) * a.c_row_stride];
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++) res_r[r] = 0.f;
  }
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const int mm = m0 + 8 * (r >> 2) + 4 * half + (r & 3);
    float v = a.alpha * acc[r] + bias_r[r] + bias_c;
    if (a.Cin) v += a.beta * res_r[r];
    v = apply_act(v, a.act, a.act_coef);
    if (col_ok && mm < a.M) Yg[ycol + (int64_t)mm * a.y_row_stride] = v;
  }
}

template <int KS>
static void launch_ks(const dnnrtContext *ctx, const IgemmArgs &a, int rsmode, int layout, int tiles) {
  const int k_per_wave = (int)(ceil_div(ceil_div(a.Kdim, KS), 8) * 8);
  dim3 grid(tiles, 1, a.Z), block(64 * KS);
#define LAUNCH(RS, LAY)                                                                         \
  hipLaunchKernelGGL((igemm_f32_direct_kernel<RS, LAY, KS>), grid, block, 0, ctx->stream, a, k_per_wave)
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
