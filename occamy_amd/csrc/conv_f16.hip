// fp16 convolution with fp32 accumulation on v_mfma_f32_32x32x16_f16.
//
// GEMM view: D[k_out, pixel] = sum_k Wt[k_out, k] * Xcol[k, pixel].  The MFMA
// wants, per lane, 8 CONSECUTIVE k of one row (A) / one column (B), so both
// operands should be k-contiguous in memory.  Channels-last activations make
// the im2col operand so: with k ordered (r, s, c) a run of 8 k is 8 adjacent
// channels of one input pixel, and the filter is stored K,R,S,C to match.
//
// Fast kernel (NHWC in, NHWC out, C % 32 == 0, K % 8 == 0, group 1):
//   tile BM k_out x BN pixels, BK = 32; per step every thread moves 16-byte
//   chunks global -> registers -> LDS (rows padded to 80 bytes, which makes
//   the ds_read_b128 operand fetches conflict-free); registers prefetch the
//   next step while the MFMAs of the current one run; LDS is double-buffered,
//   one barrier per step.  A BK step lies inside one (r, s) tap, so the tap
//   and its bounds check are wave-uniform.  The epilogue adds bias, applies the
//   activation, converts to fp16 and goes through LDS once more so that global
//   stores are full 16-byte chunks of a pixel's channel vector.
//
// Generic kernel (any C, NCHW or NHWC on either side): same MFMA structure
// with element-wise gathers; it serves the first convolution of a network
// (3 input channels, NCHW from the host) and odd shapes.
#include "conv_f16.h"

namespace dnnrt {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// 16-byte load through an explicitly GLOBAL pointer.  Left to itself the
// compiler emits flat loads here, which count against the LDS counter as well
// and so serialise the prefetch behind every LDS operand fetch.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const u32x4 *global_u32x4_ptr;
__device__ __forceinline__ u32x4 load_global_16(const void *p) { return *(global_u32x4_ptr)p; }

constexpr int BK16 = 32;      // k per step
constexpr int LDS_ROW = 40;   // halfs per LDS row: 32 + 8 pad (80 bytes)

template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(256) void conv_f16_nhwc_kernel(const ConvF16Args a) {
  static_assert(WM * WN == 4, "four wavefronts");
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int A_CH = BM * 4 / 256, B_CH = BN * 4 / 256;  // 16-byte chunks per thread per step
  static_assert(A_CH >= 1 && B_CH >= 1, "tile too small");
  constexpr int STAGE = (BM + BN) * LDS_ROW;               // halfs per pipeline stage
  constexpr int CROW = BM + 8;                             // halfs per row of the output staging tile
  constexpr int SMEM = (2 * STAGE > BN * CROW) ? 2 * STAGE : BN * CROW;
  __shared__ __attribute__((aligned(16))) _Float16 smem[SMEM];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);

  const int tiles_m = (a.K + BM - 1) / BM;
  const int tile_n = blockIdx.x / tiles_m, tile_m = blockIdx.x - tile_n * tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int NPQ = a.N * a.P * a.Q, PQ = a.P * a.Q;
  const int CRS = a.C * a.R * a.S;

  const _Float16 *__restrict__ Xg = reinterpret_cast<const _Float16 *>(a.X);
  const _Float16 *__restrict__ Wg = reinterpret_cast<const _Float16 *>(a.Wt);

  // ---- loader constants ------------------------------------------------
  // A (filters): chunk id -> (row, 16-byte chunk of the 64-byte k slice)
  // element OFFSETS, not pointers, are kept across the loop: the address is
  // formed from the kernel-argument base at each load, which keeps the loads
  // in the global address space (flat loads would tie them to the LDS counter)
  int64_t a_off[A_CH];
  bool a_ok[A_CH];
#pragma unroll
  for (int i = 0; i < A_CH; i++) {
    const int id = tid + i * 256, row = id >> 2, ch = id & 3;
    const int k_out = m0 + row;
    a_ok[i] = k_out < a.K;
    a_off[i] = (int64_t)(a_ok[i] ? k_out : 0) * CRS + ch * 8;
  }
  // B (im2col): each chunk belongs to one output pixel
  int b_ih0[B_CH], b_iw0[B_CH];
  int64_t b_off[B_CH];
  bool b_ok[B_CH];
#pragma unroll
  for (int i = 0; i < B_CH; i++) {
    const int id = tid + i * 256, row = id >> 2, ch = id & 3;
    const int pix = n0 + row;
    b_ok[i] = pix < NPQ;
    const int n = b_ok[i] ? pix / PQ : 0;
    const int pq = b_ok[i] ? pix - n * PQ : 0;
    const int p = pq / a.Q, q = pq - p * a.Q;
    b_ih0[i] = p * a.sh - a.ph;
    b_iw0[i] = q * a.sw - a.pw;
    b_off[i] = (int64_t)n * a.H * a.W * a.C + ch * 8;
  }

  // Register ring: the loads of DEPTH future steps are in flight while the
  // MFMAs of the current one run (a step is ~0.1 us of MFMA work, a global
  // load takes several times that).  Slots are indexed with compile-time
  // constants: the step loop is unrolled DEPTH times.
  constexpr int DEPTH = 4;
  u32x4 ra[DEPTH][A_CH], rb[DEPTH][B_CH];
  const u32x4 zero4 = {0u, 0u, 0u, 0u};

  const int steps_c = a.C / BK16, nk = a.R * a.S * steps_c;
  int lr = 0, ls = 0, lc0 = 0, lstep = 0;  // cursor of the next step to load

  auto load_step = [&](u32x4 (&qa)[A_CH], u32x4 (&qb)[B_CH]) {
    if (lstep < nk) {
      const int kk = (lr * a.S + ls) * a.C + lc0;
#pragma unroll
      for (int i = 0; i < A_CH; i++)
        qa[i] = a_ok[i] ? load_global_16(Wg + (a_off[i] + kk)) : zero4;
#pragma unroll
      for (int i = 0; i < B_CH; i++) {
        const int ih = b_ih0[i] + lr, iw = b_iw0[i] + ls;
        const bool ok = b_ok[i] && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
        qb[i] = ok ? load_global_16(Xg + (b_off[i] + ((int64_t)ih * a.W + iw) * a.C + lc0)) : zero4;
      }
      lc0 += BK16;
      if (lc0 == a.C) { lc0 = 0; if (++ls == a.S) { ls = 0; ++lr; } }
    }
    lstep++;
  };
  auto store_step = [&](int buf, const u32x4 (&qa)[A_CH], const u32x4 (&qb)[B_CH]) {
    _Float16 *As = smem + buf * STAGE, *Bs = As + BM * LDS_ROW;
#pragma unroll
    for (int i = 0; i < A_CH; i++) {
      const int id = tid + i * 256, row = id >> 2, ch = id & 3;
      *reinterpret_cast<u32x4 *>(As + row * LDS_ROW + ch * 8) = qa[i];
    }
#pragma unroll
    for (int i = 0; i < B_CH; i++) {
      const int id = tid + i * 256, row = id >> 2, ch = id & 3;
      *reinterpret_cast<u32x4 *>(Bs + row * LDS_ROW + ch * 8) = qb[i];
    }
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // prologue: step 0 into LDS, steps 1 .. DEPTH-1 in flight in slots 1 .. DEPTH-1
  load_step(ra[0], rb[0]);
#pragma unroll
  for (int d = 1; d < DEPTH; d++) load_step(ra[d], rb[d]);
  store_step(0, ra[0], rb[0]);
  __syncthreads();

  for (int kt0 = 0; kt0 < nk; kt0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; u++) {
      const int kt = kt0 + u;
      if (kt < nk) {
        const int buf = kt & 1;
        // slot u held step kt (already in LDS): reuse it for step kt + DEPTH
        load_step(ra[u], rb[u]);
        const _Float16 *As = smem + buf * STAGE, *Bs = As + BM * LDS_ROW;
#pragma unroll
        for (int ks = 0; ks < BK16; ks += 16) {
          half8 av[TM], bv[TN];
#pragma unroll
          for (int i = 0; i < TM; i++)
            av[i] = *reinterpret_cast<const half8 *>(As + (wm0 + i * 32 + l32) * LDS_ROW + ks + half * 8);
#pragma unroll
          for (int j = 0; j < TN; j++)
            bv[j] = *reinterpret_cast<const half8 *>(Bs + (wn0 + j * 32 + l32) * LDS_ROW + ks + half * 8);
#pragma unroll
          for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[i], bv[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) store_step(buf ^ 1, ra[(u + 1) % DEPTH], rb[(u + 1) % DEPTH]);
        __syncthreads();
      }
    }
  }

  // ---- epilogue: bias, activation, fp16, transpose through LDS ------------
  // register r of lane l in block (i, j): k_out = 8*(r/4) + 4*(l/32) + r%4,
  // pixel = l%32 -> four consecutive k_out per register group.
  const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
  const _Float16 *__restrict__ Zg = reinterpret_cast<const _Float16 *>(a.Z);
  const bool relu_now = a.act == DNNRT_ACT_RELU && !Zg;  // with a residual the activation comes after the sum
  _Float16 *Cs = smem;  // [BN pixels][CROW]
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int kl = wm0 + i * 32 + 8 * g + 4 * half;  // k_out within the tile
        half4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          float v = acc[i][j][4 * g + e];
          const int k_out = m0 + kl + e;
          if (biasg && k_out < a.K) v += (float)biasg[k_out];
          if (relu_now) v = v < 0.f ? 0.f : v;
          o[e] = (_Float16)v;
        }
        *reinterpret_cast<half4 *>(Cs + (wn0 + j * 32 + l32) * CROW + kl) = o;
      }
  __syncthreads();
  _Float16 *__restrict__ Yg = reinterpret_cast<_Float16 *>(a.Y);
  constexpr int CH_PER_ROW = BM / 8;
#pragma unroll
  for (int id = tid; id < BN * CH_PER_ROW; id += 256) {
    const int row = id / CH_PER_ROW, ch = id - row * CH_PER_ROW;
    const int pix = n0 + row, k_out = m0 + ch * 8;
    if (pix < NPQ && k_out < a.K) {
      half8 o = *reinterpret_cast<const half8 *>(Cs + row * CROW + ch * 8);
      if (Zg) {
        // conv + bias was rounded to fp16 above, as a separate convolution
        // would have stored it; the residual sum follows in fp32
        const half8 zv = *reinterpret_cast<const half8 *>(Zg + (int64_t)pix * a.K + k_out);
#pragma unroll
        for (int e = 0; e < 8; e++) {
          float v = (float)o[e] + (float)zv[e];
          if (a.act == DNNRT_ACT_RELU) v = v < 0.f ? 0.f : v;
          o[e] = (_Float16)v;
        }
      }
      *reinterpret_cast<half8 *>(Yg + (int64_t)pix * a.K + k_out) = o;
    }
  }
}

// ---- generic kernel ---------------------------------------------------------
// 64 k_out x 64 pixels, four wavefronts of 32x32 each, BK = 32, single LDS
// stage, element-wise gathers.  Layout flags are runtime values.
__global__ __launch_bounds__(256) void conv_f16_generic_kernel(const ConvF16Args a, const int in_nchw,
                                                               const int out_nhwc, const int w_krsc) {
  __shared__ __attribute__((aligned(16))) _Float16 As[64 * LDS_ROW];
  __shared__ __attribute__((aligned(16))) _Float16 Bs[64 * LDS_ROW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm0 = (wave >> 1) * 32, wn0 = (wave & 1) * 32;
  const int g = blockIdx.z, Kg = a.K / a.group;
  const int tiles_m = (Kg + 63) / 64;
  const int tile_n = blockIdx.x / tiles_m, tile_m = blockIdx.x - tile_n * tiles_m;
  const int m0 = tile_m * 64, n0 = tile_n * 64;
  const int NPQ = a.N * a.P * a.Q, PQ = a.P * a.Q, RS = a.R * a.S;
  const int CRS = a.Cg * RS;
  const _Float16 *__restrict__ Xg = reinterpret_cast<const _Float16 *>(a.X);
  const _Float16 *__restrict__ Wg = reinterpret_cast<const _Float16 *>(a.Wt);

  // each thread fills 8 elements of each tile per step: row = tid / 4, k = (tid % 4) * 8 + e
  const int lrow = tid >> 2, lk0 = (tid & 3) * 8;
  const int k_out = g * Kg + m0 + lrow;
  const bool a_row_ok = m0 + lrow < Kg;
  const int pix = n0 + lrow;
  const bool b_row_ok = pix < NPQ;
  const int n = b_row_ok ? pix / PQ : 0;
  const int pq = b_row_ok ? pix - n * PQ : 0;
  const int p = pq / a.Q, q = pq - p * a.Q;
  const int ih0 = p * a.sh - a.ph, iw0 = q * a.sw - a.pw;

  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;

  for (int k0 = 0; k0 < CRS; k0 += BK16) {
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int k = k0 + lk0 + e;
      _Float16 av = (_Float16)0.f, bv = (_Float16)0.f;
      if (k < CRS) {
        int c, r, s;
        if (w_krsc) { c = k % a.Cg; const int rs = k / a.Cg; r = rs / a.S; s = rs - r * a.S; }
        else { c = k / RS; const int rs = k - c * RS; r = rs / a.S; s = rs - r * a.S; }
        if (a_row_ok) av = Wg[(int64_t)k_out * CRS + k];  // k is the filter's own storage order
        const int ih = ih0 + r, iw = iw0 + s, cc = g * a.Cg + c;
        if (b_row_ok && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W)
          bv = in_nchw ? Xg[(((int64_t)n * a.C + cc) * a.H + ih) * a.W + iw]
                       : Xg[(((int64_t)n * a.H + ih) * a.W + iw) * a.C + cc];
      }
      As[lrow * LDS_ROW + lk0 + e] = av;
      Bs[lrow * LDS_ROW + lk0 + e] = bv;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < BK16; ks += 16) {
      const half8 av = *reinterpret_cast<const half8 *>(As + (wm0 + l32) * LDS_ROW + ks + half * 8);
      const half8 bv = *reinterpret_cast<const half8 *>(Bs + (wn0 + l32) * LDS_ROW + ks + half * 8);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, acc, 0, 0, 0);
    }
    __syncthreads();
  }

  const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
  const _Float16 *__restrict__ Zg = reinterpret_cast<const _Float16 *>(a.Z);
  _Float16 *__restrict__ Yg = reinterpret_cast<_Float16 *>(a.Y);
  const int opix = n0 + wn0 + l32;
  if (opix >= NPQ) return;
  const int on = opix / PQ, opq = opix - on * PQ;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const int ml = m0 + wm0 + 8 * (r >> 2) + 4 * half + (r & 3);
    if (ml >= Kg) continue;
    const int ko = g * Kg + ml;
    float v = acc[r];
    if (biasg) v += (float)biasg[ko];
    const int64_t off = out_nhwc ? (int64_t)opix * a.K + ko : ((int64_t)on * a.K + ko) * PQ + opq;
    if (Zg) v = (float)(_Float16)v + (float)Zg[off];
    if (a.act == DNNRT_ACT_RELU) v = v < 0.f ? 0.f : v;
    Yg[off] = (_Float16)v;
  }
}

bool launch_conv_f16(const dnnrtContext *ctx, const ConvF16Args &a) {
  const int64_t NPQ = (int64_t)a.N * a.P * a.Q;
  const bool fast = a.format == DNNRT_NHWC && a.group == 1 && a.C % 32 == 0 && a.K % 8 == 0 &&
                    aligned16(a.X) && aligned16(a.Wt) && aligned16(a.Y) && aligned16(a.Z);
  if (fast) {
    // Largest tile that still gives every CU two workgroups to overlap.
    const int64_t want = 2 * (int64_t)ctx->num_cu;
    auto tiles_of = [&](int bm, int bn) { return ceil_div(a.K, bm) * ceil_div(NPQ, bn); };
#define LAUNCH_FAST(BM_, BN_, WM_, WN_)                                                                    \
  do {                                                                                                     \
    const int64_t tiles = tiles_of(BM_, BN_);                                                              \
    if (tiles > INT32_MAX) { set_error("conv(fp16): too many tiles"); return false; }                      \
    hipLaunchKernelGGL((conv_f16_nhwc_kernel<BM_, BN_, WM_, WN_>), dim3((unsigned)tiles), dim3(256), 0,    \
                       ctx->stream, a);                                                                    \
  } while (0)
    if (a.K <= 64) {
      if (tiles_of(64, 128) >= want) LAUNCH_FAST(64, 128, 1, 4);
      else LAUNCH_FAST(64, 64, 2, 2);
    } else {
      if (tiles_of(128, 128) >= want) LAUNCH_FAST(128, 128, 2, 2);
      else if (tiles_of(128, 64) >= want) LAUNCH_FAST(128, 64, 2, 2);
      else LAUNCH_FAST(64, 64, 2, 2);
    }
#undef LAUNCH_FAST
  } else {
    const int Kg = a.K / a.group;
    const int64_t tiles = ceil_div(Kg, 64) * ceil_div(NPQ, 64);
    if (tiles > INT32_MAX || a.group > 65535) { set_error("conv(fp16): too many tiles"); return false; }
    const int in_nchw = a.format != DNNRT_NHWC, out_nhwc = a.format != DNNRT_NCHW;
    const int w_krsc = a.format != DNNRT_NCHW;  // channels-last programs store filters K,R,S,C
    hipLaunchKernelGGL(conv_f16_generic_kernel, dim3((unsigned)tiles, 1, (unsigned)a.group), dim3(256), 0, ctx->stream,
                       a, in_nchw, out_nhwc, w_krsc);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("conv(fp16): launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

}  // namespace dnnrt
