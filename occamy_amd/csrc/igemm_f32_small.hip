// Two specialisations of the small-problem fp32 implicit GEMM
// (igemm_f32_direct.hip) for the shapes that make up a batch-1 CNN or a short
// transformer: 3x3 convolutions and 1x1 convolutions / plain matrix products.
//
// Same decomposition -- one 32x32 tile of D per workgroup, KS wavefronts
// splitting the reduction, operands straight from global memory into MFMA
// registers -- but the per-element index arithmetic is gone (a wave64 VALU
// instruction costs 4 cycles, and ~30 of them per loaded element made the
// general kernel issue-bound):
//   3x3: a lane owns one output pixel; its nine tap offsets and nine validity
//        masks are computed once.  One iteration = 2 channels x 9 taps
//        (half-wave h takes channel c+h), i.e. nine MFMAs fed by nine
//        contiguous filter words and nine input words at base + tap_off[j].
//   1x1: the reduction index is the channel; addresses advance by a constant.
// All loads are unconditional (clamped addresses; what must not contribute is
// masked on the B side at the time of use), so the compiler can track the
// hardware load counter and the register ring keeps several iterations of
// loads in flight.  Offsets are 32-bit: the dispatcher only takes these
// kernels when every operand is below 2^31 elements.
#include "igemm_f32.h"

#include <type_traits>

namespace dnnrt {

typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float mask_f(float v, unsigned m) { return __uint_as_float(__float_as_uint(v) & m); }

// The 16 accumulator registers of a lane hold rows m0 + 8 * (r >> 2) + 4 * half + (r & 3)
// of output column n0 + l32.
__device__ __forceinline__ int acc_row(int m0, int half, int r) { return m0 + 8 * (r >> 2) + 4 * half + (r & 3); }
// ... that is, row m0 + 4 * half (the only part that differs between lanes) plus row_k(r), known at compile time:
// address arithmetic per row is then a uniform offset (scalar unit) added to one per-lane base.
__device__ __forceinline__ constexpr int row_k(int r) { return 8 * (r >> 2) + (r & 3); }

// Bias of the lane's 16 rows, requested at kernel start so that the values
// are there when the epilogue wants them (a load per row at that point costs
// a memory round trip each: the rows are handled under a divergent branch).
__device__ __forceinline__ void prefetch_bias(const IgemmArgs &a, int z, int m0, int half, float (&bias_r)[16]) {
  if (a.bias) {
    const float *__restrict__ biasg = a.bias + (int64_t)z * a.bias_z_stride;
    if (m0 + 32 <= a.M && (reinterpret_cast<uintptr_t>(biasg) & 15u) == 0) {
      // whole tile inside the matrix: the lane's rows are four runs of four, one 16-byte load each
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const float4 v = *reinterpret_cast<const float4 *>(biasg + m0 + 8 * g + 4 * half);
        bias_r[4 * g] = v.x; bias_r[4 * g + 1] = v.y; bias_r[4 * g + 2] = v.z; bias_r[4 * g + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; r++) bias_r[r] = biasg[min(acc_row(m0, half, r), a.M - 1)];
    }
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++) bias_r[r] = 0.f;
  }
}

// Sum the KS partial tiles in LDS, then bias / residual / activation / store by wavefront 0.
// The reduction may also be split over gridDim.y workgroups.  Each of them
// leaves its partial tile in `partials` and bumps the tile's arrival counter;
// whoever arrives last adds the partials up in split order -- the order of
// arrival does not matter, so the result is the same bits on every run -- and
// finishes the tile.  Nobody waits for anybody.  The last arriver puts the
// counter back to zero for the next kernel on the stream.
template <int KS, bool WIDE_FIXUP>
__device__ __forceinline__ void reduce_and_store(const IgemmArgs &a, floatx16 acc, const float (&bias_r)[16], float bias_c, float (*red)[16][64],
                                                 int wave, int lane, int m0, int img, int pq, bool col_ok, int z, unsigned tile,
                                                 float *partials, unsigned *counters) {
  const int half = lane >> 5;
  const bool full = m0 + 32 <= a.M;  // the whole tile lies inside the matrix (same for every lane)
  // the residual tensor's 16 values, requested before anything is waited for
  const int64_t ycol = (int64_t)img * a.y_img_stride + pq;
  float res_r[16];
  if (a.Cin) {
    if (wave == 0) {
      const float *__restrict__ Cg = a.Cin + (int64_t)z * a.c_z_stride;
      if (full) {
        const float *__restrict__ c0 = Cg + ycol + (int64_t)(m0 + 4 * half) * a.c_row_stride;
#pragma unroll
        for (int r = 0; r < 16; r++) res_r[r] = c0[(int64_t)row_k(r) * a.c_row_stride];
      } else {
#pragma unroll
        for (int r = 0; r < 16; r++) res_r[r] = Cg[ycol + (int64_t)min(acc_row(m0, half, r), a.M - 1) * a.c_row_stride];
      }
    }
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++) res_r[r] = 0.f;
  }
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
  const int splits = (int)gridDim.y;
  if (splits > 1) {
    float *mine = partials + ((size_t)tile * splits + blockIdx.y) * 1024;
#pragma unroll
    for (int r = 0; r < 16; r++) __hip_atomic_store(&mine[r * 64 + lane], acc[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The hand-over.  Every workgroup of a tile (1) writes its partial tile with device-scope atomic
    // stores, which go past the per-XCD L2 to the point where all XCDs agree, (2) waits until every one of
    // them is acknowledged (s_waitcnt 0: the counters of a wavefront reach zero only when its stores have been
    // written there), (3) adds one to the tile's arrival counter with a device-scope atomic, performed at
    // that same point.  Whoever reads splits - 1 knows that every other workgroup's step (2) is over, so its
    // device-scope atomic loads, issued after the counter's value has come back (the branch depends on it and
    // a wavefront issues in order), read the finished partial tiles.  Nobody waits for anybody: a workgroup
    // that is not last leaves.  What this rests on is the hardware's behaviour, stated above, not the
    // language's memory model, which would ask for a release on (3) and an acquire in the reader; on this
    // target a release at device scope also writes back every dirty line of the XCD's L2 (the previous
    // layer's output), which costs more than the split saves.  The signal fences keep the compiler, which
    // may reorder relaxed accesses to different addresses, from moving them across (2) and (3); they emit no
    // instruction.
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0) expcnt(0) lgkmcnt(0)
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    unsigned arrived = 0;
    if (lane == 0) arrived = __hip_atomic_fetch_add(&counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    if (arrived != (unsigned)splits - 1) return;
    // splits is a power of two >= 2: the partial tiles are requested four
    // (WIDE_FIXUP: eight) at a time, a memory round trip each time, and added in split order
    const float *all = partials + (size_t)tile * splits * 1024 + lane;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    auto part = [&](int y, float (&p)[16]) {
#pragma unroll
      for (int r = 0; r < 16; r++) p[r] = __hip_atomic_load(all + (size_t)y * 1024 + r * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    if (splits == 2) {
      float p0[16], p1[16];
      part(0, p0); part(1, p1);
#pragma unroll
      for (int r = 0; r < 16; r++) acc[r] = (acc[r] + p0[r]) + p1[r];
    } else if (splits == 4 || !WIDE_FIXUP) {
      for (int y = 0; y < splits; y += 4) {
        float p0[16], p1[16], p2[16], p3[16];
        part(y, p0); part(y + 1, p1); part(y + 2, p2); part(y + 3, p3);
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = (((acc[r] + p0[r]) + p1[r]) + p2[r]) + p3[r];
      }
    } else {  // the 3x3 kernel has the registers for it anyway
      for (int y = 0; y < splits; y += 8) {
        float p0[16], p1[16], p2[16], p3[16], p4[16], p5[16], p6[16], p7[16];
        part(y, p0); part(y + 1, p1); part(y + 2, p2); part(y + 3, p3);
        part(y + 4, p4); part(y + 5, p5); part(y + 6, p6); part(y + 7, p7);
#pragma unroll
        for (int r = 0; r < 16; r++)
          acc[r] = (((((((acc[r] + p0[r]) + p1[r]) + p2[r]) + p3[r]) + p4[r]) + p5[r]) + p6[r]) + p7[r];
      }
    }
    if (lane == 0) __hip_atomic_store(&counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (!col_ok) return;
  float *__restrict__ y0 = a.Y + (int64_t)z * a.y_z_stride + ycol + (int64_t)(m0 + 4 * half) * a.y_row_stride;
  // one copy of the store loop per activation mode, picked once (the mode is the same for every lane);
  // only a tile that sticks out of the matrix checks its rows
  auto store_rows = [&](auto mode_c, auto full_c) {
    constexpr int MODE = decltype(mode_c)::value;
    constexpr bool FULL = decltype(full_c)::value;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      if (!FULL && acc_row(m0, half, r) >= a.M) continue;
      float v = a.alpha * acc[r] + bias_r[r] + bias_c;
      if (a.Cin) v += a.beta * res_r[r];
      y0[(int64_t)row_k(r) * a.y_row_stride] = apply_act(v, MODE, a.act_coef);
    }
  };
  auto store = [&](auto mode_c) {
    if (full) store_rows(mode_c, std::true_type{});
    else store_rows(mode_c, std::false_type{});
  };
  switch (a.act) {
    case DNNRT_ACT_RELU: store(std::integral_constant<int, DNNRT_ACT_RELU>{}); break;
    case DNNRT_ACT_CLIPPED_RELU: store(std::integral_constant<int, DNNRT_ACT_CLIPPED_RELU>{}); break;
    case DNNRT_ACT_LEAKY_RELU: store(std::integral_constant<int, DNNRT_ACT_LEAKY_RELU>{}); break;
    case ACT_GELU: store(std::integral_constant<int, ACT_GELU>{}); break;
    default: store(std::integral_constant<int, DNNRT_ACT_IDENTITY>{}); break;
  }
}

template <int KS, bool AMC>
__global__ __launch_bounds__(64 * KS) void conv3x3_f32_small_kernel(const IgemmArgs a, const int c_per_wave, float *partials,
                                                                    unsigned *counters) {
  __shared__ float red[KS > 1 ? KS - 1 : 1][16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, half = lane >> 5;
  // Workgroups go round-robin over the 8 XCDs (gridDim.x is a multiple of 8, so that holds for every y and
  // z as well), each with its own L2.  The XCDs are laid out as a grid of xcd_m x (8 / xcd_m) over the
  // (filter-row tile, column tile) plane and each owns one rectangle of tiles: it fetches 1 / xcd_m of the
  // filter and xcd_m / 8 of the activations, where a run of consecutive tiles per XCD fetches all of one operand
  // into all eight L2s.  The launcher picks xcd_m from the two operands' sizes.
  const int tiles_m = (a.M + 31) / 32, tiles_n = (a.Ncols + 31) / 32, tiles = tiles_n * tiles_m;
  const int tm_per = a.tm_per, tn_per = a.tn_per;
  const int xcd = (int)(blockIdx.x & 7), in_xcd = (int)(blockIdx.x >> 3);
  const int tm_local = div_magic(in_xcd, tn_per, a.magic_tn_per);
  const int tile_m = (xcd >> a.xcd_n_log2) * tm_per + tm_local;
  const int tile_n = (xcd & ((1 << a.xcd_n_log2) - 1)) * tn_per + (in_xcd - tm_local * tn_per);
  if (tm_local >= tm_per || tile_m >= tiles_m || tile_n >= tiles_n) return;
  const int tile_id = tile_m * tiles_n + tile_n;
  const int m0 = tile_m * 32, n0 = tile_n * 32, z = blockIdx.z;
  const float *__restrict__ Ag = a.A + (int64_t)z * a.a_z_stride;
  const float *__restrict__ Xg = a.X + (int64_t)z * a.x_z_stride;

  const int m = m0 + l32, mrow = m < a.M ? m : 0;
  const int col = n0 + l32;
  const bool col_ok = col < a.Ncols;
  const int PQ = a.P * a.Q, HW = a.H * a.W, C = a.Kdim / 9;
  float bias_r[16];
  prefetch_bias(a, z, m0, half, bias_r);
  const float bias_c = 0.f;  // a per-column bias belongs to matrix products, which are never 3x3
  const int img = col_ok ? div_magic(col, PQ, a.magic_pq) : 0, pq = col_ok ? col - img * PQ : 0;
  const int p = div_magic(pq, a.Q, a.magic_q), q = pq - p * a.Q;
  const int ih0 = p * a.sh - a.ph, iw0 = q * a.sw - a.pw;
  unsigned tap_off[9], tap_mask[9];
#pragma unroll
  for (int j = 0; j < 9; j++) {
    const int ih = ih0 + j / 3, iw = iw0 + j % 3;
    const bool ok = col_ok && (unsigned)ih < (unsigned)a.H && (unsigned)iw < (unsigned)a.W;
    tap_off[j] = ok ? (unsigned)(ih * a.W + iw) : 0u;
    tap_mask[j] = ok ? 0xffffffffu : 0u;
  }
  const unsigned x_img = (unsigned)((int64_t)img * a.x_img_stride);
  const unsigned a_row = (unsigned)mrow * (unsigned)a.Kdim, lda = (unsigned)a.a_ld;

  const int cbeg = ((int)blockIdx.y * KS + wave) * c_per_wave, cend = min(C, cbeg + c_per_wave);
  const int niter = c_per_wave >> 1;

  constexpr int DEPTH = 4;
  float ra[DEPTH][9], rb[DEPTH][9];
  unsigned cm[DEPTH];
  auto load_iter = [&](int i, float (&av)[9], float (&bv)[9], unsigned &cmask) {
    const int c = cbeg + 2 * i + half;
    const unsigned cc = (unsigned)min(c, C - 1);
    cmask = c < cend ? 0xffffffffu : 0u;
    const unsigned bo = x_img + cc * (unsigned)HW;
    if (AMC) {  // filter stored [k][K_out]: 32 lanes read 32 consecutive words
      const unsigned ao = cc * 9u * lda + (unsigned)mrow;
#pragma unroll
      for (int j = 0; j < 9; j++) av[j] = Ag[ao + (unsigned)j * lda];
    } else {
      const unsigned ao = a_row + cc * 9u;
#pragma unroll
      for (int j = 0; j < 9; j++) av[j] = Ag[ao + j];
    }
#pragma unroll
    for (int j = 0; j < 9; j++) bv[j] = Xg[bo + tap_off[j]];
  };

  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
#pragma unroll
  for (int d = 0; d < DEPTH; d++) load_iter(d, ra[d], rb[d], cm[d]);
  auto mfma_iter = [&](int u) {
#pragma unroll
    for (int j = 0; j < 9; j++)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[u][j], mask_f(rb[u][j], tap_mask[j] & cm[u]), acc, 0, 0, 0);
  };
  // Iteration i lives in slot i % DEPTH and is refilled with iteration
  // i + DEPTH.  Whole groups that need every refill run without a branch; the
  // last DEPTH iterations refill nothing, and the group in between asks per
  // slot.  Most batch-1 layers have exactly DEPTH iterations per wavefront:
  // everything is requested by the prologue and nothing is loaded in vain.
  int i0 = 0;
  for (; i0 + 2 * DEPTH <= niter; i0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; u++) {
      mfma_iter(u);
      load_iter(i0 + u + DEPTH, ra[u], rb[u], cm[u]);
    }
  }
#pragma unroll
  for (int u = 0; u < DEPTH; u++) {
    if (i0 + u < niter) {
      mfma_iter(u);
      if (i0 + u + DEPTH < niter) load_iter(i0 + u + DEPTH, ra[u], rb[u], cm[u]);
    }
  }
  i0 += DEPTH;
#pragma unroll
  for (int u = 0; u < DEPTH; u++)
    if (i0 + u < niter) mfma_iter(u);
  reduce_and_store<KS, true>(a, acc, bias_r, bias_c, red, wave, lane, m0, img, pq, col_ok, z, (unsigned)(z * tiles + tile_id), partials, counters);
}

// 1x1 geometry (convolution, possibly strided, or matrix product with A rows
// k-contiguous and B columns contiguous); Kdim % 4 == 0, A rows 16-byte aligned.
template <int KS, bool AMC>
__global__ __launch_bounds__(64 * KS) void conv1x1_f32_small_kernel(const IgemmArgs a, const int k_per_wave, float *partials,
                                                                    unsigned *counters) {
  __shared__ float red[KS > 1 ? KS - 1 : 1][16][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, half = lane >> 5;
  // Workgroups go round-robin over the 8 XCDs (gridDim.x is a multiple of 8, so that holds for every y and
  // z as well), each with its own L2.  The XCDs are laid out as a grid of xcd_m x (8 / xcd_m) over the
  // (filter-row tile, column tile) plane and each owns one rectangle of tiles: it fetches 1 / xcd_m of the
  // filter and xcd_m / 8 of the activations, where a run of consecutive tiles per XCD fetches all of one operand
  // into all eight L2s.  The launcher picks xcd_m from the two operands' sizes.
  const int tiles_m = (a.M + 31) / 32, tiles_n = (a.Ncols + 31) / 32, tiles = tiles_n * tiles_m;
  const int tm_per = a.tm_per, tn_per = a.tn_per;
  const int xcd = (int)(blockIdx.x & 7), in_xcd = (int)(blockIdx.x >> 3);
  const int tm_local = div_magic(in_xcd, tn_per, a.magic_tn_per);
  const int tile_m = (xcd >> a.xcd_n_log2) * tm_per + tm_local;
  const int tile_n = (xcd & ((1 << a.xcd_n_log2) - 1)) * tn_per + (in_xcd - tm_local * tn_per);
  if (tm_local >= tm_per || tile_m >= tiles_m || tile_n >= tiles_n) return;
  const int tile_id = tile_m * tiles_n + tile_n;
  const int m0 = tile_m * 32, n0 = tile_n * 32, z = blockIdx.z;
  // With a second convolution (a.A2) the reduction is the first's followed by the second's; a wavefront's slice
  // lies in one of them (the launcher makes k_per_wave divide Kdim), so it only picks its operands here.
  const int kbeg_all = ((int)blockIdx.y * KS + wave) * k_per_wave;
  const bool second = a.A2 != nullptr && kbeg_all >= a.Kdim;
  const float *__restrict__ Ag = second ? a.A2 : a.A + (int64_t)z * a.a_z_stride;
  const float *__restrict__ Xg = second ? a.X2 : a.X + (int64_t)z * a.x_z_stride;
  const int Kd = second ? a.Kdim2 : a.Kdim;

  const int m = m0 + l32, mrow = m < a.M ? m : 0;
  const int col = n0 + l32;
  const bool col_ok = col < a.Ncols;
  const int PQ = a.P * a.Q, HW = second ? a.H2 * a.W2 : a.H * a.W;
  float bias_r[16];
  prefetch_bias(a, z, m0, half, bias_r);
  if (a.A2 != nullptr && a.bias2 != nullptr) {  // both biases ride in the one epilogue
#pragma unroll
    for (int r = 0; r < 16; r++) bias_r[r] += a.bias2[min(acc_row(m0, half, r), a.M - 1)];
  }
  const float bias_c = load_bias_col(a, col_ok ? col : 0);  // requested up front as well
  const int img = col_ok ? div_magic(col, PQ, a.magic_pq) : 0, pq = col_ok ? col - img * PQ : 0;
  const int p = div_magic(pq, a.Q, a.magic_q), q = pq - p * a.Q;
  const unsigned x_pix = second ? (unsigned)((int64_t)img * a.x2_img_stride + (int64_t)(p * a.sh2) * a.W2 + q * a.sw2)
                                : (unsigned)((int64_t)img * a.x_img_stride + (int64_t)(p * a.sh) * a.W + q * a.sw);
  const unsigned a_row = (unsigned)mrow * (unsigned)Kd, lda = (unsigned)a.a_ld;

  const int kbeg = second ? kbeg_all - a.Kdim : kbeg_all, kend = min(Kd, kbeg + k_per_wave);
  const int niter = k_per_wave >> 3;

  constexpr int DEPTH = 4;
  float4 ra[DEPTH];
  float rb[DEPTH][4];
  unsigned km[DEPTH];
  auto load_iter = [&](int i, float4 &av, float (&bv)[4], unsigned &kmask) {
    const int ka = kbeg + 8 * i + 4 * half;
    const unsigned kc = (unsigned)min(ka, Kd - 4);
    kmask = ka < kend ? 0xffffffffu : 0u;
    if (AMC) {
      const unsigned ao = kc * lda + (unsigned)mrow;
      av.x = Ag[ao]; av.y = Ag[ao + lda]; av.z = Ag[ao + 2u * lda]; av.w = Ag[ao + 3u * lda];
    } else {
      av = *reinterpret_cast<const float4 *>(Ag + (a_row + kc));
    }
    const unsigned bo = x_pix + kc * (unsigned)HW;
#pragma unroll
    for (int j = 0; j < 4; j++) bv[j] = Xg[bo + (unsigned)(j * HW)];
  };

  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
#pragma unroll
  for (int d = 0; d < DEPTH; d++) load_iter(d, ra[d], rb[d], km[d]);
  auto mfma_iter = [&](int u) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[u].x, mask_f(rb[u][0], km[u]), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[u].y, mask_f(rb[u][1], km[u]), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[u].z, mask_f(rb[u][2], km[u]), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[u].w, mask_f(rb[u][3], km[u]), acc, 0, 0, 0);
  };
  // refills as in the 3x3 kernel: branch-free groups, then one group that asks per slot, then none
  int i0 = 0;
  for (; i0 + 2 * DEPTH <= niter; i0 += DEPTH) {
#pragma unroll
    for (int u = 0; u < DEPTH; u++) {
      mfma_iter(u);
      load_iter(i0 + u + DEPTH, ra[u], rb[u], km[u]);
    }
  }
#pragma unroll
  for (int u = 0; u < DEPTH; u++) {
    if (i0 + u < niter) {
      mfma_iter(u);
      if (i0 + u + DEPTH < niter) load_iter(i0 + u + DEPTH, ra[u], rb[u], km[u]);
    }
  }
  i0 += DEPTH;
#pragma unroll
  for (int u = 0; u < DEPTH; u++)
    if (i0 + u < niter) mfma_iter(u);
  reduce_and_store<KS, false>(a, acc, bias_r, bias_c, red, wave, lane, m0, img, pq, col_ok, z, (unsigned)(z * tiles + tile_id), partials, counters);
}

// A fill kernel rather than hipMemsetAsync: a caller may be recording the stream into a graph.
__global__ void zero_counters_kernel(unsigned *counters, int n) {
  const int i = (int)(blockIdx.x * blockDim.x + threadIdx.x);
  if (i < n) counters[i] = 0u;
}

void clear_split_counters(const dnnrtContext *ctx, int n) {
  hipLaunchKernelGGL(zero_counters_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, ctx->stream, ctx->splitk_counters, n);
}

// Returns true if one of the specialised kernels took the problem.
bool launch_igemm_f32_small(const dnnrtContext *ctx, const IgemmArgs &a, int rsmode, int layout, bool &launched) {
  launched = false;
  if (layout != 0 && layout != 2) return true;
  const bool amc = layout == 2;
  // 32-bit element offsets inside the kernels
  const int64_t a_elems = amc ? (int64_t)a.Kdim * a.a_ld : (int64_t)a.M * a.Kdim;
  const int64_t x_elems = (int64_t)((a.Ncols + a.P * a.Q - 1) / (a.P * a.Q)) * a.x_img_stride + (int64_t)a.Kdim * a.H * a.W;
  if (a_elems >= (1ll << 31) || x_elems >= (1ll << 31)) return true;
  const bool is3x3 = rsmode == 3 && a.Kdim % 9 == 0 && !a.bias_col;
  const bool is1x1 = rsmode == 1 && (amc || a.a_vec4) && a.Kdim % 4 == 0 && a.Kdim >= 4;
  if (!is3x3 && !is1x1) return true;
  const bool dual = a.A2 != nullptr;
  if (dual) {
    const int64_t x2_elems = (int64_t)((a.Ncols + a.P * a.Q - 1) / (a.P * a.Q)) * a.x2_img_stride + (int64_t)a.Kdim2 * a.H2 * a.W2;
    if (!is1x1 || a.Z != 1 || a.Kdim2 % 8 != 0 || a.Kdim % 8 != 0 || x2_elems >= (1ll << 31) || (int64_t)a.Kdim2 * a.a_ld >= (1ll << 31) ||
        (int64_t)a.M * a.Kdim2 >= (1ll << 31))
      return true;
  }

  const int64_t tiles64 = ceil_div(a.M, 32) * ceil_div(a.Ncols, 32);
  if (tiles64 > INT32_MAX) return true;
  const int tiles = (int)tiles64;
  const int64_t want_waves = (int64_t)ctx->num_cu * 8;
  const int red_len = is3x3 ? a.Kdim / 9 : a.Kdim + (dual ? a.Kdim2 : 0);   // channels
  // reduction slice worth a wavefront; 1x1 problems of at most 32 tiles (the last stages of a MobileNetV2 at batch 1)
  // go down to 16 channels: 0.264 -> 0.260 ms per inference there, with more tiles it costs more than it gives
  const int min_slice = is3x3 ? 4 : (tiles <= 32 ? 16 : 32);
  int ks = 1;
  while (ks < 8 && (int64_t)tiles * a.Z * ks < want_waves && ceil_div(red_len, ks * 2) >= min_slice) ks *= 2;
  // Still far from filling the chip (deep layers at batch 1: a few dozen tiles
  // over a reduction of thousands): split the reduction over workgroups too.
  int splits = 1;
  while (splits < 16 && (int64_t)tiles * a.Z * splits * 2 <= ctx->num_cu &&
         ceil_div(red_len, ks * splits * 2) >= min_slice) {
    if ((int64_t)tiles * a.Z * splits * 2 * 4096 > ctx->splitk_partial_bytes || (int64_t)tiles * a.Z > ctx->splitk_max_tiles) {
      if (!ctx->splitk_shared) break;  // a handle's own scratch: a shallower split is as good
      set_error("igemm_f32(small): the split reduction of this problem needs %lld bytes of scratch and %lld counters, "
                "the static scratch holds %lld and %d",
                (long long)tiles * a.Z * splits * 2 * 4096, (long long)tiles * a.Z, (long long)ctx->splitk_partial_bytes,
                ctx->splitk_max_tiles);
      return false;
    }
    splits *= 2;
  }
  int k_per_wave_1x1 = (int)(ceil_div(ceil_div(red_len, ks * splits), 8) * 8);
  if (dual) {
    // a slice must not straddle the two reductions: the next power of two, which has to divide the first one's
    // length (wavefronts whose slice starts past the end find every k masked)
    int p2 = 8;
    while (p2 < k_per_wave_1x1) p2 *= 2;
    if (a.Kdim % p2 != 0) return true;  // not launched: the caller runs the two convolutions one after the other
    k_per_wave_1x1 = p2;
  }
  // The XCD grid: xcd_m x (8 / xcd_m) rectangles of tiles.  Elements fetched over all eight L2s: the filter
  // 8 / xcd_m times, the activations xcd_m times; rectangles that do not divide the tile counts leave
  // workgroups without a tile and XCDs with less work, which the estimate charges for.
  IgemmArgs am = a;
  const int tiles_m = (int)ceil_div(a.M, 32), tiles_n = (int)ceil_div(a.Ncols, 32);
  int64_t slots = 0;
  {
    const double act = (double)(a.Kdim / (a.R * a.S)) * a.H * a.W * (double)ceil_div(a.Ncols, (int64_t)a.P * a.Q), filt = (double)a.M * a.Kdim;
    double best = 0;
    for (int xm = 1; xm <= 8; xm *= 2) {
      const int xn = 8 / xm;
      if ((xm > tiles_m && xm > 1) || (xn > tiles_n && xn > 1)) continue;
      const int64_t per = ceil_div(tiles_m, xm) * ceil_div(tiles_n, xn);
      const double cost = (act * xm + filt * xn) * ((double)(8 * per) / tiles);
      if (slots == 0 || cost < best) { best = cost; am.xcd_m = xm; slots = 8 * per; }
    }
    if (slots == 0) { am.xcd_m = 1; slots = 8 * ceil_div(tiles_m, 1) * ceil_div(tiles_n, 8); }  // a single tile either way
  }
  if (slots > INT32_MAX) return true;
  {
    const int xn = 8 / am.xcd_m;
    am.xcd_n_log2 = xn == 8 ? 3 : xn == 4 ? 2 : xn == 2 ? 1 : 0;
    am.tm_per = (int)ceil_div(tiles_m, am.xcd_m);
    am.tn_per = (int)ceil_div(tiles_n, xn);
    am.magic_tn_per = magic_of(am.tn_per);
    am.magic_pq = magic_of(a.P * a.Q);
    am.magic_q = magic_of(a.Q);
  }
  dim3 grid((unsigned)slots, splits, a.Z);
  if (ctx->splitk_shared && splits > 1) clear_split_counters(ctx, tiles * a.Z);
#define LAUNCH_KS2(KERNEL, AMC_, ARG)                                                                  \
  switch (ks) {                                                                                          \
    case 1: hipLaunchKernelGGL((KERNEL<1, AMC_>), grid, dim3(64), 0, ctx->stream, am, ARG, ctx->splitk_partials, ctx->splitk_counters); break;  \
    case 2: hipLaunchKernelGGL((KERNEL<2, AMC_>), grid, dim3(128), 0, ctx->stream, am, ARG, ctx->splitk_partials, ctx->splitk_counters); break; \
    case 4: hipLaunchKernelGGL((KERNEL<4, AMC_>), grid, dim3(256), 0, ctx->stream, am, ARG, ctx->splitk_partials, ctx->splitk_counters); break; \
    default: hipLaunchKernelGGL((KERNEL<8, AMC_>), grid, dim3(512), 0, ctx->stream, am, ARG, ctx->splitk_partials, ctx->splitk_counters); break; \
  }
#define LAUNCH_KS(KERNEL, ARG)                                                                         \
  do {                                                                                                 \
    if (amc) { LAUNCH_KS2(KERNEL, true, ARG) } else { LAUNCH_KS2(KERNEL, false, ARG) }                 \
  } while (0)
  if (is3x3) {
    const int c_per_wave = (int)(ceil_div(ceil_div(red_len, ks * splits), 2) * 2);
    LAUNCH_KS(conv3x3_f32_small_kernel, c_per_wave);
  } else {
    LAUNCH_KS(conv1x1_f32_small_kernel, k_per_wave_1x1);
  }
#undef LAUNCH_KS
#undef LAUNCH_KS2
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("igemm_f32(small): launch failed: %s", hipGetErrorString(e)); return false; }
  launched = true;
  return true;
}

}  // namespace dnnrt
