// fp16 matrix product.  Out[M,N] = A[M,K] * B[N,K]^T is exactly a channels-last
// 1x1 convolution (M "pixels" of K channels, N filters), so it runs on the
// fp16 convolution kernels (a bias row is the convolution's bias).  Every
// other form -- B stored K x N, transposed A, batches, alpha / beta, a bias
// row with a residual matrix and an activation behind it -- goes to one
// generic kernel: a 64 x 64 tile of Out per workgroup, operands gathered
// into LDS in runs of eight along their contiguous direction (strides are
// runtime values; one 16-byte load per run where alignment allows), 32x32x16 MFMA,
// fp32 accumulation, one rounding to fp16 at the end; with few tiles and a
// long reduction the reduction is split over workgroups.
#include "gemm_f16.h"

#include "conv_f16.h"

namespace dnnrt {

typedef _Float16 g_half8 __attribute__((ext_vector_type(8)));
typedef float g_floatx16 __attribute__((ext_vector_type(16)));

struct GemmF16Args {
  const __half *A, *B, *C, *bias;
  __half *Out;
  int M, N, K;
  int64_t a_sm, a_sk, b_sk, b_sn;   // element strides of A along m and k, of B along k and n
  int64_t az, bz, yz;               // batch strides (0: shared)
  int64_t c_sm, cz;                 // C: row stride (0: one row for every m), batch stride
  float alpha, beta;
  int act;
  float act_coef;
  bool a_vec, b_vec;                // the contiguous direction of A / B may be read eight elements (16 bytes) at a time
  int steps_per_split;              // 64-k steps per workgroup along gridDim.y (the reduction split over workgroups)
  float *partials;                  // the handle's scratch: one 64 x 64 fp32 tile per (tile, split)
  unsigned *counters;               // ... and one arrival counter per tile, zero between kernels
};

constexpr int G_BK = 64, G_ROW = 72;  // k per step; halfs per LDS row (64 + 8 of padding)

// Tile: 64 columns n x 64 rows m; the MFMA's row operand is the B side (n), its column operand the A side (m), so
// that a lane ends up with four consecutive n of one m: an 8-byte store.
__global__ __launch_bounds__(256) void gemm_f16_generic_kernel(const GemmF16Args a) {
  __shared__ __attribute__((aligned(16))) _Float16 Ns[64 * G_ROW];  // [n][k]
  __shared__ __attribute__((aligned(16))) _Float16 Ms[64 * G_ROW];  // [m][k]
  __shared__ unsigned arrived_before;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, half = lane >> 5;
  const int wn0 = (wave >> 1) * 32, wm0 = (wave & 1) * 32;
  const int tiles_n = (a.N + 63) / 64;
  const int tile_m = blockIdx.x / tiles_n, tile_n = blockIdx.x - tile_m * tiles_n;
  const int n0 = tile_n * 64, m0 = tile_m * 64, z = blockIdx.z;
  const _Float16 *__restrict__ Ag = reinterpret_cast<const _Float16 *>(a.A) + (int64_t)z * a.az;
  const _Float16 *__restrict__ Bg = reinterpret_cast<const _Float16 *>(a.B) + (int64_t)z * a.bz;
  // Which way the 2048 elements of an operand's step are dealt to the 256 threads: along k when k is the
  // contiguous direction in memory (eight consecutive k of one row per thread), along the row index otherwise.
  const bool a_k_fast = a.a_sk == 1, b_k_fast = a.b_sk == 1;
  g_floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  // A step is 64 rows x 64 k per operand = 512 runs of eight elements along the operand's contiguous direction;
  // a thread takes two runs of each operand.  Run r along k: row r / 8, k 8 (r % 8); along the row index: k r / 8,
  // rows 8 (r % 8) ...  A run is one 16-byte load where the operand allows it, eight 2-byte loads otherwise.
  const int k_begin = (int)blockIdx.y * a.steps_per_split * G_BK, k_end = min(a.K, k_begin + a.steps_per_split * G_BK);
  // Four steps of operands are requested ahead, in registers: a workgroup of a split reduction has a handful of
  // steps, so all of its loads are in flight before the first one is used.
  constexpr int AHEAD = 4;
  g_half8 ra[AHEAD][2], rb[AHEAD][2];
  auto request = [&](g_half8 (&va)[2], g_half8 (&vb)[2], const int k0) {
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int r = tid + 256 * h;
      {  // A side
        const int row0 = a_k_fast ? r >> 3 : (r & 7) << 3, kk0 = a_k_fast ? (r & 7) << 3 : r >> 3;
        const int64_t at = (int64_t)(m0 + row0) * a.a_sm + (int64_t)(k0 + kk0) * a.a_sk;
        const bool whole = a_k_fast ? (m0 + row0 < a.M && k0 + kk0 + 8 <= a.K) : (m0 + row0 + 8 <= a.M && k0 + kk0 < a.K);
        if (a.a_vec && whole) {
          va[h] = *reinterpret_cast<const g_half8 *>(Ag + at);
        } else {
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const int gm = m0 + row0 + (a_k_fast ? 0 : e), gk = k0 + kk0 + (a_k_fast ? e : 0);
            va[h][e] = (gm < a.M && gk < a.K) ? Ag[(int64_t)gm * a.a_sm + (int64_t)gk * a.a_sk] : (_Float16)0.f;
          }
        }
      }
      {  // B side (n contiguous: the thread's two runs are rows k = 2 (tid / 8) and the next one, which go to LDS as pairs)
        const int row0 = b_k_fast ? r >> 3 : (tid & 7) << 3, kk0 = b_k_fast ? (r & 7) << 3 : 2 * (tid >> 3) + h;
        const int64_t at = (int64_t)(k0 + kk0) * a.b_sk + (int64_t)(n0 + row0) * a.b_sn;
        const bool whole = b_k_fast ? (n0 + row0 < a.N && k0 + kk0 + 8 <= a.K) : (n0 + row0 + 8 <= a.N && k0 + kk0 < a.K);
        if (a.b_vec && whole) {
          vb[h] = *reinterpret_cast<const g_half8 *>(Bg + at);
        } else {
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const int gn = n0 + row0 + (b_k_fast ? 0 : e), gk = k0 + kk0 + (b_k_fast ? e : 0);
            vb[h][e] = (gn < a.N && gk < a.K) ? Bg[(int64_t)gk * a.b_sk + (int64_t)gn * a.b_sn] : (_Float16)0.f;
          }
        }
      }
    }
  };
  auto to_lds = [&](const g_half8 (&va)[2], const g_half8 (&vb)[2]) {
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int r = tid + 256 * h;
      {  // -> Ms[m][k]
        const int row0 = a_k_fast ? r >> 3 : (r & 7) << 3, kk0 = a_k_fast ? (r & 7) << 3 : r >> 3;
        if (a_k_fast) {
          *reinterpret_cast<g_half8 *>(Ms + row0 * G_ROW + kk0) = va[h];
        } else {
#pragma unroll
          for (int e = 0; e < 8; e++) Ms[(row0 + e) * G_ROW + kk0] = va[h][e];
        }
      }
      if (b_k_fast) {  // -> Ns[n][k]
        const int row0 = r >> 3, kk0 = (r & 7) << 3;
        *reinterpret_cast<g_half8 *>(Ns + row0 * G_ROW + kk0) = vb[h];
      }
    }
    if (!b_k_fast) {
      // n contiguous in memory: -> Nd[k / 2][n], one 32-bit word per pair of consecutive k of a column n, so that the
      // thread's two runs (rows k, k + 1 of eight columns) are eight consecutive words, two 16-byte stores, and an
      // MFMA operand (eight consecutive k of one n) is four words 72 words apart.  (Element by element into
      // Ns[n][k] this was sixteen 2-byte stores a thread and step, most of them on the same banks.)
      typedef unsigned g_uintx4 __attribute__((ext_vector_type(4)));
      unsigned *Nd = reinterpret_cast<unsigned *>(Ns);
      const g_uintx4 d0 = __builtin_bit_cast(g_uintx4, vb[0]), d1 = __builtin_bit_cast(g_uintx4, vb[1]);  // word j: columns 2j, 2j + 1
      g_uintx4 lo, hi;  // columns 0..3 and 4..7, each word (row k, row k + 1)
#pragma unroll
      for (int j = 0; j < 2; j++) {
        lo[2 * j] = (d0[j] & 0xffffu) | (d1[j] << 16);
        lo[2 * j + 1] = (d0[j] >> 16) | (d1[j] & 0xffff0000u);
        hi[2 * j] = (d0[2 + j] & 0xffffu) | (d1[2 + j] << 16);
        hi[2 * j + 1] = (d0[2 + j] >> 16) | (d1[2 + j] & 0xffff0000u);
      }
      unsigned *dst = Nd + (tid >> 3) * G_ROW + ((tid & 7) << 3);
      *reinterpret_cast<g_uintx4 *>(dst) = lo;
      *reinterpret_cast<g_uintx4 *>(dst + 4) = hi;
    }
  };
#pragma unroll
  for (int s = 0; s < AHEAD; s++)
    if (k_begin + s * G_BK < k_end) request(ra[s], rb[s], k_begin + s * G_BK);
  for (int k0 = k_begin; k0 < k_end; k0 += AHEAD * G_BK) {
#pragma unroll
    for (int s = 0; s < AHEAD; s++) {
      const int ks0 = k0 + s * G_BK;
      if (ks0 >= k_end) break;  // the same for every thread
      to_lds(ra[s], rb[s]);
      __syncthreads();
      if (ks0 + AHEAD * G_BK < k_end) request(ra[s], rb[s], ks0 + AHEAD * G_BK);
#pragma unroll
      for (int ks = 0; ks < G_BK; ks += 16) {
        g_half8 nv;
        if (b_k_fast) {
          nv = *reinterpret_cast<const g_half8 *>(Ns + (wn0 + l32) * G_ROW + ks + half * 8);
        } else {
          const unsigned *Nd = reinterpret_cast<const unsigned *>(Ns) + ((ks >> 1) + half * 4) * G_ROW + wn0 + l32;
          typedef unsigned g_uintx4 __attribute__((ext_vector_type(4)));
          const g_uintx4 w4 = {Nd[0], Nd[G_ROW], Nd[2 * G_ROW], Nd[3 * G_ROW]};
          nv = __builtin_bit_cast(g_half8, w4);
        }
        const g_half8 mv = *reinterpret_cast<const g_half8 *>(Ms + (wm0 + l32) * G_ROW + ks + half * 8);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(nv, mv, acc, 0, 0, 0);
      }
      __syncthreads();
    }
  }
  // The reduction split over gridDim.y workgroups: each leaves its partial tile in the scratch and bumps the tile's
  // arrival counter; whoever arrives last adds the partial tiles up in split order (the same bits whatever the order
  // of arrival) and finishes the tile; nobody waits for anybody.  The hand-over is the one of the fp32 small-problem
  // kernels (igemm_f32_small.hip): device-scope atomic stores of the partial tile, a wait until every one of the
  // wavefront's stores is acknowledged, a barrier (all four wavefronts are there), then one device-scope atomic
  // increment; the last arriver reads with device-scope atomic loads and puts the counter back to zero.
  const int splits = (int)gridDim.y;
  if (splits > 1) {
    const unsigned tile = (unsigned)z * gridDim.x + blockIdx.x;
    float *mine = a.partials + ((size_t)tile * splits + blockIdx.y) * 4096;
#pragma unroll
    for (int r = 0; r < 16; r++) __hip_atomic_store(&mine[r * 256 + tid], acc[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __syncthreads();
    if (tid == 0) arrived_before = __hip_atomic_fetch_add(&a.counters[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrived_before != (unsigned)splits - 1) return;
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    const float *all = a.partials + (size_t)tile * splits * 4096 + tid;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    for (int y0 = 0; y0 < splits; y0 += 4) {  // four partial tiles requested at a time, added in split order
      float p[4][16];
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (y0 + j < splits) {
#pragma unroll
          for (int r = 0; r < 16; r++)
            p[j][r] = __hip_atomic_load(all + (size_t)(y0 + j) * 4096 + r * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (y0 + j < splits) {
#pragma unroll
          for (int r = 0; r < 16; r++) acc[r] += p[j][r];
        }
    }
    if (tid == 0) __hip_atomic_store(&a.counters[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // register r of a lane: n = n0 + wn0 + 8 (r >> 2) + 4 half + (r & 3), m = m0 + wm0 + l32
  const int m = m0 + wm0 + l32;
  if (m >= a.M) return;
  const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
  const _Float16 *__restrict__ Cg = a.C ? reinterpret_cast<const _Float16 *>(a.C) + (int64_t)z * a.cz + (int64_t)m * a.c_sm : nullptr;
  _Float16 *__restrict__ Og = reinterpret_cast<_Float16 *>(a.Out) + (int64_t)z * a.yz + (int64_t)m * a.N;
#pragma unroll
  for (int r = 0; r < 16; r++) {
    const int n = n0 + wn0 + 8 * (r >> 2) + 4 * half + (r & 3);
    if (n >= a.N) continue;
    float v = a.alpha * acc[r];
    if (biasg) v += (float)biasg[n];
    if (Cg) v += a.beta * (float)Cg[n];
    Og[n] = (_Float16)apply_act(v, a.act, a.act_coef);
  }
}

bool gemm_f16(const dnnrtContext *ctx, const __half *A, const __half *B, const __half *C, __half *Out, int M,
              int N, int K, float alpha, float beta, bool transA, bool transB, int Z, int64_t az, int64_t bz,
              int64_t yz, bool c_is_row, const __half *bias, int act) {
  // C: nothing, or one row of N values with beta 1 (a Gemm's bias), which is the convolution's per-filter bias
  const bool bias_row = C && c_is_row && beta == 1.f;
  const bool as_conv = !transA && transB && Z == 1 && alpha == 1.f && (bias_row || (!C || beta == 0.f)) && !bias && act == DNNRT_ACT_IDENTITY;
  if (as_conv) {
    ConvF16Args a{};
    a.X = A; a.Wt = B; a.bias = bias_row ? C : nullptr; a.Y = Out;
    a.N = M; a.C = K; a.H = 1; a.W = 1; a.K = N; a.Cg = K; a.R = 1; a.S = 1; a.P = 1; a.Q = 1;
    a.ph = 0; a.pw = 0; a.sh = 1; a.sw = 1; a.group = 1;
    a.act = DNNRT_ACT_IDENTITY;
    a.format = DNNRT_NHWC;
    return launch_conv_f16(ctx, a);
  }
  if (Z < 1 || Z > 65535) { set_error("matmul(fp16): %d batches (1..65535)", Z); return false; }
  const int64_t tiles = ceil_div(M, 64) * ceil_div(N, 64);
  if (tiles > INT32_MAX) { set_error("matmul(fp16): too many tiles"); return false; }
  GemmF16Args g{};
  g.A = A; g.B = B; g.C = (C && beta != 0.f) ? C : nullptr; g.bias = bias; g.Out = Out;
  g.M = M; g.N = N; g.K = K;
  g.a_sm = transA ? 1 : K; g.a_sk = transA ? M : 1;   // A stored M x K, or K x M when transposed
  g.b_sk = transB ? 1 : N; g.b_sn = transB ? K : 1;   // B stored K x N, or N x K when transposed
  g.az = az; g.bz = bz; g.yz = yz;
  g.c_sm = c_is_row ? 0 : N; g.cz = c_is_row ? 0 : yz;
  g.alpha = alpha; g.beta = beta; g.act = act; g.act_coef = ctx->act_coef;
  // a run of eight along the contiguous direction is one aligned 16-byte load when every run starts on a multiple
  // of eight elements: base, batch stride and the other direction's stride
  const int64_t a_other = transA ? g.a_sk : g.a_sm, b_other = transB ? g.b_sn : g.b_sk;
  g.a_vec = aligned16(A) && a_other % 8 == 0 && az % 8 == 0;
  g.b_vec = aligned16(B) && b_other % 8 == 0 && bz % 8 == 0;
  // Few tiles and a long reduction (a transformer's Linear layers at batch 1: 128 rows): the reduction is split over
  // workgroups up to about one workgroup per CU, a split keeping at least four 64-k steps (all of them in flight
  // at once), as far as the handle's scratch holds the partial tiles.  Measured on the fp16 BERT-base encoder:
  // 0.997 ms per sequence, against 1.02 with three or five steps, 1.08 with 1.75 workgroups per CU and one step,
  // 1.06 with half a workgroup per CU.
  const int steps = (int)ceil_div(K, G_BK);
  int64_t splits = 1;
  const int64_t want = ctx->num_cu, have = tiles * Z;
  if (!ctx->splitk_shared && have < want && have <= ctx->splitk_max_tiles) {
    splits = (want + have / 2) / have;
    splits = splits > 16 ? 16 : splits;
    splits = splits > steps / 4 ? steps / 4 : splits;
    splits = splits < 1 ? 1 : splits;
    while (splits > 1 && have * splits * 16384 > (int64_t)ctx->splitk_partial_bytes) splits--;  // 64 x 64 fp32 per tile and split
  }
  g.steps_per_split = (int)ceil_div(steps, splits);
  splits = ceil_div(steps, g.steps_per_split);  // no empty split: every arrival carries a partial tile
  g.partials = ctx->splitk_partials;
  g.counters = ctx->splitk_counters;
  hipLaunchKernelGGL(gemm_f16_generic_kernel, dim3((unsigned)tiles, (unsigned)splits, (unsigned)Z), dim3(256), 0, ctx->stream, g);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("matmul(fp16): launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

}  // namespace dnnrt
