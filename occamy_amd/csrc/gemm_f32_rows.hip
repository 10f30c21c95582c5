// Row-major fp32 matrix product for transformer Linear layers:
//   D[M, N] = act(A[M, K] * B[K, N] + bias_col[n] + beta * Cin[m, n]),  A and B row-major, a few hundred rows.
//
// The operand-from-global kernels (igemm_f32_small.hip) read A with one lane
// per row: 32 rows, 32 cache lines per load instruction, which is what made a
// 128 x 768 x 2304 product take 24 us.  Here both operands go through LDS:
// 16-byte coalesced global loads (rows of A along k, rows of B along n), A
// stored transposed so that every MFMA operand fetch is a conflict-free
// ds_read_b32.  64 x 64 tile per workgroup, four wavefronts (2 x 2) of one
// 32 x 32 accumulator each and four more taking the other half of every chunk, k in chunks of 32, LDS double buffered, the
// global loads of the next four chunks in flight in a register ring.
//
// Few rows mean few tiles (M = 128, N = 768: 24), so the reduction is split
// over gridDim.y workgroups: each wavefront leaves its partial 32 x 32 tile
// in the handle's scratch and bumps that tile's arrival counter; the last to
// arrive adds the partials in split order (same bits on every run), applies
// the epilogue and puts the counter back to zero.  Nobody waits for anybody.
#include "igemm_f32.h"

#include <type_traits>

namespace dnnrt {

typedef float floatx16 __attribute__((ext_vector_type(16)));

namespace rows {
constexpr int BM = 64, BN = 64, BKC = 32, LD = 68;  // LD: floats per LDS row (16-byte aligned, staggers the banks)
}

__global__ __launch_bounds__(512) void gemm_f32_rows_kernel(const IgemmArgs a, const int chunks_per_split, float *partials,
                                                            unsigned *counters) {
  using namespace rows;
  __shared__ float As[2][BKC][LD];  // [k][m]
  __shared__ float Bs[2][BKC][LD];  // [k][n]
  // Eight wavefronts: 0-3 and 4-7 own the same four 32 x 32 tiles and take the two halves of every
  // k chunk, so each SIMD holds two wavefronts and one's LDS and address work overlaps the other's MFMAs.
  const int tid = threadIdx.x, lane = tid & 63, wave = (tid >> 6) & 3, kg = tid >> 8, l32 = lane & 31, half = lane >> 5;
  const int tiles_n = (a.Ncols + BN - 1) / BN;
  const int tile = blockIdx.x, tile_m = tile / tiles_n, tile_n = tile - tile_m * tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int wm0 = (wave >> 1) * 32, wn0 = (wave & 1) * 32;
  const int nchunks = a.Kdim / BKC;
  const int c_beg = (int)blockIdx.y * chunks_per_split, c_end = min(nchunks, c_beg + chunks_per_split);

  // loader geometry: a chunk of A is 64 rows x 8 float4, of B 32 rows x 16 float4; one of each per thread
  const int a_row = tid >> 3, a_k4 = tid & 7;
  const int b_row = tid >> 4, b_n4 = tid & 15;
  const unsigned a_off0 = (unsigned)min(m0 + a_row, a.M - 1) * (unsigned)a.Kdim + a_k4 * 4;
  const int b_col = min(n0 + b_n4 * 4, a.Ncols - 4);  // columns past the end repeat the last four; they are not stored
  const unsigned b_off0 = (unsigned)b_row * (unsigned)a.Ncols + b_col;
  // A ring of DEPTH chunks in registers: the loads of chunk c + DEPTH are
  // issued when chunk c moves to LDS, so several chunks' worth of memory
  // latency overlap (a split holds only a handful of chunks and a CU only one
  // or two workgroups: nothing else would hide it).
  constexpr int DEPTH = 4;
  struct Chunk { float4 a0, b0; };
  Chunk r0, r1, r2, r3;  // separate variables, not an array: they must stay in registers
  auto load_chunk = [&](int c, Chunk &r) {
    const unsigned ka = (unsigned)min(c, c_end - 1) * BKC, kb = ka * (unsigned)a.Ncols;  // past the end: a copy nobody reads
    r.a0 = *reinterpret_cast<const float4 *>(a.A + a_off0 + ka);
    r.b0 = *reinterpret_cast<const float4 *>(a.X + b_off0 + kb);
  };
  auto store_chunk = [&](int buf, const Chunk &r) {
    float *ap = &As[buf][a_k4 * 4][a_row];
    ap[0] = r.a0.x; ap[LD] = r.a0.y; ap[2 * LD] = r.a0.z; ap[3 * LD] = r.a0.w;
    *reinterpret_cast<float4 *>(&Bs[buf][b_row][b_n4 * 4]) = r.b0;
  };

  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  // One step: chunk c (ring slot r, LDS buffer `buf`) to LDS, refill the slot,
  // barrier, MFMAs.  The barrier of step c also separates the MFMAs of step
  // c - 1 from the store of step c + 1 into the same LDS buffer.
  auto step = [&](int c, int buf, Chunk &r, bool refill) {
    store_chunk(buf, r);
    if (refill) load_chunk(c + DEPTH, r);
    __syncthreads();
    const float *ap = &As[buf][kg * (BKC / 2) + half][wm0 + l32], *bp = &Bs[buf][kg * (BKC / 2) + half][wn0 + l32];
#pragma unroll
    for (int i = 0; i < BKC / 4; i++)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ap[2 * i * LD], bp[2 * i * LD], acc, 0, 0, 0);
  };
  if (c_beg < c_end) {
    load_chunk(c_beg, r0);
    load_chunk(c_beg + 1, r1);
    load_chunk(c_beg + 2, r2);
    load_chunk(c_beg + 3, r3);
    // Whole groups of DEPTH steps that need every refill run without a
    // branch around the loads; the last DEPTH chunks refill nothing (a split
    // holds about six chunks: refills past its end were most of the loads),
    // and the group in between asks per slot.
    int c = c_beg;
    for (; c + 2 * DEPTH <= c_end; c += DEPTH) {
      step(c, 0, r0, true);
      step(c + 1, 1, r1, true);
      step(c + 2, 0, r2, true);
      step(c + 3, 1, r3, true);
    }
    if (c < c_end) step(c, 0, r0, c + DEPTH < c_end);
    if (c + 1 < c_end) step(c + 1, 1, r1, c + 1 + DEPTH < c_end);
    if (c + 2 < c_end) step(c + 2, 0, r2, c + 2 + DEPTH < c_end);
    if (c + 3 < c_end) step(c + 3, 1, r3, c + 3 + DEPTH < c_end);
    c += DEPTH;
    if (c < c_end) step(c, 0, r0, false);
    if (c + 1 < c_end) step(c + 1, 1, r1, false);
    if (c + 2 < c_end) step(c + 2, 0, r2, false);
  }

  // what the epilogue adds, requested now: the values are there long before they are used
  const int col = n0 + wn0 + l32;
  const bool col_ok = col < a.Ncols;
  const int colc = col_ok ? col : 0;
  const float bias_c = load_bias_col(a, colc);
  const int mrow0 = m0 + wm0 + 4 * half;  // the lane's rows are mrow0 + row_k(r)
  auto row_k = [](int r) { return 8 * (r >> 2) + (r & 3); };
  float res_r[16];
  if (a.Cin && kg == 0) {
#pragma unroll
    for (int r = 0; r < 16; r++) res_r[r] = a.Cin[(int64_t)min(mrow0 + row_k(r), a.M - 1) * a.c_row_stride + colc];
  } else {
#pragma unroll
    for (int r = 0; r < 16; r++) res_r[r] = 0.f;
  }

  // the second k group hands its sums to the first through LDS (the tiles are free after this barrier)
  __syncthreads();
  float *xch = &As[0][0][0];  // 4 wavefronts x 16 registers x 64 lanes = 16 KiB <= the 17 KiB of As
  if (kg == 1) {
#pragma unroll
    for (int r = 0; r < 16; r++) xch[(wave * 16 + r) * 64 + lane] = acc[r];
  }
  __syncthreads();
  if (kg == 1) return;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] += xch[(wave * 16 + r) * 64 + lane];

  // ---- split reduction: register r of lane (l32, half) is row 8*(r/4) + 4*half + r%4, column l32 of the wavefront's tile
  const int splits = (int)gridDim.y;
  if (splits > 1) {
    const unsigned slot = (unsigned)tile * 4u + (unsigned)wave;
    float *mine = partials + ((size_t)slot * splits + blockIdx.y) * 1024;
#pragma unroll
    for (int r = 0; r < 16; r++) __hip_atomic_store(&mine[r * 64 + lane], acc[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // device-scope accesses reach the point where all XCDs agree; waiting for
    // the stores' acknowledgements orders them before the arrival (a release
    // fence would write back this XCD's whole L2).  The signal fences keep the
    // compiler from moving the relaxed accesses across the wait and the arrival
    // (they emit no instruction); the hand-over protocol is described in
    // igemm_f32_small.hip.
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    unsigned arrived = 0;
    if (lane == 0) arrived = __hip_atomic_fetch_add(&counters[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    if (arrived != (unsigned)splits - 1) return;
    // the partial tiles are requested four at a time (a memory round trip each time) and added in split order
    const float *all = partials + (size_t)slot * splits * 1024 + lane;
    auto part = [&](int y, float (&p)[16]) {
#pragma unroll
      for (int r = 0; r < 16; r++) p[r] = __hip_atomic_load(all + (size_t)y * 1024 + r * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    int y = 0;
    for (; y + 4 <= splits; y += 4) {
      float p0[16], p1[16], p2[16], p3[16];
      part(y, p0); part(y + 1, p1); part(y + 2, p2); part(y + 3, p3);
#pragma unroll
      for (int r = 0; r < 16; r++) acc[r] = (((acc[r] + p0[r]) + p1[r]) + p2[r]) + p3[r];
    }
    if (y < splits) {  // one to three left: requested together as well (an absent one re-reads the last and is not added)
      float p0[16], p1[16], p2[16];
      part(y, p0); part(min(y + 1, splits - 1), p1); part(min(y + 2, splits - 1), p2);
#pragma unroll
      for (int r = 0; r < 16; r++) {
        acc[r] += p0[r];
        if (y + 1 < splits) acc[r] += p1[r];
        if (y + 2 < splits) acc[r] += p2[r];
      }
    }
    if (lane == 0) __hip_atomic_store(&counters[slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- epilogue: one copy of the store loop per activation mode; a row is one per-lane base plus a uniform offset
  if (!col_ok) return;
  float *__restrict__ y0 = a.Y + (int64_t)mrow0 * a.y_row_stride + col;
  auto store = [&](auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      if (mrow0 + row_k(r) >= a.M) continue;
      float v = a.alpha * acc[r] + bias_c;
      if (a.Cin) v += a.beta * res_r[r];
      y0[(int64_t)row_k(r) * a.y_row_stride] = apply_act(v, MODE, a.act_coef);
    }
  };
  switch (a.act) {
    case DNNRT_ACT_RELU: store(std::integral_constant<int, DNNRT_ACT_RELU>{}); break;
    case ACT_GELU: store(std::integral_constant<int, ACT_GELU>{}); break;
    case DNNRT_ACT_IDENTITY: store(std::integral_constant<int, DNNRT_ACT_IDENTITY>{}); break;
    default: {  // the remaining modes through the run-time switch
#pragma unroll
      for (int r = 0; r < 16; r++) {
        if (mrow0 + row_k(r) >= a.M) continue;
        float v = a.alpha * acc[r] + bias_c;
        if (a.Cin) v += a.beta * res_r[r];
        y0[(int64_t)row_k(r) * a.y_row_stride] = apply_act(v, a.act, a.act_coef);
      }
    }
  }
}

// Takes row-major products whose shape fits (returns launched = false otherwise).
bool launch_gemm_f32_rows(const dnnrtContext *ctx, const IgemmArgs &a, bool &launched) {
  using namespace rows;
  launched = false;
  if (a.Z != 1 || a.b_kcontig || a.a_mcontig || a.bias) return true;
  if (a.M < 32 || a.Ncols < 4 || a.Kdim % BKC || a.Ncols % 4 || !aligned16(a.A) || !aligned16(a.X)) return true;
  if ((int64_t)a.M * a.Kdim >= (1ll << 31) || (int64_t)a.Kdim * a.Ncols >= (1ll << 31)) return true;
  // below about 0.3 GFLOP the operand-from-global kernels (no LDS round trip, no barriers) are as fast or faster
  if ((double)a.M * a.Ncols * a.Kdim < 1.5e8) return true;
  const int64_t tiles = ceil_div(a.M, BM) * ceil_div(a.Ncols, BN);
  // a problem that fills the chip with unsplit tiles several times over is better off with the big-tile kernel
  if (tiles >= 4 * (int64_t)ctx->num_cu) return true;
  const int nchunks = a.Kdim / BKC;
  // about 1.75 workgroups per CU: two workgroups on a CU run out of step, so one's MFMAs overlap the
  // other's LDS and memory phases (measured on the 128-row BERT products: 5-6 splits beat both 3 and 8)
  const int64_t want = 7 * (int64_t)ctx->num_cu / 4;
  int64_t splits = tiles >= want ? 1 : (want + tiles / 2) / tiles;
  splits = splits > 8 ? 8 : splits;  // beyond eight the last arriver's reads of the partial tiles (four at a time) cost more than the
                                     // shorter slices save: 128 x 3072 x 768 at 16 splits against 8, BERT-base 0.870 -> 0.844 ms
  splits = splits > nchunks ? nchunks : splits;
  while (splits > 1 && (tiles * 4 * splits * 4096 > ctx->splitk_partial_bytes || tiles * 4 > ctx->splitk_max_tiles)) splits--;
  const int cps = (int)ceil_div(nchunks, splits);
  splits = ceil_div(nchunks, cps);  // no empty split: every arrival carries a partial tile
  if (ctx->splitk_shared && splits > 1) clear_split_counters(ctx, (int)tiles * 4);
  hipLaunchKernelGGL(gemm_f32_rows_kernel, dim3((unsigned)tiles, (unsigned)splits, 1), dim3(512), 0, ctx->stream, a, cps,
                     ctx->splitk_partials, ctx->splitk_counters);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("gemm_f32(rows): launch failed: %s", hipGetErrorString(e)); return false; }
  launched = true;
  return true;
}

}  // namespace dnnrt
