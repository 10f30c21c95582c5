// fp16 convolution with fp32 accumulation on v_mfma_f32_32x32x16_f16.
//
// GEMM view: D[k_out, pixel] = sum_k Wt[k_out, k] * Xcol[k, pixel].  The MFMA
// wants, per lane, 8 CONSECUTIVE k of one row (A) / one column (B), so both
// operands should be k-contiguous in memory.  Channels-last activations make
// the im2col operand so: with k ordered (r, s, c) a run of 8 k is 8 adjacent
// channels of one input pixel, and the filter is stored K,R,S,C to match.
//
// Fast kernel (NHWC in, NHWC out, C % 64 == 0, K % 8 == 0, group 1):
//   tile BM k_out x BN pixels, BK = 64; per step every thread moves 16-byte
//   chunks global -> registers -> LDS (128-byte rows with an XOR swizzle of the
//   chunk position, which makes both the stores and the ds_read_b128 operand
//   fetches conflict-free); two register stages of loads in flight, LDS
//   double buffered, one barrier per step.  A step lies inside one (r, s) tap,
//   so the tap and its bounds check are wave-uniform.  The epilogue adds bias,
//   applies the activation (after the residual sum, if there is one), converts
//   to fp16 and goes through LDS once more so that global stores are full
//   16-byte chunks of a pixel's channel vector.
//
// Generic kernel (any C, groups, NCHW or NHWC on either side): same MFMA
// structure with element-wise gathers, for the shapes neither the fast kernel
// nor the first-layer kernel (conv_f16_stem.hip) takes.
#include "conv_f16.h"

#include <type_traits>

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

constexpr int BK16 = 32;      // k per step of the generic kernel
constexpr int BKF = 64;       // k per step of the fast kernel: a row's slice is one 128-byte line
constexpr int LDS_ROW = 64;   // halfs per LDS row of the fast kernel: 128 bytes, no padding
constexpr int LDS_ROW_G = 40; // generic kernel: 32 + 8 pad (80 bytes)

// Fast kernel.  Tile BM k_out x BN pixels, four wavefronts in a WM x WN grid,
// each owning (BM/WM) x (BN/WN) of the tile as 32x32 MFMA blocks.
//
// Everything inside the K loop is branch-free on the vector side: every load
// is issued unconditionally from a clamped address and what must not
// contribute (padding taps, rows past the end of the tensor) is zeroed by an
// AND when the chunk goes to LDS.  Only then can the compiler count the
// outstanding loads exactly and wait for just the stage it is about to store
// (a load under a divergent branch forces a wait for ALL outstanding loads,
// which exposes the full memory latency at every step).
//
// Pipeline, one barrier per step of 64 k: two register stages of global
// loads in flight (a step's loads are issued two steps before it is
// computed), LDS double buffered, MFMA operands double buffered inside the
// step.  A row's slice of a step is one full 128-byte line: half-line requests
// cost the L2 a full slot each, and the L2 is what bounds this kernel.
//
// Workgroup ids are dealt round-robin to the 8 XCDs, each with an L2 of its
// own: the kernel renumbers them so that one XCD works on a contiguous run of
// tiles (k_out tiles of one pixel tile first), which then share their
// operands in that L2.
//
// KG = 2 doubles the workgroup to eight wavefronts: wavefronts 4-7 own the
// same output blocks as 0-3 and take the second half of every 64-k step (the
// partial sums meet in LDS once, at the end).  Same tile, same traffic, but
// two wavefronts per SIMD: a wavefront cannot overlap its own vector
// arithmetic with its MFMAs, so where a CU holds a single workgroup (few
// tiles: the 14x14 and 7x7 layers) the MFMA pipe otherwise idles during all
// address, mask and LDS work.
// FEW_STEPS = n > 0: the whole reduction is exactly n 64-k steps (a 1x1 layer
// over 64 n channels) and they take turns in ONE LDS stage instead of
// alternating between two: half the LDS, so more workgroups fit a CU, and
// what these layers need is memory requests in flight, not MFMA time.
// DUAL: two 1x1 convolutions (no padding) onto the same output tile, Y = act(fp16(conv(X, W) + bias) +
// fp16(conv(X2, W2) + bias2)) — a residual block's last convolution and its projection shortcut.  The second
// convolution's steps come first, into the same accumulators; where its reduction ends they are rounded to fp16
// with its bias, exactly what it would have stored as a convolution of its own, and set aside; the epilogue adds
// them as it adds a residual tensor, which is then never written or read.  The turns of the single-stage sequence
// are DUAL_FIRST steps of the second convolution, then the first's.
template <int BM, int BN, int WM, int WN, int DEPTH, int MIN_WAVES, bool MASKED, int KG, int FEW_STEPS = 0, bool DUAL = false,
          int DUAL_FIRST = 0>
__global__ __launch_bounds__(256 * KG, MIN_WAVES)  // second argument: wavefronts per SIMD the register budget must allow
 void conv_f16_nhwc_kernel(const ConvF16Args a, const int tiles_total) {
  static_assert(!DUAL || (KG == 1 && FEW_STEPS > 0), "the two-convolution form is written for the single-stage sequence");
  static_assert(WM * WN == 4, "four wavefronts");
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static_assert(KG == 1 || KG == 2, "one or two k groups");
  constexpr int NT = 256 * KG;
  constexpr int A_CH = BM * 8 / NT, B_CH = BN * 8 / NT;  // 16-byte chunks per thread per step
  static_assert(A_CH >= 1 && B_CH >= 1, "tile too small");
  constexpr int STAGE = (BM + BN) * LDS_ROW;               // halfs per pipeline stage
  constexpr int CROW = BM + 8;                             // halfs per row of the output staging tile
  constexpr bool ONE_STAGE = FEW_STEPS > 0;
  static_assert(!ONE_STAGE || KG == 1, "the single-stage sequence is written for one k group");
  constexpr int STAGES = ONE_STAGE ? 1 : 2;
  constexpr int SMEM = (STAGES * STAGE > BN * CROW) ? STAGES * STAGE : BN * CROW;
  static_assert(DEPTH == 2 || DEPTH == 4, "ring slots and LDS stages are indexed at compile time");
  __shared__ __attribute__((aligned(16))) _Float16 smem[SMEM];

  const int per_xcd = (tiles_total + 7) >> 3;
  const int tile = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
  if (tile >= tiles_total) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = (tid >> 6) & 3, kg = tid >> 8;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);

  const int tiles_m = (a.K + BM - 1) / BM;
  const int tile_n = tile / tiles_m, tile_m = tile - tile_n * tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int NPQ = a.N * a.P * a.Q, PQ = a.P * a.Q;
  const int CRS = a.C * a.R * a.S;

  const char *__restrict__ Xg = reinterpret_cast<const char *>(a.X);
  const char *__restrict__ Wg = reinterpret_cast<const char *>(a.Wt);
  const char *__restrict__ X2g = reinterpret_cast<const char *>(a.X2);
  const char *__restrict__ W2g = reinterpret_cast<const char *>(a.Wt2);

  // ---- loader constants ------------------------------------------------
  // chunk id -> (row of the tile, 16-byte chunk of the row's 64-byte k slice).
  // Unsigned 32-bit BYTE offsets from the kernel-argument bases (the
  // dispatcher checks the tensors are below 4 GiB), so the loads use the
  // scalar-base + 32-bit vector-offset form: no 64-bit address arithmetic and
  // no address registers that outlive the load.
  unsigned a_off[A_CH], a_msk[A_CH], a_off2[DUAL ? A_CH : 1];
#pragma unroll
  for (int i = 0; i < A_CH; i++) {
    const int id = tid + i * NT, row = id >> 3, ch = id & 7;
    const int k_out = m0 + row;
    const bool ok = k_out < a.K;
    a_off[i] = 2u * (unsigned)((ok ? k_out : 0) * CRS + ch * 8);
    if (DUAL) a_off2[i] = 2u * (unsigned)((ok ? k_out : 0) * a.C2 + ch * 8);
    a_msk[i] = ok ? 0xffffffffu : 0u;
  }
  // B (im2col): a chunk belongs to one output pixel; bit (r * S + s) of
  // b_taps says whether that tap reads inside the image.
  int b_pix[B_CH], b_pix2[DUAL ? B_CH : 1];
  unsigned b_taps[B_CH];
#pragma unroll
  for (int i = 0; i < B_CH; i++) {
    const int id = tid + i * NT, row = id >> 3, ch = id & 7;
    const int pix = n0 + row;
    const bool ok = pix < NPQ;
    const int n = ok ? div_magic(pix, PQ, a.magic_pq) : 0;
    const int pq = ok ? pix - n * PQ : 0;
    const int p = div_magic(pq, a.Q, a.magic_q), q = pq - p * a.Q;
    const int ih0 = p * a.sh - a.ph, iw0 = q * a.sw - a.pw;
    b_pix[i] = 2 * (((n * a.H + ih0) * a.W + iw0) * a.C + ch * 8);  // bytes; negative inside the padding
    if (DUAL) b_pix2[i] = 2 * (((n * a.H2 + p * a.sh2) * a.W2 + q * a.sw2) * a.C2 + ch * 8);
    unsigned taps = 0;
    if (MASKED && ok) {
      // taps (r, s) inside the image: r in [r_lo, r_hi), s in [s_lo, s_hi)
      const int r_lo = max(0, -ih0), r_hi = min(a.R, a.H - ih0);
      const int s_lo = max(0, -iw0), s_hi = min(a.S, a.W - iw0);
      const unsigned row_bits = s_hi > s_lo ? ((1u << (s_hi - s_lo)) - 1u) << s_lo : 0u;
      for (int r = 0; r < a.R; r++)
        if (r >= r_lo && r < r_hi) taps |= row_bits << (r * a.S);
    }
    b_taps[i] = taps;
  }

  u32x4 ra[DEPTH][A_CH], rb[DEPTH][B_CH];
  unsigned rm[DEPTH][B_CH];

  const int steps_c = a.C / BKF, nk2 = DUAL ? a.C2 / BKF : 0, nk = a.R * a.S * steps_c + nk2;
  // cursor of the next step to load (wave-uniform); it stops at the last step,
  // so loads issued past the end re-read that step and are never used
  int lj = 0, l_r = 0, l_s = 0, l_c0 = 0;

  auto load_step = [&](u32x4 (&qa)[A_CH], u32x4 (&qb)[B_CH], unsigned (&qm)[B_CH]) {
    if (DUAL) {  // both convolutions 1x1: step lj is 64 channels of the second one (lj < nk2), then of the first
      const bool second = lj < nk2;
      const unsigned k_off = 2u * (unsigned)(second ? lj : lj - nk2) * BKF;
      const char *__restrict__ wb = second ? W2g : Wg;
      const char *__restrict__ xb = second ? X2g : Xg;
#pragma unroll
      for (int i = 0; i < A_CH; i++) qa[i] = load_global_16(wb + ((second ? a_off2[i] : a_off[i]) + k_off));
#pragma unroll
      for (int i = 0; i < B_CH; i++) {
        const unsigned off = (unsigned)(second ? b_pix2[i] : b_pix[i]) + k_off;
        if (MASKED) {
          const unsigned m = 0u - (b_taps[i] & 1u);
          qm[i] = m;
          qb[i] = load_global_16(xb + (off & m));
        } else {
          qb[i] = load_global_16(xb + off);
        }
      }
      lj = lj + 1 < nk ? lj + 1 : lj;
      return;
    }
    const unsigned w_off = 2u * (unsigned)lj * BKF;
    const int x_off = 2 * ((l_r * a.W + l_s) * a.C + l_c0);
    const int tap = l_r * a.S + l_s;
#pragma unroll
    for (int i = 0; i < A_CH; i++) qa[i] = load_global_16(Wg + (a_off[i] + w_off));
#pragma unroll
    for (int i = 0; i < B_CH; i++) {
      if (MASKED) {
        const unsigned m = 0u - ((b_taps[i] >> tap) & 1u);
        qm[i] = m;
        qb[i] = load_global_16(Xg + ((unsigned)(b_pix[i] + x_off) & m));
      } else {
        qb[i] = load_global_16(Xg + (unsigned)(b_pix[i] + x_off));
      }
    }
    // advance, without branches (selects on the scalar unit)
    const bool more = lj + 1 < nk;
    const int c0n = l_c0 + BKF, sn = l_s + 1;
    const bool wrap_c = c0n == a.C, wrap_s = wrap_c && sn == a.S;
    lj = more ? lj + 1 : lj;
    l_c0 = more ? (wrap_c ? 0 : c0n) : l_c0;
    l_s = more ? (wrap_c ? (wrap_s ? 0 : sn) : l_s) : l_s;
    l_r = (more && wrap_s) ? l_r + 1 : l_r;
  };
  // LDS rows are 128 bytes (eight 16-byte chunks) and chunk c of row r lives at
  // position c ^ ((r >> 1) & 7).  The LDS has 64 four-byte banks and serves a
  // 16-byte access for 16 lanes per clock: with this placement 16 consecutive
  // lanes always cover all 64 banks once, both when a step is stored (two
  // rows x eight chunks) and when MFMA operands are read (16 rows, one chunk
  // each).  Measured on the same 16-byte reads: 240 B/clk per CU conflict-free,
  // 126 with two lanes per bank, 63 with four.
  const int st_swz = (tid >> 4) & 7;   // store side: row = tid / 8 + 32 * i
  const int ld_swz = (l32 >> 1) & 7;   // operand side: row = 32 * block + l32
  auto store_step = [&](int buf, const u32x4 (&qa)[A_CH], const u32x4 (&qb)[B_CH], const unsigned (&qm)[B_CH]) {
    _Float16 *As = smem + buf * STAGE, *Bs = As + BM * LDS_ROW;
#pragma unroll
    for (int i = 0; i < A_CH; i++) {
      const int id = tid + i * NT, row = id >> 3, ch = id & 7;
      u32x4 v = qa[i];
      if (MASKED) v &= a_msk[i];
      *reinterpret_cast<u32x4 *>(As + row * LDS_ROW + ((ch ^ st_swz) * 8)) = v;
    }
#pragma unroll
    for (int i = 0; i < B_CH; i++) {
      const int id = tid + i * NT, row = id >> 3, ch = id & 7;
      u32x4 v = qb[i];
      if (MASKED) v &= qm[i];
      *reinterpret_cast<u32x4 *>(Bs + row * LDS_ROW + ((ch ^ st_swz) * 8)) = v;
    }
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // Bias of the k_out this lane will hold in its accumulators: four
  // consecutive values per register group, fetched once, up front, as 8-byte
  // loads from clamped addresses (K is a multiple of 8, so a group of four is
  // inside the tensor or outside it as a whole; rows outside are never stored).
  half4 bias4[TM][4];
  {
    const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int k_out = m0 + wm0 + i * 32 + 8 * g + 4 * half;
        const half4 zero = {(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
        bias4[i][g] = biasg ? *reinterpret_cast<const half4 *>(biasg + (k_out < a.K ? k_out : 0)) : zero;
      }
  }

  // the second convolution's result, as it would have been stored: set aside when its steps are done
  floatx16 zacc[DUAL ? TM : 1][DUAL ? TN : 1];
  auto set_aside = [&]() __attribute__((always_inline)) {
    const _Float16 *__restrict__ bias2g = reinterpret_cast<const _Float16 *>(a.bias2);
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int k_out = m0 + wm0 + i * 32 + 8 * g + 4 * half;
        half4 b2 = {(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
        if (bias2g) b2 = *reinterpret_cast<const half4 *>(bias2g + (k_out < a.K ? k_out : 0));
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int e = 0; e < 4; e++) {
            zacc[DUAL ? i : 0][DUAL ? j : 0][4 * g + e] = (float)(_Float16)(acc[i][j][4 * g + e] + (float)b2[e]);
            acc[i][j][4 * g + e] = 0.f;
          }
      }
  };

  half8 fa[2][TM], fb[2][TN];
  auto read_frags = [&](int stage, half8 (&qa)[TM], half8 (&qb)[TN], int sub) {  // sub: which k16 of the step
    const _Float16 *As = smem + stage * STAGE, *Bs = As + BM * LDS_ROW;
#pragma unroll
    for (int i = 0; i < TM; i++)
      qa[i] = *reinterpret_cast<const half8 *>(As + (wm0 + i * 32 + l32) * LDS_ROW + (((2 * sub + half) ^ ld_swz) * 8));
#pragma unroll
    for (int j = 0; j < TN; j++)
      qb[j] = *reinterpret_cast<const half8 *>(Bs + (wn0 + j * 32 + l32) * LDS_ROW + (((2 * sub + half) ^ ld_swz) * 8));
  };
  auto mfma_frags = [&](const half8 (&qa)[TM], const half8 (&qb)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa[i], qb[j], acc[i][j], 0, 0, 0);
  };

  // prologue: steps 0 and 1 in flight, step 0 into LDS stage 0
  static_assert(DEPTH == 2, "the step sequence below is written for two register slots");
  load_step(ra[0], rb[0], rm[0]);
  if (ONE_STAGE ? FEW_STEPS > 1 : nk > 1) load_step(ra[1], rb[1], rm[1]);
  store_step(0, ra[0], rb[0], rm[0]);
  __syncthreads();

  // Step kt (register slot U = kt % 2, LDS stage U): refill slot U with step
  // kt + 2 if there is one; four k16 sub-steps, the operands of each read from
  // LDS while the MFMAs of the one before run; half way, step kt + 1 (if there
  // is one) goes from its slot into the other LDS stage (nobody reads that
  // stage during this step); one barrier.  The body has no branch, so the
  // scheduler is free to spread the loads, LDS traffic and address arithmetic
  // between the MFMAs.  Whether a step refills and whether it has a successor
  // are compile-time properties of its place in the sequence: nothing is
  // loaded or staged for steps past the end (a 1x1 layer over 64 channels is a
  // single step: it used to issue three steps' worth of loads).  (A ring of 4
  // register stages was measured and bought nothing over 2 on any ResNet-50 layer.)
  auto step = [&](auto slot_c, auto refill_c, auto next_c) {
    constexpr int U = decltype(slot_c)::value, S = U & 1, N = (U + 1) % DEPTH;
    constexpr bool REFILL = decltype(refill_c)::value, HAS_NEXT = decltype(next_c)::value;
    if constexpr (REFILL) load_step(ra[U], rb[U], rm[U]);
    if constexpr (KG == 1) {
      read_frags(S, fa[0], fb[0], 0);
      read_frags(S, fa[1], fb[1], 1);
      mfma_frags(fa[0], fb[0]);
      read_frags(S, fa[0], fb[0], 2);
      mfma_frags(fa[1], fb[1]);
      if constexpr (HAS_NEXT) store_step(S ^ 1, ra[N], rb[N], rm[N]);
      read_frags(S, fa[1], fb[1], 3);
      mfma_frags(fa[0], fb[0]);
      mfma_frags(fa[1], fb[1]);
    } else {  // this k group's half of the step: sub-steps 2 kg and 2 kg + 1
      read_frags(S, fa[0], fb[0], 2 * kg);
      read_frags(S, fa[1], fb[1], 2 * kg + 1);
      mfma_frags(fa[0], fb[0]);
      if constexpr (HAS_NEXT) store_step(S ^ 1, ra[N], rb[N], rm[N]);
      mfma_frags(fa[1], fb[1]);
    }
    __syncthreads();
  };
  using std::integral_constant;
  using std::true_type;
  using std::false_type;
  const integral_constant<int, 0> slot0{};
  const integral_constant<int, 1> slot1{};
  int kt = 0;
  if constexpr (!ONE_STAGE) {
    for (; kt + 4 <= nk; kt += 2) {  // both steps have a step two ahead to request
      step(slot0, true_type{}, true_type{});
      step(slot1, true_type{}, true_type{});
    }
  }
  const int rem = ONE_STAGE ? 0 : nk - kt;  // 1, 2 or 3
  if constexpr (ONE_STAGE) {
    // step T: its data goes from register slot T % 2 into the one stage (step 0's is there already), the
    // slot is refilled with step T + 2 if there is one, then the MFMAs read the stage
    auto turn = [&](auto t_c) {
      constexpr int T = decltype(t_c)::value, U = T & 1;
      if constexpr (DUAL && T == DUAL_FIRST) set_aside();
      if constexpr (T > 0) {
        store_step(0, ra[U], rb[U], rm[U]);
        __syncthreads();
      }
      if constexpr (T + 2 < FEW_STEPS) load_step(ra[U], rb[U], rm[U]);
      step(slot0, false_type{}, false_type{});  // reads stage 0, loads and stages nothing, ends on a barrier
    };
    turn(integral_constant<int, 0>{});
    if constexpr (FEW_STEPS > 1) turn(integral_constant<int, 1>{});
    if constexpr (FEW_STEPS > 2) turn(integral_constant<int, 2>{});
    if constexpr (FEW_STEPS > 3) turn(integral_constant<int, 3>{});
    if constexpr (FEW_STEPS > 4) turn(integral_constant<int, 4>{});
    if constexpr (FEW_STEPS > 5) turn(integral_constant<int, 5>{});
    static_assert(FEW_STEPS <= 6, "up to six turns are written out");
  } else if (rem == 3) {
    step(slot0, true_type{}, true_type{});
    step(slot1, false_type{}, true_type{});
    step(slot0, false_type{}, false_type{});
  } else if (rem == 2) {
    step(slot0, false_type{}, true_type{});
    step(slot1, false_type{}, false_type{});
  } else if (rem == 1) {
    step(slot0, false_type{}, false_type{});
  }

  // ---- epilogue: bias, activation, fp16, transpose through LDS ------------
  // register r of lane l in block (i, j): k_out = 8*(r/4) + 4*(l/32) + r%4,
  // pixel = l%32 -> four consecutive k_out per register group.
  if constexpr (KG == 2) {
    // the second k group hands its partial sums over through LDS (the step
    // loop ended on a barrier: nobody reads the operand stages any more)
    static_assert(4 * TM * TN * 16 * 64 * 2 <= SMEM, "partial sums must fit in the operand stages");
    float *red = reinterpret_cast<float *>(smem);
    if (kg == 1) {
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int r = 0; r < 16; r++) red[(((wave * TM + i) * TN + j) * 16 + r) * 64 + lane] = acc[i][j][r];
    }
    __syncthreads();
    if (kg == 0) {
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc[i][j][r] += red[(((wave * TM + i) * TN + j) * 16 + r) * 64 + lane];
    }
    __syncthreads();  // the output staging below reuses the same LDS
  }
  const _Float16 *__restrict__ Zg = reinterpret_cast<const _Float16 *>(a.Z);
  const int act_now = Zg ? DNNRT_ACT_IDENTITY : a.act;  // with a residual the activation comes after the sum
  _Float16 *Cs = smem;  // [BN pixels][CROW]
  // the residual chunks this thread will need, requested now (clamped
  // addresses) so that they arrive while the tile is staged through LDS
  constexpr int CH_PER_ROW = BM / 8, OUT_IT = BN * CH_PER_ROW / NT;
  half8 zpre[OUT_IT];
  if (Zg) {
#pragma unroll
    for (int it = 0; it < OUT_IT; it++) {
      const int id = tid + it * NT, row = id / CH_PER_ROW, ch = id - row * CH_PER_ROW;
      const int pix = min(n0 + row, NPQ - 1), k_out = min(m0 + ch * 8, a.K - 8);
      zpre[it] = *reinterpret_cast<const half8 *>(Zg + (int64_t)pix * a.K + k_out);
    }
  }
  // The activation mode is the same for the whole launch: each loop below is
  // instantiated per mode and picked once, so the per-element code is that of
  // the one mode (ReLU: a single max).
  auto per_mode = [&](int mode, auto &&body) {
    switch (mode) {
      case DNNRT_ACT_RELU: body(std::integral_constant<int, DNNRT_ACT_RELU>{}); break;
      case DNNRT_ACT_CLIPPED_RELU: body(std::integral_constant<int, DNNRT_ACT_CLIPPED_RELU>{}); break;
      case DNNRT_ACT_LEAKY_RELU: body(std::integral_constant<int, DNNRT_ACT_LEAKY_RELU>{}); break;
      default: body(std::integral_constant<int, DNNRT_ACT_IDENTITY>{}); break;
    }
  };
  if (KG == 1 || kg == 0)
    per_mode(act_now, [&](auto mode_c) {
      constexpr int MODE = decltype(mode_c)::value;
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
              if (DUAL)  // conv + bias rounded as a convolution of its own would store it, then the sum in fp32
                o[e] = (_Float16)apply_act((float)(_Float16)(acc[i][j][4 * g + e] + (float)bias4[i][g][e]) +
                                               zacc[DUAL ? i : 0][DUAL ? j : 0][4 * g + e], MODE, a.act_coef);
              else
                o[e] = (_Float16)apply_act(acc[i][j][4 * g + e] + (float)bias4[i][g][e], MODE, a.act_coef);
            }
            *reinterpret_cast<half4 *>(Cs + (wn0 + j * 32 + l32) * CROW + kl) = o;
          }
    });
  __syncthreads();
  _Float16 *__restrict__ Yg = reinterpret_cast<_Float16 *>(a.Y);
  per_mode(Zg ? a.act : DNNRT_ACT_IDENTITY, [&](auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
    for (int it = 0; it < OUT_IT; it++) {
      const int id = tid + it * NT;
      const int row = id / CH_PER_ROW, ch = id - row * CH_PER_ROW;
      const int pix = n0 + row, k_out = m0 + ch * 8;
      if (pix < NPQ && k_out < a.K) {
        half8 o = *reinterpret_cast<const half8 *>(Cs + row * CROW + ch * 8);
        if (Zg) {
          // conv + bias was rounded to fp16 above, as a separate convolution
          // would have stored it; the residual sum follows in fp32
          const half8 zv = zpre[it];
#pragma unroll
          for (int e = 0; e < 8; e++) o[e] = (_Float16)apply_act((float)o[e] + (float)zv[e], MODE, a.act_coef);
        }
        *reinterpret_cast<half8 *>(Yg + (int64_t)pix * a.K + k_out) = o;
      }
    }
  });
}

// ---- generic kernel ---------------------------------------------------------
// 64 k_out x 64 pixels, four wavefronts of 32x32 each, BK = 32, single LDS
// stage, element-wise gathers.  Layout flags are runtime values.
__global__ __launch_bounds__(256) void conv_f16_generic_kernel(const ConvF16Args a, const int in_nchw,
                                                               const int out_nhwc, const int w_krsc) {
  __shared__ __attribute__((aligned(16))) _Float16 As[64 * LDS_ROW_G];
  __shared__ __attribute__((aligned(16))) _Float16 Bs[64 * LDS_ROW_G];
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
      As[lrow * LDS_ROW_G + lk0 + e] = av;
      Bs[lrow * LDS_ROW_G + lk0 + e] = bv;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < BK16; ks += 16) {
      const half8 av = *reinterpret_cast<const half8 *>(As + (wm0 + l32) * LDS_ROW_G + ks + half * 8);
      const half8 bv = *reinterpret_cast<const half8 *>(Bs + (wn0 + l32) * LDS_ROW_G + ks + half * 8);
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
    v = apply_act(v, a.act, a.act_coef);
    Yg[off] = (_Float16)v;
  }
}

// ---- depthwise, channels-last -------------------------------------------------
// One input channel per filter and as many filters as channels: a memory-bound elementwise operation.  A thread owns
// eight consecutive channels of one output pixel: per tap one 16-byte load of the input and the tap's eight weights
// from LDS, where the workgroup keeps the whole filter transposed to [tap][channel] (its global layout, K,R,S with
// one channel, is the same whether the program calls it K,C,R,S or K,R,S,C); fp32 accumulation, bias, residual and
// activation as in every fp16 convolution (conv + bias rounded to fp16 before the residual is added).
__global__ __launch_bounds__(256) void dwconv_f16_nhwc_kernel(const ConvF16Args a, const int64_t total) {
  extern __shared__ __attribute__((aligned(16))) _Float16 wt[];  // [R * S][K]
  const int RS = a.R * a.S, K8 = a.K >> 3;
  const _Float16 *__restrict__ Wg = reinterpret_cast<const _Float16 *>(a.Wt);
  for (int e = threadIdx.x; e < a.K * RS; e += 256) {
    const int k = e / RS, tap = e - k * RS;
    wt[tap * a.K + k] = Wg[e];
  }
  __syncthreads();
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int c8 = (int)(i % K8);
  const int64_t pix = i / K8;
  const int q = (int)(pix % a.Q);
  const int64_t t = pix / a.Q;
  const int p = (int)(t % a.P), n = (int)(t / a.P);
  const int ih0 = p * a.sh - a.ph, iw0 = q * a.sw - a.pw;
  const _Float16 *__restrict__ Xg = reinterpret_cast<const _Float16 *>(a.X) + (int64_t)n * a.H * a.W * a.C + 8 * c8;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; e++) acc[e] = 0.f;
  for (int r = 0; r < a.R; r++) {
    const int ih = ih0 + r;
    if ((unsigned)ih >= (unsigned)a.H) continue;
    for (int s = 0; s < a.S; s++) {
      const int iw = iw0 + s;
      if ((unsigned)iw >= (unsigned)a.W) continue;
      const half8 xv = *reinterpret_cast<const half8 *>(Xg + ((int64_t)ih * a.W + iw) * a.C);
      const half8 wv = *reinterpret_cast<const half8 *>(wt + (r * a.S + s) * a.K + 8 * c8);
#pragma unroll
      for (int e = 0; e < 8; e++) acc[e] = fmaf((float)xv[e], (float)wv[e], acc[e]);
    }
  }
  const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
  const _Float16 *__restrict__ Zg = reinterpret_cast<const _Float16 *>(a.Z);
  const int64_t off = pix * a.K + 8 * c8;
  half8 out;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    float v = acc[e];
    if (biasg) v += (float)biasg[8 * c8 + e];
    if (Zg) v = (float)(_Float16)v + (float)Zg[off + e];
    out[e] = (_Float16)apply_act(v, a.act, a.act_coef);
  }
  *reinterpret_cast<half8 *>(reinterpret_cast<_Float16 *>(a.Y) + off) = out;
}

// The 3x3 depthwise layers (stride 1 or 2) again, without LDS and without a barrier: the thread's 72 filter values
// are nine 16-byte loads from the K x 3 x 3 filter as it lies in memory (eight filters are contiguous), the loops
// over the taps are unrolled, and the thread index is taken apart with multiply-high divisions.  A thread computes
// PIX neighbouring pixels of an output row, which share their input vectors: 3 x (PIX - 1) x STRIDE + 9 loads
// instead of 9 PIX (the kernel is bound by the requests it sends to L2, not by its arithmetic: without the FMAs
// it runs 13 % faster, no more).  Every load is unconditional, from a clamped address, and a tap in the padding
// has its value replaced by zero: a load under a divergent branch is waited for before the next one is issued,
// which with more than one pixel per thread costs more than the shared loads give.  WAVES: the wavefronts per
// SIMD the register allocation aims at.  MobileNetV2 at batch 64, 144 channels at 56 x 56, stride 1: 65 us with
// one pixel per thread (six wavefronts), 54 with two (five), 49 with three (four), 45.5 with four (four; 47.8 at
// three); the stride-2 layers gain less and run with two pixels (four wavefronts).  Taps are summed in the order
// of the kernel above.
template <int STRIDE, int PIX, int WAVES>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WAVES, WAVES))) void dwconv3x3_f16_nhwc_kernel(const ConvF16Args a, const int total, const int qstrips, const unsigned magic_k8,
                                                                 const unsigned magic_qs, const unsigned magic_p) {
  const int i = (int)(blockIdx.x * 256 + threadIdx.x);
  if (i >= total) return;
  constexpr int COLS = 3 + (PIX - 1) * STRIDE;
  const int K8 = a.K >> 3;
  int t = div_magic(i, K8, magic_k8);
  const int c8 = i - t * K8;
  const int row = div_magic(t, qstrips, magic_qs);
  const int q0 = PIX * (t - row * qstrips);
  const int n = div_magic(row, a.P, magic_p), p = row - n * a.P;
  const _Float16 *__restrict__ Wg = reinterpret_cast<const _Float16 *>(a.Wt) + (int64_t)c8 * 72;
  half8 wraw[9];  // filter 8 c8 + e, tap t: element 9 e + t
#pragma unroll
  for (int j = 0; j < 9; j++) wraw[j] = *reinterpret_cast<const half8 *>(Wg + 8 * j);
  const _Float16 *__restrict__ Xg = reinterpret_cast<const _Float16 *>(a.X) + (int64_t)n * a.H * a.W * a.C + 8 * c8;
  const int ih0 = p * STRIDE - a.ph, iw0 = q0 * STRIDE - a.pw;
  half8 zero8;
#pragma unroll
  for (int e = 0; e < 8; e++) zero8[e] = (_Float16)0.f;
  float acc[PIX][8];
#pragma unroll
  for (int j = 0; j < PIX; j++)
#pragma unroll
    for (int e = 0; e < 8; e++) acc[j][e] = 0.f;
#pragma unroll
  for (int r = 0; r < 3; r++) {
    const int ih = ih0 + r;
    const bool row_ok = (unsigned)ih < (unsigned)a.H;
    half8 xv[COLS];
#pragma unroll
    for (int c = 0; c < COLS; c++) {
      const int iw = iw0 + c;
      const bool ok = row_ok && (unsigned)iw < (unsigned)a.W;
      // unconditional, from a clamped address: a load under a branch is waited for before the next one is issued
      const int ihc = min(max(ih, 0), a.H - 1), iwc = min(max(iw, 0), a.W - 1);
      const half8 v = *reinterpret_cast<const half8 *>(Xg + ((int64_t)ihc * a.W + iwc) * a.C);
      xv[c] = ok ? v : zero8;
    }
#pragma unroll
    for (int j = 0; j < PIX; j++)
#pragma unroll
      for (int s = 0; s < 3; s++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const int at = 9 * e + 3 * r + s;
          acc[j][e] = fmaf((float)xv[j * STRIDE + s][e], (float)wraw[at >> 3][at & 7], acc[j][e]);
        }
  }
  const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
  const _Float16 *Zg = reinterpret_cast<const _Float16 *>(a.Z);  // may be Y itself: a thread reads an element, then writes it
  auto finish = [&](auto mode_c) {  // one copy per activation mode, picked once
    constexpr int MODE = decltype(mode_c)::value;
    float bias8[8];
#pragma unroll
    for (int e = 0; e < 8; e++) bias8[e] = biasg ? (float)biasg[8 * c8 + e] : 0.f;
#pragma unroll
    for (int j = 0; j < PIX; j++) {
      if (q0 + j >= a.Q) break;
      const int64_t off = ((((int64_t)n * a.P + p) * a.Q) + q0 + j) * a.K + 8 * c8;
      half8 z8, out;
      if (Zg) z8 = *reinterpret_cast<const half8 *>(Zg + off);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float v = acc[j][e] + bias8[e];
        if (Zg) v = (float)(_Float16)v + (float)z8[e];
        out[e] = (_Float16)apply_act(v, MODE, a.act_coef);
      }
      *reinterpret_cast<half8 *>(reinterpret_cast<_Float16 *>(a.Y) + off) = out;
    }
  };
  by_act_mode(a.act, finish);
}

static bool dwconv_f16_applies(const ConvF16Args &a) {
  return a.format == DNNRT_NHWC && a.group > 1 && a.group == a.C && a.K == a.C && a.Cg == 1 && a.C % 8 == 0 &&
         (int64_t)a.K * a.R * a.S * 2 <= 48 * 1024 && aligned16(a.X) && aligned16(a.Y) && aligned16(a.Z);
}

// Y = act(fp16(conv(X, W) + bias) + fp16(conv(X2, W2) + bias2)): `a` with its X2 / Wt2 / bias2 / C2 / H2 / W2 / sh2 / sw2
// fields set.  Both convolutions 1x1 without padding onto the same N x K x P x Q result (dual_conv_applies).
bool dual_conv_applies(const ConvF16Args &a) {
  return a.format == DNNRT_NHWC && a.group == 1 && a.R == 1 && a.S == 1 && a.ph == 0 && a.pw == 0 && a.Z == nullptr && a.X2 && a.Wt2 &&
         a.C % 64 == 0 && a.C2 % 64 == 0 && a.K % 8 == 0 && (a.H2 - 1) / a.sh2 + 1 == a.P && (a.W2 - 1) / a.sw2 + 1 == a.Q &&
         (int64_t)a.N * a.H * a.W * a.C < (1ll << 31) && (int64_t)a.N * a.H2 * a.W2 * a.C2 < (1ll << 31) &&
         (int64_t)a.K * a.C < (1ll << 31) && (int64_t)a.K * a.C2 < (1ll << 31) && aligned16(a.X) && aligned16(a.Wt) && aligned16(a.Y) &&
         aligned16(a.X2) && aligned16(a.Wt2) && (reinterpret_cast<uintptr_t>(a.bias) & 7u) == 0 &&
         (reinterpret_cast<uintptr_t>(a.bias2) & 7u) == 0;
}

bool launch_conv_f16_dual(const dnnrtContext *ctx, const ConvF16Args &a) {
  const int64_t NPQ = (int64_t)a.N * a.P * a.Q;
  ConvF16Args am = a;
  am.magic_pq = magic_of(a.P * a.Q);
  am.magic_q = magic_of(a.Q);
  auto tiles_of = [&](int bm, int bn) { return ceil_div(a.K, bm) * ceil_div(NPQ, bn); };
#define LAUNCH_DUAL(BM_, BN_, MINW_, FEW_, FIRST_)                                                                                      \
  do {                                                                                                                         \
    const int64_t tiles = tiles_of(BM_, BN_);                                                                                  \
    if (tiles + 8 > INT32_MAX) { set_error("conv(fp16): too many tiles"); return false; }                                      \
    const unsigned grid = (unsigned)(ceil_div(tiles, 8) * 8);                                                                  \
    if (NPQ % BN_ != 0 || a.K % BM_ != 0)                                                                                      \
      hipLaunchKernelGGL((conv_f16_nhwc_kernel<BM_, BN_, 2, 2, 2, MINW_, true, 1, FEW_, true, FIRST_>), dim3(grid), dim3(256), 0,  \
                         ctx->stream, am, (int)tiles);                                                                         \
    else                                                                                                                       \
      hipLaunchKernelGGL((conv_f16_nhwc_kernel<BM_, BN_, 2, 2, 2, MINW_, false, 1, FEW_, true, FIRST_>), dim3(grid), dim3(256), 0, \
                         ctx->stream, am, (int)tiles);                                                                         \
  } while (0)
  // Two steps in all (64 + 64 channels, the first block of a ResNet), or six (256 strided + 128, the first block of its
  // second stage): the single-stage 64 x 64 tiles that such short reductions run best on; 89 -> 56 us and 55 -> 50 us
  // at batch 64, where the pair is bound by the bytes the shortcut's result would be written and read with.  Longer
  // reductions were slower this way than as two calls (on plain 64 x 64 tiles, and on 128 x 128 ones, where the
  // second accumulator set no longer fits 256 registers: 53 vs 45 us on 512 + 256 -> 1024 channels at 14 x 14, 43 vs
  // 41 us on the last stage); the entry point runs those as the two calls.
  if (a.C == 64 && a.C2 == 64) LAUNCH_DUAL(64, 64, 2, 2, 1);
  else if (a.C == 128 && a.C2 == 256) LAUNCH_DUAL(64, 64, 2, 6, 4);
  else { set_error("conv(fp16): the two-convolution kernel takes 64 + 64 or 128 + 256 input channels"); return false; }
#undef LAUNCH_DUAL
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("conv(fp16): launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

bool launch_conv_f16(const dnnrtContext *ctx, const ConvF16Args &a) {
  bool stem_launched = false;
  if (!launch_conv_f16_stem(ctx, a, stem_launched)) return false;
  if (stem_launched) return true;
  bool first_launched = false;
  if (!launch_conv_f16_first(ctx, a, first_launched)) return false;
  if (first_launched) return true;
  bool few_launched = false;
  if (!launch_conv_f16_fewpix(ctx, a, few_launched)) return false;
  if (few_launched) return true;
  const int64_t NPQ = (int64_t)a.N * a.P * a.Q;
  const bool fast = a.format == DNNRT_NHWC && a.group == 1 && a.C % 64 == 0 && a.K % 8 == 0 && a.R * a.S <= 32 &&
                    (int64_t)a.N * a.H * a.W * a.C < (1ll << 31) && (int64_t)a.K * a.C * a.R * a.S < (1ll << 31) &&
                    aligned16(a.X) && aligned16(a.Wt) && aligned16(a.Y) && aligned16(a.Z) &&
                    (reinterpret_cast<uintptr_t>(a.bias) & 7u) == 0;
  if (fast) {
    ConvF16Args am = a;
    am.magic_pq = magic_of(a.P * a.Q);
    am.magic_q = magic_of(a.Q);
    auto tiles_of = [&](int bm, int bn) { return ceil_div(a.K, bm) * ceil_div(NPQ, bn); };
    const bool pad = a.ph != 0 || a.pw != 0;
#define LAUNCH_FAST(BM_, BN_, WM_, WN_, DEPTH_, MIN_WAVES_, KG_, FEW_)                                                  \
  do {                                                                                                     \
    const int64_t tiles = tiles_of(BM_, BN_);                                                              \
    if (tiles + 8 > INT32_MAX) { set_error("conv(fp16): too many tiles"); return false; }                  \
    const unsigned grid = (unsigned)(ceil_div(tiles, 8) * 8);                                              \
    if (pad || NPQ % BN_ != 0 || a.K % BM_ != 0)                                                           \
      hipLaunchKernelGGL((conv_f16_nhwc_kernel<BM_, BN_, WM_, WN_, DEPTH_, MIN_WAVES_, true, KG_, FEW_>), dim3(grid), \
                         dim3(256 * KG_), 0, ctx->stream, am, (int)tiles);                                 \
    else                                                                                                   \
      hipLaunchKernelGGL((conv_f16_nhwc_kernel<BM_, BN_, WM_, WN_, DEPTH_, MIN_WAVES_, false, KG_, FEW_>), dim3(grid), \
                         dim3(256 * KG_), 0, ctx->stream, am, (int)tiles);                                 \
  } while (0)
    // Tile choice, from per-layer timings of the ResNet-50 shapes at batch 64
    // (14.8 GFLOP 3x3 layers run in 25-35 us, 1x1 layers near their HBM time):
    // 128x128 when there are enough tiles for more than one workgroup per CU;
    // with about one per CU, the eight-wavefront 128x128 variant, which keeps
    // two wavefronts on every SIMD; with fewer still, 64x64 (see below); 64x64 when K_out <= 64 (64x128, case 15, was ahead on
    // its 3x3 layers until the step sequence stopped loading past the end and
    // fell behind after: 37 vs 33 us;
    // walking an XCD's run of tiles pixel tiles first instead of k_out tiles
    // first, so that an XCD touches a slice of a large filter only, changed
    // nothing on the 7x7 layers).
    // 0 = automatic; > 0 forced (tuning and tests); < 0: that variant where it can run the problem, else automatic
    // the handle's forced variant (tests, sweeps) goes before the call's own (its `algo` operand, a tuned program)
    const int tile_sel = ctx->f16_tile ? ctx->f16_tile : -a.variant;
    int sel = tile_sel;
    if (sel < 0) {
      const int want = -sel, steps = a.R * a.S * (a.C / BKF);
      bool can = true;
      if ((want >= 31 && want <= 40) || (want >= 60 && want <= 69)) can = dma_conv_applies(am);
      else if (want >= 41 && want <= 59) can = patch_conv_applies(am) && patch_variant_fits(am, want);
      else if (want == 70) can = c64_conv_applies(am);
      else if (want == 18) can = steps <= 4;
      else if (want == 17) can = steps == 1 || steps == 2 || steps == 4;
      sel = can ? want : 0;
    }
    if (sel == 0) {
      const int nk = a.R * a.S * (a.C / BKF);
      const int64_t t128 = tiles_of(128, 128), cus = ctx->num_cu;
      const bool dma_ok = dma_conv_applies(am);
      const int patch_cap = patch_conv_applies(am) ? patch_conv_capacity(am, 128) : 0;
      const bool one_per_cu = 5 * t128 >= 3 * cus && 4 * t128 < 5 * cus, fewer = 5 * t128 < 3 * cus;
      // 3x3 stride-1 layers with up to two 128x128 tiles per CU (28x28, 14x14 and 7x7 images at batch 64): the
      // input patch stays in LDS (inside the network 33 -> 24 us on 256 -> 256 at 14x14, 41 -> 27 us on 512 -> 512
      // at 7x7, where 64-row tiles give twice the workgroups); with more tiles per CU the im2col tiles are as fast.
      // Inside a network the filters come from HBM (activations pass through the caches in between), so the
      // variants that keep four (128-row tiles) or six (64-row tiles) filter steps in flight are the ones
      // chosen: 27 -> 25 us and 36 -> 26 us against two steps in flight.  With 128-row tiles the eight wavefronts
      // split the tile (two rows by four columns of 64 x 32 blocks) rather than the reduction: no partial sums to
      // hand over at the end (25 -> 22 us on 256 -> 256 at 14x14, 28.3 -> 26.5 us on 128 -> 128 at 28x28).
      // 64 -> 64 channels, 3x3, on images wide enough to fill the persistent kernel's two-row tiles and with several
      // tiles per workgroup: its filter stays in registers (inside the network 36 -> 27.5 us at 56x56, batch 64)
      const int64_t c64_tiles = (int64_t)a.N * ((a.H + 1) / 2) * ceil_div(a.K, 64);
      if (c64_conv_applies(am) && 2 * a.W >= 96 && c64_tiles >= 4 * cus) sel = 70;
      else if (patch_cap && 5 * t128 >= 3 * cus && t128 < 2 * cus) sel = patch_cap == 256 ? 54 : 57;
      else if (patch_cap && fewer) sel = patch_cap == 256 ? 47 : 49;
      else if (nk <= 4) sel = 18;  // up to four steps (1x1 over up to 256 channels): the single-stage 64x64 variant
                              // (27 vs 34 us on 64 -> 256 at 56x56, 22.6 vs 26.6 on 128 -> 512 at 28x28, 18.3 vs 21.7 on 256 -> 1024 at 14x14)
      else if (a.K <= 64) sel = 4;
      // From about one 128x128 tile per CU to two (14x14 layers and the long reductions of the 28x28 layers at
      // batch 64): operands straight into a four-stage LDS ring, two steps in flight, on eight wavefronts: with
      // two wavefronts per SIMD one computes while the other waits for its operands (inside the network, against
      // the same ring on four wavefronts: 17.5 -> 14.8 us on 1x1 1024 -> 256 at 14x14, 29 -> 24 us on the strided
      // 3x3 256 -> 256, 26 -> 24.5 us on 1x1 1024 -> 512; against the register-staged 128x128 tiles 29.5 -> 28.3 us
      // on the 3x3 layers over 128 channels at 28x28).
      else if (dma_ok && 5 * t128 >= 3 * cus && t128 < 2 * cus && (one_per_cu || nk >= 16)) sel = 64;
      else if (4 * t128 >= 5 * cus) sel = 3;
      else if (one_per_cu) sel = 12;
      // Fewer 128x128 tiles than that (7x7 layers at batch 64): 64-row tiles on eight wavefronts (1x1 2048 -> 512:
      // 20.5 -> 17 us inside the network, strided 3x3 512 -> 512: 35 -> 30 us); short reductions keep the 64x64 tiles.
      else sel = dma_ok && nk >= 8 ? 66 : 4;
    }
    if ((sel >= 31 && sel <= 40) || (sel >= 60 && sel <= 69)) {
      if (!dma_conv_applies(am)) { set_error("conv(fp16): tile %d needs tensors below 2 GiB", sel); return false; }
      if (!launch_conv_f16_dma(ctx, am, sel)) return false;
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) { set_error("conv(fp16): launch failed: %s", hipGetErrorString(e)); return false; }
      return true;
    }
    if (sel == 70) {
      if (!c64_conv_applies(am)) { set_error("conv(fp16): tile 70 is for 3x3 stride-1 pad-1 layers over 64 channels, at most 62 pixels wide, without a residual"); return false; }
      if (!launch_conv_f16_c64(ctx, am)) return false;
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) { set_error("conv(fp16): launch failed: %s", hipGetErrorString(e)); return false; }
      return true;
    }
    if (sel >= 41 && sel <= 59) {
      if (!patch_conv_applies(am)) { set_error("conv(fp16): tile %d is for 3x3 stride-1 pad-1 layers over 128 channels or more", sel); return false; }
      if (!launch_conv_f16_patch(ctx, am, sel)) return false;
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) { set_error("conv(fp16): launch failed: %s", hipGetErrorString(e)); return false; }
      return true;
    }
    switch (sel) {
      case 3: LAUNCH_FAST(128, 128, 2, 2, 2, 2, 1, 0); break;
      case 11: LAUNCH_FAST(128, 64, 2, 2, 2, 1, 2, 0); break;
      case 12: LAUNCH_FAST(128, 128, 2, 2, 2, 1, 2, 0); break;
      case 15: LAUNCH_FAST(64, 128, 2, 2, 2, 2, 1, 0); break;
      case 18: {  // 64 x 64, one LDS stage, for reductions of one to four steps
        const int steps = a.R * a.S * (a.C / BKF);
        if (steps == 1) LAUNCH_FAST(64, 64, 2, 2, 2, 2, 1, 1);
        else if (steps == 2) LAUNCH_FAST(64, 64, 2, 2, 2, 2, 1, 2);
        else if (steps == 3) LAUNCH_FAST(64, 64, 2, 2, 2, 2, 1, 3);
        else if (steps == 4) LAUNCH_FAST(64, 64, 2, 2, 2, 2, 1, 4);
        else { set_error("conv(fp16): tile 18 is for reductions of one to four steps"); return false; }
        break;
      }
      case 17: {  // the same with 128 x 64 tiles
        const int steps = a.R * a.S * (a.C / BKF);
        if (steps == 1) LAUNCH_FAST(128, 64, 2, 2, 2, 2, 1, 1);
        else if (steps == 2) LAUNCH_FAST(128, 64, 2, 2, 2, 2, 1, 2);
        else if (steps == 4) LAUNCH_FAST(128, 64, 2, 2, 2, 2, 1, 4);
        else { set_error("conv(fp16): tile 17 is for reductions of one, two or four steps"); return false; }
        break;
      }
      default: LAUNCH_FAST(64, 64, 2, 2, 2, 2, 1, 0); break;
    }
#undef LAUNCH_FAST
  } else if (pointwise_conv_applies(a)) {
    return launch_conv_f16_pointwise(ctx, a);
  } else if (dwconv_f16_applies(a)) {
    const int64_t total = NPQ * (a.K / 8), blocks = ceil_div(total, 256);
    if (blocks > INT32_MAX) { set_error("conv(fp16): depthwise output too large"); return false; }
    if (a.R == 3 && a.S == 3 && a.sh == a.sw && (a.sh == 1 || a.sh == 2) && aligned16(a.Wt) && total + 256 < (1ll << 31)) {
      const int pix = a.sh == 1 ? 4 : 2;  // pixels of an output row per thread
      const int qstrips = (a.Q + pix - 1) / pix;
      const int64_t threads = (int64_t)a.N * a.P * qstrips * (a.K / 8);
      const unsigned grid = (unsigned)ceil_div(threads, 256);
      const unsigned m_k8 = magic_of(a.K / 8), m_qs = magic_of(qstrips), m_p = magic_of(a.P);
#define DW_LAUNCH(ST, PX, WV) hipLaunchKernelGGL((dwconv3x3_f16_nhwc_kernel<ST, PX, WV>), dim3(grid), dim3(256), 0, ctx->stream, a, (int)threads, qstrips, m_k8, m_qs, m_p)
      if (a.sh == 1) DW_LAUNCH(1, 4, 4);
      else DW_LAUNCH(2, 2, 4);
#undef DW_LAUNCH
    } else
    hipLaunchKernelGGL(dwconv_f16_nhwc_kernel, dim3((unsigned)blocks), dim3(256), (size_t)a.K * a.R * a.S * 2, ctx->stream, a, total);
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
