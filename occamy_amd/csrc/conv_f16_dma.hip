// fp16 channels-last convolution whose operands go from global memory
// straight into LDS (buffer_load_dwordx4 ... lds), without passing through
// vector registers.
//
// GEMM view, operand order and LDS layout are those of conv_f16.hip:
// D[k_out, pixel] = sum_k Wt[k_out, k] * Xcol[k, pixel] with k ordered
// (r, s, c), filters K,R,S,C, activations N,H,W,C, steps of 64 k so that a
// row's slice of a step is one 128-byte line, chunk c of row r kept at
// position c ^ ((r >> 1) & 7) of its LDS row.
//
// What is different is how a step gets there.  One buffer load with the LDS
// bit set moves 16 bytes per lane to LDS address M0 + 16 * lane: a wavefront
// fills eight consecutive 128-byte rows per instruction, and which global
// chunk lands in which slot is decided by the lane's buffer offset alone, so
// the XOR placement costs nothing.  Out-of-range offsets read as zeros:
// padding taps, pixels past the end of the tensor and filters past K_out are
// lanes whose offset has bit 31 set (tensors are kept below 2 GiB).  A step
// therefore costs no register, no LDS store instruction and no masking
// arithmetic; per lane and step what is left is three integer operations per
// padded chunk (none without padding: the tap offset rides in the scalar
// offset of the instruction).
//
// Pipeline: a ring of NS LDS stages, NS - 2 steps in flight beyond the one
// being computed, one barrier per step, waits by exact count (vmcnt) so that
// only the step about to be read has to have landed; within a step, fragment
// reads, MFMA groups and the next loads alternate in a pinned order.
#include "conv_f16.h"

#include <type_traits>

namespace dnnrt {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void *lds_ptr;

[[maybe_unused]] constexpr unsigned DMA_OUT_OF_RANGE = 0x80000000u;  // at or above every num_records used here: reads as zeros

// s_waitcnt that waits for the vector-memory counter only (gfx9 encoding:
// vmcnt in bits 3:0 and 15:14, expcnt 6:4 and lgkmcnt 11:8 left at "any").
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// A barrier the compiler neither adds waits to (__syncthreads() would wait
// for every outstanding load, the prefetched steps included) nor moves LDS
// accesses across.
__device__ __forceinline__ void ring_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// BM k_out x BN pixels per workgroup, WM x WN wavefronts each owning
// (BM / WM) x (BN / WN) of it as 32x32 MFMA blocks, NS LDS stages.
// MASKED: some lane of some step may have to read zeros in place of an
// activation (padding, or pixel rows past the end of the tensor).
// DUAL: two 1x1 convolutions without padding onto the same result as ONE reduction (a residual block's projection
// shortcut and its last convolution): the steps over the second convolution's channels (X2, Wt2) come first, then
// those over the first one's; a step differs from another only in which tensors and per-lane offsets its loads
// use.  The sum of both reductions and both biases is formed in fp32 and rounded once.
template <int BM, int BN, int WM, int WN, int NS, bool MASKED, bool DUAL = false>
__global__ __launch_bounds__(64 * WM * WN) void conv_f16_dma_kernel(const ConvF16Args a, const int tiles_total) {
  // The buffer-resource type exists for the device target only: the host pass, which needs just the launch stub,
  // would silently drop a kernel whose body it cannot type-check.
#if __HIP_DEVICE_COMPILE__
  constexpr int NW = WM * WN, NT = 64 * NW;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int A_L = BM / 8 / NW, B_L = BN / 8 / NW;  // loads (8 rows each) per wavefront and step
  constexpr int L = A_L + B_L;
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0 && TM >= 1 && TN >= 1, "tile does not divide over the wavefronts");
  static_assert(NS >= 3, "ring depth");
  constexpr int STAGE = (BM + BN) * 128;  // bytes
  constexpr int CROW = BM + 8;            // halfs per row of the output staging tile
  static_assert(BN * CROW * 2 <= NS * STAGE, "the output tile is staged in the operand ring");
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int per_xcd = (tiles_total + 7) >> 3;
  const int tile = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
  if (tile >= tiles_total) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, half = lane >> 5;
  const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);

  const int tiles_m = (a.K + BM - 1) / BM;
  const int tile_n = tile / tiles_m, tile_m = tile - tile_n * tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int NPQ = a.N * a.P * a.Q, PQ = a.P * a.Q;
  const int CRS = a.C * a.R * a.S;

  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.Wt), 0, 2 * a.K * CRS, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_x =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.X), 0, 2 * a.N * a.H * a.W * a.C, 0x00020000);

  // ---- loader constants --------------------------------------------------
  // Load i of this wavefront fills rows 8 * (wave + i * NW) .. + 7 of the A
  // (or B) part of a stage; lane -> (row, slot); the chunk that belongs in
  // that slot is slot ^ ((row >> 1) & 7).
  unsigned a_off[A_L];
#pragma unroll
  for (int i = 0; i < A_L; i++) {
    const int row = 8 * (wave + i * NW) + (lane >> 3), ch = (lane & 7) ^ ((row >> 1) & 7);
    const int k_out = m0 + row;
    a_off[i] = k_out < a.K ? 2u * (unsigned)(k_out * CRS + ch * 8) : DMA_OUT_OF_RANGE;
  }
  // B (im2col): a lane's chunk belongs to one output pixel.  b_base is the
  // byte offset of tap (0, 0), channel chunk ch (negative inside the padding);
  // bit (r * S + s) of b_out says that tap (r, s) reads OUTSIDE the image.
  int b_base[B_L];
  unsigned b_out[B_L];
#pragma unroll
  for (int i = 0; i < B_L; i++) {
    const int row = 8 * (wave + i * NW) + (lane >> 3), ch = (lane & 7) ^ ((row >> 1) & 7);
    const int pix = n0 + row;
    const bool ok = pix < NPQ;
    const int n = ok ? div_magic(pix, PQ, a.magic_pq) : 0;
    const int pq = ok ? pix - n * PQ : 0;
    const int p = div_magic(pq, a.Q, a.magic_q), q = pq - p * a.Q;
    const int ih0 = p * a.sh - a.ph, iw0 = q * a.sw - a.pw;
    b_base[i] = 2 * (((n * a.H + ih0) * a.W + iw0) * a.C + ch * 8);
    unsigned in = 0;
    if (MASKED && ok) {
      const int r_lo = max(0, -ih0), r_hi = min(a.R, a.H - ih0);
      const int s_lo = max(0, -iw0), s_hi = min(a.S, a.W - iw0);
      const unsigned row_bits = s_hi > s_lo ? ((1u << (s_hi - s_lo)) - 1u) << s_lo : 0u;
      for (int r = 0; r < a.R; r++)
        if (r >= r_lo && r < r_hi) in |= row_bits << (r * a.S);
    }
    b_out[i] = ~in;
  }

  // DUAL: the same for the second convolution (1x1, no padding: one tap, always inside; a pixel past the end of the
  // tensor is an out-of-range offset, and so it is for the first convolution in this form)
  [[maybe_unused]] unsigned a2_off[DUAL ? A_L : 1], b2_base[DUAL ? B_L : 1];
  [[maybe_unused]] __amdgpu_buffer_rsrc_t rsrc_w2 = rsrc_w, rsrc_x2 = rsrc_x;
  if constexpr (DUAL) {
    rsrc_w2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.Wt2), 0, 2 * a.K * a.C2, 0x00020000);
    rsrc_x2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.X2), 0, 2 * a.N * a.H2 * a.W2 * a.C2, 0x00020000);
#pragma unroll
    for (int i = 0; i < A_L; i++) {
      const int row = 8 * (wave + i * NW) + (lane >> 3), ch = (lane & 7) ^ ((row >> 1) & 7);
      const int k_out = m0 + row;
      a2_off[i] = k_out < a.K ? 2u * (unsigned)(k_out * a.C2 + ch * 8) : DMA_OUT_OF_RANGE;
    }
#pragma unroll
    for (int i = 0; i < B_L; i++) {
      const int row = 8 * (wave + i * NW) + (lane >> 3), ch = (lane & 7) ^ ((row >> 1) & 7);
      const int pix = n0 + row;
      const bool ok = pix < NPQ;
      const int n = ok ? div_magic(pix, PQ, a.magic_pq) : 0;
      const int pq = ok ? pix - n * PQ : 0;
      const int p = div_magic(pq, a.Q, a.magic_q), q = pq - p * a.Q;
      b2_base[i] = ok ? 2u * (unsigned)(((n * a.H2 + p * a.sh2) * a.W2 + q * a.sw2) * a.C2 + ch * 8) : DMA_OUT_OF_RANGE;
      if (!ok) b_base[i] = (int)DMA_OUT_OF_RANGE;
    }
  }

  const int steps_c = a.C >> 6, steps_2 = DUAL ? a.C2 >> 6 : 0, nk = a.R * a.S * steps_c + steps_2;
  // cursor of the next step to load (all scalar)
  int l_r = 0, l_s = 0, l_c0 = 0, l_stage = 0, l_k = 0;
  [[maybe_unused]] int l_it = 0;

  // The loads of one step, in three parts so that they can be issued between the MFMA groups of another step
  // (a wavefront that issues them all at once sits in the memory pipeline's queue while its MFMA queue drains).
  auto issue_loads = [&](auto lo_c, auto hi_c) {
    constexpr int LO = decltype(lo_c)::value, HI = decltype(hi_c)::value;
    char *As = smem + l_stage * STAGE, *Bs = As + BM * 128;
    if constexpr (DUAL) {
      if (l_it < steps_2) {
#pragma unroll
        for (int n = LO; n < HI; n++) {
          if (n < A_L) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w2, (lds_ptr)(As + 1024 * (wave + n * NW)), 16, a2_off[n], 2 * l_c0, 0, 0);
          else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x2, (lds_ptr)(Bs + 1024 * (wave + (n - A_L) * NW)), 16, b2_base[n - A_L], 2 * l_c0, 0, 0);
        }
      } else {
#pragma unroll
        for (int n = LO; n < HI; n++) {
          if (n < A_L) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_ptr)(As + 1024 * (wave + n * NW)), 16, a_off[n], 2 * l_c0, 0, 0);
          else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_ptr)(Bs + 1024 * (wave + (n - A_L) * NW)), 16, (unsigned)b_base[n - A_L], 2 * l_c0, 0, 0);
        }
      }
      return;
    }
    const int tap = l_r * a.S + l_s;
    const int x_tap = 2 * ((l_r * a.W + l_s) * a.C);  // bytes from tap (0, 0) to this tap
#pragma unroll
    for (int n = LO; n < HI; n++) {
      if (n < A_L) {
        const int i = n;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_ptr)(As + 1024 * (wave + i * NW)), 16, a_off[i], 2 * l_k, 0, 0);
      } else {
        const int i = n - A_L;
        if (MASKED) {
          // bit 31 set when the tap is outside (or the address is negative): out of range, zeros
          const unsigned voff = (unsigned)(b_base[i] + x_tap) | ((b_out[i] >> tap) << 31);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_ptr)(Bs + 1024 * (wave + i * NW)), 16, voff, 2 * l_c0, 0, 0);
        } else {
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_ptr)(Bs + 1024 * (wave + i * NW)), 16, (unsigned)b_base[i],
                                                   x_tap + 2 * l_c0, 0, 0);
        }
      }
    }
  };
  auto advance_loader = [&]() {
    l_stage = l_stage + 1 == NS ? 0 : l_stage + 1;
    if constexpr (DUAL) {  // channel offset inside the convolution the step belongs to
      l_it++;
      l_c0 = l_it == steps_2 ? 0 : l_c0 + 64;
      return;
    }
    l_k += 64;
    const int c0n = l_c0 + 64, sn = l_s + 1;
    const bool wrap_c = c0n == a.C, wrap_s = wrap_c && sn == a.S;
    l_c0 = wrap_c ? 0 : c0n;
    l_s = wrap_c ? (wrap_s ? 0 : sn) : l_s;
    l_r = wrap_s ? l_r + 1 : l_r;
  };
  constexpr int L1 = (L + 2) / 3, L2 = L1 + (L - L1 + 1) / 2;  // part boundaries
  auto issue_part = [&](auto part_c) {
    constexpr int PART = decltype(part_c)::value;
    if constexpr (PART == 0) issue_loads(std::integral_constant<int, 0>{}, std::integral_constant<int, L1>{});
    if constexpr (PART == 1) issue_loads(std::integral_constant<int, L1>{}, std::integral_constant<int, L2>{});
    if constexpr (PART == 2) { issue_loads(std::integral_constant<int, L2>{}, std::integral_constant<int, L>{}); advance_loader(); }
  };
  auto issue_step = [&]() {
    issue_loads(std::integral_constant<int, 0>{}, std::integral_constant<int, L>{});
    advance_loader();
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // Bias of the k_out this lane will hold in its accumulators, requested
  // before the ring starts (older loads complete first, so the ring's counted
  // waits cover them).
  half4 bias4[TM][4];
  [[maybe_unused]] half4 bias4b[DUAL ? TM : 1][4];  // DUAL: the second convolution's
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
    if constexpr (DUAL) {
      const _Float16 *__restrict__ bias2g = reinterpret_cast<const _Float16 *>(a.bias2);
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const int k_out = m0 + wm0 + i * 32 + 8 * g + 4 * half;
          const half4 zero = {(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
          bias4b[i][g] = bias2g ? *reinterpret_cast<const half4 *>(bias2g + (k_out < a.K ? k_out : 0)) : zero;
        }
    }
    // The counted waits below assume these loads are older than every ring load: nothing may move across here.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  }

  // operand fetch: lane reads 16 bytes of row (block row + l32) at slot (2 sub + half) ^ swizzle(row);
  // 2 sub and half occupy different bits, so the address of sub-step `sub` is that of sub-step 0 ^ (32 sub)
  const unsigned ld_a0 = (unsigned)((wm0 + l32) * 128 + ((half ^ ((l32 >> 1) & 7)) * 16));
  const unsigned ld_b0 = (unsigned)((BM + wn0 + l32) * 128 + ((half ^ ((l32 >> 1) & 7)) * 16));
  half8 fa[2][TM], fb[2][TN];
  auto read_frags = [&](const char *stage, half8 (&qa)[TM], half8 (&qb)[TN], int sub) {
#pragma unroll
    for (int i = 0; i < TM; i++) qa[i] = *reinterpret_cast<const half8 *>(stage + ((ld_a0 ^ (32u * sub)) + i * 4096));
#pragma unroll
    for (int j = 0; j < TN; j++) qb[j] = *reinterpret_cast<const half8 *>(stage + ((ld_b0 ^ (32u * sub)) + j * 4096));
  };
  auto mfma_frags = [&](const half8 (&qa)[TM], const half8 (&qb)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa[i], qb[j], acc[i][j], 0, 0, 0);
  };
  // ---- the ring -------------------------------------------------------------
  // P = NS - 2 steps are in flight beyond the one being computed.  Inside step `it` a wavefront alternates
  // fragment reads, MFMA groups and the loads of step it + P, each a sub-step ahead of its use:
  //   read(sub 1)  mfma(sub 0)  loads 1/3  |  read(sub 2)  mfma(sub 1)  loads 2/3  |  read(sub 3)  mfma(sub 2)  loads 3/3
  //   wait until step it + 1 has landed, barrier, read(sub 0 of step it + 1), mfma(sub 3)
  // so an MFMA group never waits for the LDS read issued right before it, and the MFMA pipe has a group queued
  // while the wavefront sits at the barrier or in the memory pipeline's queue.  The compiler's scheduler would
  // sink the reads below the MFMAs that do not depend on them: scheduling barriers pin the order.
  // The stage step it + P lands in was last read in step it - 2; the barrier inside step it - 1 came after
  // everybody's reads of it (their MFMAs of sub-step 3 had those operands).
  constexpr int P = NS - 2;
  static_assert(P >= 1 && P <= 6 && (P - 1) * L < 64, "ring depth");
  int c_stage = 0;
  auto stage_ptr = [&]() { return smem + c_stage * STAGE; };
  auto next_stage = [&]() { c_stage = c_stage + 1 == NS ? 0 : c_stage + 1; };
#define PIN() __builtin_amdgcn_sched_barrier(0)
  // G: steps still in flight behind step `it` when it ends (P while loads are being issued); LOADS: issue step it + P
  auto step_body = [&](auto g_c, auto loads_c) {
    constexpr int G = decltype(g_c)::value;
    constexpr bool LOADS = decltype(loads_c)::value;
    const char *stage = stage_ptr();
    read_frags(stage, fa[1], fb[1], 1); PIN();
    mfma_frags(fa[0], fb[0]); PIN();
    if constexpr (LOADS) { issue_part(std::integral_constant<int, 0>{}); PIN(); }
    read_frags(stage, fa[0], fb[0], 2); PIN();
    mfma_frags(fa[1], fb[1]); PIN();
    if constexpr (LOADS) { issue_part(std::integral_constant<int, 1>{}); PIN(); }
    read_frags(stage, fa[1], fb[1], 3); PIN();
    mfma_frags(fa[0], fb[0]); PIN();
    if constexpr (LOADS) { issue_part(std::integral_constant<int, 2>{}); PIN(); }
    next_stage();
    if constexpr (G > 0) {
      wait_vmcnt<(G - 1) * L>();  // this wavefront's part of the next step has landed; the barrier covers the others'
      ring_barrier();
      read_frags(stage_ptr(), fa[0], fb[0], 0); PIN();
    }
    mfma_frags(fa[1], fb[1]); PIN();
  };
  {
    // prologue: steps 0 .. P - 1 (those that exist), then wait for step 0
    const int pre = nk < P ? nk : P;
#pragma unroll
    for (int q = 0; q < P; q++)
      if (q < pre) issue_step();
    if (pre == 1) wait_vmcnt<0>();
    else if (pre == 2) wait_vmcnt<(P > 1 ? 1 : 0) * L>();
    else if (pre == 3) wait_vmcnt<(P > 2 ? 2 : 0) * L>();
    else if (pre == 4) wait_vmcnt<(P > 3 ? 3 : 0) * L>();
    else if (pre == 5) wait_vmcnt<(P > 4 ? 4 : 0) * L>();
    else wait_vmcnt<(P > 5 ? 5 : 0) * L>();
    ring_barrier();
    read_frags(stage_ptr(), fa[0], fb[0], 0); PIN();
  }
  for (int it = 0; it < nk - P; it++) step_body(std::integral_constant<int, P>{}, std::true_type{});
  // the last P steps (fewer if the reduction is shorter): nothing left to load, one step fewer in flight each time
  if constexpr (P > 5) { if (nk > 5) step_body(std::integral_constant<int, 5>{}, std::false_type{}); }
  if constexpr (P > 4) { if (nk > 4) step_body(std::integral_constant<int, 4>{}, std::false_type{}); }
  if constexpr (P > 3) { if (nk > 3) step_body(std::integral_constant<int, 3>{}, std::false_type{}); }
  if constexpr (P > 2) { if (nk > 2) step_body(std::integral_constant<int, 2>{}, std::false_type{}); }
  if constexpr (P > 1) { if (nk > 1) step_body(std::integral_constant<int, 1>{}, std::false_type{}); }
  step_body(std::integral_constant<int, 0>{}, std::false_type{});
#undef PIN
  ring_barrier();  // nobody reads the operand stages any more

  // ---- epilogue: bias, activation, fp16, transpose through LDS ------------
  // register r of lane l in block (i, j): k_out = 8*(r/4) + 4*(l/32) + r%4, pixel = l%32
  const _Float16 *__restrict__ Zg = reinterpret_cast<const _Float16 *>(a.Z);
  const int act_now = Zg ? DNNRT_ACT_IDENTITY : a.act;  // with a residual the activation comes after the sum
  _Float16 *Cs = reinterpret_cast<_Float16 *>(smem);    // [BN pixels][CROW]
  constexpr int CH_PER_ROW = BM / 8, OUT_IT = BN * CH_PER_ROW / NT;
  static_assert(BN * CH_PER_ROW % NT == 0, "output chunks divide over the threads");
  half8 zpre[OUT_IT];
  if (Zg) {
#pragma unroll
    for (int o = 0; o < OUT_IT; o++) {
      const int id = tid + o * NT, row = id / CH_PER_ROW, ch = id - row * CH_PER_ROW;
      const int pix = min(n0 + row, NPQ - 1), k_out = min(m0 + ch * 8, a.K - 8);
      zpre[o] = *reinterpret_cast<const half8 *>(Zg + (int64_t)pix * a.K + k_out);
    }
  }
  auto per_mode = [&](int mode, auto &&body) {
    switch (mode) {
      case DNNRT_ACT_RELU: body(std::integral_constant<int, DNNRT_ACT_RELU>{}); break;
      case DNNRT_ACT_CLIPPED_RELU: body(std::integral_constant<int, DNNRT_ACT_CLIPPED_RELU>{}); break;
      case DNNRT_ACT_LEAKY_RELU: body(std::integral_constant<int, DNNRT_ACT_LEAKY_RELU>{}); break;
      default: body(std::integral_constant<int, DNNRT_ACT_IDENTITY>{}); break;
    }
  };
  per_mode(act_now, [&](auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const int kl = wm0 + i * 32 + 8 * g + 4 * half;
          half4 o;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            float v = acc[i][j][4 * g + e] + (float)bias4[i][g][e];
            if constexpr (DUAL) v += (float)bias4b[i][g][e];
            o[e] = (_Float16)apply_act(v, MODE, a.act_coef);
          }
          *reinterpret_cast<half4 *>(Cs + (wn0 + j * 32 + l32) * CROW + kl) = o;
        }
  });
  __syncthreads();
  _Float16 *__restrict__ Yg = reinterpret_cast<_Float16 *>(a.Y);
  per_mode(Zg ? a.act : DNNRT_ACT_IDENTITY, [&](auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
    for (int o = 0; o < OUT_IT; o++) {
      const int id = tid + o * NT;
      const int row = id / CH_PER_ROW, ch = id - row * CH_PER_ROW;
      const int pix = n0 + row, k_out = m0 + ch * 8;
      if (pix < NPQ && k_out < a.K) {
        half8 v = *reinterpret_cast<const half8 *>(Cs + row * CROW + ch * 8);
        if (Zg) {
          // conv + bias was rounded to fp16 above, as a separate convolution
          // would have stored it; the residual sum follows in fp32
          const half8 zv = zpre[o];
#pragma unroll
          for (int e = 0; e < 8; e++) v[e] = (_Float16)apply_act((float)v[e] + (float)zv[e], MODE, a.act_coef);
        }
        *reinterpret_cast<half8 *>(Yg + (int64_t)pix * a.K + k_out) = v;
      }
    }
  });
#endif
}

// More than 64 KiB of LDS per workgroup has to be asked for, once per kernel and device.
template <int BM, int BN, int WM, int WN, int NS, bool MASKED, bool DUAL = false>
static bool launch_dma_masked(const dnnrtContext *ctx, const ConvF16Args &a, unsigned grid, int tiles) {
  constexpr int SMEM = NS * (BM + BN) * 128;
  static bool raised[16] = {};
  if (ctx->device < 0 || ctx->device >= 16) { set_error("conv(fp16): device ordinal %d", ctx->device); return false; }
  if (!raised[ctx->device]) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(&conv_f16_dma_kernel<BM, BN, WM, WN, NS, MASKED, DUAL>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, SMEM) != hipSuccess) {
      set_error("conv(fp16): cannot reserve %d bytes of LDS", SMEM);
      return false;
    }
    raised[ctx->device] = true;
  }
  hipLaunchKernelGGL((conv_f16_dma_kernel<BM, BN, WM, WN, NS, MASKED, DUAL>), dim3(grid), dim3(64 * WM * WN), SMEM, ctx->stream, a, tiles);
  return true;
}

template <int BM, int BN, int WM, int WN, int NS>
static bool launch_dma_dual(const dnnrtContext *ctx, const ConvF16Args &a) {
  const int64_t NPQ = (int64_t)a.N * a.P * a.Q;
  const int64_t tiles = ceil_div(a.K, BM) * ceil_div(NPQ, BN);
  if (tiles + 8 > INT32_MAX) { set_error("conv(fp16): too many tiles"); return false; }
  return launch_dma_masked<BM, BN, WM, WN, NS, false, true>(ctx, a, (unsigned)(ceil_div(tiles, 8) * 8), (int)tiles);
}

template <int BM, int BN, int WM, int WN, int NS>
static bool launch_dma(const dnnrtContext *ctx, const ConvF16Args &a) {
  const int64_t NPQ = (int64_t)a.N * a.P * a.Q;
  const int64_t tiles = ceil_div(a.K, BM) * ceil_div(NPQ, BN);
  if (tiles + 8 > INT32_MAX) { set_error("conv(fp16): too many tiles"); return false; }
  const unsigned grid = (unsigned)(ceil_div(tiles, 8) * 8);
  const bool masked = a.ph != 0 || a.pw != 0 || NPQ % BN != 0;
  return masked ? launch_dma_masked<BM, BN, WM, WN, NS, true>(ctx, a, grid, (int)tiles)
                : launch_dma_masked<BM, BN, WM, WN, NS, false>(ctx, a, grid, (int)tiles);
}

// The variants of this file, by id (conv_f16.hip owns the choice).  `a` must
// satisfy dma_conv_applies and carry the division constants.
bool launch_conv_f16_dma(const dnnrtContext *ctx, const ConvF16Args &a, int variant) {
  switch (variant) {
    case 31: return launch_dma<128, 64, 2, 2, 4>(ctx, a);
    case 32: return launch_dma<128, 128, 2, 2, 3>(ctx, a);
    case 33: return launch_dma<128, 128, 2, 2, 4>(ctx, a);
    case 34: return launch_dma<128, 256, 2, 2, 3>(ctx, a);
    case 35: return launch_dma<128, 256, 2, 4, 3>(ctx, a);
    case 36: return launch_dma<64, 256, 1, 4, 3>(ctx, a);
    case 37: return launch_dma<64, 128, 1, 4, 4>(ctx, a);
    case 38: return launch_dma<64, 64, 2, 2, 4>(ctx, a);
    case 39: return launch_dma<256, 128, 2, 2, 3>(ctx, a);
    case 40: return launch_dma<64, 64, 2, 2, 8>(ctx, a);    // six steps in flight: filters that come from HBM
    case 60: return launch_dma<128, 64, 2, 2, 6>(ctx, a);
    case 61: return launch_dma<128, 128, 2, 2, 5>(ctx, a);
    case 62: return launch_dma<64, 128, 1, 4, 6>(ctx, a);
    // three stages only: 72 KiB (48 KiB) of LDS, so that two (three) workgroups share a compute unit and one's epilogue
    // runs under another's reduction
    case 63: return launch_dma<128, 64, 2, 2, 3>(ctx, a);
    case 65: return launch_dma<64, 128, 2, 2, 3>(ctx, a);
    case 67: return launch_dma<64, 128, 1, 4, 3>(ctx, a);
    case 69: return launch_dma<64, 64, 2, 2, 3>(ctx, a);
    case 64: return launch_dma<128, 128, 4, 2, 4>(ctx, a);  // eight wavefronts: two per SIMD, one fills the other's waits
    case 66: return launch_dma<64, 128, 2, 4, 4>(ctx, a);   // the same on 64-row tiles
    default: set_error("conv(fp16): no direct-to-LDS variant %d", variant); return false;
  }
}

// The two-convolution form (one reduction over both, one rounding): `a` must satisfy dma_dual_applies and carry the
// division constants; variant 0 picks by the number of tiles.
bool dma_dual_variant(int variant) { return variant == 33 || variant == 39 || variant == 61 || variant == 64 || variant == 66 || variant == 37; }
bool launch_conv_f16_dma_dual(const dnnrtContext *ctx, const ConvF16Args &a, int variant) {
  if (!dma_dual_variant(variant)) {
    const int64_t t128 = ceil_div(a.K, 128) * ceil_div((int64_t)a.N * a.P * a.Q, 128);
    variant = 2 * t128 >= 3 * ctx->num_cu ? 64 : 66;
  }
  switch (variant) {
    case 33: return launch_dma_dual<128, 128, 2, 2, 4>(ctx, a);
    case 37: return launch_dma_dual<64, 128, 1, 4, 4>(ctx, a);
    case 39: return launch_dma_dual<256, 128, 2, 2, 3>(ctx, a);
    case 61: return launch_dma_dual<128, 128, 2, 2, 5>(ctx, a);
    case 64: return launch_dma_dual<128, 128, 4, 2, 4>(ctx, a);
    default: return launch_dma_dual<64, 128, 2, 4, 4>(ctx, a);
  }
}

bool dma_dual_applies(const ConvF16Args &a) {
  return a.format == DNNRT_NHWC && a.group == 1 && a.R == 1 && a.S == 1 && a.ph == 0 && a.pw == 0 && a.Z == nullptr && a.X2 && a.Wt2 &&
         a.C % 64 == 0 && a.C2 % 64 == 0 && a.K % 8 == 0 && (a.H - 1) / a.sh + 1 == a.P && (a.W - 1) / a.sw + 1 == a.Q &&
         (a.H2 - 1) / a.sh2 + 1 == a.P && (a.W2 - 1) / a.sw2 + 1 == a.Q &&
         (int64_t)a.N * a.H * a.W * a.C < (1ll << 30) && (int64_t)a.N * a.H2 * a.W2 * a.C2 < (1ll << 30) &&
         (int64_t)a.K * a.C < (1ll << 30) && (int64_t)a.K * a.C2 < (1ll << 30) && aligned16(a.X) && aligned16(a.Wt) && aligned16(a.Y) &&
         aligned16(a.X2) && aligned16(a.Wt2) && (reinterpret_cast<uintptr_t>(a.bias) & 7u) == 0 &&
         (reinterpret_cast<uintptr_t>(a.bias2) & 7u) == 0;
}

bool dma_conv_applies(const ConvF16Args &a) {
  return a.format == DNNRT_NHWC && a.group == 1 && a.C % 64 == 0 && a.K % 8 == 0 && a.R * a.S <= 32 &&
         (int64_t)a.N * a.H * a.W * a.C < (1ll << 30) && (int64_t)a.K * a.C * a.R * a.S < (1ll << 30) &&
         aligned16(a.X) && aligned16(a.Wt) && aligned16(a.Y) && aligned16(a.Z) && (reinterpret_cast<uintptr_t>(a.bias) & 7u) == 0;
}

}  // namespace dnnrt
