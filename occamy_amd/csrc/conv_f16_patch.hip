// fp16 channels-last 3x3 convolution (stride 1, padding 1) that keeps the
// input patch of its pixel tile in LDS.
//
// GEMM view as in conv_f16.hip: D[k_out, pixel] = sum_k Wt[k_out, k] * Xcol[k, pixel],
// filters K,R,S,C, activations N,H,W,C.  An im2col kernel fetches every input
// pixel nine times, once per tap; on a 128 x 128 tile that is as many bytes
// through the compute unit's vector memory path (64 bytes per clock) as the
// MFMAs of the step take clocks, so such a kernel cannot pass half of the MFMA
// peak.  Here a workgroup loads, per slab of 64 input channels, the rows of
// the image its pixels' windows touch (with a one-pixel frame of zeros) once,
// and the nine taps read their B operands out of that patch at nine offsets;
// only the filter slices stream through a ring of LDS stages.
//
// Patch geometry.  The batch is treated as one tall image in which every
// image is framed by a zero row above and below: padded row n * (H + 2) + h + 1
// holds input row h of image n.  Output pixel (n, p, q) reads, for tap (r, s),
// padded row n * (H + 2) + p + r and patch column q + s (patch column c holds
// input column c - 1, columns 0 and W + 1 are zeros), so a tap is the uniform
// offset r * (W + 2) + s from the pixel's own patch index, whatever image
// boundaries the tile's run of pixels crosses.  Frame pixels are buffer loads
// with an out-of-range offset: they arrive as zeros.
//
// LDS layout: a slab is [patch pixel][128 bytes], the 16-byte chunk c of patch
// pixel p kept at position c ^ ((u >> 1) & 7) with u = p - 2 * (p / (W + 2)),
// the pixel's index with the two frame columns of every patch row before it
// taken out.  An MFMA operand read takes one chunk of 32 consecutive output
// pixels at one tap; their patch indices jump by two wherever the run goes
// on to the next image row, but their u are consecutive (the pixel behind a
// row's last one has the next row's column `s`, which is W further in u), so
// 16 lanes always land in 16 different 16-byte bank groups: u mod 16 picks
// the group, its lowest bit through the address (p and u have the same
// parity) and the next three through the position.  With p in place of u
// every row change inside a run of 16 lanes put two lanes on one group, and
// on 14 x 14 images every such run has one.  The direct-to-LDS writes are
// linear, so conflict-free either way.  Two slabs (the one being read, the
// next one landing); filter stages [k_out][128 bytes], chunk c of row k at
// c ^ ((k >> 1) & 7).
//
// Reduction order: slab-major, tap-minor (the filter row of k_out holds, for
// tap t, its C channels contiguously: step (slab, t) reads 128 bytes at
// t * C + 64 * slab).  The nine taps of a slab are unrolled, so every wait is
// an exact count.  Loads past the end of the reduction are still issued, out
// of range (zeros into stages nobody reads any more): the counts never change.
//
// Wavefronts: WM x WN wavefronts tile the BM x BN output, and KG such groups
// split the four 16-k sub-steps of every 64-k step between them (partial sums
// meet in LDS at the end), which puts two wavefronts on every SIMD: one's
// operand reads overlap the other's MFMAs.
#include "conv_f16.h"

#include <type_traits>

namespace dnnrt {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void *lds_ptr;

[[maybe_unused]] constexpr unsigned PATCH_OUT_OF_RANGE = 0x80000000u;  // at or above every num_records used here

template <int N>
__device__ __forceinline__ void patch_wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}
__device__ __forceinline__ void patch_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// The p_l patch loads of the next slab are issued in taps 1 .. 8 - p (load i in tap 1 + i % (8 - p)): after the
// barrier that follows the last reads of the slab they overwrite, and before the first filter loads of the next
// slab (tap 9 - p), so that a wait for those covers them.
constexpr int patch_loads_at(int tap, int p, int p_l) {
  const int taps = 8 - p;
  return tap >= 1 && tap <= taps ? (p_l - (tap - 1) + taps - 1) / taps : 0;
}
// Loads younger than the filter loads of step it + 1 when step it (tap `tap`) ends: the steps it + 2 .. it + P
// were requested in steps it + 2 - P .. it, each after that step's patch loads.
constexpr int younger_loads(int tap, int p, int a_l, int p_l) {
  int n = 0;
  for (int d = 0; d <= p - 2; d++) n += a_l + patch_loads_at((tap - d + 9) % 9, p, p_l);
  return n;
}

template <int BM, int BN, int WM, int WN, int KG, int PCAP, int NS>
__global__ __launch_bounds__(64 * WM * WN * KG) void conv3x3_f16_patch_kernel(const ConvF16Args a, const int tiles_total) {
  // The buffer-resource type exists for the device target only (the host pass needs just the launch stub).
#if __HIP_DEVICE_COMPILE__
  constexpr int NWG = WM * WN, NW = NWG * KG, NT = 64 * NW;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int SUBS = 4 / KG;
  constexpr int A_L = BM / 8 / NW, P_L = PCAP / 8 / NW;
  constexpr int A_STAGE = BM * 128, SLAB = PCAP * 128;
  constexpr int P = NS - 2;
  static_assert(KG == 1 || KG == 2 || KG == 4, "the four sub-steps divide over the groups");
  static_assert(BM % (8 * NW) == 0 && PCAP % (8 * NW) == 0 && TM >= 1 && TN >= 1, "loads divide over the wavefronts");
  static_assert(P >= 1 && P <= 6, "ring depth");
  constexpr int CROW = BM + 8;  // halfs per row of the output staging tile
  constexpr int CS_BYTES = BN * CROW * 2;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char *const patch = smem;             // [2][SLAB]
  char *const ring = smem + 2 * SLAB;   // [NS][A_STAGE]

  const int per_xcd = (tiles_total + 7) >> 3;
  const int tile = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
  if (tile >= tiles_total) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kg = wave / NWG, wq = wave - kg * NWG;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm0 = (wq / WN) * (BM / WM), wn0 = (wq % WN) * (BN / WN);

  const int tiles_m = (a.K + BM - 1) / BM;
  const int tile_n = tile / tiles_m, tile_m = tile - tile_n * tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int PQ = a.P * a.Q, NPQ = a.N * PQ;
  const int CRS = a.C * 9;
  const int Hp = a.H + 2, PW = a.W + 2;

  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.Wt), 0, 2 * a.K * CRS, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_x =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.X), 0, 2 * a.N * a.H * a.W * a.C, 0x00020000);

  // ---- the tile's patch ---------------------------------------------------
  const int img0 = div_magic(n0, PQ, a.magic_pq);
  const int p0 = div_magic(n0 - img0 * PQ, a.Q, a.magic_q);
  const int prow0 = img0 * Hp + p0;  // padded row of the first pixel's tap row 0
  int pp_needed;
  {
    const int last = min(n0 + BN, NPQ) - 1;
    const int img1 = div_magic(last, PQ, a.magic_pq);
    const int p1 = div_magic(last - img1 * PQ, a.Q, a.magic_q);
    pp_needed = (img1 * Hp + p1 + 2 - prow0 + 1) * PW;  // through the last pixel's tap row 2
  }
  // patch load i of this wavefront fills patch pixels 8 * (wave + i * NW) .. + 7 of a slab
  unsigned p_off[P_L];
#pragma unroll
  for (int i = 0; i < P_L; i++) {
    const int pp = 8 * (wave + i * NW) + (lane >> 3);
    const int prow_rel = div_magic(pp, PW, a.magic_pw), col = pp - prow_rel * PW;
    const int ch = (lane & 7) ^ (((pp - 2 * prow_rel) >> 1) & 7);
    const int prow = prow0 + prow_rel;
    const int n = div_magic(prow, Hp, a.magic_hp), hr = prow - n * Hp;
    const bool ok = pp < pp_needed && n < a.N && hr >= 1 && hr <= a.H && col >= 1 && col <= a.W;
    p_off[i] = ok ? 2u * (unsigned)(((n * a.H + hr - 1) * a.W + col - 1) * a.C + ch * 8) : PATCH_OUT_OF_RANGE;
  }
  // filter load i fills rows 8 * (wave + i * NW) .. + 7 of a stage
  unsigned a_off[A_L];
#pragma unroll
  for (int i = 0; i < A_L; i++) {
    const int row = 8 * (wave + i * NW) + (lane >> 3), ch = (lane & 7) ^ ((row >> 1) & 7);
    const int k_out = m0 + row;
    a_off[i] = k_out < a.K ? 2u * (unsigned)(k_out * CRS + ch * 8) : PATCH_OUT_OF_RANGE;
  }
  // operand fetch: patch index of tap (0, 0) of the pixel whose column of D this lane holds, per 32-pixel block
  // ... and the same index with the frame columns of the patch rows before it taken out (what the swizzle goes by)
  int pp00[TN], uu00[TN];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int pix = min(n0 + wn0 + j * 32 + l32, NPQ - 1);  // a column past the end computes a copy that is never stored
    const int n = div_magic(pix, PQ, a.magic_pq), pq = pix - n * PQ;
    const int p = div_magic(pq, a.Q, a.magic_q), q = pq - p * a.Q;
    pp00[j] = (n * Hp + p - prow0) * PW + q;
    uu00[j] = pp00[j] - 2 * (n * Hp + p - prow0);
  }
  const unsigned ld_a0 = (unsigned)((wm0 + l32) * 128 + ((half ^ ((l32 >> 1) & 7)) * 16));

  const int nslab = a.C >> 6, nk = 9 * nslab;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // Bias of the k_out this lane holds in its accumulators, requested before the ring starts (older loads
  // complete first, so the ring's counted waits cover them).
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
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- loaders (all cursors scalar) -----------------------------------------
  int l_it = 0, l_tap = 0, l_slab = 0, l_stage = 0;
  auto issue_filter = [&]() {  // the filter slice of step l_it (zeros past the end of the reduction)
    char *As = ring + l_stage * A_STAGE;
    const unsigned dead = l_it >= nk ? PATCH_OUT_OF_RANGE : 0u;
    const int soff = 2 * (l_tap * a.C + l_slab * 64);
#pragma unroll
    for (int i = 0; i < A_L; i++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_ptr)(As + 1024 * (wave + i * NW)), 16, a_off[i] | dead, soff, 0, 0);
    l_it++;
    l_stage = l_stage + 1 == NS ? 0 : l_stage + 1;
    const bool wrap = l_tap == 8;
    l_tap = wrap ? 0 : l_tap + 1;
    l_slab += wrap ? 1 : 0;
  };
  auto issue_patch = [&](int slab, int i) {  // load i of slab `slab` (zeros if there is no such slab); i unrolls to a constant
    const unsigned dead = slab >= nslab ? PATCH_OUT_OF_RANGE : 0u;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_ptr)(patch + (slab & 1) * SLAB + 1024 * (wave + i * NW)), 16,
                                             p_off[i] | dead, slab * 128, 0, 0);
  };

  // ---- operand fetch -----------------------------------------------------------
  half8 fa[2][TM], fb[2][TN];
  unsigned bad[TN];  // this lane's patch addresses of the current tap (chunk of sub-step 0)
  auto tap_addresses = [&](int tap_r, int tap_s) {  // tap (r, s): r patch rows down, s columns right
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int pp = pp00[j] + tap_r * PW + tap_s, u = uu00[j] + tap_r * a.W + tap_s;
      bad[j] = (unsigned)(pp * 128 + (((half ^ (u >> 1)) & 7) << 4));
    }
  };
  auto read_frags = [&](const char *stage, const char *slab, half8 (&qa)[TM], half8 (&qb)[TN], int sub) {
#pragma unroll
    for (int i = 0; i < TM; i++) qa[i] = *reinterpret_cast<const half8 *>(stage + ((ld_a0 ^ (32u * sub)) + i * 4096));
#pragma unroll
    for (int j = 0; j < TN; j++) qb[j] = *reinterpret_cast<const half8 *>(slab + (bad[j] ^ (32u * sub)));
  };
  auto mfma_frags = [&](const half8 (&qa)[TM], const half8 (&qb)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa[i], qb[j], acc[i][j], 0, 0, 0);
  };

  // ---- the ring -------------------------------------------------------------
  // Step (slab, tap): this wavefront's sub-steps are kg, kg + KG, ...  The operands of a step's first sub-step
  // are fetched at the end of the step before (after its barrier), those of the others one sub-step ahead of
  // their MFMAs; the scheduler would sink the fetches below the MFMAs they do not feed, so the order is pinned.
  int c_stage = 0;
#define PIN() __builtin_amdgcn_sched_barrier(0)
  auto step = [&](int slab, auto tap_c) {
    constexpr int TAP = decltype(tap_c)::value;
    constexpr int NEXT = (TAP + 1) % 9;
    const char *stage = ring + c_stage * A_STAGE;
    const char *cur = patch + (slab & 1) * SLAB;
    if constexpr (SUBS == 4) {
      read_frags(stage, cur, fa[1], fb[1], 1); PIN();
      mfma_frags(fa[0], fb[0]); PIN();
      read_frags(stage, cur, fa[0], fb[0], 2); PIN();
      mfma_frags(fa[1], fb[1]); PIN();
      read_frags(stage, cur, fa[1], fb[1], 3); PIN();
      mfma_frags(fa[0], fb[0]); PIN();
    } else if constexpr (SUBS == 2) {
      read_frags(stage, cur, fa[1], fb[1], kg + KG); PIN();
      mfma_frags(fa[0], fb[0]); PIN();
    }
    if constexpr (patch_loads_at(TAP, P, P_L) > 0) {
#pragma unroll
      for (int i = TAP - 1; i < P_L; i += 8 - P) issue_patch(slab + 1, i);
    }
    issue_filter(); PIN();
    c_stage = c_stage + 1 == NS ? 0 : c_stage + 1;
    // the next step's filter slice (and, when this is a slab's last tap, the next slab, requested before it)
    patch_wait_vmcnt<younger_loads(TAP, P, A_L, P_L)>();
    patch_barrier();
    const char *nstage = ring + c_stage * A_STAGE;
    const char *nslab_ptr = NEXT == 0 ? patch + ((slab + 1) & 1) * SLAB : cur;
    if constexpr (SUBS == 1) { mfma_frags(fa[0], fb[0]); PIN(); }  // before its operand registers are fetched into again
    tap_addresses(NEXT / 3, NEXT % 3);
    read_frags(nstage, nslab_ptr, fa[0], fb[0], kg); PIN();
    if constexpr (SUBS > 1) { mfma_frags(fa[1], fb[1]); PIN(); }
  };
  // prologue: slab 0, then the filter slices of steps 0 .. P - 1; wait for step 0 (the slab is older)
#pragma unroll
  for (int i = 0; i < P_L; i++) issue_patch(0, i);
#pragma unroll
  for (int q = 0; q < P; q++) issue_filter();
  patch_wait_vmcnt<(P - 1) * A_L>();
  patch_barrier();
  tap_addresses(0, 0);
  read_frags(ring, patch, fa[0], fb[0], kg); PIN();
  for (int slab = 0; slab < nslab; slab++) {
    step(slab, std::integral_constant<int, 0>{});
    step(slab, std::integral_constant<int, 1>{});
    step(slab, std::integral_constant<int, 2>{});
    step(slab, std::integral_constant<int, 3>{});
    step(slab, std::integral_constant<int, 4>{});
    step(slab, std::integral_constant<int, 5>{});
    step(slab, std::integral_constant<int, 6>{});
    step(slab, std::integral_constant<int, 7>{});
    step(slab, std::integral_constant<int, 8>{});
  }
#undef PIN
  // the fetch after the last step read zeros that nobody uses; the loads past the end must have landed before
  // the stages are used for anything else
  patch_wait_vmcnt<0>();
  patch_barrier();

  // ---- partial sums of the other groups ---------------------------------------
  if constexpr (KG > 1) {
    float *red = reinterpret_cast<float *>(smem + CS_BYTES);  // [(KG - 1) * NWG wavefronts][TM * TN * 16 registers][64 lanes]
    if (kg > 0) {
      float *mine = red + (size_t)((kg - 1) * NWG + wq) * (TM * TN * 16 * 64) + lane;
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int r = 0; r < 16; r++) mine[((i * TN + j) * 16 + r) * 64] = acc[i][j][r];
    }
    __syncthreads();
    if (kg == 0) {
#pragma unroll
      for (int g = 1; g < KG; g++) {
        const float *theirs = red + (size_t)((g - 1) * NWG + wq) * (TM * TN * 16 * 64) + lane;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] += theirs[((i * TN + j) * 16 + r) * 64];
      }
    }
  }

  // ---- epilogue: bias, activation, fp16, transpose through LDS ------------
  // register r of lane l in block (i, j): k_out = 8*(r/4) + 4*(l/32) + r%4, pixel = l%32
  const _Float16 *__restrict__ Zg = reinterpret_cast<const _Float16 *>(a.Z);
  const int act_now = Zg ? DNNRT_ACT_IDENTITY : a.act;  // with a residual the activation comes after the sum
  _Float16 *Cs = reinterpret_cast<_Float16 *>(smem);    // [BN pixels][CROW], below the partial sums
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
  if (kg == 0) {
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
            for (int e = 0; e < 4; e++) o[e] = (_Float16)apply_act(acc[i][j][4 * g + e] + (float)bias4[i][g][e], MODE, a.act_coef);
            *reinterpret_cast<half4 *>(Cs + (wn0 + j * 32 + l32) * CROW + kl) = o;
          }
    });
  }
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
          // conv + bias was rounded to fp16 above, as a separate convolution would have stored it; the
          // residual sum follows in fp32
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

// Patch pixels a tile of bn consecutive output pixels can need at most: the rows its pixels lie in, one above and
// one below, and two frame rows per image boundary the run crosses, each W + 2 wide.
static int64_t patch_pixels_bound(const ConvF16Args &a, int bn) {
  const int64_t row_steps = (a.W - 1 + bn - 1) / a.W;  // row changes inside the run, at most
  const int64_t crossings = (row_steps + a.H - 1) / a.H;
  return (row_steps + 1 + 2 + 2 * crossings) * (a.W + 2);
}

template <int BM, int BN, int WM, int WN, int KG, int PCAP, int NS>
static bool launch_patch(const dnnrtContext *ctx, const ConvF16Args &a, bool only_ask) {
  constexpr int NWG = WM * WN;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int LOOP = 2 * PCAP * 128 + NS * BM * 128;
  constexpr int TAIL = BN * (BM + 8) * 2 + (KG - 1) * NWG * TM * TN * 16 * 64 * 4;
  constexpr int SMEM = LOOP > TAIL ? LOOP : TAIL;
  static_assert(SMEM <= 160 * 1024, "LDS of a compute unit");
  if (only_ask) return patch_pixels_bound(a, BN) <= PCAP;
  if (patch_pixels_bound(a, BN) > PCAP) {
    set_error("conv(fp16): this variant holds %d patch pixels, a run of %d pixels of a %d x %d image can need more", PCAP, BN, a.H, a.W);
    return false;
  }
  const int64_t NPQ = (int64_t)a.N * a.P * a.Q;
  const int64_t tiles = ceil_div(a.K, BM) * ceil_div(NPQ, BN);
  if (tiles + 8 > INT32_MAX) { set_error("conv(fp16): too many tiles"); return false; }
  static bool raised[16] = {};
  if (ctx->device < 0 || ctx->device >= 16) { set_error("conv(fp16): device ordinal %d", ctx->device); return false; }
  if (!raised[ctx->device]) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(&conv3x3_f16_patch_kernel<BM, BN, WM, WN, KG, PCAP, NS>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, SMEM) != hipSuccess) {
      set_error("conv(fp16): cannot reserve %d bytes of LDS", SMEM);
      return false;
    }
    raised[ctx->device] = true;
  }
  ConvF16Args am = a;
  am.magic_pw = magic_of(a.W + 2);
  am.magic_hp = magic_of(a.H + 2);
  hipLaunchKernelGGL((conv3x3_f16_patch_kernel<BM, BN, WM, WN, KG, PCAP, NS>), dim3((unsigned)(ceil_div(tiles, 8) * 8)),
                     dim3(64 * NWG * KG), SMEM, ctx->stream, am, (int)tiles);
  return true;
}

bool patch_conv_applies(const ConvF16Args &a) {
  return a.format == DNNRT_NHWC && a.group == 1 && a.R == 3 && a.S == 3 && a.sh == 1 && a.sw == 1 && a.ph == 1 && a.pw == 1 &&
         a.C % 64 == 0 && a.C >= 128 && a.K % 8 == 0 && (int64_t)a.N * a.H * a.W * a.C < (1ll << 30) &&
         (int64_t)a.K * a.C * 9 < (1ll << 30) && (int64_t)a.N * (a.H + 2) < (1 << 24) && aligned16(a.X) && aligned16(a.Wt) &&
         aligned16(a.Y) && aligned16(a.Z) && (reinterpret_cast<uintptr_t>(a.bias) & 7u) == 0;
}

// The smallest patch capacity compiled for tile width bn that holds this problem's patches, or 0.
int patch_conv_capacity(const ConvF16Args &a, int bn) {
  const int64_t need = patch_pixels_bound(a, bn);
  return need <= 256 ? 256 : need <= 320 ? 320 : 0;
}

// The variants of this file, by id (conv_f16.hip owns the choice).  `a` must satisfy patch_conv_applies and carry
// the division constants of P * Q and Q.  only_ask: launch nothing, say whether the variant's patch capacity fits.
static bool patch_variant(const dnnrtContext *ctx, const ConvF16Args &a, int variant, bool only_ask) {
  switch (variant) {
    case 41: return launch_patch<128, 128, 2, 2, 2, 256, 4>(ctx, a, only_ask);
    case 42: return launch_patch<128, 128, 2, 2, 2, 320, 4>(ctx, a, only_ask);
    case 43: return launch_patch<64, 128, 1, 2, 4, 256, 4>(ctx, a, only_ask);
    case 44: return launch_patch<64, 128, 1, 2, 4, 320, 4>(ctx, a, only_ask);
    case 45: return launch_patch<128, 128, 2, 2, 1, 256, 4>(ctx, a, only_ask);
    case 46: return launch_patch<64, 128, 1, 2, 2, 256, 4>(ctx, a, only_ask);
    case 47: return launch_patch<64, 128, 1, 2, 4, 256, 8>(ctx, a, only_ask);   // six filter steps in flight
    case 48: return launch_patch<128, 128, 2, 2, 2, 256, 5>(ctx, a, only_ask);  // three
    case 49: return launch_patch<64, 128, 1, 2, 4, 320, 8>(ctx, a, only_ask);
    case 51: return launch_patch<128, 128, 2, 2, 2, 256, 6>(ctx, a, only_ask);  // four (all of the LDS)
    case 52: return launch_patch<128, 128, 2, 2, 2, 320, 5>(ctx, a, only_ask);
    case 54: return launch_patch<128, 128, 2, 4, 1, 256, 6>(ctx, a, only_ask);  // eight wavefronts over the tile, none over the reduction
    case 57: return launch_patch<128, 128, 2, 4, 1, 320, 5>(ctx, a, only_ask);
    default: if (!only_ask) set_error("conv(fp16): no patch variant %d", variant); return false;
  }
}
bool launch_conv_f16_patch(const dnnrtContext *ctx, const ConvF16Args &a, int variant) { return patch_variant(ctx, a, variant, false); }
bool patch_variant_fits(const ConvF16Args &a, int variant) { return patch_variant(nullptr, a, variant, true); }

}  // namespace dnnrt
