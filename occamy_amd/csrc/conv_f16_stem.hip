// First convolution of an ImageNet CNN in fp16: 3 input channels, 7x7 filter,
// stride 2, pad 3, 64 output channels; input N,C,H,W as the host sent it,
// output channels-last (the DNNRT_NCHW_TO_NHWC format), filter K,R,S,C.
//
// With 3 channels the im2col operand has no run of 8 contiguous k in memory,
// so the implicit-GEMM kernels in conv_f16.hip would gather it element by
// element.  Here a workgroup stages the input patch of an 8 x 16 tile of
// output pixels in LDS (3 x 21 x 37 values, zero-filled outside the image) and
// orders the reduction as (c, r, s) with s padded from 7 to 8: the 8 k of one
// MFMA lane are then 8 adjacent halfs of one patch row, i.e. four aligned
// 32-bit LDS reads.  A k16 step pairs patch rows (c, r) = 2j and 2j + 1 (lower
// and upper half-wave); 21 rows make 11 steps, the 22nd row and the 8th tap
// carry zero weights (and the B side is zeroed there as well, so that a
// non-finite input value cannot leak through 0 * x).
//
// The filter (64 x 147) lives in registers as MFMA A operands for the whole
// kernel (it gets there through LDS, see below): workgroups are persistent and
// walk over tiles, loading the next tile's patch into registers while the
// current one is computed.  The bias is one more term of the reduction (see below).
//
// Wavefront w owns output rows 2w, 2w+1 of the tile (32 pixels) and all 64
// output channels (two 32x32 MFMA blocks).  Results go through a
// wave-private LDS buffer so that each pixel's 64 channels leave as one
// 128-byte line.
#include "conv_f16.h"

#include <type_traits>

namespace dnnrt {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short ushort8 __attribute__((ext_vector_type(8)));
typedef unsigned short ushort2v __attribute__((ext_vector_type(2)));

namespace stem {
constexpr int TP = 8, TQ = 16;               // output pixels per tile
constexpr int PY = 2 * TP + 5, PX = 2 * TQ + 5;  // 21 x 37 input patch per channel
constexpr int PROW = 48;                     // halfs per patch row in LDS (row pairs land 64 bytes apart mod 128)
constexpr int PATCH = 3 * PY * PROW;         // halfs per patch buffer
constexpr int NEL = 3 * PY * PX;             // 2331 patch elements
constexpr int PER_THREAD = (NEL + 255) / 256;  // 10
constexpr int STEPS = 11;
constexpr int OROW = 72;                     // halfs per pixel in the output staging buffer (64 + 8 pad)
}  // namespace stem

template <bool RELU>
__global__ __launch_bounds__(256, 2) void conv_f16_stem_kernel(const ConvF16Args a, const int tiles_p, const int tiles_q,
                                                               const int total) {
  using namespace stem;
  // one LDS block: the two patch buffers, then the four wavefronts' output staging; at start-up the whole filter passes through it
  __shared__ __attribute__((aligned(16))) _Float16 smem[2 * PATCH + 4 * 32 * OROW];
  static_assert(2 * PATCH + 4 * 32 * OROW >= 64 * 147, "the filter is staged in the same block");
  _Float16(*patch)[PATCH] = reinterpret_cast<_Float16(*)[PATCH]>(smem);
  _Float16 *ostage = smem + 2 * PATCH;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, half = lane >> 5;
  const _Float16 *__restrict__ Xg = reinterpret_cast<const _Float16 *>(a.X);
  const _Float16 *__restrict__ Wg = reinterpret_cast<const _Float16 *>(a.Wt);
  _Float16 *__restrict__ Yg = reinterpret_cast<_Float16 *>(a.Y);

  // ---- filter into A-operand registers ---------------------------------
  // Through LDS: read from global memory a lane's 176 two-byte elements lie in
  // 64 different cache lines per load instruction (one filter per lane, 294
  // bytes apart), which kept the vector memory pipe busy for longer than all
  // the tiles of the workgroup together; the copy below reads each line once.
  {
    // 64 * 147 halfs = 1176 units of 16 bytes (the launcher checked the alignment): five loads per thread, all
    // issued before the first store (a loop of load-then-store would pay the memory latency once per unit)
    constexpr int UNITS = 64 * 147 / 8, PER = (UNITS + 255) / 256;
    const u32x4 *__restrict__ w128 = reinterpret_cast<const u32x4 *>(Wg);
    u32x4 *s128 = reinterpret_cast<u32x4 *>(smem);
    u32x4 wv[PER];
#pragma unroll
    for (int k = 0; k < PER; k++) wv[k] = w128[min(tid + k * 256, UNITS - 1)];
#pragma unroll
    for (int k = 0; k < PER; k++)
      if (tid + k * 256 < UNITS) s128[tid + k * 256] = wv[k];
  }
  __syncthreads();
  half8 afr[2][STEPS];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < STEPS; j++) {
      const int cr = 2 * j + half, c = cr / 7, r = cr - c * 7;
      const int k_out = 32 * i + l32;
#pragma unroll
      for (int s = 0; s < 8; s++) {
        _Float16 v = (_Float16)0.f;
        if (s < 7 && cr < 21) v = smem[((k_out * 7 + r) * 7 + s) * 3 + c];
        afr[i][j][s] = v;
      }
    }
  // The bias rides in the reduction: tap s = 7 does not exist, so in patch row (c, r) = (0, 0) its weight is the
  // bias and its input value a one (bias x 1 is exact in the fp32 sum).  The accumulators then start from zero,
  // and there is no bias to convert for every tile.
  if (a.bias != nullptr) {
    const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const _Float16 bv = biasg[32 * i + l32];
      if (half == 0) afr[i][0][7] = bv;
    }
  }

  __syncthreads();  // every lane has its part of the filter: the block is free
  // zero both patch buffers once: the columns past PX stay zero for good
  for (int e = tid; e < 2 * PATCH / 8; e += 256)
    reinterpret_cast<u32x4 *>(&patch[0][0])[e] = (u32x4){0u, 0u, 0u, 0u};

  // patch element e of this thread: (c, y, x), fixed for the whole kernel
  int pe_lds[PER_THREAD], pe_off[PER_THREAD], pe_y[PER_THREAD], pe_x[PER_THREAD];
  const int HW = a.H * a.W;
#pragma unroll
  for (int k = 0; k < PER_THREAD; k++) {
    const int e = tid + k * 256;
    const int ee = e < NEL ? e : 0;
    const int c = ee / (PY * PX), rem = ee - c * (PY * PX), y = rem / PX, x = rem - y * PX;
    pe_y[k] = y; pe_x[k] = e < NEL ? x : -100000;  // far outside: reads as zero
    pe_off[k] = c * HW + y * a.W + x;                // offset from the patch's corner (which may lie outside the image)
    pe_lds[k] = (c * PY + y) * PROW + x;
  }
  auto load_patch = [&](int tile, _Float16 (&v)[PER_THREAD]) {
    const int tq = tile % tiles_q, t2 = tile / tiles_q, tp = t2 % tiles_p, n = t2 / tiles_p;
    const int iy0 = 2 * tp * TP - 3, ix0 = 2 * tq * TQ - 3;
    const _Float16 *xb = Xg + (int64_t)n * 3 * HW;
    const int corner = iy0 * a.W + ix0;              // uniform; negative at the top and left borders
#pragma unroll
    for (int k = 0; k < PER_THREAD; k++) {
      const int iy = iy0 + pe_y[k], ix = ix0 + pe_x[k];
      const bool ok = (unsigned)iy < (unsigned)a.H && (unsigned)ix < (unsigned)a.W;
      const _Float16 t = xb[ok ? corner + pe_off[k] : 0];
      v[k] = ok ? t : (_Float16)0.f;
    }
  };
  auto store_patch = [&](int buf, const _Float16 (&v)[PER_THREAD]) {
#pragma unroll
    for (int k = 0; k < PER_THREAD; k++)
      if (tid + k * 256 < NEL) patch[buf][pe_lds[k]] = v[k];
  };

  // B operand address of this lane inside a patch: pixel (2 * wave + l32 / 16, l32 % 16)
  const int b_base = (2 * (2 * wave + (l32 >> 4))) * PROW + 2 * (l32 & 15);

  _Float16 pv[PER_THREAD];
  int tile = blockIdx.x;
  __syncthreads();  // zero fill done
  if (tile < total) load_patch(tile, pv);
  store_patch(0, pv);
  __syncthreads();

  int cur = 0;
  for (; tile < total; tile += gridDim.x) {
    const int nxt = tile + (int)gridDim.x;
    load_patch(nxt < total ? nxt : tile, pv);  // unconditional: a repeat of this tile when there is no next one

    floatx16 acc[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
    const _Float16 *pb = &patch[cur][0];
#pragma unroll
    for (int j = 0; j < STEPS; j++) {
      const int cr = 2 * j + half, crc = cr < 21 ? cr : 20;
      const int c = crc / 7, r = crc - c * 7;
      const unsigned *src = reinterpret_cast<const unsigned *>(pb + (c * PY + r) * PROW + b_base);
      u32x4 w;
      w[0] = src[0]; w[1] = src[1]; w[2] = src[2]; w[3] = src[3] & 0x0000ffffu;  // tap s = 7 does not exist
      if (j == 0 && half == 0) w[3] |= 0x3c000000u;                               // but the bias's one (fp16 1.0) does
      if (j == STEPS - 1 && half) w = (u32x4){0u, 0u, 0u, 0u};                    // nor does patch row 21
      half8 bv;
      __builtin_memcpy(&bv, &w, 16);
      acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][j], bv, acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[1][j], bv, acc[1], 0, 0, 0);
    }

    // ---- epilogue: bias, activation, 128-byte lines per pixel -------------
    const int tq = tile % tiles_q, t2 = tile / tiles_q, tp = t2 % tiles_p, n = t2 / tiles_p;
    _Float16 *os = ostage + wave * (32 * OROW);
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        half4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          float v = acc[i][4 * g + e];
          if (RELU) v = v < 0.f ? 0.f : v;
          o[e] = (_Float16)v;
        }
        *reinterpret_cast<half4 *>(os + l32 * OROW + 32 * i + 8 * g + 4 * half) = o;
      }
    // same wavefront reads what it wrote: LDS keeps a wavefront's accesses in order
    // pixel (row it / 2 of the wavefront's two, column 8 * (it % 2) + lane / 8), channels 8 * (lane % 8) ... + 7:
    // a uniform base per tile and wavefront, one per-lane offset, and constants per `it`
    const int p_w = tp * TP + 2 * wave, q_l = tq * TQ + (lane >> 3);
    _Float16 *yt = Yg + (((int64_t)n * a.P + p_w) * a.Q + tq * TQ) * 64 + (lane >> 3) * 64 + (lane & 7) * 8;
#pragma unroll
    for (int it = 0; it < 4; it++) {
      const int pl = it * 8 + (lane >> 3);
      const u32x4 v = *reinterpret_cast<const u32x4 *>(os + pl * OROW + (lane & 7) * 8);
      if (p_w + (it >> 1) < a.P && q_l + 8 * (it & 1) < a.Q)
        *reinterpret_cast<u32x4 *>(yt + (int64_t)(it >> 1) * a.Q * 64 + (it & 1) * 512) = v;
    }

    store_patch(cur ^ 1, pv);
    __syncthreads();
    cur ^= 1;
  }
}

// ---- the same convolution with the 3x3 / stride 2 / pad 1 max-pool that follows it in ResNets ----------------
// The convolution's result (N x 112 x 112 x 64 at 224 x 224: four times the pooled tensor) is never stored.
// A workgroup owns a strip of seven pooled columns of one image and walks down it: the tile at step t holds
// convolution rows 8 t .. 8 t + 7 and columns 14 qs - 1 .. 14 qs + 14 (fifteen are needed, the sixteenth comes
// free with the tile shape), staged in LDS after the activation; with the last row of the step before, kept in
// LDS, that is every window of pooled rows 4 t .. 4 t + 3.  Convolution outputs outside the image (column -1 of
// the first strip, rows and columns past the end) are staged as -inf, which is what the pooling's padding is.
// Two staging tiles and two carried rows alternate, so that the one barrier per step the patch double buffer
// already needs is enough: step i is pooled after its barrier (at the start of step i + 1, behind the loads that
// step issues) from tile i % 2 and carry i % 2, and writes carry (i + 1) % 2; step i + 1 writes tile
// (i + 1) % 2 before the next barrier, and nobody reads that one in between.
//
// The kernel is bound by the number of vector instructions it issues, not by memory or the MFMA pipe, so:
//   * the patch is loaded two input values at a time.  The reduction window of a pixel starts one input column
//     early (eight taps x = 2 q - 4 .. 2 q + 3, the first with weight zero, instead of 2 q - 3 .. 2 q + 4 with the
//     last zero), which puts every window, and with an even image width every pair, on a 4-byte boundary both
//     in global memory and in LDS;
//   * everything about a thread's place in the pooling is computed once; NaN (which must reach the result, and
//     which the packed fp16 maximum drops) is looked for with one more packed maximum per load and handled in a
//     branch that a wavefront takes only if one of its windows saw one.
namespace stem {
constexpr int PXP = TQ + 3;                          // 19 pairs = 38 input columns per patch row
constexpr int NELP = 3 * PY * PXP;                   // 1197 pairs
[[maybe_unused]] constexpr int PER_THREAD_P = (NELP + 255) / 256;  // 5 (device code only)
}  // namespace stem

template <bool RELU>
__global__ __launch_bounds__(256, 2) void conv_f16_stem_pool_kernel(const ConvF16Args a, const int PP, const int QQ, const int strips,
                                                                    const unsigned magic_strips, const int steps_per_unit,
                                                                    const int units, _Float16 *__restrict__ Yp) {
  // The buffer-resource type exists for the device target only (the host pass needs just the launch stub).
#if __HIP_DEVICE_COMPILE__
  using namespace stem;
  constexpr int STAGE = 128 * OROW, CARRY = 16 * OROW;
  __shared__ __attribute__((aligned(16))) _Float16 smem[2 * PATCH + 2 * STAGE + 2 * CARRY];
  __shared__ int nonfinite;  // set, for good, once a non-finite input, weight or bias value has been seen
  static_assert(2 * PATCH + 2 * STAGE >= 64 * 147, "the filter is staged in the same block");
  static_assert(2 * PXP <= PROW, "patch row");
  _Float16(*patch)[PATCH] = reinterpret_cast<_Float16(*)[PATCH]>(smem);
  _Float16 *const stage = smem + 2 * PATCH;
  _Float16 *const carry = stage + 2 * STAGE;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, half = lane >> 5;
  const _Float16 *__restrict__ Wg = reinterpret_cast<const _Float16 *>(a.Wt);
  // bit 15 / 31 of the result is set iff the fp16 value in that half has all exponent bits set (infinity or NaN)
  auto non_finite_bits = [](unsigned v) { return (v & 0x7c007c00u) + 0x04000400u; };

  // ---- filter into A-operand registers (as in the kernel above, taps moved up by one) --------
  unsigned nf = 0;
  if (tid == 0) nonfinite = 0;
  {
    constexpr int UNITS = 64 * 147 / 8, PER = (UNITS + 255) / 256;
    const u32x4 *__restrict__ w128 = reinterpret_cast<const u32x4 *>(Wg);
    u32x4 *s128 = reinterpret_cast<u32x4 *>(smem);
    u32x4 wv[PER];
#pragma unroll
    for (int k = 0; k < PER; k++) wv[k] = w128[min(tid + k * 256, UNITS - 1)];
#pragma unroll
    for (int k = 0; k < PER; k++) {
      if (tid + k * 256 < UNITS) s128[tid + k * 256] = wv[k];
#pragma unroll
      for (int d = 0; d < 4; d++) nf |= non_finite_bits(wv[k][d]);
    }
  }
  __syncthreads();
  half8 afr[2][STEPS];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < STEPS; j++) {
      const int cr = 2 * j + half, c = cr / 7, r = cr - c * 7;
      const int k_out = 32 * i + l32;
#pragma unroll
      for (int s = 0; s < 8; s++) {
        _Float16 v = (_Float16)0.f;
        if (s >= 1 && cr < 21) v = smem[((k_out * 7 + r) * 7 + s - 1) * 3 + c];
        afr[i][j][s] = v;
      }
    }
  // The bias rides in the reduction: the window's first column carries no tap, so in patch row (c, r) = (0, 0) its
  // weight is the bias and its input value a one (bias x 1 is exact in the fp32 sum).  The accumulators then start
  // from zero, and there is no bias to convert at every step.
  if (a.bias != nullptr) {
    const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const _Float16 bv = biasg[32 * i + l32];
      if (half == 0) afr[i][0][0] = bv;
      unsigned short bb;
      __builtin_memcpy(&bb, &bv, 2);
      nf |= non_finite_bits(bb);
    }
  }
  if (__builtin_amdgcn_ballot_w64((nf & 0x80008000u) != 0) != 0 && lane == 0) nonfinite = 1;
  __syncthreads();  // every lane has its part of the filter: the block is free
  for (int e = tid; e < 2 * PATCH / 8; e += 256)  // the columns past 2 PXP stay zero for good
    reinterpret_cast<u32x4 *>(&patch[0][0])[e] = (u32x4){0u, 0u, 0u, 0u};

  // pair e of this thread: (c, y, xp), fixed for the whole kernel: its byte offset from the patch's corner in the
  // image, its position in LDS, and (y, x) as two 16-bit fields, so that one packed add, one packed minimum and one
  // compare say whether the pair lies inside the image (a coordinate below zero wraps to a large unsigned value).
  // A pair outside gets an offset past the end of the buffer and reads as zero.
  const __amdgpu_buffer_rsrc_t rsrc_x =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.X), 0, 2 * a.N * 3 * a.H * a.W, 0x00020000);
  int pe_off[PER_THREAD_P], pe_lds[PER_THREAD_P];
  ushort2v pe_yx[PER_THREAD_P];
  const int HW = a.H * a.W;
#pragma unroll
  for (int k = 0; k < PER_THREAD_P; k++) {
    const int e = tid + k * 256;
    const int ee = e < NELP ? e : 0;
    const int c = ee / (PY * PXP), rem = ee - c * (PY * PXP), y = rem / PXP, xp = rem - y * PXP;
    pe_lds[k] = e < NELP ? (c * PY + y) * PROW + 2 * xp : -1;
    pe_off[k] = 2 * (c * HW + y * a.W + 2 * xp);
    pe_yx[k] = (ushort2v){(unsigned short)(e < NELP ? y : 0x6000), (unsigned short)(2 * xp)};  // 0x6000: beyond any image (height <= 16384)
  }
  const ushort2v yx_last = {(unsigned short)(a.H - 1), (unsigned short)(a.W - 2)};  // even width: a pair starts at an even column
  // step (unit, t): unit = image * strips + strip.  Convolution pixel (8 t, 14 qs - 1) reads input rows from
  // 2 p - 3 and input columns from 2 q - 4
  auto load_patch = [&](int unit, int t, unsigned (&v)[PER_THREAD_P]) {
    const int n = div_magic(unit, strips, magic_strips), qs = unit - n * strips;
    const int iy0 = 16 * t - 3, ix0 = 28 * qs - 6;
    const int image = 2 * n * 3 * HW, corner = 2 * (iy0 * a.W + ix0);
    const ushort2v yx0 = {(unsigned short)iy0, (unsigned short)ix0};
#pragma unroll
    for (int k = 0; k < PER_THREAD_P; k++) {
      const ushort2v yx = pe_yx[k] + yx0, in = __builtin_elementwise_min(yx, yx_last);
      unsigned yxu, inu;
      __builtin_memcpy(&yxu, &yx, 4);
      __builtin_memcpy(&inu, &in, 4);
      const int off = yxu == inu ? corner + pe_off[k] : (int)0x80000000;
      v[k] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_x, off, image, 0);
    }
  };
  auto store_patch = [&](int buf, const unsigned (&v)[PER_THREAD_P]) {
    unsigned seen = 0;
#pragma unroll
    for (int k = 0; k < PER_THREAD_P; k++) {
      if (pe_lds[k] >= 0) *reinterpret_cast<unsigned *>(&patch[buf][pe_lds[k]]) = v[k];
      seen |= non_finite_bits(v[k]);
    }
    if (__builtin_amdgcn_ballot_w64((seen & 0x80008000u) != 0) != 0 && lane == 0) nonfinite = 1;
  };
  const int b_base = (2 * (2 * wave + (l32 >> 4))) * PROW + 2 * (l32 & 15);

  // ---- a thread's place in the pooling: pooled row tid / 56 and column tid / 8 % 7 of the step's 4 x 7, channels
  // 8 (tid % 8) .. + 7; window row r is tile row 2 prow - 1 + r (row -1: the carried one) ----
  const int ch = tid & 7, cell = tid >> 3, prow = cell / 7, pcol = cell - 7 * prow;
  const int win_off = ((2 * prow - 1) * 16 + 2 * pcol) * OROW + 8 * ch;  // of window (0, 0) in the staging tile (negative for prow 0)
  const int carry_off = (2 * pcol) * OROW + 8 * ch;                      // the same in the carried row
  const bool pools = tid < 224;

  auto advance = [&](int &u, int &tt) {
    if (++tt == steps_per_unit) { tt = 0; u += (int)gridDim.x; }
  };
  auto pool_step = [&](int unit, int t, int cur) {
    const int n = div_magic(unit, strips, magic_strips), qs = unit - n * strips;
    const int pp = 4 * t + prow, pq = 7 * qs + pcol;
    const _Float16 *st = stage + cur * STAGE, *cy = carry + cur * CARRY;
    // A NaN among the convolution's results needs a non-finite input, weight or bias value (finite fp16 products
    // cannot overflow an fp32 sum).  Until one has been seen the packed fp16 maximum, which drops NaN, is all
    // there is to do; from then on the largest magnitude bit pattern of a window is tracked beside the maximum
    // (above 0x7c00: a NaN), at two more instructions per pair of values.
    auto windows = [&](auto track_c) {
      constexpr bool TRACK = decltype(track_c)::value;
      half8 m;
      ushort8 big = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int e = 0; e < 8; e++) m[e] = (_Float16)(-INFINITY);
#pragma unroll
      for (int r = 0; r < 3; r++) {
        if (r == 0 && prow == 0 && t == 0) continue;  // nothing above the first tile: padding
        const _Float16 *row = (r == 0 && prow == 0) ? cy + carry_off : st + win_off + r * 16 * OROW;
#pragma unroll
        for (int sx = 0; sx < 3; sx++) {
          const half8 v = *reinterpret_cast<const half8 *>(row + sx * OROW);
          m = __builtin_elementwise_max(m, v);
          if (TRACK) {
            ushort8 bits;
            __builtin_memcpy(&bits, &v, 16);
            big = __builtin_elementwise_max(big, (ushort8)(bits & (unsigned short)0x7fff));
          }
        }
      }
      if (RELU) {  // max(relu(x)) = relu(max(x)); a window always holds at least one value, so m is never the padding
        const half8 zero8 = {(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
        m = __builtin_elementwise_max(m, zero8);
      }
      ushort8 mb;
      __builtin_memcpy(&mb, &m, 16);
      if (TRACK) {
#pragma unroll
        for (int e = 0; e < 8; e++) mb[e] = big[e] > 0x7c00 ? (unsigned short)0x7e00 : mb[e];
      }
      if (pp < PP && pq < QQ)
        *reinterpret_cast<ushort8 *>(Yp + (((int64_t)n * PP + pp) * QQ + pq) * 64 + 8 * ch) = mb;
    };
    if (pools) {
      if (__builtin_amdgcn_readfirstlane(nonfinite) != 0) windows(std::true_type{});
      else windows(std::false_type{});
    }
    // the tile's last row is the next step's row -1: 16 pixels x 8 chunks of 16 bytes
    if (tid < 128)
      *reinterpret_cast<half8 *>(carry + (cur ^ 1) * CARRY + tid * 8 + (tid >> 3) * (OROW - 64)) =
          *reinterpret_cast<const half8 *>(st + 7 * 16 * OROW + tid * 8 + (tid >> 3) * (OROW - 64));
  };

  // ---- the walk: patches are loaded two steps ahead (registers), stored to LDS one step ahead --------------
  // Step i: issue the loads of step i + 2; pool step i - 1 (its tile is complete since the last barrier);
  // multiply step i; stage its tile; store the patch of step i + 1, loaded a whole step ago; barrier.
  // Workgroup b runs on XCD b % 8; neighbouring strips of an image read overlapping input columns (and every strip
  // whole 128-byte lines of them): an XCD's workgroups take consecutive strips, so the overlap is read from its L2.
  const int first_unit = (gridDim.x & 7) == 0 ? (int)(blockIdx.x & 7) * (int)(gridDim.x >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  int u0 = first_unit, t0 = 0;  // this step
  int u1 = u0, t1 = 0;          // the next one
  advance(u1, t1);
  int u2 = u1, t2 = t1;         // the one after
  advance(u2, t2);
  int pu = -1, pt = 0;          // the step before (not pooled yet)
  int cur = 0;
  unsigned pvA[PER_THREAD_P], pvB[PER_THREAD_P];
  __syncthreads();  // zero fill done
  load_patch(u0 < units ? u0 : 0, t0, pvA);
  store_patch(0, pvA);
  load_patch(u1 < units ? u1 : 0, t1, pvA);  // (a repeat of some existing patch when nothing follows: the loads are unconditional)
  __syncthreads();

  auto step = [&](unsigned (&ld)[PER_THREAD_P], unsigned (&st)[PER_THREAD_P]) {
    load_patch(u2 < units ? u2 : u0, u2 < units ? t2 : t0, ld);
    if (pu >= 0) pool_step(pu, pt, cur ^ 1);

    floatx16 acc[2];
    const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const _Float16 *pb = &patch[cur][0];
#pragma unroll
    for (int j = 0; j < STEPS; j++) {
      const int cr = 2 * j + half, crc = cr < 21 ? cr : 20;
      const int c = crc / 7, r = crc - c * 7;
      const unsigned *src = reinterpret_cast<const unsigned *>(pb + (c * PY + r) * PROW + b_base);
      u32x4 w;
      w[0] = src[0] & 0xffff0000u; w[1] = src[1]; w[2] = src[2]; w[3] = src[3];  // the window's first column is no tap
      if (j == 0 && half == 0) w[0] |= 0x3c00u;                                   // but the bias's one (fp16 1.0)
      if (j == STEPS - 1 && half) w = (u32x4){0u, 0u, 0u, 0u};                    // nor is patch row 21 a row
      half8 bv;
      __builtin_memcpy(&bv, &w, 16);
      acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][j], bv, j == 0 ? zero16 : acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[1][j], bv, j == 0 ? zero16 : acc[1], 0, 0, 0);
    }

    // the tile into LDS, rounded to fp16: pixel 32 wave + l32 = (row 2 wave + l32 / 16, column l32 % 16).  The ReLU
    // waits until after the pooling (a quarter of the values, and it commutes with the maximum and the rounding)
    {
      const int n = div_magic(u0, strips, magic_strips), qs = u0 - n * strips;
      const int p = 8 * t0 + 2 * wave + (l32 >> 4), q = 14 * qs - 1 + (l32 & 15);
      const bool exists = p < a.P && q >= 0 && q < a.Q;
      const bool all_exist = __builtin_amdgcn_ballot_w64(!exists) == 0;
      _Float16 *os = stage + cur * STAGE + (32 * wave + l32) * OROW;
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
          half4 o;
#pragma unroll
          for (int e = 0; e < 4; e++) o[e] = (_Float16)acc[i][4 * g + e];
          if (!all_exist && !exists) o = (half4){(_Float16)(-INFINITY), (_Float16)(-INFINITY), (_Float16)(-INFINITY), (_Float16)(-INFINITY)};
          *reinterpret_cast<half4 *>(os + 32 * i + 8 * g + 4 * half) = o;
        }
    }
    store_patch(cur ^ 1, st);
    __syncthreads();
    pu = u0; pt = t0;
    u0 = u1; t0 = t1; u1 = u2; t1 = t2;
    advance(u2, t2);
    cur ^= 1;
  };
  while (u0 < units) {
    step(pvB, pvA);
    if (u0 >= units) break;
    step(pvA, pvB);
  }
  if (pu >= 0) pool_step(pu, pt, cur ^ 1);
#endif
}

bool launch_conv_f16_stem(const dnnrtContext *ctx, const ConvF16Args &a, bool &launched) {
  launched = false;
  if (a.format != DNNRT_NCHW_TO_NHWC || a.group != 1 || a.C != 3 || a.R != 7 || a.S != 7 || a.sh != 2 || a.sw != 2 ||
      a.ph != 3 || a.pw != 3 || a.K != 64 || a.Z != nullptr || !aligned16(a.Y) || !aligned16(a.Wt) || (reinterpret_cast<uintptr_t>(a.bias) & 7u) != 0 ||
      (a.act != DNNRT_ACT_RELU && a.act != DNNRT_ACT_IDENTITY))
    return true;
  if ((int64_t)3 * a.H * a.W >= (1ll << 31)) return true;
  const int tiles_p = (a.P + stem::TP - 1) / stem::TP, tiles_q = (a.Q + stem::TQ - 1) / stem::TQ;
  const int64_t total = (int64_t)a.N * tiles_p * tiles_q;
  if (total > INT32_MAX) return true;
  const int64_t grid = total < 2 * (int64_t)ctx->num_cu ? total : 2 * (int64_t)ctx->num_cu;
  if (a.act == DNNRT_ACT_RELU)
    hipLaunchKernelGGL(conv_f16_stem_kernel<true>, dim3((unsigned)grid), dim3(256), 0, ctx->stream, a, tiles_p, tiles_q, (int)total);
  else
    hipLaunchKernelGGL(conv_f16_stem_kernel<false>, dim3((unsigned)grid), dim3(256), 0, ctx->stream, a, tiles_p, tiles_q, (int)total);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("conv(fp16 stem): launch failed: %s", hipGetErrorString(e)); return false; }
  launched = true;
  return true;
}

// The fused first layer: `a` describes the convolution (a.Y unused), Yp receives the pooled tensor N x PP x QQ x 64.
// Refuses, with an error, everything but the shape the kernel is written for.
bool launch_conv_f16_stem_pool(const dnnrtContext *ctx, const ConvF16Args &a, __half *Yp, int PP, int QQ) {
  if (a.format != DNNRT_NCHW_TO_NHWC) { set_error("conv+maxpool: only for an N,C,H,W input and channels-last output (DNNRT_NCHW_TO_NHWC)"); return false; }
  if (a.group != 1 || a.C != 3 || a.R != 7 || a.S != 7 || a.sh != 2 || a.sw != 2 || a.ph != 3 || a.pw != 3 || a.K != 64) {
    set_error("conv+maxpool: the convolution must be 3 -> 64 channels, 7x7, stride 2, pad 3");
    return false;
  }
  if (a.act != DNNRT_ACT_RELU && a.act != DNNRT_ACT_IDENTITY) { set_error("conv+maxpool: activation must be ReLU or identity"); return false; }
  if (!aligned16(Yp) || !aligned16(a.Wt) || (reinterpret_cast<uintptr_t>(a.bias) & 7u) != 0) {
    set_error("conv+maxpool: the filter and the result must be 16-byte aligned, the bias 8-byte aligned");
    return false;
  }
  if ((int64_t)3 * a.H * a.W >= (1ll << 31)) { set_error("conv+maxpool: image too large"); return false; }
  if (a.H > 16384 || a.W > 16384 || (int64_t)2 * a.N * 3 * a.H * a.W >= (1ll << 31)) {
    set_error("conv+maxpool: images up to 16384 x 16384 and an input below 2 GiB");
    return false;
  }
  if ((a.W & 1) || (reinterpret_cast<uintptr_t>(a.X) & 3u)) {  // the input is read two columns at a time
    set_error("conv+maxpool: the input must have an even width and be 4-byte aligned");
    return false;
  }
  const int strips = (QQ + 6) / 7, steps = (a.P + stem::TP - 1) / stem::TP;
  const int64_t units = (int64_t)a.N * strips;
  if (units > INT32_MAX) { set_error("conv+maxpool: batch too large"); return false; }
  const int64_t grid = units < 2 * (int64_t)ctx->num_cu ? units : 2 * (int64_t)ctx->num_cu;
  _Float16 *yp = reinterpret_cast<_Float16 *>(Yp);
  if (a.act == DNNRT_ACT_RELU)
    hipLaunchKernelGGL(conv_f16_stem_pool_kernel<true>, dim3((unsigned)grid), dim3(256), 0, ctx->stream, a, PP, QQ, strips, magic_of(strips), steps, (int)units, yp);
  else
    hipLaunchKernelGGL(conv_f16_stem_pool_kernel<false>, dim3((unsigned)grid), dim3(256), 0, ctx->stream, a, PP, QQ, strips, magic_of(strips), steps, (int)units, yp);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("conv+maxpool: launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

}  // namespace dnnrt
