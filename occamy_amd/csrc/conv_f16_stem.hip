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
// current one is computed.  The bias is the accumulators' starting value.
//
// Wavefront w owns output rows 2w, 2w+1 of the tile (32 pixels) and all 64
// output channels (two 32x32 MFMA blocks).  Results go through a
// wave-private LDS buffer so that each pixel's 64 channels leave as one
// 128-byte line.
#include "conv_f16.h"

namespace dnnrt {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

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
  half4 bias4[2][4];
  {
    // eight unconditional 8-byte loads (from the filter when there is no bias, then zeroed): a load under a
    // branch is waited for before the next one is issued, and 32 of them in a row took longer than ten tiles
    const bool has_bias = a.bias != nullptr;
    const _Float16 *__restrict__ biasg = has_bias ? reinterpret_cast<const _Float16 *>(a.bias) : Wg;
    const half4 zero4 = {(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const half4 b = *reinterpret_cast<const half4 *>(biasg + 32 * i + 8 * g + 4 * half);
        bias4[i][g] = has_bias ? b : zero4;
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
      for (int r = 0; r < 16; r++) acc[i][r] = (float)bias4[i][r >> 2][r & 3];  // the sum starts from the bias
    const _Float16 *pb = &patch[cur][0];
#pragma unroll
    for (int j = 0; j < STEPS; j++) {
      const int cr = 2 * j + half, crc = cr < 21 ? cr : 20;
      const int c = crc / 7, r = crc - c * 7;
      const unsigned *src = reinterpret_cast<const unsigned *>(pb + (c * PY + r) * PROW + b_base);
      u32x4 w;
      w[0] = src[0]; w[1] = src[1]; w[2] = src[2]; w[3] = src[3] & 0x0000ffffu;  // tap s = 7 does not exist
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

}  // namespace dnnrt
