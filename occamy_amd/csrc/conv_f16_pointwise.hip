// Channels-last fp16 1x1 stride-1 convolutions over a channel count the tiled
// kernels do not take (a multiple of 8 up to 256 that is not a multiple of 64:
// the 16, 24, 32, 96, 144 and 160 channels of a MobileNetV2).
//
// Such a layer is a product of a tall matrix (pixels x C, contiguous in
// memory) with a small one (C x K) and is bound by the bytes of its input and
// result.  There is no workgroup tile and no barrier: a wavefront owns 32
// consecutive pixels, reads their channels once, straight in the MFMA's
// operand shape (lane l of half h holds channels 16 s + 8 h .. + 7 of pixel
// l, for every 16-channel step s), and walks the filters in blocks of 32: per
// block one v_mfma_f32_32x32x16_f16 per step, the filter block read from
// global memory in the same shape (the whole filter is a few KB to a few
// hundred KB and stays in the caches), then bias, residual and activation on
// the lane's sixteen results (four runs of four consecutive filters of one
// pixel), which leave through a small staging tile of the wavefront's own so
// that the stores are 16 bytes a lane and contiguous per pixel.  The next
// block's filter values are requested before the current block's MFMAs.  With few pixels the filter
// blocks are dealt over gridDim.y, so that the launch still has a few
// thousand wavefronts.
#include "conv_f16.h"

namespace dnnrt {

typedef _Float16 pw_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 pw_half4 __attribute__((ext_vector_type(4)));
typedef float pw_floatx16 __attribute__((ext_vector_type(16)));

constexpr int PW_MAX_C = 256;
constexpr int PW_CHUNK = 4;                        // filter blocks per pass through the staging tile
constexpr int PW_STAGE_ROW = 32 * PW_CHUNK + 8;     // halfs per pixel row of the tile (16 bytes of padding)

template <int STEPS, bool STAGED>
__global__ __launch_bounds__(256) void conv1x1_f16_pointwise_kernel(const ConvF16Args a, const int npq, const int kblocks,
                                                                    const int kblocks_per_group) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, half = lane >> 5;
  const int64_t p0 = ((int64_t)blockIdx.x * 4 + wave) * 32;
  if (p0 >= npq) return;  // the whole wavefront
  const int64_t pix = p0 + l32;
  const bool pix_ok = pix < npq;
  const _Float16 *__restrict__ Xg = reinterpret_cast<const _Float16 *>(a.X);
  const _Float16 *__restrict__ Wg = reinterpret_cast<const _Float16 *>(a.Wt);
  const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
  const _Float16 *Zg = reinterpret_cast<const _Float16 *>(a.Z);  // may be Y itself: a thread reads an element, then writes it
  _Float16 *Yg = reinterpret_cast<_Float16 *>(a.Y);

  pw_half8 zero8;
#pragma unroll
  for (int e = 0; e < 8; e++) zero8[e] = (_Float16)0.f;
  pw_half8 xf[STEPS];
#pragma unroll
  for (int s = 0; s < STEPS; s++) {
    // loads are unconditional, from clamped addresses (a load under a branch is waited for before the next one
    // is issued); what must not contribute is replaced by zeros afterwards
    const int ch = (2 * s + half) * 8;
    const pw_half8 v = *reinterpret_cast<const pw_half8 *>(Xg + (pix_ok ? pix : (int64_t)npq - 1) * a.C + (ch < a.C ? ch : 0));
    xf[s] = (pix_ok && ch < a.C) ? v : zero8;
  }
  auto filter_block = [&](pw_half8 (&wf)[STEPS], const int kb) {
    const int krow = kb * 32 + l32;
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
      const int ch = (2 * s + half) * 8;
      const pw_half8 v = *reinterpret_cast<const pw_half8 *>(Wg + (int64_t)min(krow, a.K - 1) * a.C + (ch < a.C ? ch : 0));
      wf[s] = (krow < a.K && ch < a.C) ? v : zero8;
    }
  };
  // Results leave through a staging tile of the wavefront's own (32 pixels x up to four filter blocks, fp16): the
  // accumulators hold four filters of one pixel per lane, the tile is read back sixteen bytes a lane with a pixel's
  // filters side by side, so a store instruction covers runs of 64 to 256 bytes instead of 32 runs of 16.
  // (STAGED: layers with few input channels and many filters, where the stores are what takes the time; elsewhere
  // the tile's LDS costs more in wavefronts per CU than the wider stores give back, and the lanes store their runs
  // of four filters themselves: 96 -> 576 channels at 14 x 14, batch 64: 21 us against 27.)
  __shared__ __attribute__((aligned(16))) _Float16 stage_all[STAGED ? 4 : 1][STAGED ? 32 * PW_STAGE_ROW : 8];
  _Float16 *const stage = stage_all[STAGED ? wave : 0];
  const int kb_begin = (int)blockIdx.y * kblocks_per_group, kb_end = min(kblocks, kb_begin + kblocks_per_group);
  pw_half8 wf[STEPS], wn[STEPS];
  if (kb_begin < kb_end) filter_block(wf, kb_begin);
  for (int kc = kb_begin; kc < kb_end; kc += PW_CHUNK) {
    const int nb = min(PW_CHUNK, kb_end - kc);
    for (int j = 0; j < nb; j++) {
      const int kb = kc + j;
      if (kb + 1 < kb_end) filter_block(wn, kb + 1);
      pw_floatx16 acc;
#pragma unroll
      for (int r = 0; r < 16; r++) acc[r] = 0.f;
#pragma unroll
      for (int s = 0; s < STEPS; s++) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[s], xf[s], acc, 0, 0, 0);
      // acc[4 g + i]: filter 32 kb + 8 g + 4 half + i of pixel l32.  With a residual the tile holds the rounded
      // sum of product and bias, the rest follows when the tile is read back; without, the finished value.
      // one copy of the loop per activation mode, picked once: the mode is the same for every lane
      auto finish_block = [&](auto mode_c) {
        constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const int kk = kb * 32 + 8 * g + 4 * half;
          pw_half4 b4, z4, o4;
          const bool k_ok = kk < a.K;  // K is a multiple of four: a run of four is inside or outside as a whole
          const int64_t at = pix * a.K + kk;
          if (biasg && k_ok) b4 = *reinterpret_cast<const pw_half4 *>(biasg + kk);
          if (!STAGED && Zg && k_ok && pix_ok) z4 = *reinterpret_cast<const pw_half4 *>(Zg + at);
#pragma unroll
          for (int i = 0; i < 4; i++) {
            float v = acc[4 * g + i];
            if (biasg && k_ok) v += (float)b4[i];
            if (!STAGED && Zg && k_ok && pix_ok) v = (float)(_Float16)v + (float)z4[i];
            o4[i] = (_Float16)((STAGED && Zg) ? v : apply_act(v, MODE, a.act_coef));
          }
          if (STAGED) *reinterpret_cast<pw_half4 *>(stage + l32 * PW_STAGE_ROW + j * 32 + 8 * g + 4 * half) = o4;
          else if (k_ok && pix_ok) *reinterpret_cast<pw_half4 *>(Yg + at) = o4;
        }
      };
      by_act_mode(a.act, finish_block);
#pragma unroll
      for (int s = 0; s < STEPS; s++) wf[s] = wn[s];
    }
    if (!STAGED) continue;
    // LDS serves a wavefront's instructions in order: what the compiler must not do is move the tile's reads
    // above its writes (a fence that waits for the global stores in flight as well would cost their latency).
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_wave_barrier();
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    const int parts = 4 * nb;  // 16-byte parts of a pixel's row in the tile
    const unsigned by_parts = nb == 1 ? 16384u : nb == 2 ? 8192u : nb == 3 ? 5462u : 4096u;  // ceil(2^16 / parts): i / parts for i < 512
    auto finish_tile = [&](auto mode_c) {
      constexpr int MODE = decltype(mode_c)::value;
      for (int i = lane; i < 32 * parts; i += 64) {
        const int prow = (int)(((unsigned)i * by_parts) >> 16), part = i - prow * parts;
        const int kk = kc * 32 + 8 * part;
        if (p0 + prow < npq && kk < a.K) {  // K is a multiple of eight
          const int64_t at = (p0 + prow) * a.K + kk;
          pw_half8 v8 = *reinterpret_cast<const pw_half8 *>(stage + prow * PW_STAGE_ROW + 8 * part);
          if (Zg) {
            const pw_half8 z8 = *reinterpret_cast<const pw_half8 *>(Zg + at);
#pragma unroll
            for (int e = 0; e < 8; e++) v8[e] = (_Float16)apply_act((float)v8[e] + (float)z8[e], MODE, a.act_coef);
          }
          *reinterpret_cast<pw_half8 *>(Yg + at) = v8;
        }
      }
    };
    by_act_mode(a.act, finish_tile);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_wave_barrier();
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
  }
}

constexpr int PW_STAGED_MAX_C = 32;  // the staged variant is compiled for one and two steps only

template <int STEPS>
static void pointwise_launch(const dnnrtContext *ctx, const ConvF16Args &a, dim3 grid, bool staged, int npq, int kblocks, int per_group) {
  if constexpr (16 * STEPS <= PW_STAGED_MAX_C) {
    if (staged) {
      hipLaunchKernelGGL((conv1x1_f16_pointwise_kernel<STEPS, true>), grid, dim3(256), 0, ctx->stream, a, npq, kblocks, per_group);
      return;
    }
  }
  hipLaunchKernelGGL((conv1x1_f16_pointwise_kernel<STEPS, false>), grid, dim3(256), 0, ctx->stream, a, npq, kblocks, per_group);
}

bool pointwise_conv_applies(const ConvF16Args &a) {
  auto aligned = [](const void *p, uintptr_t to) { return (reinterpret_cast<uintptr_t>(p) & (to - 1)) == 0; };
  return a.format == DNNRT_NHWC && a.group == 1 && a.R == 1 && a.S == 1 && a.sh == 1 && a.sw == 1 && a.ph == 0 && a.pw == 0 &&
         a.C % 8 == 0 && a.C >= 8 && a.C <= PW_MAX_C && a.K % 8 == 0 && a.K >= 8 &&
         (int64_t)a.N * a.P * a.Q + 128 < (1ll << 31) && aligned(a.X, 16) && aligned(a.Wt, 16) && aligned(a.Y, 16) &&
         aligned(a.Z, 16) && aligned(a.bias, 8);
}

bool launch_conv_f16_pointwise(const dnnrtContext *ctx, const ConvF16Args &a) {
  const int npq = (int)((int64_t)a.N * a.P * a.Q);
  if (npq == 0) return true;
  const int waves = (npq + 31) / 32, kblocks = (a.K + 31) / 32;
  // a few thousand wavefronts: eight per CU where the pixels alone do not give them
  const int want = 8 * ctx->num_cu;
  int groups = waves >= want ? 1 : (want + waves - 1) / waves;
  groups = groups > kblocks ? kblocks : groups;
  const int per_group = (kblocks + groups - 1) / groups;
  groups = (kblocks + per_group - 1) / per_group;
  const dim3 grid((unsigned)((waves + 3) / 4), (unsigned)groups);
  const int steps = (a.C + 15) / 16;
  const bool staged = a.C <= PW_STAGED_MAX_C && a.K >= 64;
#define PW_CASE(S) \
  case S: pointwise_launch<S>(ctx, a, grid, staged, npq, kblocks, per_group); break
  switch (steps) {
    PW_CASE(1); PW_CASE(2); PW_CASE(3); PW_CASE(4); PW_CASE(5); PW_CASE(6); PW_CASE(7); PW_CASE(8);
    PW_CASE(9); PW_CASE(10); PW_CASE(11); PW_CASE(12); PW_CASE(13); PW_CASE(14); PW_CASE(15); PW_CASE(16);
    default: set_error("conv(fp16): the pointwise kernel takes up to %d channels", PW_MAX_C); return false;
  }
#undef PW_CASE
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("conv(fp16): launch failed: %s", hipGetErrorString(e)); return false; }
  return true;
}

}  // namespace dnnrt
