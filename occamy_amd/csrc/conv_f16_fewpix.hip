// fp16 1x1 convolution / matrix product over few output pixels (a fully
// connected layer at small batch): Y[pix][k_out] = sum_c X[pix][c] * Wt[k_out][c].
//
// With at most a few dozen pixels the tiled kernels have a handful of tiles
// and walk the whole reduction in one workgroup each: 8 workgroups and 32
// serial steps for 64 x 2048 -> 1000.  The work is reading the filter once, so
// here a workgroup owns 16 filters and 32 pixels, its four wavefronts share the
// channels (64-channel chunks dealt round-robin), every wavefront keeps four
// chunks of loads in flight, and the four partial sums meet in LDS.
//
// v_mfma_f32_16x16x32_f16: lane l holds row/column l % 16 and the eight
// reduction indices 8 * (l / 16) ... + 7 of both operands.  Any bijection of
// the channels onto (instruction, lane group, element) gives the same sum, so
// a lane reads 16 consecutive channels (32 bytes) per chunk and feeds the two
// halves to two instructions: a filter row is read in 128-byte runs.
#include "conv_f16.h"

namespace dnnrt {

typedef _Float16 fp_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 fp_half4 __attribute__((ext_vector_type(4)));
typedef float fp_float4 __attribute__((ext_vector_type(4)));

struct FewChunk {
  fp_half8 w0, w1;        // 16 channels of this lane's filter
  fp_half8 x00, x01;      // the same channels of its pixel in the first block of 16 pixels
  fp_half8 x10, x11;      // and in the second block
};

__global__ __launch_bounds__(256) void conv_f16_fewpix_kernel(ConvF16Args a, int npix) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, lr = lane & 15, lg = lane >> 4;
  const int f = min((int)blockIdx.x * 16 + lr, a.K - 1);
  const int p0 = min((int)blockIdx.y * 32 + lr, npix - 1), p1 = min((int)blockIdx.y * 32 + 16 + lr, npix - 1);
  const _Float16 *__restrict__ wrow = reinterpret_cast<const _Float16 *>(a.Wt) + (int64_t)f * a.C + lg * 16;
  const _Float16 *__restrict__ xrow0 = reinterpret_cast<const _Float16 *>(a.X) + (int64_t)p0 * a.C + lg * 16;
  const _Float16 *__restrict__ xrow1 = reinterpret_cast<const _Float16 *>(a.X) + (int64_t)p1 * a.C + lg * 16;
  const int nch = a.C >> 6;                    // 64-channel chunks; this wavefront takes chunks wave, wave + 4, ...
  const int mine = (nch - wave + 3) >> 2;      // how many of them (0 when nch <= wave)
  const int rounds = (nch + 3) >> 2;           // the most any wavefront takes
  const int last = max(mine - 1, 0);

  // chunk i of this wavefront; past its last one the last is read again (a valid address) and not used
  auto fetch = [&](FewChunk &c, int i) {
    const int off = (wave + 4 * min(i, last)) * 64;
    c.w0 = *reinterpret_cast<const fp_half8 *>(wrow + off);
    c.w1 = *reinterpret_cast<const fp_half8 *>(wrow + off + 8);
    c.x00 = *reinterpret_cast<const fp_half8 *>(xrow0 + off);
    c.x01 = *reinterpret_cast<const fp_half8 *>(xrow0 + off + 8);
    c.x10 = *reinterpret_cast<const fp_half8 *>(xrow1 + off);
    c.x11 = *reinterpret_cast<const fp_half8 *>(xrow1 + off + 8);
  };
  fp_float4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  auto use = [&](const FewChunk &c, int i) {
    const bool live = i < mine;
    const fp_half8 zero = {};
    const fp_half8 w0 = live ? c.w0 : zero, w1 = live ? c.w1 : zero;
    acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, c.x00, acc0, 0, 0, 0);
    acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, c.x10, acc1, 0, 0, 0);
    acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, c.x01, acc0, 0, 0, 0);
    acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, c.x11, acc1, 0, 0, 0);
  };
  FewChunk c0, c1, c2, c3;
  fetch(c0, 0); fetch(c1, 1); fetch(c2, 2); fetch(c3, 3);
  int i = 0;
  for (; i + 4 < rounds; i += 4) {
    use(c0, i);     fetch(c0, i + 4);
    use(c1, i + 1); fetch(c1, i + 5);
    use(c2, i + 2); fetch(c2, i + 6);
    use(c3, i + 3); fetch(c3, i + 7);
  }
  use(c0, i); use(c1, i + 1); use(c2, i + 2); use(c3, i + 3);

  // the four wavefronts' sums meet in LDS; 128 threads finish one (pixel block, lane) each
  __shared__ fp_float4 red[4][2][64];
  red[wave][0][lane] = acc0;
  red[wave][1][lane] = acc1;
  __syncthreads();
  if (tid >= 128) return;
  const int pb = tid >> 6;
  fp_float4 v = red[0][pb][lane];
#pragma unroll
  for (int w = 1; w < 4; w++) {
    const fp_float4 o = red[w][pb][lane];
    v[0] += o[0]; v[1] += o[1]; v[2] += o[2]; v[3] += o[3];
  }
  // lane l of the result holds pixel l % 16 and filters 4 * (l / 16) ... + 3
  const int pix = (int)blockIdx.y * 32 + pb * 16 + lr, k_out = (int)blockIdx.x * 16 + 4 * lg;
  if (pix >= npix || k_out >= a.K) return;     // K_out % 4 == 0: a group of four is inside or outside as a whole
  const int64_t off = (int64_t)pix * a.K + k_out;
  if (a.bias) {
    const fp_half4 b = *reinterpret_cast<const fp_half4 *>(reinterpret_cast<const _Float16 *>(a.bias) + k_out);
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] += (float)b[e];
  }
  if (a.Z) {
    // convolution + bias is rounded to fp16 as a separate convolution would have stored it; the residual sum follows in fp32
    const fp_half4 z = *reinterpret_cast<const fp_half4 *>(reinterpret_cast<const _Float16 *>(a.Z) + off);
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] = (float)(_Float16)v[e] + (float)z[e];
  }
  fp_half4 o;
#pragma unroll
  for (int e = 0; e < 4; e++) o[e] = (_Float16)apply_act(v[e], a.act, a.act_coef);
  *reinterpret_cast<fp_half4 *>(reinterpret_cast<_Float16 *>(a.Y) + off) = o;
}

bool launch_conv_f16_fewpix(const dnnrtContext *ctx, const ConvF16Args &a, bool &launched) {
  launched = false;
  const int64_t npix = (int64_t)a.N * a.P * a.Q;
  const bool fits = a.format == DNNRT_NHWC && a.group == 1 && a.R == 1 && a.S == 1 && a.ph == 0 && a.pw == 0 &&
                    a.sh == 1 && a.sw == 1 && a.P == a.H && a.Q == a.W && a.C % 64 == 0 && a.C >= 256 && a.K % 4 == 0 &&
                    npix >= 1 && npix <= FEWPIX_MAX_PIXELS && (int64_t)a.K * a.C < (1ll << 31) &&
                    aligned16(a.X) && aligned16(a.Wt) && (reinterpret_cast<uintptr_t>(a.Y) & 7u) == 0 &&
                    (reinterpret_cast<uintptr_t>(a.Z) & 7u) == 0 && (reinterpret_cast<uintptr_t>(a.bias) & 7u) == 0;
  const int forced = ctx->f16_tile;
  if (!fits || forced != 0) return true;  // another kernel's problem (or another tile is forced)
  const dim3 grid((unsigned)ceil_div(a.K, 16), (unsigned)ceil_div(npix, 32));
  hipLaunchKernelGGL(conv_f16_fewpix_kernel, grid, dim3(256), 0, ctx->stream, a, (int)npix);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { set_error("conv(fp16): launch failed: %s", hipGetErrorString(e)); return false; }
  launched = true;
  return true;
}

}  // namespace dnnrt
