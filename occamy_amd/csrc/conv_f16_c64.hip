// fp16 channels-last 3x3 convolution (stride 1, padding 1) over exactly 64
// input channels on images up to 62 pixels wide: persistent workgroups, the
// filter in registers, the input patch in LDS.
//
// With 64 channels a tap is one 64-k step and the whole reduction is nine
// steps: a tile-per-workgroup kernel spends more time starting and finishing
// a tile than multiplying, and an im2col kernel fetches every input pixel nine
// times for a layer whose whole input is read in the time its MFMAs take.
// Here two workgroups of four wavefronts are launched per compute unit and
// each walks over its tiles:
//   * a tile is two image rows (2 W <= 128 output pixels); its input patch,
//     four rows with a one-pixel frame, goes straight into LDS (buffer loads
//     with the LDS bit; frame pixels are out-of-range offsets and arrive as
//     zeros) while the previous tile is being multiplied: two patch buffers
//     per workgroup;
//   * the filter never passes through LDS inside the loop: wavefront (mh, nh)
//     owns output channels 32 mh .. + 31 and pixels 64 nh .. + 63 and keeps its
//     32 x 576 slice of the filter as 36 MFMA A operands in registers for the
//     whole kernel, so LDS carries only the B operand (one 16-byte read per
//     MFMA).  The slice reaches the registers through LDS once: a lane's
//     operand is 16 bytes of its own filter row, and 32 rows 1152 bytes apart
//     per load instruction cost more than all the MFMAs of the kernel; as
//     whole 128-byte lines (row, tap) written straight to LDS and read back
//     swizzled the set-up takes a third of that;
//   * results are staged in LDS and stored as whole 128-byte pixel rows (a lane
//     holds four consecutive output channels of one pixel: stored from the
//     registers, an instruction would touch 32 lines with 16 bytes each, and
//     the stores then take longer than the MFMAs).  A tile's staged output is
//     stored at the start of the next tile, so the wait for the next patch —
//     every outstanding vector-memory operation of the wavefront, stores
//     included: loads and stores do not complete in order with each other, so
//     a count would not say which are done — finds the stores long done.  Two
//     barriers per tile, none inside it; the other workgroup of the compute
//     unit, out of step with this one, has the MFMA pipes meanwhile.
// LDS layout of a patch as in conv_f16_patch.hip: [patch pixel][128 bytes],
// chunk c of patch pixel p at position c ^ ((p >> 1) & 7).
#include "conv_f16.h"

#include <type_traits>

namespace dnnrt {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void *lds_ptr;

constexpr int C64_CROW = 64 + 8;  // halfs per row of the output staging tile

// LDS of a workgroup: two patches of `patch_px` pixels (a multiple of 8), the staging tile of 2 W pixel rows, the bias
static int c64_lds_bytes(int patch_px, int W) { return 2 * patch_px * 128 + 2 * W * C64_CROW * 2 + 64 * 2; }

__global__ __launch_bounds__(256, 2) void conv3x3_f16_c64_kernel(const ConvF16Args a, const int tiles_n, const int tiles_per_image,
                                                                 const unsigned magic_tpi, const int patch_px) {
  // The buffer-resource type exists for the device target only (the host pass needs just the launch stub).
#if __HIP_DEVICE_COMPILE__
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  // [2][patch_px pixels][128 bytes], then the staging tile [2 W pixels][C64_CROW], then the bias [64]
  _Float16 *const Cs = reinterpret_cast<_Float16 *>(smem + 2 * patch_px * 128);
  _Float16 *const biasl = Cs + 2 * a.W * C64_CROW;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int mh = wave & 1, nh = wave >> 1;
  const int l32 = lane & 31, half = lane >> 5;
  const int m0 = (int)blockIdx.y * 64;
  const int PW = a.W + 2;
  // Workgroup b runs on XCD b % 8.  Neighbouring tiles share two of their four input rows: the workgroups of one XCD
  // take a run of consecutive tiles at a time, so that the second reader of a row finds it in that XCD's L2.
  const int workers = (int)gridDim.x;
  const int worker = (workers & 7) == 0 ? (int)(blockIdx.x & 7) * (workers >> 3) + (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  if (worker >= tiles_n) return;

  const __amdgpu_buffer_rsrc_t rsrc_x =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.X), 0, 2 * a.N * a.H * a.W * 64, 0x00020000);

  // the bias of the tile's 64 output channels waits in LDS (the registers hold the filter)
  if (tid < 64) {
    const _Float16 *__restrict__ biasg = reinterpret_cast<const _Float16 *>(a.bias);
    biasl[tid] = biasg && m0 + tid < a.K ? biasg[m0 + tid] : (_Float16)0.f;
  }

  // ---- patch loads: up to eight per wavefront and tile -------------------------
  // load i fills patch pixels 8 (wave + 4 i) .. + 7; patch pixel pp = prow * PW + pcol holds input pixel
  // (r0 - 1 + prow, pcol - 1) of the tile's image.  rel[i]: byte offset from input pixel (r0 - 1, 0) to this
  // lane's chunk; whether the row exists depends on the tile.
  // (Recomputed for every tile: sixteen registers held across the loop are sixteen too many beside the filter.)
  auto issue_patch = [&](int tile, int buf) {
    // tile -> image and first row; rows r0 - 1 .. r0 + 2 of the image, those outside it read as zeros, and so
    // does a tile past the end
    const int img = div_magic(tile, tiles_per_image, magic_tpi);
    const int r0 = 2 * (tile - img * tiles_per_image);
    const int base = 2 * (((img * a.H + r0 - 1) * a.W) * 64);  // negative for the first rows of the first image: those lanes are invalid
    const bool dead = tile >= tiles_n;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      if (8 * (wave + 4 * i) >= patch_px) break;  // (uniform) the patch ends before this group of eight pixels
      const int pp = 8 * (wave + 4 * i) + (lane >> 3), ch = (lane & 7) ^ ((pp >> 1) & 7);
      const int prow = div_magic(pp, PW, a.magic_pw), pcol = pp - prow * PW;
      const int row = r0 - 1 + prow;
      const bool out = dead || prow > 3 || pcol < 1 || pcol > a.W || row < 0 || row >= a.H;
      const unsigned off = out ? 0x80000000u : (unsigned)(base + 2 * ((prow * a.W + pcol - 1) * 64 + ch * 8));
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_ptr)(smem + buf * patch_px * 128 + 1024 * (wave + 4 * i)), 16, off, 0, 0, 0);
    }
  };

  // ---- operand fetch: this lane's two pixels at each tap --------------------------
  // slot s = 64 nh + 32 j + l32 is pixel (s / W, s % W) of the tile's two rows; tap (r, c) reads patch pixel
  // (s / W + r) * PW + s % W + c.  Slots past 2 W compute a copy of slot 0 that is never stored.
  unsigned bad[2][9];
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int s0 = 64 * nh + 32 * j + l32, s = s0 < 2 * a.W ? s0 : 0;
    const int row = s >= a.W ? 1 : 0, q = s - row * a.W;
#pragma unroll
    for (int t = 0; t < 9; t++) {
      const int pp = (row + t / 3) * PW + q + t % 3;
      bad[j][t] = (unsigned)(pp * 128 + (((half ^ (pp >> 1)) & 7) << 4));
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
  _Float16 *__restrict__ Yg = reinterpret_cast<_Float16 *>(a.Y);
  auto store_tile = [&](int tile) {  // the staged tile to global memory, 16 bytes per thread and round
    const int img = div_magic(tile, tiles_per_image, magic_tpi);
    const int r0 = 2 * (tile - img * tiles_per_image);
    const int valid = (r0 + 1 < a.H ? 2 : 1) * a.W;
    const int64_t pix0 = (int64_t)(img * a.H + r0) * a.W;  // the tile's pixels are consecutive in N,H,W order
#pragma unroll
    for (int o = 0; o < 4; o++) {
      const int id = tid + 256 * o, slot = id >> 3, ch = id & 7;
      const int k_out = m0 + 8 * ch;
      if (slot < valid && k_out < a.K)
        *reinterpret_cast<half8 *>(Yg + (pix0 + slot) * a.K + k_out) = *reinterpret_cast<const half8 *>(Cs + slot * C64_CROW + 8 * ch);
    }
  };

  issue_patch(worker, 0);

  // ---- the filter slice of this wavefront, as MFMA A operands -----------------
  // operand (tap, sub): row l32 of the slice, k = 64 tap + 16 sub + 8 half .. + 7.
  // Through LDS (the second patch buffer and the staging tile, not yet in use, while the first tile's patch is
  // already on its way into the first buffer), one half of the output channels at a time: line
  // 9 row + tap holds the 128 bytes of (row, tap), chunk c at position c ^ ((line >> 1) & 7), which spreads the
  // 32 rows a fetch reads over all banks.
  half8 fa[9][4];
  {
    char *const fstage = smem + patch_px * 128;
    const __amdgpu_buffer_rsrc_t rsrc_w =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<__half *>(a.Wt), 0, 2 * a.K * 576, 0x00020000);
#pragma unroll
    for (int pass = 0; pass < 2; pass++) {
#pragma unroll
      for (int i = 0; i < 9; i++) {  // 288 lines of 128 bytes, eight per load instruction, nine instructions per wavefront
        const int line = 8 * (wave + 4 * i) + (lane >> 3), ch = (lane & 7) ^ ((line >> 1) & 7);
        const int row = line / 9, tap = line - 9 * row, k_out = m0 + 32 * pass + row;
        const unsigned off = k_out < a.K ? 2u * (unsigned)(k_out * 576 + tap * 64 + ch * 8) : 0x80000000u;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_ptr)(fstage + 1024 * (wave + 4 * i)), 16, off, 0, 0, 0);
      }
      __builtin_amdgcn_s_waitcnt(0);
      __syncthreads();
      if (mh == pass) {
#pragma unroll
        for (int t = 0; t < 9; t++) {
          const int line = 9 * l32 + t;
          const char *at = fstage + line * 128;
          const unsigned sw = (unsigned)((line >> 1) & 7);
#pragma unroll
          for (int sub = 0; sub < 4; sub++) fa[t][sub] = *reinterpret_cast<const half8 *>(at + ((((unsigned)(2 * sub + half)) ^ sw) << 4));
        }
      }
      __syncthreads();  // the lines have been read: the space is free for the other half, then for the patches
    }
  }
  // ---- the walk over this workgroup's tiles --------------------------------------
  int buf = 0, prev = -1;
  for (int tile = worker; tile < tiles_n; tile += workers) {
    // this tile's patch has landed (the stores of the tile before last, issued a tile ago, are done as well), and
    // this wavefront's writes to the staging tile and of the bias; after the barrier everybody is also done reading
    // the other buffer, so the next tile's patch can land there while this tile is multiplied
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (prev >= 0) store_tile(prev);
    if (tile + workers < tiles_n) issue_patch(tile + workers, buf ^ 1);

    // (keeps the compiler from carrying the 72 operand addresses of a tile, which do not depend on the tile,
    // in registers across the loop)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int t = 0; t < 9; t++) asm volatile("" : "+v"(bad[j][t]));
    const char *slab = smem + buf * patch_px * 128;
    floatx16 acc[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[j][r] = 0.f;
    half8 fb[2][2];
    fb[0][0] = *reinterpret_cast<const half8 *>(slab + bad[0][0]);
    fb[0][1] = *reinterpret_cast<const half8 *>(slab + bad[1][0]);
#pragma unroll
    for (int t = 0; t < 9; t++) {
#pragma unroll
      for (int sub = 0; sub < 4; sub++) {
        // the operands of the next sub-step are requested before this one's MFMAs
        const int cur = sub & 1, nxt = cur ^ 1;
        if (sub < 3) {
          fb[nxt][0] = *reinterpret_cast<const half8 *>(slab + (bad[0][t] ^ (32u * (sub + 1))));
          fb[nxt][1] = *reinterpret_cast<const half8 *>(slab + (bad[1][t] ^ (32u * (sub + 1))));
        } else if (t < 8) {
          fb[nxt][0] = *reinterpret_cast<const half8 *>(slab + bad[0][t < 8 ? t + 1 : 8]);
          fb[nxt][1] = *reinterpret_cast<const half8 *>(slab + bad[1][t < 8 ? t + 1 : 8]);
        }
        __builtin_amdgcn_sched_barrier(0);
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[t][sub], fb[cur][0], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[t][sub], fb[cur][1], acc[1], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- results: register r of lane l in block j is k_out 8 (r / 4) + 4 (l / 32) + r % 4, pixel 32 j + l % 32.
    // Everybody's copies of the previous tile out of the staging tile are done before it is written again.
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    per_mode(a.act, [&](auto mode_c) {
      constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int kl = 32 * mh + 8 * g + 4 * half;
        const half4 b4 = *reinterpret_cast<const half4 *>(biasl + kl);
#pragma unroll
        for (int j = 0; j < 2; j++) {
          const int slot = 64 * nh + 32 * j + l32;
          half4 o;
#pragma unroll
          for (int e = 0; e < 4; e++) o[e] = (_Float16)apply_act(acc[j][4 * g + e] + (float)b4[e], MODE, a.act_coef);
          if (slot < 2 * a.W) *reinterpret_cast<half4 *>(Cs + slot * C64_CROW + kl) = o;
        }
      }
    });
    prev = tile;
    buf ^= 1;
  }
  __syncthreads();
  if (prev >= 0) store_tile(prev);
#endif
}

bool c64_conv_applies(const ConvF16Args &a) {
  return a.format == DNNRT_NHWC && a.group == 1 && a.R == 3 && a.S == 3 && a.sh == 1 && a.sw == 1 && a.ph == 1 && a.pw == 1 &&
         a.C == 64 && a.K % 8 == 0 && a.W <= 62 && a.Z == nullptr && (int64_t)a.N * a.H * a.W * 64 < (1ll << 30) &&
         (int64_t)a.K * 576 < (1ll << 30) && (int64_t)a.N * ((a.H + 1) / 2) < (1 << 30) && aligned16(a.X) && aligned16(a.Wt) &&
         aligned16(a.Y) && (reinterpret_cast<uintptr_t>(a.bias) & 7u) == 0;
}

// `a` must satisfy c64_conv_applies.
bool launch_conv_f16_c64(const dnnrtContext *ctx, const ConvF16Args &a) {
  const int tiles_per_image = (a.H + 1) / 2;
  const int tiles_n = a.N * tiles_per_image;
  const int tiles_m = (int)ceil_div(a.K, 64);
  if (tiles_m > 65535) { set_error("conv(fp16): too many output channels for the 64-channel kernel"); return false; }
  // two workgroups per compute unit walk the tiles (each wavefront holds its filter slice in registers: eight
  // wavefronts fill a CU's register files)
  const int slots = 2 * ctx->num_cu / tiles_m > 0 ? 2 * ctx->num_cu / tiles_m : 1;
  const int workers = tiles_n < slots ? tiles_n : slots;
  ConvF16Args am = a;
  am.magic_pw = magic_of(a.W + 2);
  // four patch rows, rounded up to whole load instructions (eight pixels); the filter passes through the space
  // behind the first patch at start-up, 36 KiB at a time
  int patch_px = (int)ceil_div(4 * (a.W + 2), 8) * 8;
  while (c64_lds_bytes(patch_px, a.W) - 64 * 2 - patch_px * 128 < 36 * 1024) patch_px += 8;
  const int smem = c64_lds_bytes(patch_px, a.W);
  static bool raised[16] = {};
  if (ctx->device < 0 || ctx->device >= 16) { set_error("conv(fp16): device ordinal %d", ctx->device); return false; }
  if (!raised[ctx->device]) {  // more than 64 KiB of LDS has to be asked for, once per device (the largest any width needs)
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(&conv3x3_f16_c64_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            c64_lds_bytes(256, 62)) != hipSuccess) {
      set_error("conv(fp16): cannot reserve %d bytes of LDS", c64_lds_bytes(256, 62));
      return false;
    }
    raised[ctx->device] = true;
  }
  hipLaunchKernelGGL(conv3x3_f16_c64_kernel, dim3((unsigned)workers, (unsigned)tiles_m), dim3(256), (size_t)smem, ctx->stream, am,
                     tiles_n, tiles_per_image, magic_of(tiles_per_image), patch_px);
  return true;
}

}  // namespace dnnrt
