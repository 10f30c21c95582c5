// fp32 implicit-GEMM on gfx950 MFMA: one kernel family serves dense
// convolution (NCHW), 2-D GEMM and batched matmul.
//
//   D[m, col] = act(alpha * sum_k A[m, k] * B[k, col] + bias[m] + bias_col[col] + beta * Cin[m, col])
//
// A is the weight / left matrix, B the im2col view of the input / right
// matrix.  Columns are output pixels (n, p, q) flattened; for a plain matrix
// product the "image" is 1 x Ncols.
#pragma once
#include "common.h"

namespace dnnrt {

struct IgemmArgs {
  const float *A;     // [M][Kdim] (k contiguous), or [Kdim][a_ld] when a_mcontig
  int64_t a_ld;       // a_mcontig: elements between consecutive k (>= M)
  const float *X;     // conv input / right matrix
  float *Y;
  const float *bias;  // per row m, may be null
  const float *bias_col;  // per column (shared by every z), may be null
  const float *Cin;   // same indexing as Y, scaled by beta, may be null
  float alpha, beta;
  int act;            // DNNRT_ACT_{IDENTITY, RELU, CLIPPED_RELU, LEAKY_RELU}
  float act_coef;     // ceiling / slope of the last two
  int M, Kdim, Ncols;
  // geometry of B: column -> (img, p, q); k -> (c, r, s)
  int H, W, R, S, P, Q, ph, pw, sh, sw;
  int64_t x_img_stride;   // elements between images of X (C*H*W)
  int64_t y_img_stride;   // elements between images of Y (K*P*Q)
  int64_t y_row_stride;   // elements between rows m of Y (P*Q, or ldc)
  int64_t c_row_stride;   // the same for Cin (0: one row added to every row of D)
  int64_t c_z_stride;     // elements between the Cin of consecutive z
  // blockIdx.z: group of a grouped convolution or batch of a batched matmul
  int Z;
  int64_t a_z_stride, x_z_stride, y_z_stride, bias_z_stride;
  unsigned magic_rs, magic_s;  // filled in by launch_igemm_f32: magic_of(R * S), magic_of(S), for the generic filter sizes
  int xcd_m;          // (small kernels, set by their launcher) the XCDs form an xcd_m x (8 / xcd_m) grid over the tile plane
  // ... and what the kernels would otherwise divide for at their start, before any load can be issued (a
  // division is some twenty dependent instructions): log2(8 / xcd_m), tiles per XCD along m and n, and the
  // multiply-high constants of tn_per, P * Q and Q
  int xcd_n_log2, tm_per, tn_per;
  unsigned magic_tn_per, magic_pq, magic_q;
  // (conv1x1_f32_small_kernel) a second 1x1 convolution onto the same result, its reduction appended to the first's:
  // filter A2 ([M][Kdim2] or, a_mcontig, [Kdim2][a_ld]), input X2 of H2 x W2 pixels per channel read with strides sh2, sw2,
  // bias2 per row or null.  A2 == nullptr: none.
  const float *A2, *X2, *bias2;
  int Kdim2, H2, W2, sh2, sw2;
  int64_t x2_img_stride;
  bool b_kcontig;     // B stored [Ncols][Kdim] (k contiguous): GEMM with transB
  bool a_mcontig;     // A stored [Kdim][M]: GEMM with transA
  bool a_vec4;        // A rows may be read as aligned float4
  bool b_vec4;        // (b_kcontig) B rows may be read as aligned float4
};

// The per-column bias of a lane's column, or 0 without one.  The load is
// unconditional (with no bias_col it reads A[0], which always exists, and the
// value is dropped): a load under a branch makes the compiler wait for every
// outstanding load where it is first used, which cost the small kernels over
// a microsecond.
__device__ __forceinline__ float load_bias_col(const IgemmArgs &a, int col) {
  const float *at = a.bias_col ? a.bias_col + col : a.A;
  const float v = *at;
  return a.bias_col ? v : 0.f;
}

// Launches the kernel on `stream`; returns false (with the error text set) if
// the shape cannot be handled.
bool launch_igemm_f32(const dnnrtContext *ctx, const IgemmArgs &a);
// The variant for problems too small to fill the chip with LDS-staged tiles
// (igemm_f32_direct.hip); rsmode / layout as computed by launch_igemm_f32.
bool launch_igemm_f32_direct(const dnnrtContext *ctx, const IgemmArgs &a, int rsmode, int layout);
// 3x3 convolutions large enough for LDS-staged tiles (igemm_f32_3x3.hip); `launched` says whether it applied.
bool launch_conv3x3_f32_tiled(const dnnrtContext *ctx, const IgemmArgs &a, int layout, bool &launched);
// Row-major products with a few hundred rows (gemm_f32_rows.hip); `launched` says whether it applied.
bool launch_gemm_f32_rows(const dnnrtContext *ctx, const IgemmArgs &a, bool &launched);
// Zeroes the first n arrival counters of the context's split-reduction scratch on its stream.  For scratch that
// is shared beyond one handle (splitk_shared): whoever used the counters last may have died half-way.
void clear_split_counters(const dnnrtContext *ctx, int n);
// 3x3 / 1x1 specialisations of the above (igemm_f32_small.hip); `launched` says whether one applied.
bool launch_igemm_f32_small(const dnnrtContext *ctx, const IgemmArgs &a, int rsmode, int layout, bool &launched);

}  // namespace dnnrt
