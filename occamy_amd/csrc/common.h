// Shared declarations of the gfx950 runtime library: the handle, error
// reporting and small host helpers.  Everything here is internal; the public
// surface is include/dnnrt.h.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/dnnrt.h"

struct dnnrtContext {
  hipStream_t stream;  // kernels of this handle are launched here
  int format;          // DNNRT_NCHW / DNNRT_NHWC / DNNRT_NCHW_TO_NHWC
  int filter_layout;   // DNNRT_FILTER_KCRS / DNNRT_FILTER_CRSK (fp32 convolutions)
  float act_coef;      // ceiling of CLIPPED_RELU / slope of LEAKY_RELU
  int device;
  int num_cu;
  // Scratch for reductions split over workgroups: partial tiles and one
  // arrival counter per output tile (all zero between kernels).  The library's
  // static array for the first live handle of a device, allocated for any
  // further one; kernels of one handle run in stream order, so they share it.
  float *splitk_partials;
  unsigned *splitk_counters;
  int64_t splitk_partial_bytes;  // what the two buffers hold
  int splitk_max_tiles;
  // The buffers are shared with callers this handle knows nothing of (the process-wide static scratch of
  // dnnrtConvBiasActivNoAlloc): clear the counters a launch uses before it, and refuse a problem whose
  // split would have to shrink to fit instead of shrinking it.
  bool splitk_shared;
  bool scratch_is_static;  // the two buffers are the library's static array (held by one handle per device), not allocations
  int f16_tile;        // dnnrtSetConvTile: 0 = pick the fp16 convolution variant by problem size, otherwise one of F16_TILE_IDS
};

namespace dnnrt {

constexpr int64_t SPLITK_PARTIAL_BYTES = 8ll << 20;  // a handle's scratch: 2048 partial 32x32 fp32 tiles
constexpr int SPLITK_MAX_TILES = 16384;               // ... and arrival counters
// The static scratch of dnnrtConvBiasActivNoAlloc (conv.hip): the split-reduction convolution kernels ask for
// at most one partial tile per compute unit, 1 MiB on 256 of them.
constexpr int64_t NOALLOC_PARTIAL_BYTES = 1ll << 20;
constexpr int NOALLOC_MAX_TILES = 1024;

// The fp16 channels-last convolution variants dnnrtSetConvTile can force
// (zero-terminated; what each one is: launch_conv_f16 in conv_f16.hip).
constexpr int F16_TILE_IDS[] = {3, 4, 11, 12, 15, 17, 18, 31, 32, 33, 34, 35, 36, 37, 38, 39, 40, 60, 61, 62, 63, 64, 65, 66, 67, 69,
                                  41, 42, 43, 44, 45, 46, 47, 48, 49, 51, 52, 54, 57, 70, 0};

void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

// Compute entry points return NULL on error.
#define DNNRT_FAIL(...)                                                        \
  do {                                                                         \
    ::dnnrt::set_error(__VA_ARGS__);                                           \
    return nullptr;                                                            \
  } while (0)

#define DNNRT_CHECK_LAUNCH(what)                                               \
  do {                                                                         \
    hipError_t e_ = hipGetLastError();                                         \
    if (e_ != hipSuccess) DNNRT_FAIL("%s: launch failed: %s", what, hipGetErrorString(e_)); \
  } while (0)

inline int64_t numel(const int64_t *d, int64_t rank) {
  int64_t n = 1;
  for (int64_t i = 0; i < rank; i++) n *= d[i];
  return n;
}
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool float_dtype(int32_t dt) { return dt == DNNRT_F32 || dt == DNNRT_F16; }

// Gelu as an epilogue of the matrix products only (not an activMode of the convolution calls).
constexpr int ACT_GELU = 7;

// The activations a convolution epilogue can apply (sigmoid and tanh are
// separate calls, as in the reference).
// x / d for 0 <= x < 2^31 with magic = magic_of(d) from the host: one
// multiply-high and a correction instead of ~40 instructions of integer division.
__device__ __forceinline__ int div_magic(int x, int d, unsigned magic) {
  int q = (int)__umulhi((unsigned)x, magic);
  int r = x - q * d;
  if (r < 0) { q--; r += d; }
  if (r >= d) q++;
  return q;
}
inline unsigned magic_of(int d) {  // ceil(2^32 / d), saturated (d == 1)
  const uint64_t m = (((uint64_t)1 << 32) + (uint64_t)d - 1) / (uint64_t)d;
  return (unsigned)(m > 0xffffffffull ? 0xffffffffull : m);
}

__device__ __forceinline__ float apply_act(float v, int act, float coef) {
  if (act == DNNRT_ACT_RELU) return v < 0.f ? 0.f : v;
  if (act == DNNRT_ACT_CLIPPED_RELU) { v = v < 0.f ? 0.f : v; return v > coef ? coef : v; }
  if (act == DNNRT_ACT_LEAKY_RELU) return v < 0.f ? coef * v : v;
  if (act == ACT_GELU) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752f));
  return v;
}
__host__ __device__ inline bool fusable_act(int64_t act) {
  return act == DNNRT_ACT_RELU || act == DNNRT_ACT_IDENTITY || act == DNNRT_ACT_CLIPPED_RELU || act == DNNRT_ACT_LEAKY_RELU;
}

}  // namespace dnnrt
