// Multi-head attention core for transformer encoders:
//   Y[b, q, h*DH + d] = sum_k softmax_k(scale * <Q[b,q,h,:], K[b,k,h,:]>) * V[b,k,h,d]
// with Q, K, V, Y stored [batch, seq, heads * DH] (the layout the Linear layers
// write), fp32 or fp16 (widened on the way into LDS, everything in between in
// fp32, one rounding on the way out).  It stands for the chain the reference runs call by call --
// Reshape + Transpose of each operand (CUDAReshapeFunc, CUDATranspose4DFloatFunc),
// CUDAMatmulNdFunc, the scaling Mul, CUDASoftmaxFunc, CUDAMatmulNdFunc, Transpose
// + Reshape back -- twelve launches and eleven round trips through memory.
//
// One workgroup = 32 queries of one head; its four wavefronts split every block
// of 128 keys (32 each).  Scores are computed transposed (keys x queries) so
// that a lane owns one query: the soft-max statistics are per lane, and the
// exponentiated scores already sit in the register layout the second product
// wants as its B operand (the 16 accumulator registers of a lane are 16 keys,
// which is just an ordering of the reduction index).  Keys are streamed in
// blocks with a running maximum and sum, so any sequence length works.
#include "common.h"

namespace dnnrt {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 att_half4 __attribute__((ext_vector_type(4)));

// four consecutive elements of a stored tensor as fp32, and back
__device__ __forceinline__ float4 load4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 load4(const __half *p) {
  const att_half4 h = *reinterpret_cast<const att_half4 *>(p);
  return make_float4((float)h[0], (float)h[1], (float)h[2], (float)h[3]);
}
__device__ __forceinline__ void store4(float *p, float4 v) { *reinterpret_cast<float4 *>(p) = v; }
__device__ __forceinline__ void store4(__half *p, float4 v) {
  const att_half4 h = {(_Float16)v.x, (_Float16)v.y, (_Float16)v.z, (_Float16)v.w};
  *reinterpret_cast<att_half4 *>(p) = h;
}

constexpr int ATT_QB = 32, ATT_KB = 128;

template <int DH, typename T>
__global__ __launch_bounds__(256) void attention_kernel(const T *__restrict__ Q, const T *__restrict__ K,
                                                        const T *__restrict__ V, T *__restrict__ Y, int Sq,
                                                        int Sk, int ld_in, int ld, float scale) {
  constexpr int ROW = DH + 4;       // LDS row stride in floats: 16-byte aligned rows, 16-byte reads spread over the banks
  constexpr int TD = DH / 32;       // 32-wide tiles of the head dimension
  extern __shared__ float smem[];
  float *Qs = smem;                 // [32][ROW]
  float *Ks = Qs + ATT_QB * ROW;    // [128][ROW]
  float *Vs = Ks + ATT_KB * ROW;    // [128][ROW]
  float *mx = Vs + ATT_KB * ROW;    // [4][32] block maxima per wavefront
  float *sm = mx + 4 * 32;          // [4][32] final sums per wavefront
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5;
  const int q0 = blockIdx.x * ATT_QB, head = blockIdx.y, b = blockIdx.z;
  const T *Qg = Q + (int64_t)b * Sq * ld_in + head * DH;
  const T *Kg = K + (int64_t)b * Sk * ld_in + head * DH;
  const T *Vg = V + (int64_t)b * Sk * ld_in + head * DH;

  // the query tile (rows past the end repeat the last query; they are not stored)
  // All of a tile's loads are requested before the first value goes to LDS (as a load-then-store loop the
  // compiler keeps one round trip to memory per turn: two for the queries, eight per block of keys and values,
  // most of the kernel's time at sequence length 128).
  constexpr int Q_TURNS = ATT_QB * (DH / 4) / 256, KV_TURNS = ATT_KB * (DH / 4) / 256, KV_CHUNK = KV_TURNS < 8 ? KV_TURNS : 8;
  static_assert(ATT_QB * (DH / 4) % 256 == 0 && ATT_KB * (DH / 4) % 256 == 0, "tile loads divide over the threads");
  {
    float4 qv[Q_TURNS];
#pragma unroll
    for (int u = 0; u < Q_TURNS; u++) {
      const int i = tid + 256 * u, r = i / (DH / 4), c4 = i - r * (DH / 4);
      qv[u] = load4(Qg + (int64_t)min(q0 + r, Sq - 1) * ld_in + c4 * 4);
    }
#pragma unroll
    for (int u = 0; u < Q_TURNS; u++) {
      const int i = tid + 256 * u, r = i / (DH / 4), c4 = i - r * (DH / 4);
      *reinterpret_cast<float4 *>(Qs + r * ROW + c4 * 4) = qv[u];
    }
  }

  floatx16 o[TD];
#pragma unroll
  for (int t = 0; t < TD; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[t][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  for (int kb = 0; kb < Sk; kb += ATT_KB) {
    __syncthreads();  // everyone is done with the previous block's K and V
#pragma unroll
    for (int u0 = 0; u0 < KV_TURNS; u0 += KV_CHUNK) {  // at most eight turns (64 registers) in flight
      float4 kv[KV_CHUNK], vv[KV_CHUNK];
#pragma unroll
      for (int u = 0; u < KV_CHUNK; u++) {
        const int i = tid + 256 * (u0 + u), r = i / (DH / 4), c4 = i - r * (DH / 4);
        const int64_t row = (int64_t)min(kb + r, Sk - 1) * ld_in + c4 * 4;
        kv[u] = load4(Kg + row);
        vv[u] = load4(Vg + row);
      }
#pragma unroll
      for (int u = 0; u < KV_CHUNK; u++) {
        const int i = tid + 256 * (u0 + u), r = i / (DH / 4), c4 = i - r * (DH / 4);
        *reinterpret_cast<float4 *>(Ks + r * ROW + c4 * 4) = kv[u];
        *reinterpret_cast<float4 *>(Vs + r * ROW + c4 * 4) = vv[u];
      }
    }
    __syncthreads();

    // scores, transposed: S[key][query] over this wavefront's 32 keys.  The
    // reduction index d is ordered so that lane half h walks d = h*DH/2 + i:
    // four consecutive MFMA operands are one 16-byte LDS read.
    floatx16 s;
#pragma unroll
    for (int r = 0; r < 16; r++) s[r] = 0.f;
    const float *krow = Ks + (wave * 32 + l32) * ROW + half * (DH / 2);
    const float *qrow = Qs + l32 * ROW + half * (DH / 2);
#pragma unroll
    for (int j = 0; j < DH / 8; j++) {
      const float4 ka = *reinterpret_cast<const float4 *>(krow + 4 * j);
      const float4 qa = *reinterpret_cast<const float4 *>(qrow + 4 * j);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.x, qa.x, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.y, qa.y, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.z, qa.z, s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.w, qa.w, s, 0, 0, 0);
    }
    // register r of lane (l32, half) is key 8*(r/4) + 4*half + r%4 of the wavefront's 32, query l32
    float mloc = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int key = kb + wave * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
      s[r] = key < Sk ? s[r] * scale : -INFINITY;
      mloc = fmaxf(mloc, s[r]);
    }
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
    if (half == 0) mx[wave * 32 + l32] = mloc;
    __syncthreads();
    const float mblk = fmaxf(fmaxf(mx[l32], mx[32 + l32]), fmaxf(mx[64 + l32], mx[96 + l32]));
    const float m_new = fmaxf(m_run, mblk);            // finite: every block holds at least one key
    const float alpha = expf(m_run - m_new);           // 0 on the first block
    float lsum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) { s[r] = expf(s[r] - m_new); lsum += s[r]; }
    l_run = l_run * alpha + lsum;                      // this lane's 16 keys; halves and wavefronts are added at the end
    m_run = m_new;
#pragma unroll
    for (int t = 0; t < TD; t++)
#pragma unroll
      for (int r = 0; r < 16; r++) o[t][r] *= alpha;
    // O^T[d][query] += V^T[d][key] * P^T[key][query]: step r takes, in lane
    // half h, key 8*(r/4) + 4*h + r%4 -- the key register r holds
    const float *vbase = Vs + (wave * 32 + 4 * half) * ROW + l32;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const float *vrow = vbase + (8 * (r >> 2) + (r & 3)) * ROW;
#pragma unroll
      for (int t = 0; t < TD; t++) o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[32 * t], s[r], o[t], 0, 0, 0);
    }
  }

  // add the four wavefronts' partial outputs and sums, normalise, store
  __syncthreads();
  float *red = Ks;  // [4][32 queries][ROW], reusing the K and V tiles (4 * 32 rows <= 256 rows)
  l_run += __shfl_xor(l_run, 32, 64);
  if (half == 0) sm[wave * 32 + l32] = l_run;
#pragma unroll
  for (int t = 0; t < TD; t++)
#pragma unroll
    for (int g = 0; g < 4; g++)
      *reinterpret_cast<float4 *>(red + (wave * 32 + l32) * ROW + 32 * t + 8 * g + 4 * half) =
          make_float4(o[t][4 * g], o[t][4 * g + 1], o[t][4 * g + 2], o[t][4 * g + 3]);
  __syncthreads();
  T *Yg = Y + (int64_t)b * Sq * ld + head * DH;
  for (int i = tid; i < ATT_QB * (DH / 4); i += 256) {
    const int q = i / (DH / 4), c4 = i - q * (DH / 4);
    if (q0 + q >= Sq) continue;
    const float inv = 1.0f / (sm[q] + sm[32 + q] + sm[64 + q] + sm[96 + q]);
    float4 acc = *reinterpret_cast<const float4 *>(red + q * ROW + c4 * 4);
#pragma unroll
    for (int w = 1; w < 4; w++) {
      const float4 p = *reinterpret_cast<const float4 *>(red + (w * 32 + q) * ROW + c4 * 4);
      acc.x += p.x; acc.y += p.y; acc.z += p.z; acc.w += p.w;
    }
    store4(Yg + (int64_t)(q0 + q) * ld + c4 * 4, make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv));
  }
}

template <int DH, typename T>
static void launch_attention(const dnnrtContext *ctx, const T *Q, const T *K, const T *V, T *Y, int B,
                             int Sq, int Sk, int H, int ld_in, float scale) {
  constexpr int ROW = DH + 4;
  const size_t lds = (size_t)((ATT_QB + 2 * ATT_KB) * ROW + 8 * 32) * sizeof(float);
  static bool raised = false;  // per instantiation: more than 64 KiB of dynamic LDS must be asked for once
  if (!raised) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&attention_kernel<DH, T>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised = true;
  }
  hipLaunchKernelGGL((attention_kernel<DH, T>), dim3((unsigned)ceil_div(Sq, ATT_QB), (unsigned)H, (unsigned)B), dim3(256),
                     lds, ctx->stream, Q, K, V, Y, Sq, Sk, ld_in, H * DH, scale);
}

}  // namespace dnnrt

using namespace dnnrt;

extern "C" void *dnnrtAttention(dnnrtHandle_t handle, const void *Q, const void *K, const void *V, void *Y,
                                int64_t batch, int64_t seqQ, int64_t seqK, int64_t heads, int64_t headDim,
                                int64_t ldIn, float scale, int32_t dtype) {
  if (!handle) DNNRT_FAIL("dnnrtAttention: null handle");
  if (!Q || !K || !V || !Y) DNNRT_FAIL("dnnrtAttention: null argument");
  if (dtype != DNNRT_F32 && dtype != DNNRT_F16) DNNRT_FAIL("dnnrtAttention: dtype %d (fp32 and fp16)", dtype);
  if (batch < 0 || seqQ < 0) DNNRT_FAIL("dnnrtAttention: bad dims");
  if (batch == 0 || seqQ == 0) return Y;  // no queries: no work
  if (seqK <= 0 || heads <= 0) DNNRT_FAIL("dnnrtAttention: bad dims");
  if (batch > 65535 || heads > 65535 || seqQ > (1 << 24) || seqK > (1 << 24)) DNNRT_FAIL("dnnrtAttention: dims too large");
  if (headDim != 32 && headDim != 64 && headDim != 128) DNNRT_FAIL("dnnrtAttention: head dim %ld (32, 64, 128)", (long)headDim);
  if (!aligned16(Q) || !aligned16(K) || !aligned16(V) || !aligned16(Y)) DNNRT_FAIL("dnnrtAttention: operands must be 16-byte aligned");
  if (Y == Q || Y == K || Y == V) DNNRT_FAIL("dnnrtAttention: Y must not alias an input");
  if (ldIn == 0) ldIn = heads * headDim;
  if (ldIn < heads * headDim || ldIn % 4 || ldIn > INT32_MAX) DNNRT_FAIL("dnnrtAttention: ldIn %ld (>= heads * headDim, multiple of 4)", (long)ldIn);
  auto run = [&](auto *q, auto *k, auto *v, auto *y) {
    if (headDim == 32) launch_attention<32>(handle, q, k, v, y, (int)batch, (int)seqQ, (int)seqK, (int)heads, (int)ldIn, scale);
    else if (headDim == 64) launch_attention<64>(handle, q, k, v, y, (int)batch, (int)seqQ, (int)seqK, (int)heads, (int)ldIn, scale);
    else launch_attention<128>(handle, q, k, v, y, (int)batch, (int)seqQ, (int)seqK, (int)heads, (int)ldIn, scale);
  };
  if (dtype == DNNRT_F32) run((const float *)Q, (const float *)K, (const float *)V, (float *)Y);
  else run((const __half *)Q, (const __half *)K, (const __half *)V, (__half *)Y);
  DNNRT_CHECK_LAUNCH("dnnrtAttention");
  return Y;
}
