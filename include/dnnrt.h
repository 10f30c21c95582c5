/* dnnrt.h -- C ABI of the gfx950 (MI355X) runtime that Occamy's DNN dialect
 * lowers to.
 *
 * Every entry point below stands where one row of the reference's runtime API
 * table stands (src/Conversion/DNNToLLVM/DNNAPISpecs.inc); the row and the
 * wrapper it replaces are cited on each declaration.  Calling convention is
 * the reference's: plain C, arguments by value, every tensor passed as its raw
 * device pointer plus a HOST array of int64 dims (dense, row-major, no
 * strides), scalar attributes as i64 / i32 / float.  Compute functions return
 * the output device pointer (NULL on error, dnnrtLastError() says why);
 * memory functions return 0 on success and non-zero on error (the reference
 * printf()s and exit(-1)s instead, src/Tools/dnn-wrapper/cuda/wrapDNNMalloc.cpp:11-16).
 *
 * Differences from the reference table, all deliberate:
 *   - a dnnrtHandle_t replaces cudnnHandle_t and is the first argument of
 *     EVERY compute call (the reference passes a handle to the 7 cuDNN-backed
 *     calls only).  The handle carries the stream kernels are launched on.
 *   - every compute call takes a trailing `int32_t dtype` (DNNRT_F32 /
 *     DNNRT_F16).  The reference is float-only.
 *   - dnnrtConvBiasActiv takes `group` (the reference drops it,
 *     src/Transform/DNN/opFusing/fuseConvBiasRelu.cpp:107-114).
 *   - dnnrtMemOffset does not clear the slot (the reference memsets it,
 *     src/Tools/dnn-wrapper/cuda/wrapDNNMemOffset.cpp:27); every kernel here
 *     fully overwrites its output.
 *   - one dnnrtTranspose replaces the per-rank Transpose{2,3,4,6}D symbols.
 *   - new: dnnrtSync, dnnrtSetStream, dnnrtSetTensorFormat,
 *     dnnrtSetFilterLayout, dnnrtSetConvTile, dnnrtListConvTiles, dnnrtLayerNorm,
 *     dnnrtGelu, dnnrtHostAlloc/Free, dnnrtLastError.
 *
 * A tensor with no elements (a zero batch, a zero row count) is accepted by
 * every operator: nothing is launched, the output buffer is left as it is and
 * the call returns it, as the reference's zero-block launches do nothing.
 * Negative dims and empty reduction ranges (K = 0) are refused.
 *
 * The library is not re-entrant per handle; calls on one handle must come
 * from one host thread at a time (the reference keeps its handles in
 * file-scope globals, src/Conversion/DNNToLLVM/Ops/cudnn/ConvForward.cpp:15).
 */
#ifndef DNNRT_H
#define DNNRT_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dnnrtContext *dnnrtHandle_t; /* replaces cudnnHandle_t */
typedef void *dnnrtStream_t;                /* a hipStream_t */

enum { DNNRT_F32 = 0, DNNRT_F16 = 1, DNNRT_I64 = 2 };

/* Physical layout of rank-4 activation tensors.  Dims are always passed in
 * logical N,C,H,W order; the format says how they lie in memory.
 * DNNRT_NCHW_TO_NHWC is honoured by the convolution calls only: X is read as
 * NCHW, Y is written as NHWC (used for the first convolution of an fp16
 * channels-last program, whose input arrives from the host as NCHW). */
enum { DNNRT_NCHW = 0, DNNRT_NHWC = 1, DNNRT_NCHW_TO_NHWC = 2 };

/* Physical layout of fp32 convolution filters.  dimW is always passed in
 * logical K,C/group,R,S order.  KCRS is the reference's (ONNX initializers as
 * they come).  CRSK stores element (k, c, r, s) at ((c*R + r)*S + s)*K + k, so
 * consecutive output channels are adjacent: a caller that owns the constants
 * permutes them once on the host and the batch-1 kernels read them coalesced.
 * fp16 filters follow the tensor format instead (NHWC => K,R,S,C). */
enum { DNNRT_FILTER_KCRS = 0, DNNRT_FILTER_CRSK = 1 };

/* activation modes: cudnnActivationMode_t values the reference emits
 * (src/Tools/dnn-wrapper/cudnn/CUDNNActiveFunc.cpp:8-91;
 *  fusedOp/CUDNNConvBiasReluFunc.cpp:65-68). */
enum { DNNRT_ACT_SIGMOID = 0, DNNRT_ACT_RELU = 1, DNNRT_ACT_TANH = 2,
       DNNRT_ACT_CLIPPED_RELU = 3, /* min(max(x, 0), coef): cuDNN's mode 3 */
       DNNRT_ACT_IDENTITY = 5,
       DNNRT_ACT_LEAKY_RELU = 6    /* x < 0 ? coef * x : x: no cuDNN mode */ };

/* tensor-op modes: cudnnOpTensorOp_t values the reference emits
 * (src/Conversion/DNNToLLVM/Ops/cudnn/Add.cpp:148, Mul.cpp:144, Sqrt.cpp:112). */
enum { DNNRT_OP_ADD = 0, DNNRT_OP_MUL = 1, DNNRT_OP_SQRT = 4 };

/* reduce mode: only AVG (5) is ever emitted
 * (src/Conversion/ONNXToDNN/Ops/cudnn/ReduceMeanV13.cpp:37). */
enum { DNNRT_REDUCE_AVG = 5 };

/* memcpy kinds (src/Dialect/DNN/DNN.td:61-83). */
enum { DNNRT_H2D = 1, DNNRT_D2H = 2, DNNRT_D2D = 3 };

/* `algo` operand of the convolution calls: BASE + a variant id of dnnrtListConvTiles */
enum { DNNRT_CONV_ALGO_BASE = 1000 };

/* ---- handle / stream ------------------------------------------------- */

/* DNNAPISpecs.inc:92 "cudnnCreate" (emitted at function entry,
 * src/Conversion/DNNToLLVM/DNNToLLVMCommon.cpp:172-177). */
int32_t dnnrtCreate(dnnrtHandle_t *handle);
/* New, for accounting; no counterpart in the reference.  Every byte the
 * library has taken from the device allocator and not yet returned
 * (`allocated_now`: pools, dnnrtMalloc, and a handle's reduction scratch when
 * it could not have the static one), the largest value that sum has had
 * (`allocated_peak`; reset_peak != 0 makes it `allocated_now` after the read),
 * and the size of the library's static device arrays (`static_bytes`: the
 * reduction scratch that the first live handle of a device uses, 8 MiB +
 * 64 KiB, and that of dnnrtConvBiasActivNoAlloc, 1 MiB + 4 KiB; they are part
 * of the loaded code object and taken from no allocator).  A program that
 * runs on the only handle of its device therefore holds its pool and nothing
 * else.  Counted per process, over all handles; any pointer may be null. */
int32_t dnnrtDeviceMemoryStats(int64_t *allocated_now, int64_t *allocated_peak,
                               int64_t *static_bytes, int32_t reset_peak);
/* DNNAPISpecs.inc:93 "cudnnDestroy". */
int32_t dnnrtDestroy(dnnrtHandle_t handle);
/* DNNAPISpecs.inc:94 "cudaStreamCreate" (DNNToLLVMCommon.cpp:208-213). */
int32_t dnnrtStreamCreate(dnnrtStream_t *stream);
/* DNNAPISpecs.inc:95 "cudaStreamDestroy". */
int32_t dnnrtStreamDestroy(dnnrtStream_t stream);
/* New.  Kernels of `handle` are launched on `stream` from now on (the
 * reference launches kernels on the NULL stream and copies on its one stream). */
int32_t dnnrtSetStream(dnnrtHandle_t handle, dnnrtStream_t stream);
/* New.  Physical layout of rank-4 activations for subsequent calls. */
int32_t dnnrtSetTensorFormat(dnnrtHandle_t handle, int32_t format);
/* New.  Physical layout of fp32 convolution filters for subsequent calls
 * (DNNRT_FILTER_KCRS is the default and the reference's). */
int32_t dnnrtSetFilterLayout(dnnrtHandle_t handle, int32_t layout);
/* New, for tuning and tests; no counterpart in the reference (cuDNN picks its
 * algorithm from the `algo` argument, which the reference always passes as 0).
 * The fp16 channels-last convolution is compiled in several variants (tile
 * shape, wavefronts per workgroup, pipeline depth); by default each call picks
 * one from the problem size.  dnnrtListConvTiles writes the ids of the
 * variants of this build into ids[0..capacity) and returns how many there
 * are; dnnrtSetConvTile(handle, id) makes every following fp16 channels-last
 * convolution of the handle use that variant (and switches the few-pixel 1x1
 * kernel off), 0 restores the automatic choice.  A variant that cannot run a
 * given problem makes that convolution call fail with an error, never
 * fall back.  -id states a preference instead: the variant runs the problems
 * it can run, every other convolution gets the automatic choice (for timing
 * a variant inside a whole network). */
int32_t dnnrtListConvTiles(int32_t *ids, int32_t capacity);
int32_t dnnrtSetConvTile(dnnrtHandle_t handle, int32_t tile);
/* The coefficient of the activation modes that take one: the ceiling of
 * DNNRT_ACT_CLIPPED_RELU, the slope of DNNRT_ACT_LEAKY_RELU.  It stands where
 * the `coef` of cudnnSetActivationDescriptor stands (the reference sets up one
 * descriptor per call with coef 0, src/Tools/dnn-wrapper/cudnn/fusedOp/
 * CUDNNConvBiasReluFunc.cpp); sticky per handle like the tensor format,
 * default 0.  Read by dnnrtConvBiasActiv, dnnrtConvBiasAddActiv, dnnrtActive. */
int32_t dnnrtSetActivationCoef(dnnrtHandle_t handle, float coef);
/* New.  Blocks until all work on the handle's stream is done; the reference
 * returns to the host without waiting for its device-to-host copies
 * (src/Tools/dnn-wrapper/cuda/wrapDNNMemcpy.cpp:32). */
int32_t dnnrtSync(dnnrtHandle_t handle);
/* New.  Stream capture: the kernels that compute calls launch on the handle's
 * stream between Begin and End are recorded instead of run, and replayed by
 * Launch.  The handle must have a stream set (dnnrtSetStream); pointers seen
 * during capture are baked in.  Not available in a host-only build. */
int32_t dnnrtGraphBegin(dnnrtHandle_t handle);
int32_t dnnrtGraphEnd(dnnrtHandle_t handle, void **graph);
int32_t dnnrtGraphLaunch(dnnrtHandle_t handle, void *graph);
int32_t dnnrtGraphDestroy(void *graph);
/* New.  Device-side timestamps on a stream, for per-call timing. */
int32_t dnnrtEventCreate(void **event);
int32_t dnnrtEventRecord(void *event, dnnrtStream_t stream);
/* waits for `stop`, then gives the time from `start` to `stop` in milliseconds */
int32_t dnnrtEventElapsedMs(void *start, void *stop, float *ms);
int32_t dnnrtEventDestroy(void *event);
/* New.  Text of the calling thread's last error ("" if none). */
const char *dnnrtLastError(void);
/* New.  0 when built for the GPU, 1 for a host-only build of the same ABI. */
int32_t dnnrtIsHostBackend(void);

/* ---- memory ---------------------------------------------------------- */

/* DNNAPISpecs.inc:49 "wrapDNNMemPoolInit"
 * (src/Tools/dnn-wrapper/cuda/wrapDNNMemPoolInit.cpp:19-29). */
int32_t dnnrtMemPoolInit(void **pool, int64_t bytes);
/* DNNAPISpecs.inc:47 "wrapDNNMemOffset" (wrapDNNMemOffset.cpp:19-34). */
int32_t dnnrtMemOffset(void **ptr, void *base, int64_t offset, int64_t bytes);
/* New, for debugging.  Fills bytes [ptr, ptr + bytes) with `byte` on `stream` (a
 * kernel, so it can be captured into a graph).  The reference clears every
 * tensor's slot as it carves it out of the pool
 * (src/Tools/dnn-wrapper/cuda/wrapDNNMemOffset.cpp:27); dnnrtMemOffset does not,
 * and nothing needs it: every kernel writes all of its output.  A caller that
 * wants to see that claim tested fills each slot with 0xFF (a NaN in fp16 and
 * fp32) before its producer runs and looks for NaNs in the results. */
int32_t dnnrtMemFill(void *ptr, int32_t byte, int64_t bytes, dnnrtStream_t stream);
/* DNNAPISpecs.inc:45 "wrapDNNMemcpy" (wrapDNNMemcpy.cpp:17-61). */
int32_t dnnrtMemcpy(void *dst, void *src, int64_t bytes, int32_t kind,
                    dnnrtStream_t stream);
/* DNNAPISpecs.inc:40 "wrapDNNMalloc" (wrapDNNMalloc.cpp). */
int32_t dnnrtMalloc(void **ptr, int64_t bytes);
/* DNNAPISpecs.inc:19 "wrapDNNDealloc" (wrapDNNDealloc.cpp). */
int32_t dnnrtDealloc(void *ptr);
/* New.  Pinned host staging memory for constants and results. */
int32_t dnnrtHostAlloc(void **ptr, int64_t bytes);
int32_t dnnrtHostFree(void *ptr);

/* ---- convolution ----------------------------------------------------- */

/* DNNAPISpecs.inc:108 "DNNConvFunc"
 * (src/Tools/dnn-wrapper/cudnn/CUDNNConvFunc.cpp:9-105).
 * Y = conv2d(X[N,C,H,W], W[K,C/group,R,S]); cross-correlation, dilation 1,
 * pads = {pad_h, pad_w} (symmetric), strides = {stride_h, stride_w}.
 * `workspace` and `workspaceBytes` are accepted and ignored (no kernel here
 * needs one).  `algo`: the reference times cuDNN's algorithms when it compiles
 * a model and passes the winner's number
 * (src/Conversion/ONNXToDNN/ONNXToDNNCommonCUDA.cu:57-111, Ops/cudnn/Conv.cpp:82-83).
 * Here DNNRT_CONV_ALGO_BASE + id names the fp16 channels-last variant `id` of
 * dnnrtListConvTiles: the call uses it where it can run the problem, and the
 * automatic choice otherwise, as for every other value of `algo` (cuDNN's
 * numbers name nothing here).  Every variant gives results to the same
 * tolerance; a handle's dnnrtSetConvTile goes first. */
void *dnnrtConv(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                const void *W, const int64_t *dimW, void *workspace,
                int64_t workspaceBytes, int64_t algo, int64_t group,
                const int64_t *pads, const int64_t *strides, void *Y,
                int32_t dtype);
/* DNNAPISpecs.inc:121 "DNNConvBiasActivFunc"
 * (src/Tools/dnn-wrapper/cudnn/fusedOp/CUDNNConvBiasReluFunc.cpp:8-140).
 * Y = act(conv(X, W) + B), B holds K values (dimB is {1,K,1,1}),
 * activMode DNNRT_ACT_RELU or DNNRT_ACT_IDENTITY (what the reference emits),
 * or DNNRT_ACT_CLIPPED_RELU / DNNRT_ACT_LEAKY_RELU with the handle's
 * activation coefficient. */
void *dnnrtConvBiasActiv(dnnrtHandle_t handle, const void *X,
                         const int64_t *dimX, const void *W,
                         const int64_t *dimW, const void *B,
                         const int64_t *dimB, void *workspace,
                         int64_t workspaceBytes, int64_t algo, int64_t group,
                         const int64_t *pads, const int64_t *strides,
                         int64_t activMode, void *Y, int32_t dtype);
/* New: the same call with the residual operand that
 * cudnnConvolutionBiasActivationForward has and the reference passes with a
 * zero weight (CUDNNConvBiasReluFunc.cpp:94-112: alpha2 = 0, z = y).
 * Y = act((conv(X, W) + B) + Z), Z shaped and laid out like Y: either Y
 * itself (the result is written over the residual operand, which
 * cudnnConvolutionBiasActivationForward allows as well: every kernel adds an
 * element of Z in the thread that stores that element of Y) or not
 * overlapping Y at all; X must not overlap Y.
 * It replaces the conv -> add -> relu chain that closes a residual block; the
 * sums are formed in that chain's order. */
void *dnnrtConvBiasAddActiv(dnnrtHandle_t handle, const void *X,
                            const int64_t *dimX, const void *W,
                            const int64_t *dimW, const void *B,
                            const int64_t *dimB, const void *Z,
                            void *workspace, int64_t workspaceBytes,
                            int64_t algo, int64_t group, const int64_t *pads,
                            const int64_t *strides, int64_t activMode, void *Y,
                            int32_t dtype);
/* New: dnnrtConvBiasActiv followed by dnnrtMaxPool in one kernel, for the
 * first layer of an ImageNet ResNet: Y = maxpool(act(conv(X, W) + B)) with
 * the convolution's result (four times the pooled tensor) never stored.  It
 * replaces the reference's two calls (CUDNNConvBiasReluFunc.cpp:8-140, then
 * CUDNNMaxPoolFunc.cpp:8-78); every element is what that chain stores: the
 * activation's output in the tensors' type, then the maximum over the window,
 * padding ignored, NaN propagated.  One shape only, anything else fails with
 * an error (nothing falls back to the two calls, which would need a buffer
 * for the intermediate tensor): 3 -> 64 channels, 7x7, stride 2, pad 3,
 * group 1, activMode ReLU or identity; pooling 3x3, stride 2, pad 1; either
 * fp16 with tensor format DNNRT_NCHW_TO_NHWC (X is the N,C,H,W function
 * argument with an even width, Y is N,H,W,C, filter K,R,S,C) or fp32 with
 * format DNNRT_NCHW (filter in the handle's filter layout).
 * dimY = [N, 64, PP, QQ], the pooled extents. */
void *dnnrtConvBiasActivMaxPool(dnnrtHandle_t handle, const void *X,
                                const int64_t *dimX, const void *W,
                                const int64_t *dimW, const void *B,
                                const int64_t *dimB, int64_t group,
                                const int64_t *pads, const int64_t *strides,
                                int64_t activMode, const int64_t *poolKernel,
                                const int64_t *poolPads,
                                const int64_t *poolStrides, void *Y,
                                const int64_t *dimY, int32_t dtype);
/* New: a residual block's last convolution and its projection shortcut in
 * one call: Y = act((conv(X, W) + B) + (conv(X2, W2) + B2)).  It replaces
 * dnnrtConvBiasActiv (identity) on the shortcut followed by
 * dnnrtConvBiasAddActiv with that result as Z; no tensor for the shortcut's
 * result is needed.  Any two convolutions (group 1) onto the same
 * [N, K, P, Q] result, fp32 or fp16, in the handle's tensor format and filter
 * layout; B and B2 may be null.
 * One kernel where that is the faster way: fp16 DNNRT_NHWC, both 1x1 without
 * padding, the first with stride 1, over 64 + 64 or 128 + 256 input channels
 * (every element is then what the two calls would store: each conv + bias
 * rounded to fp16 on its own, the sum and the activation in fp32); fp32
 * DNNRT_NCHW, both 1x1 without padding, on problems small enough for the
 * batch-1 kernels (the two reductions are then one sum, rounded once: within
 * an fp32 ulp or two of the chain).  Everywhere else the call runs the two
 * convolutions one after the other with the shortcut's result passing through
 * Y, which gives the chain's bits; `algo` and `algo2` are then the `algo`
 * operands of the first (closing) and the second (shortcut) convolution. */
void *dnnrtConvBiasAddConvBiasActiv(
    dnnrtHandle_t handle, const void *X, const int64_t *dimX, const void *W,
    const int64_t *dimW, const void *B, const int64_t *pads,
    const int64_t *strides, const void *X2, const int64_t *dimX2,
    const void *W2, const int64_t *dimW2, const void *B2, const int64_t *pads2,
    const int64_t *strides2, int64_t activMode, int64_t algo, int64_t algo2,
    void *Y, int32_t dtype);
/* No counterpart in the reference.  dnnrtConvBiasActiv for callers that cannot
 * allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It takes the stream where the other calls
 * take a handle (dnnrtCreate may allocate the handle's reduction scratch) and
 * calls no hipMalloc, hipFree or allocating library routine; the scratch its
 * split-reduction kernels need (partial tiles and arrival counters) is a static
 * device array of 1 MiB + 4 KiB that every GPU the library runs on holds until
 * the process ends.  Tensors are NCHW, filters K,C,R,S, the activation
 * coefficient is 0 (the defaults of a fresh handle); DNNRT_ACT_RELU and
 * DNNRT_ACT_IDENTITY are the useful modes.  A convolution whose split reduction
 * would need more than the static array holds (more than one partial 32x32
 * tile per compute unit of a 256-unit device, or more than 1024 output tiles
 * under a split) is refused with an error, never run with another split:
 * results are bit-identical to dnnrtConvBiasActiv's on a fresh handle.
 * All calls on one GPU share that GPU's array: two calls that overlap in time
 * on one GPU (different streams, or several threads) race; calls on one stream
 * do not.  The arrival counters are cleared by a fill kernel ahead of every
 * launch that uses them, so a launch that died half-way leaves nothing behind. */
void *dnnrtConvBiasActivNoAlloc(dnnrtStream_t stream, const void *X,
                                const int64_t *dimX, const void *W,
                                const int64_t *dimW, const void *B,
                                const int64_t *dimB, int64_t group,
                                const int64_t *pads, const int64_t *strides,
                                int64_t activMode, void *Y, int32_t dtype);

/* ---- elementwise / broadcast ----------------------------------------- */

/* DNNAPISpecs.inc:97 "DNNActiveFunc"
 * (src/Tools/dnn-wrapper/cudnn/CUDNNActiveFunc.cpp:8-91); dimX has 4 entries. */
void *dnnrtActive(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                  int32_t mode, void *Y, int32_t dtype);
/* DNNAPISpecs.inc:99 "DNNTensorOpFunc"
 * (src/Tools/dnn-wrapper/cudnn/CUDNNTensorOpFunc.cpp:8-149).
 * O = op(A, coefB * B); B is broadcast along every dim where dimB[i] == 1;
 * dimA == dimO; the three ranks are equal.  SQRT ignores B. */
void *dnnrtTensorOp(dnnrtHandle_t handle, int64_t op, const void *A,
                    const int64_t *dimA, int32_t rankA, const void *B,
                    const int64_t *dimB, int32_t rankB, void *O,
                    const int64_t *dimO, int32_t rankO, float coefB,
                    int32_t dtype);
/* DNNAPISpecs.inc:13 "CUDAClipFunc" (cuda/CUDAClipFunc.cu:5-28). */
void *dnnrtClip(dnnrtHandle_t handle, const void *X, void *Y,
                const int64_t *dimY, float lo, float hi, int64_t rank,
                int32_t dtype);
/* DNNAPISpecs.inc:38 "CUDALeakyReluFunc" (cuda/CUDALeakyReluFunc.cu:4-34):
 * Y = X < 0 ? alpha * X : X. */
void *dnnrtLeakyRelu(dnnrtHandle_t handle, const void *X, void *Y,
                     const int64_t *dimY, float alpha, int64_t rank,
                     int32_t dtype);
/* DNNAPISpecs.inc:58 "CUDAPReluFunc" (cuda/CUDAPReluFunc.cu:4-34):
 * Y = X < 0 ? slope * X : X.  The reference kernel reads slope[0] only (one
 * slope for the whole tensor); here the slope tensor carries its dims
 * (`rank` entries, right-aligned to dimY by the caller) and is broadcast
 * along every dim where dimSlope[i] == 1, as ONNX PRelu specifies -- a
 * one-element slope gives the reference's result. */
void *dnnrtPRelu(dnnrtHandle_t handle, const void *X, void *Y,
                 const int64_t *dimY, const void *slope,
                 const int64_t *dimSlope, int64_t rank, int32_t dtype);
/* DNNAPISpecs.inc:30 "CUDAErfFunc" (cuda/CUDAErfFunc.cu:4-27). */
void *dnnrtErf(dnnrtHandle_t handle, const void *X, void *Y,
               const int64_t *dim, int64_t rank, int32_t dtype);
/* DNNAPISpecs.inc:50 "CUDANegativeFunc" (cuda/CUDANegativeFunc.cu:4-28). */
void *dnnrtNegative(dnnrtHandle_t handle, const void *X, void *Y,
                    const int64_t *dim, int64_t rank, int32_t dtype);
/* DNNAPISpecs.inc:60 "CUDAReciprocalFunc" (cuda/CUDAReciprocalFunc.cu:4-28). */
void *dnnrtReciprocal(dnnrtHandle_t handle, const void *X, void *Y,
                      const int64_t *dim, int64_t rank, int32_t dtype);
/* DNNAPISpecs.inc:56 "CUDAPowFunc" (cuda/CUDAPowFunc.cu:4-32): the exponent
 * is read from a one-element DEVICE tensor. */
void *dnnrtPow(dnnrtHandle_t handle, const void *X, const void *exponent,
               void *Y, const int64_t *dimY, int64_t rank, int32_t dtype);
/* DNNAPISpecs.inc:11 "CUDACastI64toFloatFunc" (cuda/CUDACastI64toFloatFunc.cu:4-26).
 * Returns Y (the reference returns its input pointer). */
void *dnnrtCastI64toFloat(dnnrtHandle_t handle, const int64_t *X, void *Y,
                          const int64_t *dimY, int64_t rank, int32_t dtype);
/* New (no row in the reference table; the reference lowers GELU to
 * Div, Erf, Add, Mul, Mul): Y = 0.5 x (1 + erf(x / sqrt 2)). */
void *dnnrtGelu(dnnrtHandle_t handle, const void *X, void *Y,
                const int64_t *dim, int64_t rank, int32_t dtype);

/* ---- reductions / normalisation -------------------------------------- */

/* DNNAPISpecs.inc:116 "DNNReduceFunc"
 * (src/Tools/dnn-wrapper/cudnn/CUDNNReduceFunc.cpp:8-142): reduces every dim
 * where dimY[i] == 1 and dimX[i] != 1; dimY keeps the rank of dimX. */
void *dnnrtReduce(dnnrtHandle_t handle, int32_t rank, const void *X,
                  const int64_t *dimX, void *Y, const int64_t *dimY,
                  int32_t mode, int32_t dtype);
/* DNNAPISpecs.inc:64 "CUDASoftmaxFunc" (cuda/CUDASoftmaxFunc.cu:7-128);
 * softmax along `axis` (negative axes count from the back). */
void *dnnrtSoftmax(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                   void *Y, const int64_t *dimY, int64_t axis, int64_t rank,
                   int32_t dtype);
/* New (the reference lowers LayerNorm to 9 primitive calls):
 * Y = (X - mean) / sqrt(var + eps) * gamma + beta over the last dim. */
void *dnnrtLayerNorm(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                     int64_t rank, const void *gamma, const void *beta,
                     float eps, void *Y, int32_t dtype);

/* ---- pooling --------------------------------------------------------- */

/* DNNAPISpecs.inc:113 "DNNMaxPoolFunc"
 * (src/Tools/dnn-wrapper/cudnn/CUDNNMaxPoolFunc.cpp:8-78): kernel[2],
 * pads[4] = {h_begin, w_begin, h_end, w_end} of which [0] and [1] are used
 * symmetrically, strides[2]; padding never wins the max. */
void *dnnrtMaxPool(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                   void *Y, const int64_t *dimY, const int64_t *kernel,
                   const int64_t *pads, const int64_t *strides, int32_t dtype);
/* DNNAPISpecs.inc:105 "DNNAveragePoolFunc"
 * (src/Tools/dnn-wrapper/cudnn/CUDNNAveragePoolFunc.cpp:8-78); padding is
 * counted in the divisor as the reference does (:44). */
void *dnnrtAveragePool(dnnrtHandle_t handle, const void *X,
                       const int64_t *dimX, void *Y, const int64_t *dimY,
                       const int64_t *kernel, const int64_t *pads,
                       const int64_t *strides, int32_t dtype);

/* ---- matrix products ------------------------------------------------- */

/* DNNAPISpecs.inc:4 "CUBLASMatmul2dFunc"
 * (src/Tools/dnn-wrapper/cublas/CUBLASMatmul2dFunc.cu:9-153):
 * Out = alpha op(A) op(B) + beta C, row-major; C may be NULL when beta == 0.
 * C is [M,N] as in the reference (which sizes it by dimOut, :32) or, with
 * dimC = [1,N], one row added to every row of the product.  fp16 tensors:
 * fp32 accumulation and one rounding of alpha op(A) op(B) + beta C. */
void *dnnrtMatmul2d(dnnrtHandle_t handle, int64_t rank, const void *A,
                    const int64_t *dimA, const void *B, const int64_t *dimB,
                    const void *C, const int64_t *dimC, void *Out,
                    const int64_t *dimOut, float alpha, float beta,
                    int64_t transA, int64_t transB, int32_t dtype);
/* DNNAPISpecs.inc:41 "CUDAMatmulNdFunc" (cuda/CUDAMatmulNdFunc.cu:14-173):
 * numpy.matmul for ranks 2..4; an operand of lower rank is broadcast over the
 * leading (batch) dims of the other. */
void *dnnrtMatmulNd(dnnrtHandle_t handle, const void *A, const int64_t *dimA,
                    int32_t rankA, const void *B, const int64_t *dimB,
                    int32_t rankB, void *Y, const int64_t *dimY, int32_t rankY,
                    int32_t dtype);
/* The same with a Linear layer's epilogue: Y = act((A B + bias) + Z), bias one
 * row of N values added to every row of every product, Z an optional residual
 * tensor shaped like Y (NULL: none), act = Gelu if `gelu` != 0 else identity.
 * No reference wrapper: the reference runs CUDAMatmulNdFunc and then the
 * broadcast add of the bias (Ops/cudnn/Add.cpp), the residual add, and Gelu
 * operator by operator (Div, Erf, Add, Mul, Mul).  fp32 and fp16 (fp32
 * accumulation, everything up to the activation in fp32, one rounding). */
void *dnnrtMatmulNdBias(dnnrtHandle_t handle, const void *A, const int64_t *dimA,
                        int32_t rankA, const void *B, const int64_t *dimB,
                        int32_t rankB, const void *bias, const void *Z,
                        int32_t gelu, void *Y, const int64_t *dimY,
                        int32_t rankY, int32_t dtype);
/* Multi-head attention core, Y = softmax(scale * Q K^T) V per head, with Q
 * [batch, seqQ, heads*headDim], K and V [batch, seqK, heads*headDim] and Y like
 * Q.  No reference wrapper: it stands for the chain the reference runs call
 * by call for an exported transformer (CUDAReshapeFunc + CUDATranspose4DFloatFunc
 * per operand, CUDAMatmulNdFunc, the scaling Mul, CUDASoftmaxFunc,
 * CUDAMatmulNdFunc, Transpose + Reshape back).  ldIn is the row stride of Q, K
 * and V in elements (0: heads*headDim); with the three projections computed
 * by one product into a [batch, seq, 3*heads*headDim] tensor, Q, K and V are
 * that tensor's base plus 0, 1 and 2 times heads*headDim and ldIn is its row
 * length.  Y's rows are heads*headDim long.  fp32 or fp16 (widened on the way
 * in, fp32 in between, one rounding on the way out), headDim 32 / 64 / 128,
 * 16-byte aligned operands, Y distinct from the inputs. */
void *dnnrtAttention(dnnrtHandle_t handle, const void *Q, const void *K,
                     const void *V, void *Y, int64_t batch, int64_t seqQ,
                     int64_t seqK, int64_t heads, int64_t headDim, int64_t ldIn,
                     float scale, int32_t dtype);

/* ---- data movement --------------------------------------------------- */

/* DNNAPISpecs.inc:36 "CUDAFlattenFunc" (cuda/CUDAFlattenFunc.cpp): copy. */
void *dnnrtFlatten(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                   void *Y, const int64_t *dimY, int32_t axis, int64_t rank,
                   int32_t dtype);
/* DNNAPISpecs.inc:62 "CUDAReshapeFunc" (cuda/CUDAReshapeFunc.cpp): copy. */
void *dnnrtReshape(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                   int64_t rankX, void *Y, int32_t dtype);
/* DNNAPISpecs.inc:66-69 "CUDASqueeze{Int64,Float}Func"
 * (cuda/CUDASqueezeFloatFunc.cpp:6-45) and :86-89
 * "CUDAUnsqueeze{Int64,Float}Func": copies; dimY must be dimX with size-1
 * dims removed / inserted (the reference passes the axes and ignores them). */
void *dnnrtSqueeze(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                   int64_t rankX, void *Y, const int64_t *dimY, int64_t rankY,
                   int32_t dtype);
void *dnnrtUnsqueeze(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                     int64_t rankX, void *Y, const int64_t *dimY,
                     int64_t rankY, int32_t dtype);
/* DNNAPISpecs.inc:32-35 "CUDAExpandInt64Func"
 * (cuda/CUDAExpandInt64Func.cu:5-19), for every dtype.  The reference copies
 * prod(dimX) elements and leaves the rest of Y unwritten, which is ONNX Expand
 * only when dimY equals dimX; this entry point broadcasts (dimX aligned with
 * the trailing dims of dimY, size-1 dims repeated) and so agrees with the
 * reference wherever the reference's result is defined.  The reference's
 * `shape` operand is not taken: dimY already is its value.  rankY <= 8. */
void *dnnrtExpand(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                  int64_t rankX, void *Y, const int64_t *dimY, int64_t rankY,
                  int32_t dtype);
/* DNNAPISpecs.inc:52-55 "CUDANonZero{Int64,Float}Func"
 * (cuda/CUDANonZeroFloatFunc.cu:4-34): the flat indices of the elements of X
 * that are not zero, ascending, converted to X's own element type, written to
 * the front of Y; the rest of Y keeps its contents.  Indices beyond
 * prod(dimY) entries are dropped (the reference writes past the end); the
 * reference passes one rank, the input's, for both dim arrays. */
void *dnnrtNonZero(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                   int64_t rankX, void *Y, const int64_t *dimY, int64_t rankY,
                   int32_t dtype);
/* DNNAPISpecs.inc:15-18 "CUDAConcat{Int64,Float}Func"
 * (cuda/CUDAConcatFloatFunc.cu:64-99): Y = concatenation of numInputs tensors
 * along `axis`.  X and dimX are HOST arrays (of device pointers / of host dim
 * arrays with `rank` entries each); nothing is allocated per call, where the
 * reference uploads both lists with cudaMalloc on every call.  Up to 16
 * inputs (reference: 10) of rank <= 8 (reference: 4). */
void *dnnrtConcat(dnnrtHandle_t handle, const void *const *X,
                  const int64_t *const *dimX, void *Y, const int64_t *dimY,
                  int64_t axis, int64_t numInputs, int32_t rank,
                  int32_t dtype);
/* DNNAPISpecs.inc:72-87 "CUDATranspose{2,3,4,6}D{Float,Int64}Func"
 * (cuda/CUDATranspose4DFloatFunc.cu): Y = numpy.transpose(X, perm), rank <= 6;
 * dtype DNNRT_I64 selects the Int64 variants. */
void *dnnrtTranspose(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                     void *Y, const int64_t *dimY, const int64_t *perm,
                     int64_t rank, int32_t dtype);
/* DNNAPISpecs.inc:25 "CUDAGatherFloatFunc" (cuda/CUDAGatherFloatFunc.cu:7-82):
 * numpy.take(X, indices, axis); negative indices count from the back.
 * Indices live in device memory, so the call cannot inspect them: an index
 * outside [-dimX[axis], dimX[axis]) reads nothing and its slice of Y is
 * written as zeros (the reference kernel reads out of bounds there,
 * CUDAGatherFloatFunc.cu:27-34).  A host-side build of this interface may
 * reject such an index with an error instead. */
void *dnnrtGather(dnnrtHandle_t handle, const void *X, const int64_t *dimX,
                  int64_t rankX, void *Y, const int64_t *dimY, int64_t rankY,
                  const int64_t *indices, const int64_t *dimIndices,
                  int64_t rankIndices, int64_t axis, int32_t dtype);

#ifdef __cplusplus
}
#endif
#endif /* DNNRT_H */
