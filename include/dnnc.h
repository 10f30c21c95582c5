/* dnnc.h -- C API of the host-side DNN program compiler and executor.
 *
 * It stands where the reference's compiler passes and generated model code
 * stand for the hot path: ONNX-level graph -> DNN program
 * (src/Conversion/ONNXToDNN), function arguments to device memory
 * (src/Transform/DNN/FunctionArgument.cpp), removal of unused constant uploads
 * (eraseDummyConstants.cpp), optional conv+bias+relu fusion
 * (opFusing/fuseConvBiasRelu.cpp), dealloc placement (DNNDeallocOpt.cpp), the
 * memory-pool planner (mallocPoolOpt.{hpp,cpp}), and the straight-line call
 * sequence into the runtime that src/Conversion/DNNToLLVM emits.
 * All functions return 0 / non-NULL on success; dnncLastError() gives the text
 * of the calling thread's last failure.
 */
#ifndef DNNC_H
#define DNNC_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct dnncGraph dnncGraph;
typedef struct dnncProgram dnncProgram;
typedef struct dnncSession dnncSession;

enum { DNNC_F32 = 0, DNNC_F16 = 1, DNNC_I64 = 2 };

const char *dnncLastError(void);

/* ---- graph building (what the ONNX importer hands to the reference) ---- */
dnncGraph *dnncGraphCreate(void);
void dnncGraphDestroy(dnncGraph *g);
int32_t dnncGraphAddInput(dnncGraph *g, const char *name, int32_t dtype, int32_t rank, const int64_t *dims);
/* the bytes are copied */
int32_t dnncGraphAddConstant(dnncGraph *g, const char *name, int32_t dtype, int32_t rank, const int64_t *dims, const void *data);
/* attrs: "key=v1,v2;key2=v" -- integer lists, or a float when the value has a '.' or 'e' */
int32_t dnncGraphAddNode(dnncGraph *g, const char *op_type, int32_t n_inputs, const char *const *inputs, const char *output, const char *attrs);
int32_t dnncGraphAddOutput(dnncGraph *g, const char *name);
/* The reference's own input format: an ONNX model file
 * (`core-dnn --EmitLib ... model.onnx`, test/models/simpleconv/run.py:56-60 of
 * the reference).  `bytes` is the whole file (a serialized ModelProto); the
 * tensors are copied.  Static shapes, float / float16 / int64 tensors, one
 * output per node; NULL on error (dnncLastError says which construct). */
dnncGraph *dnncGraphFromOnnx(const void *bytes, int64_t nbytes);
int32_t dnncGraphNumInputs(const dnncGraph *g);
int32_t dnncGraphNumOutputs(const dnncGraph *g);
const char *dnncGraphInputName(const dnncGraph *g, int32_t i);   /* valid while the graph lives */
const char *dnncGraphOutputName(const dnncGraph *g, int32_t i);
int32_t dnncGraphInputInfo(const dnncGraph *g, int32_t i, int32_t *dtype, int32_t *rank, int64_t *dims, int32_t cap);

/* ---- compilation ---- */
typedef struct {
  int32_t const_at_use;   /* reference flag --onnx-const-at-use (default 1) */
  int32_t fusion;         /* --dnn-kernel-fusion (default 0) */
  int32_t dealloc_opt;    /* --dnn-dealloc-opt (the reference's tests set 1) */
  int32_t pool_opt;       /* --dnn-malloc-pool-opt (the reference's tests set 1) */
  int32_t channels_last;  /* fp16 only: rank-4 activations are NHWC on the device */
  int32_t fuse_residual;  /* no reference flag: with `fusion`, conv+bias -> add -> relu
                             closing a residual block becomes one call (default 0) */
  int32_t fuse_activations; /* no reference flag: with `fusion`, conv+bias -> Clip(0, c) /
                             LeakyRelu / one-slope PRelu becomes one call (default 0) */
  int32_t recompose;      /* no reference flag: LayerNormalization and Gelu written out in
                             primitive operators become one call each (default 0) */
  int32_t fuse_matmul_bias; /* no reference flag: with `fusion`, MatMul -> Add(bias row)
                             becomes one call (default 0) */
  int32_t fuse_attention; /* no reference flag: the head split, QK^T, scaling, Softmax, PV and
                             head merge of an exported attention block become one call (default 0) */
  int32_t fuse_first_layer_maxpool; /* no reference flag: with `fusion`, a ResNet's first convolution (3 -> 64
                             channels, 7x7, stride 2, pad 3, ReLU or identity) and the 3x3 / stride 2 / pad 1
                             max-pool behind it become one call that never stores the convolution's result;
                             fp32 programs, and fp16 programs with `channels_last` and an even image width
                             (default 0) */
  int32_t fuse_projection_shortcut; /* no reference flag: with `fusion` and `fuse_residual`, the projection shortcut of a
                             residual block (conv + bias) and the block's last convolution (+ add + activation)
                             become one call, and the shortcut's result has no tensor of its own (fp16 programs:
                             with `channels_last` only; default 0) */
  int32_t alias_copies;   /* no reference flag: Flatten / Reshape / Squeeze / Unsqueeze name their input's buffer
                             as their output, so nothing is copied and nothing launched (default 0) */
  int32_t inplace_residual; /* no reference flag: with `fusion` and `fuse_residual`, a fused conv + add + activation
                             whose residual operand nothing reads afterwards writes its result over that operand
                             (one tensor fewer in the pool, one fewer in the caches; default 0) */
  int32_t compact_pool;   /* no reference flag: with `pool_opt`, offsets from a planner that knows every lifetime
                             before it places anything (largest tensor first, lowest free offset) instead of the
                             reference's first fit in program order; the pool is then usually the bytes alive at
                             once.  dnncProgramPoolBytes is that pool, not the reference's maxAllocByte (default 0) */
} dnncOptions;
/* the graph must outlive the program: constants are not copied again */
dnncProgram *dnncCompile(dnncGraph *g, const dnncOptions *opt);
void dnncProgramDestroy(dnncProgram *p);
/* the program as text, one operation per line (valid until the program is destroyed) */
const char *dnncProgramText(dnncProgram *p);
/* pool size as the reference planner reports it (its `maxAllocByte`) */
int64_t dnncProgramPoolBytes(const dnncProgram *p);
/* highest planned byte + 1; equal to the above for every trace the emission
 * rules produce.  The executor allocates the larger of the two. */
int64_t dnncProgramPoolExtent(const dnncProgram *p);
/* allocation events in execution order; returns the count (pass NULLs to query).
 * kind 0 = malloc, 1 = dealloc; bytes = unrounded size (malloc only);
 * offset = planned pool offset (malloc only, -1 before the pool pass). */
int64_t dnncProgramEvents(const dnncProgram *p, int32_t *kind, int64_t *id, int64_t *bytes, int64_t *offset, int64_t cap);
int32_t dnncProgramNumInputs(const dnncProgram *p);
int32_t dnncProgramNumOutputs(const dnncProgram *p);
/* rank, dims (up to 8) and dtype of output i */
int32_t dnncProgramOutputInfo(const dnncProgram *p, int32_t i, int32_t *dtype, int32_t *rank, int64_t *dims);
int64_t dnncProgramNumOps(const dnncProgram *p, int32_t compute_only);
/* i-th compute operation in program order: its mnemonic, its work class
 * (conv_dense, conv_depthwise, gemm, matmul, softmax, layernorm, reduce, pool,
 * attention, move, elementwise) and its algorithmic FLOPs and bytes (each tensor read or
 * written counted once at its dense size) */
int32_t dnncProgramComputeOp(const dnncProgram *p, int64_t i, const char **name, const char **work_class, double *flops, double *bytes);

/* ---- the planner alone (mallocPoolOpt.hpp:21-140, 212-218) ----
 * kind/id/bytes as above; writes one offset per event (-1 for deallocs) and
 * returns the pool size, or -1 on a dealloc of a tensor that is not live. */
int64_t dnncPlanPool(int64_t n, const int32_t *kind, const int64_t *id, const int64_t *bytes, int64_t *offset);
/* free list after the first `upto + 1` events as (first, last) byte pairs; returns the number of blocks */
int64_t dnncPlanFreeList(int64_t n, const int32_t *kind, const int64_t *id, const int64_t *bytes, int64_t upto, int64_t *out, int64_t cap);

/* ---- execution ---- */
enum { DNNC_MODE_OCCAMY = 0, DNNC_MODE_RESIDENT = 1 };
/* runtime_library: path of a shared object exporting include/dnnrt.h */
dnncSession *dnncSessionCreate(dnncProgram *p, const char *runtime_library, int32_t mode);
void dnncSessionDestroy(dnncSession *s);
/* host buffers in, host buffers out; returns when the results are in `outputs` */
int32_t dnncSessionRun(dnncSession *s, const void *const *inputs, void *const *outputs);
/* resident mode only.  on_device != 0: inputs/outputs are device buffers and the call does not
 * wait (dnncSessionSync does); on_device == 2: the kernels read the input buffers where they
 * are instead of copying them into the pool first, and the operations that produce the
 * results write them into `outputs` instead of a pool tensor that is copied there afterwards
 * -- the caller leaves the inputs unchanged and the result buffers alone until the run is
 * over, no buffer overlaps another, and passing other addresses than last time records the
 * graph again (the graphs of the last four other sets of addresses are kept and come back
 * when those addresses do); use_graph: replay the kernels from a captured graph (programs
 * of up to three kernels are issued directly all the same: a graph launch costs more) */
int32_t dnncSessionRunResident(dnncSession *s, const void *const *inputs, void *const *outputs, int32_t on_device, int32_t use_graph);
int32_t dnncSessionSync(dnncSession *s);
/* Tuning and tests: dnnrtSetConvTile on the session's handle (0 = automatic choice); a captured
 * graph is dropped and recorded again by the next replayed run. */
int32_t dnncSessionSetConvTile(dnncSession *s, int32_t tile);
/* The measured choice of convolution variant: the reference times cuDNN's algorithms on the build machine's GPU
 * when it compiles a model and passes the winner as each convolution's `algo` operand
 * (src/Conversion/ONNXToDNN/ONNXToDNNCommonCUDA.cu:57-111 calculateConvAlgo, Ops/cudnn/Conv.cpp:82-83).  Here a
 * resident session on the GPU runtime times every variant dnnrtListConvTiles names on every fp16 channels-last
 * convolution of its program, in place (inside whole passes over the program, `reps` passes per variant, on the
 * given inputs; on_device: they are device buffers), and an operation gets a variant as its `algo` operand
 * (DNNRT_CONV_ALGO_BASE + id) when that is faster than the runtime's own choice by more than 3 % in the median.
 * Returns how many operations got one (0 for programs with nothing to tune and on the host build of the ABI),
 * -1 on error.  Every variant computes the same sums in the same order per output element or to the kernels'
 * common tolerance; recorded graphs are dropped.
 * dnncSessionGetAlgos / SetAlgos: the choices as two variant ids per operation that launches
 * (dnncProgramComputeOp order; the second is for the second convolution of a fused shortcut pair; 0 = the
 * runtime's own choice), so that a tuning can be kept beside the model and applied to a later session. */
int64_t dnncSessionTune(dnncSession *s, const void *const *inputs, int32_t on_device, int32_t reps);
int64_t dnncSessionGetAlgos(const dnncSession *s, int64_t *algos, int64_t cap);
int32_t dnncSessionSetAlgos(dnncSession *s, const int64_t *algos, int64_t n);
/* Debugging, per-inference (occamy) mode: fill the pool when it is allocated, and every tensor's slot when it
 * is carved out of the pool, with `byte` (0..255; -1 switches it off).  With 0xFF a byte that a kernel leaves
 * unwritten, or that is read before its producer ran, shows up as NaN in the results. */
int32_t dnncSessionSetDebugFill(dnncSession *s, int32_t byte);
/* resident mode: one eager pass with device timestamps around every compute
 * operation; ms[i] belongs to dnncProgramComputeOp(i).  Returns the count.
 * on_device bit 0: the inputs are device buffers; bit 1: one pair of
 * timestamps per operation class around that class's launches issued back to
 * back, ms[i] = the class average (a timestamp between kernels of a few
 * microseconds costs about as much as the kernels). */
int64_t dnncSessionProfile(dnncSession *s, const void *const *inputs, int32_t on_device, float *ms, int64_t cap);
int64_t dnncSessionWeightsBytes(const dnncSession *s);
/* bytes the last occamy-mode run requested from dnnrtMemPoolInit (-1 before any run) */
int64_t dnncSessionLastPoolBytes(const dnncSession *s);
/* The runtime library's device-memory accounting (dnnrtDeviceMemoryStats of the library the session is bound
 * to): bytes it holds from the device allocator now, the peak of that sum (reset_peak != 0: the peak restarts from
 * the current value after the read), and the size of the library's static device arrays.  Per process, over all
 * sessions bound to that library. */
int32_t dnncSessionDeviceBytes(const dnncSession *s, int64_t *allocated_now, int64_t *allocated_peak,
                               int64_t *static_bytes, int32_t reset_peak);

#ifdef __cplusplus
}
#endif
#endif /* DNNC_H */
