// In-memory form of an ONNX-level graph and of the DNN program it lowers to.
//
// The DNN program mirrors the reference's DNN dialect (src/Dialect/DNN/DNN.td):
// a single block of operations in execution order; every compute operation
// takes its inputs, then its output buffer (a value produced by dnn.malloc) as
// LAST operand, and returns a result that aliases that buffer.  The passes in
// passes.cpp depend on exactly that convention, as the reference's do.
#pragma once

#include <cstdint>
#include <list>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace dnnc {

enum DType { F32 = 0, F16 = 1, I64 = 2 };
inline int64_t dtype_bytes(DType d) { return d == F32 ? 4 : d == F16 ? 2 : 8; }
inline const char *dtype_name(DType d) { return d == F32 ? "f32" : d == F16 ? "f16" : "i64"; }

typedef std::vector<int64_t> Shape;
inline int64_t shape_numel(const Shape &s) {
  int64_t n = 1;
  for (int64_t d : s) n *= d;
  return n;
}

// ---------------------------------------------------------------- ONNX level
struct GTensor {           // a value of the ONNX-level graph
  std::string name;
  DType dtype = F32;
  Shape shape;
  bool is_input = false, is_const = false;
  std::vector<uint8_t> data;  // constants only
};

struct GNode {
  std::string op_type;               // ONNX operator name, or "Constant"
  std::vector<std::string> inputs;   // "" = absent optional input
  std::string output;
  std::map<std::string, std::vector<int64_t>> ints;
  std::map<std::string, double> floats;
};

struct Graph {
  std::map<std::string, GTensor> tensors;
  std::vector<std::string> inputs, outputs;
  std::vector<GNode> nodes;  // block order; constants are "Constant" nodes
  int64_t opset = 0;         // version of the default operator set an ONNX file declares; 0: built in memory (current semantics)
};

// ---------------------------------------------------------------- DNN program
enum OpKind {
  // memory
  OP_MALLOC, OP_DEALLOC, OP_MEMCPY, OP_MEMPOOL_INIT, OP_MEM_OFFSET,
  // host-side values that device ops refer to
  OP_HOST_CONST,  // the constant's bytes in host memory (krnl.global in the reference)
  OP_HOST_ALLOC,  // host buffer of a returned value (memref.alloc in the reference)
  // compute (DNN.td)
  OP_CONVFWD, OP_CONV_BIAS_ACTIV, OP_ACTIVATION, OP_ADD, OP_MUL, OP_SQRT, OP_NEGATIVE,
  OP_RECIPROCAL, OP_REDUCE, OP_MAXPOOL, OP_AVGPOOL, OP_SOFTMAX, OP_FLATTEN, OP_RESHAPE,
  OP_TRANSPOSE, OP_GATHER, OP_MATMUL2D, OP_MATMULND, OP_POW, OP_ERF, OP_CAST, OP_CLIP,
  OP_LEAKYRELU, OP_PRELU, OP_CONCAT, OP_SQUEEZE, OP_UNSQUEEZE, OP_EXPAND,
  // fused operators that have no counterpart in DNN.td
  OP_LAYERNORM, OP_GELU,
  OP_CONV_BIAS_ADD_ACTIV,  // conv + bias + residual tensor + activation (cuDNN's z operand)
  OP_MATMUL_BIAS,          // batched matrix product + one row added to every row
  OP_ATTENTION,            // softmax(scale * Q K^T) V per head on [batch, seq, heads * dim] tensors
  OP_CONV_BIAS_ACTIV_MAXPOOL,  // conv + bias + activation, then the max-pool behind it (a ResNet's first two layers)
  OP_CONV_ADD_CONV_ACTIV,      // act((conv + bias) + (conv2 + bias2)): a residual block's last convolution and its projection shortcut
  OP_RETURN
};
const char *op_name(OpKind k);
inline bool is_compute_kind(OpKind k) { return k >= OP_CONVFWD && k < OP_RETURN; }

struct Op;
struct Value {
  int id = -1;
  Op *def = nullptr;    // null for function arguments
  int arg_index = -1;   // function argument number, or -1
  DType dtype = F32;
  Shape shape;          // memref shape; the planner sizes mallocs from it
  std::vector<std::pair<Op *, int>> uses;  // newest first, as MLIR keeps them
};

struct Op {
  OpKind kind;
  std::vector<Value *> operands;
  Value *result = nullptr;
  // attributes (only those the kind uses are meaningful)
  Shape dimA, dimB, dimOut;        // dim attributes as the reference emits them
  Shape pads, strides, kernel, perm;
  Shape pool_pads, pool_strides;   // OP_CONV_BIAS_ACTIV_MAXPOOL: the pooling's (`kernel` is its window; pads, strides: the convolution's)
  Shape dimA2, dimB2, pads2, strides2;  // OP_CONV_ADD_CONV_ACTIV: the second convolution's input dims, filter dims, pads, strides
  int64_t group = 1, axis = 0, mode = 0, algo = 0, trans_a = 0, trans_b = 0;
  int64_t bytes = 0;               // malloc / memcpy / mem-offset size
  int64_t offset = 0;              // mem-offset
  float alpha = 1.f, beta = 0.f, coef = 1.f, lo = 0.f, hi = 0.f, eps = 0.f;
  std::string const_name;          // OP_HOST_CONST: tensor name in the graph
  int out_index = -1;              // OP_HOST_ALLOC: which function result
  std::list<Op *>::iterator pos;   // position in Program::ops
};

// A Flatten / Reshape / Squeeze / Unsqueeze whose output buffer is the buffer its input lives in (the alias_copies
// pass): it launches nothing.
inline bool is_aliased_copy(const Op *op) {
  if ((op->kind != OP_FLATTEN && op->kind != OP_RESHAPE && op->kind != OP_SQUEEZE && op->kind != OP_UNSQUEEZE) || op->operands.size() != 2)
    return false;
  const Value *x = op->operands[0], *out = op->operands[1];
  return x == out || (x->def && is_compute_kind(x->def->kind) && !x->def->operands.empty() && x->def->operands.back() == out);
}
// One runtime call per such operation
inline bool launches(const Op *op) { return is_compute_kind(op->kind) && !is_aliased_copy(op); }

// One allocation event of the final program, in execution order.
struct PoolEvent {
  int kind;        // 0 malloc, 1 dealloc
  int64_t id;      // value id of the malloc
  int64_t bytes;   // malloc: prod(shape) * element bytes, before rounding
  int64_t offset;  // malloc: planned pool offset (-1 when not planned)
};

struct Program {
  std::list<Op *> ops;
  std::vector<PoolEvent> trace;      // what the pool pass replayed (it erases the deallocs)
  std::vector<std::unique_ptr<Op>> op_store;
  std::vector<std::unique_ptr<Value>> value_store;
  std::vector<Value *> args;         // function arguments, graph input order
  std::vector<std::string> arg_names;
  std::vector<std::string> out_names;
  const Graph *graph = nullptr;      // owner of constant data
  int64_t pool_bytes = -1;           // set by the pool pass: the size the reference planner reports
  int64_t pool_extent = -1;          // highest planned byte + 1 (equals pool_bytes unless the planner under-reports)
  bool channels_last = false;        // fp16 programs: rank-4 activations are NHWC on the device
  bool channels_last_requested = false;  // set before the passes run (channels_last itself after the layout checks)

  Value *new_value(DType dt, const Shape &s);
  Op *new_op(OpKind k);                       // not yet in the block
  void append(Op *op);                        // before the terminator if one exists
  void insert_before(Op *op, Op *anchor);
  void insert_after(Op *op, Op *anchor);
  void move_after(Op *op, Op *anchor);
  void move_before(Op *op, Op *anchor);
  void erase(Op *op);                         // must have no remaining uses
  void set_operands(Op *op, const std::vector<Value *> &v);
  void replace_all_uses(Value *from, Value *to);
  void renumber();                            // refresh order indices
  int order(const Op *op) const;
  Op *last_user(const Value *v);              // latest op in the block using v, or null
  Op *terminator();
  std::string to_text() const;

 private:
  mutable std::map<const Op *, int> order_;
  mutable bool order_valid_ = false;
  int next_value_id_ = 0;
  void invalidate() { order_valid_ = false; }
};

struct CompileOptions {
  bool const_at_use = true;   // --onnx-const-at-use (reference default true)
  bool fusion = false;        // --dnn-kernel-fusion
  bool dealloc_opt = true;    // --dnn-dealloc-opt
  bool pool_opt = true;       // --dnn-malloc-pool-opt
  bool channels_last = false; // fp16 only: keep rank-4 activations NHWC on the device
};

// graph.cpp
bool infer_shapes(Graph &g, bool recompose_norms, bool fuse_attention, std::string &err);
void constant_at_use(Graph &g);
// emit.cpp
bool emit_program(const Graph &g, Program &p, std::string &err);
void func_args_to_device(Program &p);
void erase_dummy_constants(Program &p);
// work.cpp
const char *op_class(const Op *op);
void op_work(const Op *op, double &flops, double &bytes);
// onnx_reader.cpp: an ONNX ModelProto (the reference's input format) -> Graph
bool graph_from_onnx(const uint8_t *data, size_t nbytes, Graph &g, std::string &err);
// passes.cpp
void fuse_conv_bias_activ(Program &p);
void fuse_residual_add(Program &p);
void fuse_conv_activations(Program &p);
void fuse_matmul_bias(Program &p);
void fuse_first_layer_maxpool(Program &p);
void alias_copies(Program &p);
void inplace_residual(Program &p);
void fuse_projection_shortcut(Program &p);
void dealloc_opt(Program &p);
std::vector<PoolEvent> pool_events(const Program &p);
bool malloc_pool_opt(Program &p, std::string &err, bool compact = false);

}  // namespace dnnc
