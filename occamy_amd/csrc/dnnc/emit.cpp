// ONNX graph -> DNN program.  One emission rule per ONNX operator, restating
// which dnn.malloc / compute / dnn.dealloc operations the reference's
// conversion patterns create and in which order
// (src/Conversion/ONNXToDNN/Ops/**, helpers in ONNXToDNNCommon.cpp:111-224):
//   - results are written into a fresh dnn.malloc placed right before the op;
//   - every malloc gets a dnn.dealloc parked in front of the terminator, in
//     creation order (ONNXToDNNCommon.cpp:218-224);
//   - a value the function returns is copied to a host buffer right after the
//     op that produced it (ONNXToDNNCommon.cpp:129-213).
// Followed by the two clean-up passes the reference runs right after the
// conversion: function arguments to device memory and removal of constant
// uploads nothing reads.
#include <cmath>
#include <cstring>

#include "ir.h"

namespace dnnc {

namespace {

struct Emitter {
  const Graph &g;
  Program &p;
  std::map<std::string, Value *> env;
  Op *ret = nullptr;
  Op *first_parked = nullptr;
  Op *first_op = nullptr;
  std::string err;

  Emitter(const Graph &g_, Program &p_) : g(g_), p(p_) {}

  void emit(Op *op) {  // at the "insertion point": after everything emitted, before parked deallocs
    p.insert_before(op, first_parked ? first_parked : ret);
  }
  Value *malloc_(DType dt, const Shape &s) {
    Op *m = p.new_op(OP_MALLOC);
    m->bytes = shape_numel(s) * dtype_bytes(dt);
    m->result = p.new_value(dt, s);
    m->result->def = m;
    emit(m);
    return m->result;
  }
  void park_dealloc(Value *v) {
    Op *d = p.new_op(OP_DEALLOC);
    p.insert_before(d, ret);
    p.set_operands(d, {v});
    if (!first_parked) first_parked = d;
  }
  Op *compute(OpKind k, const std::vector<Value *> &operands) {
    Op *op = p.new_op(k);
    emit(op);
    p.set_operands(op, operands);
    Value *out = operands.back();
    op->result = p.new_value(out->dtype, out->shape);
    op->result->def = op;
    return op;
  }
  // copy to host if the function returns this node's value
  void maybe_return(const std::string &name, Value *dev) {
    for (size_t i = 0; i < g.outputs.size(); i++) {
      if (g.outputs[i] != name) continue;
      Op *ha = p.new_op(OP_HOST_ALLOC);
      ha->out_index = (int)i;
      ha->bytes = shape_numel(dev->shape) * dtype_bytes(dev->dtype);
      ha->result = p.new_value(dev->dtype, dev->shape);
      ha->result->def = ha;
      p.insert_before(ha, p.ops.front());  // known-size host buffers go to the block front
      Op *cp = p.new_op(OP_MEMCPY);
      cp->bytes = ha->bytes;
      cp->mode = 2;  // device to host
      emit(cp);
      p.set_operands(cp, {ha->result, dev});
      std::vector<Value *> r = ret->operands;
      r[i] = ha->result;
      p.set_operands(ret, r);
    }
  }

  static Shape pad_front(const Shape &small, size_t rank) {
    Shape o(rank - small.size(), 1);
    o.insert(o.end(), small.begin(), small.end());
    return o;
  }

  float const_scalar(const std::string &name, float dflt) {
    if (name.empty()) return dflt;
    auto it = g.tensors.find(name);
    if (it == g.tensors.end() || !it->second.is_const || it->second.data.empty()) return dflt;
    const GTensor &t = it->second;
    if (t.dtype == F32) { float v; std::memcpy(&v, t.data.data(), 4); return v; }
    if (t.dtype == F16) {
      uint16_t h; std::memcpy(&h, t.data.data(), 2);
      const int s = h >> 15, e = (h >> 10) & 31, m = h & 1023;
      float v = e == 0 ? std::ldexp((float)m, -24) : e == 31 ? (m ? NAN : INFINITY) : std::ldexp((float)(m + 1024), e - 25);
      return s ? -v : v;
    }
    int64_t v; std::memcpy(&v, t.data.data(), 8); return (float)v;
  }

  bool node(const GNode &n) {
    const std::string &t = n.op_type;
    auto in = [&](size_t i) -> Value * {
      if (i >= n.inputs.size() || n.inputs[i].empty()) return nullptr;
      auto it = env.find(n.inputs[i]);
      return it == env.end() ? nullptr : it->second;
    };
    auto ints = [&](const char *k, std::vector<int64_t> d) { auto it = n.ints.find(k); return it == n.ints.end() ? d : it->second; };
    auto int1 = [&](const char *k, int64_t d) { auto it = n.ints.find(k); return (it == n.ints.end() || it->second.empty()) ? d : it->second[0]; };
    auto flt = [&](const char *k, double d) { auto it = n.floats.find(k); return it == n.floats.end() ? d : it->second; };
    const GTensor &ot = g.tensors.at(n.output);
    Value *result = nullptr, *out_buf = nullptr;

    if (t == "Constant") {  // Ops/Constant.cpp:44-104
      Op *hc = p.new_op(OP_HOST_CONST);
      hc->const_name = n.output;
      hc->result = p.new_value(ot.dtype, ot.shape);
      hc->result->def = hc;
      emit(hc);
      Value *m = malloc_(ot.dtype, ot.shape);
      Op *cp = p.new_op(OP_MEMCPY);
      cp->bytes = m->def->bytes;
      cp->mode = 1;  // host to device
      emit(cp);
      p.set_operands(cp, {m, hc->result});
      park_dealloc(m);
      env[n.output] = m;
      return true;
    }
    Value *x = in(0);
    if (!x) { err = t + " '" + n.output + "': input not available"; return false; }

    if (t == "Conv") {  // Ops/cudnn/Conv.cpp:82-158
      Value *w = in(1), *b = in(2);
      // the workspace is a memref<1 x ws x f32>; implicit GEMM needs none, so ws = 0
      Value *ws = malloc_(F32, {1, 0});
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *c = compute(OP_CONVFWD, {x, w, ws, out_buf});
      const std::vector<int64_t> pads = ints("pads", {0, 0, 0, 0});
      c->pads = {pads[0], pads[1]};  // (h, w); emit checks symmetry in shape inference
      c->strides = ints("strides", {1, 1});
      c->group = int1("group", 1);
      c->dimA = x->shape;
      c->dimB = w->shape;
      result = c->result;
      if (b) {
        Op *a = compute(OP_ADD, {c->result, b, out_buf});
        a->dimA = ot.shape;
        a->dimB = {1, ot.shape[1], 1, 1};  // bias on the channel axis
        a->coef = 1.f;
        result = a->result;
      }
      park_dealloc(out_buf);
      park_dealloc(ws);
    } else if (t == "Relu" || t == "Sigmoid" || t == "Tanh") {  // Ops/cudnn/Relu.cpp:50-58
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *a = compute(OP_ACTIVATION, {x, out_buf});
      a->mode = t == "Relu" ? 1 : t == "Sigmoid" ? 0 : 2;
      a->dimA = x->shape;
      result = a->result;
      park_dealloc(out_buf);
    } else if (t == "Add" || t == "Mul") {  // Ops/cudnn/Add.cpp:50-75, Mul.cpp:49-71
      Value *y = in(1);
      if (!y) { err = t + ": second input not available"; return false; }
      out_buf = malloc_(ot.dtype, ot.shape);
      // the operand that has the result's shape goes first; the other is
      // right-aligned and broadcast where its dim is 1
      Value *a = x, *b = y;
      if (a->shape.size() < b->shape.size() || (a->shape.size() == b->shape.size() && a->shape != ot.shape)) std::swap(a, b);
      if (pad_front(a->shape, ot.shape.size()) != ot.shape) { err = t + ": neither operand has the result's shape"; return false; }
      Op *o = compute(t == "Add" ? OP_ADD : OP_MUL, {a, b, out_buf});
      o->dimA = ot.shape;
      o->dimB = pad_front(b->shape, ot.shape.size());
      o->coef = 1.f;
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Sub") {  // Ops/cudnn/Sub.cpp:59-98: negative(B), then add
      Value *y = in(1);
      if (!y) { err = "Sub: second input not available"; return false; }
      Value *neg = malloc_(y->dtype, y->shape);
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *ng = compute(OP_NEGATIVE, {y, neg});
      ng->dimA = y->shape;
      if (pad_front(x->shape, ot.shape.size()) != ot.shape) { err = "Sub: the minuend must have the result's shape"; return false; }
      Op *o = compute(OP_ADD, {x, neg, out_buf});  // uses the malloc itself, as the reference does
      o->dimA = ot.shape;
      o->dimB = pad_front(y->shape, ot.shape.size());
      o->coef = 1.f;
      result = o->result;
      park_dealloc(neg);
      park_dealloc(out_buf);
    } else if (t == "Div") {  // Ops/cudnn/Div.cpp:47-77: reciprocal(B) into a RESULT-sized buffer, then mul
      Value *y = in(1);
      if (!y) { err = "Div: second input not available"; return false; }
      Value *rc = malloc_(ot.dtype, ot.shape);
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *r = compute(OP_RECIPROCAL, {y, rc});
      r->dimA = y->shape;
      r->result->shape = y->shape;
      if (pad_front(x->shape, ot.shape.size()) != ot.shape) { err = "Div: the dividend must have the result's shape"; return false; }
      Op *o = compute(OP_MUL, {x, rc, out_buf});
      o->dimA = ot.shape;
      o->dimB = pad_front(y->shape, ot.shape.size());
      o->coef = 1.f;
      result = o->result;
      park_dealloc(rc);
      park_dealloc(out_buf);
    } else if (t == "Sqrt" || t == "Erf" || t == "Gelu") {
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(t == "Sqrt" ? OP_SQRT : t == "Erf" ? OP_ERF : OP_GELU, {x, out_buf});
      o->dimA = ot.shape;
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Pow") {  // Ops/cuda/Pow.cpp: the exponent stays a device tensor
      Value *e = in(1);
      if (!e || shape_numel(e->shape) != 1) { err = "Pow: the exponent must be a one-element tensor"; return false; }
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_POW, {x, e, out_buf});
      o->dimA = ot.shape;
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Clip") {  // Ops/cuda/Clip.cpp:34-66: min/max folded to attributes
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_CLIP, {x, out_buf});
      o->lo = const_scalar(n.inputs.size() > 1 ? n.inputs[1] : "", -INFINITY);
      o->hi = const_scalar(n.inputs.size() > 2 ? n.inputs[2] : "", INFINITY);
      o->dimA = ot.shape;
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "LeakyRelu") {  // Ops/cuda/LeakyRelu.cpp
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_LEAKYRELU, {x, out_buf});
      o->alpha = (float)flt("alpha", 0.01);
      o->dimA = ot.shape;
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "PRelu") {  // Ops/cuda/PRelu.cpp: the slope stays a device tensor
      Value *sl = in(1);
      if (!sl) { err = "PRelu: slope not available"; return false; }
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_PRELU, {x, sl, out_buf});
      o->dimA = ot.shape;
      o->dimB = pad_front(sl->shape, ot.shape.size());
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Concat") {  // Ops/cuda/Concat.cpp: all inputs, then the output buffer
      std::vector<Value *> operands;
      for (size_t i = 0; i < n.inputs.size(); i++) {
        Value *v = in(i);
        if (!v) { err = "Concat: input not available"; return false; }
        operands.push_back(v);
      }
      if (operands.size() > 16) { err = "Concat: more than 16 inputs"; return false; }
      out_buf = malloc_(ot.dtype, ot.shape);
      operands.push_back(out_buf);
      Op *o = compute(OP_CONCAT, operands);
      o->dimOut = ot.shape;
      o->axis = int1("axis", 0);
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Squeeze" || t == "Unsqueeze" || t == "Identity") {  // Ops/cuda/Squeeze.cpp, Unsqueeze.cpp
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(t == "Squeeze" ? OP_SQUEEZE : t == "Unsqueeze" ? OP_UNSQUEEZE : OP_RESHAPE, {x, out_buf});
      o->dimA = x->shape;
      o->dimOut = ot.shape;
      o->perm = ints("axes", {});
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Expand") {
      // Ops/cuda/Expand.cpp:40-47.  The shape constant stays a device tensor
      // and an operand, as there; the output buffer is kept as the LAST
      // operand (the reference puts the shape last), because the dealloc
      // placement takes an op's last operand for the buffer its result lives
      // in: with the reference's order the output would be released right
      // after the call and the shape constant kept alive in its place.
      Value *sh = in(1);
      if (!sh) { err = "Expand: shape not available"; return false; }
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_EXPAND, {x, sh, out_buf});
      o->dimA = x->shape;
      o->dimOut = ot.shape;
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Cast") {
      if (x->dtype != I64 || ot.dtype == I64) { err = "Cast: only int64 -> float is covered"; return false; }
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_CAST, {x, out_buf});
      o->dimA = ot.shape;
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "ReduceMean") {  // Ops/cudnn/ReduceMeanV13.cpp:37-80
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_REDUCE, {x, out_buf});
      o->dimA = x->shape;
      o->dimOut = x->shape;  // the keep-dims shape, whatever keepdims says
      std::vector<int64_t> axes = ints("axes", {});
      if (axes.empty()) for (size_t i = 0; i < x->shape.size(); i++) axes.push_back((int64_t)i);
      for (int64_t a : axes) o->dimOut[(size_t)(a < 0 ? a + (int64_t)x->shape.size() : a)] = 1;
      o->mode = 5;
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "MaxPool" || t == "AveragePool") {
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(t == "MaxPool" ? OP_MAXPOOL : OP_AVGPOOL, {x, out_buf});
      o->dimA = x->shape;
      o->dimOut = ot.shape;
      o->kernel = ints("kernel_shape", {1, 1});
      o->pads = ints("pads", {0, 0, 0, 0});
      o->strides = ints("strides", {1, 1});
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Softmax") {
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_SOFTMAX, {x, out_buf});
      o->dimA = x->shape;
      o->axis = int1("axis", -1);
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Flatten" || t == "Reshape") {
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(t == "Flatten" ? OP_FLATTEN : OP_RESHAPE, {x, out_buf});
      o->dimA = x->shape;
      o->dimOut = ot.shape;
      o->axis = int1("axis", 1);
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Transpose") {
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_TRANSPOSE, {x, out_buf});
      o->dimA = x->shape;
      o->dimOut = ot.shape;
      o->perm = ints("perm", {});
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Gather") {
      Value *idx = in(1);
      if (!idx || idx->dtype != I64) { err = "Gather: indices must be an int64 tensor"; return false; }
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_GATHER, {x, idx, out_buf});
      o->dimA = x->shape;
      o->dimB = idx->shape;
      o->dimOut = ot.shape;
      o->axis = int1("axis", 0);
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "MatMul") {  // Ops/cuda/MatMul.cpp
      Value *y = in(1);
      if (!y) { err = "MatMul: second input not available"; return false; }
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_MATMULND, {x, y, out_buf});
      o->dimA = x->shape;
      o->dimB = y->shape;
      o->dimOut = ot.shape;
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "Gemm") {  // Ops/cublas/Gemm.cpp:60-81: matmul2d, then add of C onto the same buffer
      Value *y = in(1), *c = in(2);
      if (!y) { err = "Gemm: second input not available"; return false; }
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *mm = compute(OP_MATMUL2D, {x, y, out_buf});
      mm->dimA = x->shape;
      mm->dimB = y->shape;
      mm->dimOut = ot.shape;
      mm->alpha = (float)flt("alpha", 1.0);
      // the reference forwards ONNX's beta to a product whose output buffer is
      // freshly zeroed, which makes it a no-op; C is added with coefficient 1
      mm->beta = 0.f;
      mm->trans_a = int1("transA", 0);
      mm->trans_b = int1("transB", 0);
      result = mm->result;
      if (c) {
        Op *a = compute(OP_ADD, {out_buf, c, out_buf});
        a->dimA = ot.shape;
        a->dimB = pad_front(c->shape, 2);
        a->coef = 1.f;
        result = a->result;
      }
      park_dealloc(out_buf);
    } else if (t == "FusedAttention") {
      Value *k = in(1), *v = in(2);
      if (!k || !v) { err = "FusedAttention: K or V not available"; return false; }
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_ATTENTION, {x, k, v, out_buf});
      o->axis = int1("packed", 0);  // 1: the three operands are one [B, S, 3*hidden] tensor
      o->dimA = ot.shape;
      o->dimB = o->axis ? ot.shape : k->shape;
      o->group = int1("heads", 1);
      o->alpha = (float)flt("scale", 1.0);
      result = o->result;
      park_dealloc(out_buf);
    } else if (t == "LayerNormalization") {
      Value *gm = in(1), *bt = in(2);
      if (!gm || !bt) { err = "LayerNormalization: scale and bias are required"; return false; }
      if (int1("axis", -1) != -1 && int1("axis", -1) != (int64_t)x->shape.size() - 1) {
        err = "LayerNormalization: only the last axis is covered";
        return false;
      }
      out_buf = malloc_(ot.dtype, ot.shape);
      Op *o = compute(OP_LAYERNORM, {x, gm, bt, out_buf});
      o->dimA = x->shape;
      o->eps = (float)flt("epsilon", 1e-5);
      result = o->result;
      park_dealloc(out_buf);
    } else {
      err = t + ": no emission rule";
      return false;
    }
    maybe_return(n.output, out_buf);
    env[n.output] = result;
    return true;
  }
};

}  // namespace

bool emit_program(const Graph &g, Program &p, std::string &err) {
  p.graph = &g;
  Emitter e(g, p);
  e.ret = p.new_op(OP_RETURN);
  p.append(e.ret);
  // function arguments
  for (size_t i = 0; i < g.inputs.size(); i++) {
    const GTensor &t = g.tensors.at(g.inputs[i]);
    Value *a = p.new_value(t.dtype, t.shape);
    a->arg_index = (int)i;
    p.args.push_back(a);
    p.arg_names.push_back(t.name);
    e.env[t.name] = a;
  }
  // placeholder return operands, replaced as producers are emitted
  std::vector<Value *> rets;
  for (size_t i = 0; i < g.outputs.size(); i++) rets.push_back(p.new_value(F32, {}));
  p.set_operands(e.ret, rets);
  p.out_names = g.outputs;
  for (const GNode &n : g.nodes)
    if (!e.node(n)) { err = e.err; return false; }
  for (size_t i = 0; i < g.outputs.size(); i++)
    if (e.ret->operands[i] == rets[i]) { err = "output '" + g.outputs[i] + "' has no producer in the graph"; return false; }
  return true;
}

// src/Transform/DNN/FunctionArgument.cpp:30-53: every argument becomes
// malloc + host-to-device memcpy at the top of the block and a dealloc in
// front of the terminator.
void func_args_to_device(Program &p) {
  Op *ret = p.terminator();
  for (Value *arg : p.args) {
    Op *m = p.new_op(OP_MALLOC);
    m->bytes = shape_numel(arg->shape) * dtype_bytes(arg->dtype);
    m->result = p.new_value(arg->dtype, arg->shape);
    m->result->def = m;
    p.replace_all_uses(arg, m->result);
    Op *cp = p.new_op(OP_MEMCPY);
    cp->bytes = m->bytes;
    cp->mode = 1;
    p.insert_before(m, p.ops.front());
    p.insert_after(cp, m);
    p.set_operands(cp, {m->result, arg});
    Op *d = p.new_op(OP_DEALLOC);
    p.insert_before(d, ret);
    p.set_operands(d, {m->result});
  }
}

// src/Transform/DNN/eraseDummyConstants.cpp:28-57: a malloc used by nothing
// but memcpy and dealloc is removed together with those users and the host
// constant behind the memcpy.
void erase_dummy_constants(Program &p) {
  std::vector<Op *> doomed;
  for (Op *op : p.ops) {
    if (op->kind != OP_MALLOC) continue;
    bool dummy = true;
    for (const auto &u : op->result->uses)
      if (u.first->kind != OP_MEMCPY && u.first->kind != OP_DEALLOC) dummy = false;
    if (!dummy) continue;
    Op *host = nullptr;
    for (const auto &u : op->result->uses) {
      if (u.first->kind == OP_MEMCPY && u.first->operands[1]->def) host = u.first->operands[1]->def;
      doomed.push_back(u.first);
    }
    if (host && host->kind == OP_HOST_CONST) doomed.push_back(host);
    doomed.push_back(op);
  }
  for (Op *op : doomed)
    if (op->pos != p.ops.end()) p.erase(op);
}

}  // namespace dnnc
