// DNN-level passes: conv+bias(+relu) fusion, dealloc placement by last use,
// and the memory-pool rewrite.  Each restates one pass of the reference:
//   src/Transform/DNN/opFusing/fuseConvBiasRelu.cpp:35-152
//   src/Transform/DNN/DNNDeallocOpt.cpp:26-45
//   src/Transform/DNN/mallocPoolOpt.cpp:41-80 (+ mallocPoolOpt.hpp:239-265)
#include "ir.h"
#include "planner.h"

#include <map>
#include <limits>
#include <algorithm>
#include <algorithm>
#include <cmath>
#include <cstring>

namespace dnnc {

// conv -> add(bias) [-> relu] becomes one conv-bias-relufwd.  With a ReLU the
// fused op writes the ReLU's buffer and the convolution's own buffer (malloc
// and dealloc) disappears; without, it writes the convolution's buffer.
// Unlike the reference the fused op keeps `group`.
void fuse_conv_bias_activ(Program &p) {
  std::vector<Op *> convs;
  for (Op *op : p.ops)
    if (op->kind == OP_CONVFWD) convs.push_back(op);
  for (Op *conv : convs) {
    // every user of the convolution's result must be a dnn.add
    if (conv->result->uses.empty()) continue;
    Op *add = nullptr;
    bool ok = true;
    for (const auto &u : conv->result->uses) {
      if (u.first->kind != OP_ADD) { ok = false; break; }
      add = u.first;
    }
    if (!ok || !add) continue;
    // the add must be the bias add emitted with the convolution: A is the
    // conv result, the output buffer is the conv's buffer, B is [1,K,1,1]
    if (add->operands[0] != conv->result || add->operands[2] != conv->operands[3]) continue;
    if (add->dimB.size() != 4 || add->dimB[0] != 1 || add->dimB[2] != 1 || add->dimB[3] != 1) continue;
    // first user of the add decides: ReLU -> CONVBIASRELU, anything else -> CONVBIAS
    Op *relu = nullptr;
    if (!add->result->uses.empty()) {
      Op *u0 = add->result->uses.front().first;
      if (u0->kind == OP_ACTIVATION && u0->mode == 1 && u0->operands[0] == add->result) relu = u0;
    }
    // fusing the ReLU away is only sound when nothing else reads the un-activated value
    if (relu && add->result->uses.size() != 1) relu = nullptr;

    Value *x = conv->operands[0], *w = conv->operands[1], *ws = conv->operands[2], *bias = add->operands[1];
    Value *out = relu ? relu->operands[1] : conv->operands[3];
    Op *fused = p.new_op(OP_CONV_BIAS_ACTIV);
    fused->pads = conv->pads;
    fused->strides = conv->strides;
    fused->group = conv->group;
    fused->dimA = conv->dimA;
    fused->dimB = conv->dimB;
    fused->mode = relu ? 1 : 5;
    fused->result = p.new_value(out->dtype, out->shape);
    fused->result->def = fused;
    p.insert_after(fused, out->def);  // right behind the malloc it writes
    p.set_operands(fused, {x, w, bias, ws, out});
    if (relu) {
      p.replace_all_uses(relu->result, fused->result);
      Value *dead_buf = conv->operands[3];
      Op *dead_malloc = dead_buf->def;
      p.erase(relu);
      p.erase(add);
      p.erase(conv);
      std::vector<Op *> deallocs;
      for (const auto &u : dead_buf->uses)
        if (u.first->kind == OP_DEALLOC) deallocs.push_back(u.first);
      for (Op *d : deallocs) p.erase(d);
      if (dead_buf->uses.empty()) p.erase(dead_malloc);
    } else {
      p.replace_all_uses(add->result, fused->result);
      p.erase(add);
      p.erase(conv);
    }
  }
}

// conv+bias (identity) -> add(full-shape tensor Z) [-> relu], the convolution's
// result read by nothing else (and the sum by nothing but the ReLU), becomes
// one conv-bias-add-activation writing the last buffer of the chain.  The
// reference has no such pattern; cuDNN's fused call has the z operand for it
// (the reference passes it with weight 0,
// src/Tools/dnn-wrapper/cudnn/fusedOp/CUDNNConvBiasReluFunc.cpp:94-112).
void fuse_residual_add(Program &p) {
  std::vector<Op *> convs;
  for (Op *op : p.ops)
    if (op->kind == OP_CONV_BIAS_ACTIV && op->mode == 5) convs.push_back(op);
  auto drop_buffer = [&](Value *buf) {
    std::vector<Op *> deallocs;
    for (const auto &u : buf->uses)
      if (u.first->kind == OP_DEALLOC) deallocs.push_back(u.first);
    for (Op *d : deallocs) p.erase(d);
    if (buf->uses.empty() && buf->def) p.erase(buf->def);
  };
  for (Op *conv : convs) {
    if (conv->result->uses.size() != 1) continue;
    Op *add = conv->result->uses.front().first;
    if (add->kind != OP_ADD || add->coef != 1.f || add->dimA != add->dimB) continue;
    Value *z = add->operands[0] == conv->result ? add->operands[1] : add->operands[0];
    if (z == conv->result || z->shape != conv->result->shape) continue;
    // a ReLU that is the sum's only reader joins in; else the fused call stops at the sum
    Op *relu = nullptr;
    if (add->result->uses.size() == 1) {
      Op *u = add->result->uses.front().first;
      if (u->kind == OP_ACTIVATION && u->mode == 1 && u->operands[0] == add->result) relu = u;
    }
    Value *out = relu ? relu->operands[1] : add->operands[2];
    Op *fused = p.new_op(OP_CONV_BIAS_ADD_ACTIV);
    fused->pads = conv->pads;
    fused->strides = conv->strides;
    fused->group = conv->group;
    fused->dimA = conv->dimA;
    fused->dimB = conv->dimB;
    fused->mode = relu ? 1 : 5;
    fused->result = p.new_value(out->dtype, out->shape);
    fused->result->def = fused;
    // where the last fused operation stood: Z and the output buffer both exist by then
    p.insert_after(fused, relu ? relu : add);
    p.set_operands(fused, {conv->operands[0], conv->operands[1], conv->operands[2], conv->operands[3], z, out});
    p.replace_all_uses(relu ? relu->result : add->result, fused->result);
    Value *conv_buf = conv->operands[4], *add_buf = add->operands[2];
    if (relu) p.erase(relu);
    p.erase(add);
    p.erase(conv);
    if (conv_buf != out) drop_buffer(conv_buf);
    if (!relu) continue;
    if (add_buf != conv_buf) drop_buffer(add_buf);
  }
}

// The first two layers of an ImageNet ResNet, conv 7x7 / stride 2 / pad 3 over the 3-channel function argument
// (+ bias, ReLU or identity) -> max-pool 3x3 / stride 2 / pad 1, the convolution's result read by nothing else,
// become one call that never stores that result (four times the pooled tensor).  Channels-last fp16 programs (even
// image width, input straight from the function argument) and N,C,H,W fp32 programs, and only this shape: it is
// the one the runtime's kernels are written for, and the runtime refuses everything else rather than fall back.
// The reference has no such pattern
// (src/Dialect/DNN/Transforms/fuseConvBiasRelu.cpp stops at the activation).
void fuse_first_layer_maxpool(Program &p) {
  std::vector<Op *> convs;
  for (Op *op : p.ops)
    if (op->kind == OP_CONV_BIAS_ACTIV && (op->mode == 1 || op->mode == 5)) convs.push_back(op);
  for (Op *conv : convs) {
    const Shape &dx = conv->dimA, &dw = conv->dimB;
    const bool f16 = conv->result->dtype == F16;
    if (dx.size() != 4 || dw.size() != 4) continue;
    if (f16 ? !p.channels_last_requested : (conv->result->dtype != F32 || p.channels_last_requested)) continue;
    if (dw[0] != 64 || dw[1] != 3 || dw[2] != 7 || dw[3] != 7 || conv->group != 1 || (f16 && (dx[3] & 1))) continue;
    if (conv->pads != Shape{3, 3} || conv->strides != Shape{2, 2}) continue;
    // the input must be the device copy of a function argument (N,C,H,W as the host sent it)
    bool from_arg = false;
    for (const auto &u : conv->operands[0]->uses)
      if (u.first->kind == OP_MEMCPY && u.first->mode == 1 && u.second == 0 && u.first->operands[1]->arg_index >= 0) from_arg = true;
    if ((f16 && !from_arg) || conv->result->uses.size() != 1) continue;
    Op *pool = conv->result->uses.front().first;
    if (pool->kind != OP_MAXPOOL || pool->operands[0] != conv->result) continue;
    if (pool->kernel != Shape{3, 3} || pool->strides != Shape{2, 2} || pool->pads.size() < 2 || pool->pads[0] != 1 || pool->pads[1] != 1)
      continue;
    if (pool->pads.size() == 4 && (pool->pads[2] != 1 || pool->pads[3] != 1)) continue;
    Value *out = pool->operands[1];
    Op *fused = p.new_op(OP_CONV_BIAS_ACTIV_MAXPOOL);
    fused->pads = conv->pads;
    fused->strides = conv->strides;
    fused->group = conv->group;
    fused->dimA = conv->dimA;
    fused->dimB = conv->dimB;
    fused->mode = conv->mode;
    fused->kernel = pool->kernel;
    fused->pool_pads = pool->pads;
    fused->pool_strides = pool->strides;
    fused->dimOut = pool->dimOut;
    fused->result = p.new_value(out->dtype, out->shape);
    fused->result->def = fused;
    p.insert_after(fused, pool);  // where the pooling stood: its output buffer exists by then
    p.set_operands(fused, {conv->operands[0], conv->operands[1], conv->operands[2], conv->operands[3], out});
    p.replace_all_uses(pool->result, fused->result);
    Value *conv_buf = conv->operands[4];
    p.erase(pool);
    p.erase(conv);
    std::vector<Op *> deallocs;
    for (const auto &u : conv_buf->uses)
      if (u.first->kind == OP_DEALLOC) deallocs.push_back(u.first);
    for (Op *d : deallocs) p.erase(d);
    if (conv_buf->uses.empty() && conv_buf->def) p.erase(conv_buf->def);
  }
}

// conv + bias (identity: the projection shortcut of a residual block) whose only reader is the residual operand of a
// conv + bias + add + activation (the block's last convolution): one call computes both, and no tensor is allocated
// for the shortcut's result, the largest of the block.  The runtime runs the pair as one kernel where that is faster
// (fp16 channels-last over 64 + 64 and 128 + 256 channels: 89 -> 56 us and 55 -> 50 us at batch 64; fp32 at batch-1
// sizes: one launch fewer per shortcut) and as the two convolutions through the output buffer elsewhere.  fp16
// programs must be channels-last.  The reference has no such pattern.
void fuse_projection_shortcut(Program &p) {
  std::vector<Op *> closers;
  for (Op *op : p.ops)
    if (op->kind == OP_CONV_BIAS_ADD_ACTIV) closers.push_back(op);
  for (Op *m : closers) {  // operands: x, w, bias, workspace, z, out
    if (m->group != 1 || m->dimB.size() != 4) continue;
    if (m->result->dtype == F16 && !p.channels_last_requested) continue;
    Value *z = m->operands[4];
    Op *sc = z->def;
    if (!sc || sc->kind != OP_CONV_BIAS_ACTIV || sc->mode != 5 || sc->group != 1 || sc->dimB.size() != 4 || z->uses.size() != 1) continue;
    if (z->shape != m->result->shape || sc->operands[0]->shape.size() != 4) continue;
    Value *out = m->operands[5];
    Op *fused = p.new_op(OP_CONV_ADD_CONV_ACTIV);
    fused->pads = m->pads; fused->strides = m->strides; fused->group = 1;
    fused->dimA = m->dimA; fused->dimB = m->dimB; fused->mode = m->mode; fused->coef = m->coef;
    fused->dimA2 = sc->dimA; fused->dimB2 = sc->dimB; fused->pads2 = sc->pads; fused->strides2 = sc->strides;
    fused->result = p.new_value(out->dtype, out->shape);
    fused->result->def = fused;
    p.insert_after(fused, m);
    p.set_operands(fused, {m->operands[0], m->operands[1], m->operands[2], m->operands[3], sc->operands[0], sc->operands[1],
                           sc->operands[2], sc->operands[3], out});
    p.replace_all_uses(m->result, fused->result);
    Value *sc_buf = sc->operands[4];
    p.erase(m);
    p.erase(sc);
    std::vector<Op *> deallocs;
    for (const auto &u : sc_buf->uses)
      if (u.first->kind == OP_DEALLOC) deallocs.push_back(u.first);
    for (Op *d : deallocs) p.erase(d);
    if (sc_buf->uses.empty() && sc_buf->def) p.erase(sc_buf->def);
  }
}

// Flatten, Reshape, Squeeze and Unsqueeze move no element: the reference copies the tensor into a buffer of its
// own (src/Tools/dnn-wrapper/cuda/CUDAFlattenFunc.cu and its three siblings are device-to-device copies), here the
// operation can instead name its input's buffer as its output buffer.  The executor launches nothing for an
// operation whose input and output are the same address; the buffer lives on under the result's readers (the
// dealloc pass follows a result back to the buffer its producer names last), and the copy's own buffer and
// launch are gone.  Not done when anything else writes the input's buffer.
void alias_copies(Program &p) {
  std::vector<Op *> copies;
  for (Op *op : p.ops)
    if ((op->kind == OP_FLATTEN || op->kind == OP_RESHAPE || op->kind == OP_SQUEEZE || op->kind == OP_UNSQUEEZE) &&
        op->operands.size() == 2)
      copies.push_back(op);
  for (Op *op : copies) {
    Value *x = op->operands[0], *old_out = op->operands[1];
    Value *buf = nullptr;
    if (x->def && x->def->kind == OP_MALLOC) buf = x;
    else if (x->def && x->def->kind >= OP_CONVFWD && x->def->kind < OP_RETURN && !x->def->operands.empty()) buf = x->def->operands.back();
    if (!buf || !buf->def || buf->def->kind != OP_MALLOC || buf == old_out) continue;
    if (shape_numel(buf->shape) * dtype_bytes(buf->dtype) != shape_numel(old_out->shape) * dtype_bytes(old_out->dtype)) continue;
    bool other_writer = false;
    for (const auto &u : buf->uses)
      if (u.first != x->def && u.first->kind != OP_MEMCPY && u.first->kind != OP_DEALLOC && !u.first->operands.empty() &&
          u.first->operands.back() == buf)
        other_writer = true;
    if (other_writer) continue;
    // Something besides the copy and the deallocs names the copy's own buffer (the copy to the host of a returned
    // tensor reads the buffer, not the result): the copy stays a copy.
    std::vector<Op *> deallocs;
    bool other_user = false;
    for (const auto &u : old_out->uses) {
      if (u.first->kind == OP_DEALLOC) deallocs.push_back(u.first);
      else if (u.first != op) other_user = true;
    }
    if (other_user) continue;
    p.set_operands(op, {x, buf});
    for (Op *d : deallocs) p.erase(d);
    if (old_out->def && old_out->def->kind == OP_MALLOC) p.erase(old_out->def);
  }
}

// conv + bias + add + activation whose residual operand is read by nothing later writes its result over that
// operand: the output names the residual's buffer, and its own buffer is never allocated.  Every convolution kernel
// of the runtime adds the residual element by element in the thread that stores the element, so the call may be
// given Z == Y.  Besides the smaller pool, the call then touches the residual's lines once instead of two tensors':
// at batch 64 the last convolution of a ResNet-50 first-stage block reads 129 MB and writes 103 MB, and with a
// separate output what it leaves in the memory-side cache is no longer the whole tensor the next layer reads.
// Not done when the residual's buffer is also the convolution's input, or is used (a reader of anything written
// there, a copy to the host) after the call.  The reference
// has no such pattern (src/Transform/DNN/mallocPoolOpt.cpp places every result in a slot of its own).
void inplace_residual(Program &p) {
  std::vector<Op *> closers;
  for (Op *op : p.ops)
    if (op->kind == OP_CONV_BIAS_ADD_ACTIV) closers.push_back(op);
  auto buffer_of = [](const Value *v) -> Value * {
    if (!v->def) return nullptr;
    if (v->def->kind == OP_MALLOC) return const_cast<Value *>(v);
    if (v->def->kind >= OP_CONVFWD && v->def->kind < OP_RETURN && !v->def->operands.empty()) return v->def->operands.back();
    return nullptr;
  };
  for (Op *m : closers) {  // operands: x, w, bias, workspace, z, out
    Value *z = m->operands[4], *old_out = m->operands[5];
    Value *zbuf = buffer_of(z);
    if (!zbuf || zbuf == z || !zbuf->def || zbuf->def->kind != OP_MALLOC || zbuf == old_out) continue;
    if (!old_out->def || old_out->def->kind != OP_MALLOC) continue;
    if (buffer_of(m->operands[0]) == zbuf) continue;
    if (shape_numel(zbuf->shape) * dtype_bytes(zbuf->dtype) != shape_numel(old_out->shape) * dtype_bytes(old_out->dtype)) continue;
    const int at = p.order(m);
    bool ok = true;
    for (const auto &u : zbuf->uses) {  // direct users of the buffer: whoever wrote it (the residual's producer last), copies, the dealloc
      if (u.first == m || u.first->kind == OP_DEALLOC) continue;
      if (p.order(u.first) > at) ok = false;
      const bool writes = u.first->kind != OP_MEMCPY && !u.first->operands.empty() && u.first->operands.back() == zbuf;
      if (writes && u.first->result)
        for (const auto &r : u.first->result->uses)  // readers of what was written there
          if (r.first != m && p.order(r.first) > at) ok = false;
    }
    std::vector<Op *> deallocs;
    for (const auto &u : old_out->uses) {
      if (u.first->kind == OP_DEALLOC) deallocs.push_back(u.first);
      else if (u.first != m) ok = false;  // something else names the output buffer (a copy to the host)
    }
    if (!ok) continue;
    p.set_operands(m, {m->operands[0], m->operands[1], m->operands[2], m->operands[3], z, zbuf});
    for (Op *d : deallocs) p.erase(d);
    p.erase(old_out->def);
    // the residual's buffer now lives on under this call's result: its dealloc belongs behind the result's readers
    for (const auto &u : zbuf->uses)
      if (u.first->kind == OP_DEALLOC && p.order(u.first) < p.order(p.ops.back())) {
        Op *last = p.last_user(m->result);
        if (last && p.order(last) > p.order(u.first)) p.move_after(u.first, last);
      }
  }
}

// conv+bias (identity) -> Clip(0, c) | LeakyRelu(alpha) | PRelu(one constant
// slope), the convolution's result read by nothing else, becomes one fused
// call with activation mode 3 (clipped ReLU, ceiling c) or 6 (leaky ReLU,
// slope alpha) writing the activation's buffer; the convolution's own buffer
// disappears.  The reference has no such pattern (cuDNN's fused call knows
// ReLU and identity only, CUDNNConvBiasReluFunc.cpp:60-71); MobileNetV2's
// ReLU6, YOLO's LeakyRelu and SRGAN's shared-slope PRelu are its cases.
static bool constant_scalar(const Program &p, const Value *dev, float &out) {
  if (!dev->def || dev->def->kind != OP_MALLOC) return false;
  for (const auto &u : dev->uses) {
    const Op *cp = u.first;
    if (cp->kind != OP_MEMCPY || cp->mode != 1 || u.second != 0) continue;
    const Op *hc = cp->operands[1]->def;
    if (!hc || hc->kind != OP_HOST_CONST) return false;
    const GTensor &t = p.graph->tensors.at(hc->const_name);
    if (shape_numel(t.shape) != 1 || t.dtype == I64) return false;
    if (t.dtype == F32) { std::memcpy(&out, t.data.data(), 4); return true; }
    uint16_t h;
    std::memcpy(&h, t.data.data(), 2);
    const int s = h >> 15, e = (h >> 10) & 31, m = h & 1023;
    const float v = e == 0 ? std::ldexp((float)m, -24) : e == 31 ? (m ? NAN : INFINITY) : std::ldexp((float)(m + 1024), e - 25);
    out = s ? -v : v;
    return true;
  }
  return false;
}

void fuse_conv_activations(Program &p) {
  std::vector<Op *> convs;
  for (Op *op : p.ops)
    if (op->kind == OP_CONV_BIAS_ACTIV && op->mode == 5) convs.push_back(op);
  for (Op *conv : convs) {
    if (conv->result->uses.size() != 1) continue;
    Op *act = conv->result->uses.front().first;
    if (act->operands[0] != conv->result) continue;
    int64_t mode;
    float coef;
    if (act->kind == OP_CLIP && act->lo == 0.f && act->hi > 0.f && act->hi < INFINITY) { mode = 3; coef = act->hi; }
    else if (act->kind == OP_LEAKYRELU) { mode = 6; coef = act->alpha; }
    else if (act->kind == OP_PRELU && constant_scalar(p, act->operands[1], coef)) mode = 6;
    else continue;
    Value *out = act->operands.back();
    Op *fused = p.new_op(OP_CONV_BIAS_ACTIV);
    fused->pads = conv->pads;
    fused->strides = conv->strides;
    fused->group = conv->group;
    fused->dimA = conv->dimA;
    fused->dimB = conv->dimB;
    fused->mode = mode;
    fused->coef = coef;
    fused->result = p.new_value(out->dtype, out->shape);
    fused->result->def = fused;
    p.insert_after(fused, act);  // the activation's buffer exists by then
    p.set_operands(fused, {conv->operands[0], conv->operands[1], conv->operands[2], conv->operands[3], out});
    p.replace_all_uses(act->result, fused->result);
    Value *conv_buf = conv->operands[4];
    p.erase(act);
    p.erase(conv);
    std::vector<Op *> deallocs;
    for (const auto &u : conv_buf->uses)
      if (u.first->kind == OP_DEALLOC) deallocs.push_back(u.first);
    for (Op *d : deallocs) p.erase(d);
    if (conv_buf->uses.empty() && conv_buf->def) p.erase(conv_buf->def);
  }
  erase_dummy_constants(p);  // a PRelu slope that nothing reads any more
}

// matmulnd -> add(one row of N values), the product read by nothing else,
// becomes one matmulnd-bias writing the sum's buffer: the Linear layers of a
// transformer as exporters write them (MatMul, then Add of the bias).  No
// counterpart in the reference.
void fuse_matmul_bias(Program &p) {
  std::vector<Op *> mms;
  for (Op *op : p.ops)
    if (op->kind == OP_MATMULND) mms.push_back(op);
  for (Op *mm : mms) {
    if ((mm->result->dtype != F32 && mm->result->dtype != F16) || mm->result->uses.size() != 1) continue;
    Op *add = mm->result->uses.front().first;
    if (add->kind != OP_ADD || add->coef != 1.f || add->operands[0] != mm->result) continue;
    bool row = !add->dimB.empty() && add->dimB.back() == mm->dimOut.back();
    for (size_t i = 0; i + 1 < add->dimB.size(); i++) row = row && add->dimB[i] == 1;
    if (!row) continue;
    Value *out = add->operands[2], *buf = mm->operands[2];
    Op *fused = p.new_op(OP_MATMUL_BIAS);
    fused->dimA = mm->dimA;
    fused->dimB = mm->dimB;
    fused->dimOut = mm->dimOut;
    fused->mode = 5;
    fused->result = p.new_value(out->dtype, out->shape);
    fused->result->def = fused;
    p.insert_after(fused, add);
    p.set_operands(fused, {mm->operands[0], mm->operands[1], add->operands[1], out});
    p.replace_all_uses(add->result, fused->result);
    p.erase(add);
    p.erase(mm);
    if (buf != out) {
      std::vector<Op *> deallocs;
      for (const auto &u : buf->uses)
        if (u.first->kind == OP_DEALLOC) deallocs.push_back(u.first);
      for (Op *d : deallocs) p.erase(d);
      if (buf->uses.empty() && buf->def) p.erase(buf->def);
    }
  }
  // Gemm (Ops/cublas/Gemm.cpp:60-81: a product with beta 0, then C added onto
  // the same buffer): C becomes the product's own C operand with beta 1.
  std::vector<Op *> gemms;
  for (Op *op : p.ops)
    if (op->kind == OP_MATMUL2D && op->operands.size() == 3 && op->beta == 0.f) gemms.push_back(op);
  for (Op *mm : gemms) {
    // the add works on the product's BUFFER (first operand and output), not on the product's result value
    Value *buf = mm->operands[2];
    if (!mm->result->uses.empty()) continue;
    // fp16: only the shape the fp16 product is built for, with the bias as one row
    if (mm->result->dtype == F16 && !(mm->alpha == 1.f && !mm->trans_a && mm->trans_b)) continue;
    if (mm->result->dtype != F32 && mm->result->dtype != F16) continue;
    Op *add = nullptr;
    for (const auto &u : buf->uses) {
      Op *o = u.first;
      if (o == mm || p.order(o) < p.order(mm)) continue;
      if (!add || p.order(o) < p.order(add)) add = o;  // the buffer's next user
    }
    if (!add || add->kind != OP_ADD || add->coef != 1.f || add->operands[0] != buf || add->operands[2] != buf ||
        add->operands[1] == buf)
      continue;
    if (add->dimB.size() != 2 || add->dimB[1] != mm->dimOut[1] || (add->dimB[0] != 1 && add->dimB[0] != mm->dimOut[0])) continue;
    if (mm->result->dtype == F16 && add->dimB[0] != 1) continue;
    Value *out = buf;
    Op *fused = p.new_op(OP_MATMUL2D);
    fused->dimA = mm->dimA;
    fused->dimB = mm->dimB;
    fused->dimOut = mm->dimOut;
    fused->kernel = add->dimB;  // dims of C
    fused->alpha = mm->alpha;
    fused->beta = 1.f;
    fused->trans_a = mm->trans_a;
    fused->trans_b = mm->trans_b;
    fused->result = p.new_value(out->dtype, out->shape);
    fused->result->def = fused;
    p.insert_after(fused, add);
    p.set_operands(fused, {mm->operands[0], mm->operands[1], add->operands[1], out});
    p.replace_all_uses(add->result, fused->result);
    p.erase(add);
    p.erase(mm);
  }
  // second step: the Linear layer's consumer joins in when it is the only
  // reader -- Gelu (mode 7), or the sum with a residual tensor of the same shape
  std::vector<Op *> linears;
  for (Op *op : p.ops)
    if (op->kind == OP_MATMUL_BIAS && op->operands.size() == 4 && op->mode != 7) linears.push_back(op);
  for (Op *lin : linears) {
    if (lin->result->uses.size() != 1) continue;
    Op *next = lin->result->uses.front().first;
    Value *z = nullptr;
    if (next->kind == OP_GELU && next->operands[0] == lin->result) {
    } else if (next->kind == OP_ADD && next->coef == 1.f && next->dimA == next->dimB &&
               (next->operands[0] == lin->result) != (next->operands[1] == lin->result)) {
      z = next->operands[0] == lin->result ? next->operands[1] : next->operands[0];
      if (z->shape != lin->result->shape) continue;
    } else {
      continue;
    }
    Value *out = next->operands.back(), *buf = lin->operands[3];
    Op *fused = p.new_op(OP_MATMUL_BIAS);
    fused->dimA = lin->dimA;
    fused->dimB = lin->dimB;
    fused->dimOut = lin->dimOut;
    fused->mode = z ? 5 : 7;
    fused->result = p.new_value(out->dtype, out->shape);
    fused->result->def = fused;
    p.insert_after(fused, next);
    if (z) p.set_operands(fused, {lin->operands[0], lin->operands[1], lin->operands[2], z, out});
    else p.set_operands(fused, {lin->operands[0], lin->operands[1], lin->operands[2], out});
    p.replace_all_uses(next->result, fused->result);
    p.erase(next);
    p.erase(lin);
    if (buf != out) {
      std::vector<Op *> deallocs;
      for (const auto &u : buf->uses)
        if (u.first->kind == OP_DEALLOC) deallocs.push_back(u.first);
      for (Op *d : deallocs) p.erase(d);
      if (buf->uses.empty() && buf->def) p.erase(buf->def);
    }
  }
}

// Each dealloc (visited in block order, i.e. creation order of the parked
// deallocs) is moved to just after its tensor's last use.  If the last direct
// user writes the tensor (the malloc is that op's last operand), the tensor
// lives on under the op's result, and the dealloc goes after the result's last
// user instead (src/Transform/DNN/DNNDeallocOpt.cpp:24-43).
//
// One case is handled differently from the reference, on purpose: a tensor
// that the function returns AND a later operation reads (SRGAN's feature map).
// There the last direct user is the device-to-host copy, which does not write
// the tensor, so the reference frees it right after the copy although the
// producer's result is still read afterwards; with the pool pass a later
// tensor can then land on it.  Here the readers of every writer's result
// count as uses, which gives the reference's placement in every other case.
// The same rule keeps a buffer alive that an aliasing copy (alias_copies)
// writes a second time while the first writer's result still has readers.
void dealloc_opt(Program &p) {
  std::vector<Op *> deallocs;
  for (Op *op : p.ops)
    if (op->kind == OP_DEALLOC) deallocs.push_back(op);
  for (Op *d : deallocs) {
    Value *buf = d->operands[0];
    Op *m = buf->def;
    if (!m) continue;
    p.move_after(d, m);
    Op *ldu = p.last_user(buf);
    if (!ldu || ldu == d) continue;  // nothing but the dealloc uses it
    // dnn.memcpy carries its byte count as last operand in the reference, so
    // it never counts as "writes its last operand"
    auto writes = [&](const Op *u) { return u->kind != OP_MEMCPY && u->kind != OP_DEALLOC && !u->operands.empty() && u->operands.back() == buf; };
    // The latest reader of ANY writer's result: with one writer, or a chain of in-place writers each read only
    // by the next (convolution, then the bias added in place), that is the reader of the last writer's result,
    // the reference's placement.  A copy that shares its input's buffer (alias_copies) is a second writer whose
    // result can have its last reader before the first writer's has.
    Op *last = ldu;
    for (const auto &u : buf->uses) {
      if (!writes(u.first) || !u.first->result) continue;
      Op *r = p.last_user(u.first->result);
      if (r && p.order(r) > p.order(last)) last = r;
    }
    p.move_after(d, last);
  }
}

std::vector<PoolEvent> pool_events(const Program &p) {
  std::vector<PoolEvent> ev;
  for (const Op *op : p.ops) {
    if (op->kind == OP_MALLOC)
      ev.push_back({0, op->result->id, shape_numel(op->result->shape) * dtype_bytes(op->result->dtype), -1});
    else if (op->kind == OP_DEALLOC && op->operands[0]->def && op->operands[0]->def->kind == OP_MALLOC)
      ev.push_back({1, op->operands[0]->id, 0, -1});
  }
  return ev;
}

// Every malloc becomes mem-offset(pool, offset, size) with the offset the
// simulator assigns; all deallocs go; the pool is created once near the top
// and released in front of the terminator.
// compact: offsets from compact_offsets() instead of the reference's first fit (the events, and everything else
// about the program, are the same).
//
// The reference's planner takes tensors in program order and gives each the first hole it fits, which is what the
// kernel library does at run time there and must be reproduced bit for bit for its `maxAllocByte`.  With every
// lifetime known before anything is placed, the same tensors pack tighter: largest first, each at the lowest
// offset where it overlaps, in address, no already-placed tensor that is alive at the same time.  ResNet-50 at
// batch 64 in fp16: 250 MB -> the 167 MB that are alive at once.  What that buys is not the memory: pool plus
// weights then fit the 256 MB memory-side cache, and a serving loop that replays the same program finds its
// activations there.
static std::vector<int64_t> compact_offsets(const std::vector<int64_t> &size, const std::vector<int> &born, const std::vector<int> &dies) {
  const size_t n = size.size();
  std::vector<size_t> order(n);
  for (size_t i = 0; i < n; i++) order[i] = i;
  std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) { return size[a] > size[b]; });
  std::vector<int64_t> off(n, -1);
  std::vector<size_t> placed;
  for (size_t i : order) {
    if (size[i] == 0) { off[i] = 0; continue; }
    std::vector<std::pair<int64_t, int64_t>> busy;  // address ranges of placed tensors alive together with i
    for (size_t j : placed)
      if (born[j] < dies[i] && born[i] < dies[j]) busy.push_back({off[j], off[j] + size[j]});
    std::sort(busy.begin(), busy.end());
    int64_t at = 0;
    for (const auto &b : busy) {
      if (b.first - at >= size[i]) break;
      at = std::max(at, b.second);
    }
    off[i] = at;
    placed.push_back(i);
  }
  return off;
}

bool malloc_pool_opt(Program &p, std::string &err, bool compact) {
  PoolSimulator sim;
  Op *init = p.new_op(OP_MEMPOOL_INIT);
  init->result = p.new_value(F32, {1});
  init->result->def = init;
  p.insert_before(init, p.ops.front());  // ahead of every mem-offset that will refer to it
  std::vector<Op *> mallocs, deallocs;
  std::vector<int64_t> planned;  // compact: offset per malloc, in program order
  if (compact) {
    std::vector<int64_t> size;
    std::vector<int> born, dies;
    std::map<int64_t, size_t> index;  // value id -> position
    int t = 0;
    for (Op *op : p.ops) {
      if (op->kind == OP_MALLOC) {
        const int64_t bytes = shape_numel(op->result->shape) * dtype_bytes(op->result->dtype);
        index[op->result->id] = size.size();
        size.push_back(bytes <= 0 ? 0 : ((bytes - 1) / 256 + 1) * 256);  // whole cache lines, and then some
        born.push_back(t++);
        dies.push_back(std::numeric_limits<int>::max());
      } else if (op->kind == OP_DEALLOC) {
        const auto it = index.find(op->operands[0]->id);
        if (it == index.end() || dies[it->second] != std::numeric_limits<int>::max()) { err = "dealloc of a tensor that is not live"; return false; }
        dies[it->second] = t++;
      }
    }
    planned = compact_offsets(size, born, dies);
  }
  size_t nth = 0;
  for (Op *op : p.ops) {
    if (op->kind == OP_MALLOC) {
      const int64_t bytes_now = shape_numel(op->result->shape) * dtype_bytes(op->result->dtype);
      const int64_t size = compact ? (bytes_now <= 0 ? 0 : ((bytes_now - 1) / 256 + 1) * 256) : PoolSimulator::round_size(bytes_now);
      const int64_t first_fit = sim.reserve(op->result->id, size);
      const int64_t off = compact ? planned[nth++] : first_fit;
      if (off < 0 || first_fit < 0) { err = "pool simulator ran out of address space"; return false; }
      p.trace.push_back({0, op->result->id, shape_numel(op->result->shape) * dtype_bytes(op->result->dtype), off});
      op->offset = off;
      op->bytes = size;
      mallocs.push_back(op);
    } else if (op->kind == OP_DEALLOC) {
      if (!sim.release(op->operands[0]->id)) { err = "dealloc of a tensor that is not live"; return false; }
      p.trace.push_back({1, op->operands[0]->id, 0, -1});
      deallocs.push_back(op);
    }
  }
  for (Op *m : mallocs) {
    m->kind = OP_MEM_OFFSET;
    p.set_operands(m, {init->result});
  }
  for (Op *d : deallocs) p.erase(d);
  Op *release = p.new_op(OP_DEALLOC);
  p.insert_before(release, p.terminator());
  p.set_operands(release, {init->result});
  // The reference takes the pool size from the start of the LAST free block.
  // When an empty (0-byte) tensor is released while it lies inside a free
  // region, its degenerate block is appended behind the unbounded tail block
  // and that reading goes stale (too small).  Traces the emission rules
  // produce never do this (a convolution's empty workspace is released while
  // its output, at the same address, is live), but the executor must never
  // under-allocate, so the arena also covers the highest planned byte.
  int64_t extent = 0;
  for (Op *m : mallocs) extent = std::max(extent, m->offset + m->bytes);
  p.pool_bytes = compact ? extent : sim.peak();
  p.pool_extent = extent;
  init->bytes = compact ? extent : std::max(sim.peak(), extent);
  return true;
}

}  // namespace dnnc
