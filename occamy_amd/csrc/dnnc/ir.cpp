#include "ir.h"

#include <algorithm>
#include <cstdio>
#include <sstream>

namespace dnnc {

const char *op_name(OpKind k) {
  switch (k) {
    case OP_MALLOC: return "dnn.malloc";
    case OP_DEALLOC: return "dnn.dealloc";
    case OP_MEMCPY: return "dnn.memcpy";
    case OP_MEMPOOL_INIT: return "dnn.mempool-init";
    case OP_MEM_OFFSET: return "dnn.mem-offset";
    case OP_HOST_CONST: return "host.constant";
    case OP_HOST_ALLOC: return "host.alloc";
    case OP_CONVFWD: return "dnn.convfwd";
    case OP_CONV_BIAS_ACTIV: return "dnn.conv-bias-relufwd";
    case OP_ACTIVATION: return "dnn.activationfwd";
    case OP_ADD: return "dnn.add";
    case OP_MUL: return "dnn.mul";
    case OP_SQRT: return "dnn.sqrt";
    case OP_NEGATIVE: return "dnn.negative";
    case OP_RECIPROCAL: return "dnn.reciprocal";
    case OP_REDUCE: return "dnn.reduce";
    case OP_MAXPOOL: return "dnn.maxpool";
    case OP_AVGPOOL: return "dnn.averagepool";
    case OP_SOFTMAX: return "dnn.softmax";
    case OP_FLATTEN: return "dnn.flatten";
    case OP_RESHAPE: return "dnn.reshape";
    case OP_TRANSPOSE: return "dnn.transpose";
    case OP_GATHER: return "dnn.gather";
    case OP_MATMUL2D: return "dnn.matmul2d";
    case OP_MATMULND: return "dnn.matmulnd";
    case OP_POW: return "dnn.pow";
    case OP_ERF: return "dnn.erf";
    case OP_CAST: return "dnn.cast";
    case OP_CLIP: return "dnn.clip";
    case OP_LEAKYRELU: return "dnn.leakyrelu";
    case OP_PRELU: return "dnn.prelu";
    case OP_CONCAT: return "dnn.concat";
    case OP_SQUEEZE: return "dnn.squeeze";
    case OP_UNSQUEEZE: return "dnn.unsqueeze";
    case OP_EXPAND: return "dnn.expand";
    case OP_LAYERNORM: return "dnn.layernorm";
    case OP_GELU: return "dnn.gelu";
    case OP_CONV_BIAS_ADD_ACTIV: return "dnn.conv-bias-add-relufwd";
    case OP_MATMUL_BIAS: return "dnn.matmulnd-bias";
    case OP_ATTENTION: return "dnn.attention";
    case OP_CONV_BIAS_ACTIV_MAXPOOL: return "dnn.conv-bias-relu-maxpoolfwd";
    case OP_CONV_ADD_CONV_ACTIV: return "dnn.conv-bias-add-conv-bias-relufwd";
    case OP_RETURN: return "return";
  }
  return "?";
}

Value *Program::new_value(DType dt, const Shape &s) {
  value_store.emplace_back(new Value());
  Value *v = value_store.back().get();
  v->id = next_value_id_++;
  v->dtype = dt;
  v->shape = s;
  return v;
}

Op *Program::new_op(OpKind k) {
  op_store.emplace_back(new Op());
  Op *op = op_store.back().get();
  op->kind = k;
  op->pos = ops.end();
  return op;
}

Op *Program::terminator() {
  if (!ops.empty() && ops.back()->kind == OP_RETURN) return ops.back();
  return nullptr;
}

void Program::append(Op *op) {
  Op *t = terminator();
  op->pos = ops.insert(t ? t->pos : ops.end(), op);
  invalidate();
}
void Program::insert_before(Op *op, Op *anchor) {
  op->pos = ops.insert(anchor->pos, op);
  invalidate();
}
void Program::insert_after(Op *op, Op *anchor) {
  op->pos = ops.insert(std::next(anchor->pos), op);
  invalidate();
}
void Program::move_after(Op *op, Op *anchor) {
  if (op == anchor) return;
  ops.erase(op->pos);
  op->pos = ops.insert(std::next(anchor->pos), op);
  invalidate();
}
void Program::move_before(Op *op, Op *anchor) {
  if (op == anchor) return;
  ops.erase(op->pos);
  op->pos = ops.insert(anchor->pos, op);
  invalidate();
}

void Program::set_operands(Op *op, const std::vector<Value *> &v) {
  for (size_t i = 0; i < op->operands.size(); i++) {
    auto &u = op->operands[i]->uses;
    u.erase(std::remove(u.begin(), u.end(), std::make_pair(op, (int)i)), u.end());
  }
  op->operands = v;
  for (size_t i = 0; i < v.size(); i++) v[i]->uses.insert(v[i]->uses.begin(), {op, (int)i});
}

void Program::erase(Op *op) {
  set_operands(op, {});
  if (op->pos != ops.end()) ops.erase(op->pos);
  op->pos = ops.end();
  invalidate();
}

void Program::replace_all_uses(Value *from, Value *to) {
  if (from == to) return;
  // each use is unhooked from `from` and pushed on the front of `to`'s list
  const auto old = from->uses;
  from->uses.clear();
  for (const auto &u : old) {
    u.first->operands[(size_t)u.second] = to;
    to->uses.insert(to->uses.begin(), u);
  }
}

void Program::renumber() {
  order_.clear();
  int i = 0;
  for (const Op *op : ops) order_[op] = i++;
  order_valid_ = true;
}
int Program::order(const Op *op) const {
  if (!order_valid_) const_cast<Program *>(this)->renumber();
  auto it = order_.find(op);
  return it == order_.end() ? -1 : it->second;
}

Op *Program::last_user(const Value *v) {
  Op *best = nullptr;
  for (const auto &u : v->uses)
    if (!best || order(u.first) > order(best)) best = u.first;
  return best;
}

static void print_shape(std::ostringstream &os, const Shape &s) {
  os << "[";
  for (size_t i = 0; i < s.size(); i++) os << (i ? "," : "") << s[i];
  os << "]";
}

std::string Program::to_text() const {
  std::ostringstream os;
  for (const Op *op : ops) {
    if (op->result) os << "%" << op->result->id << " = ";
    os << op_name(op->kind);
    for (size_t i = 0; i < op->operands.size(); i++) {
      const Value *v = op->operands[i];
      os << (i ? ", " : " ");
      if (v->arg_index >= 0) os << "%arg" << v->arg_index;
      else os << "%" << v->id;
    }
    switch (op->kind) {
      case OP_MALLOC: os << " {bytes=" << op->bytes << "}"; break;
      case OP_MEMCPY: os << " {count=" << op->bytes << ", mode=" << op->mode << "}"; break;
      case OP_MEM_OFFSET: os << " {offset=" << op->offset << ", size=" << op->bytes << "}"; break;
      case OP_MEMPOOL_INIT: os << " {bytes=" << op->bytes << "}"; break;
      case OP_HOST_CONST: os << " @" << op->const_name; break;
      case OP_HOST_ALLOC: os << " {result=" << op->out_index << "}"; break;
      case OP_CONVFWD:
      case OP_CONV_BIAS_ACTIV:
      case OP_CONV_BIAS_ADD_ACTIV:
        os << " {pads=";
        print_shape(os, op->pads);
        os << ", strides=";
        print_shape(os, op->strides);
        os << ", group=" << op->group;
        if (op->kind != OP_CONVFWD) os << ", activMode=" << op->mode;
        if (op->kind != OP_CONVFWD && (op->mode == 3 || op->mode == 6)) os << ", activCoef=" << op->coef;
        os << "}";
        break;
      case OP_CONV_BIAS_ACTIV_MAXPOOL:
        os << " {pads=";
        print_shape(os, op->pads);
        os << ", strides=";
        print_shape(os, op->strides);
        os << ", group=" << op->group << ", activMode=" << op->mode << ", poolKernel=";
        print_shape(os, op->kernel);
        os << ", poolPads=";
        print_shape(os, op->pool_pads);
        os << ", poolStrides=";
        print_shape(os, op->pool_strides);
        os << "}";
        break;
      case OP_CONV_ADD_CONV_ACTIV:
        os << " {pads=";
        print_shape(os, op->pads);
        os << ", strides=";
        print_shape(os, op->strides);
        os << ", pads2=";
        print_shape(os, op->pads2);
        os << ", strides2=";
        print_shape(os, op->strides2);
        os << ", activMode=" << op->mode;
        if (op->mode == 3 || op->mode == 6) os << ", activCoef=" << op->coef;
        os << "}";
        break;
      case OP_ACTIVATION: os << " {mode=" << op->mode << "}"; break;
      case OP_ADD: os << " {dimB="; print_shape(os, op->dimB); os << ", biasB=" << op->coef << "}"; break;
      case OP_MUL: os << " {dimB="; print_shape(os, op->dimB); os << "}"; break;
      case OP_REDUCE: os << " {dimOutput="; print_shape(os, op->dimOut); os << ", mode=" << op->mode << "}"; break;
      case OP_MAXPOOL:
      case OP_AVGPOOL:
        os << " {kernel=";
        print_shape(os, op->kernel);
        os << ", pads=";
        print_shape(os, op->pads);
        os << ", strides=";
        print_shape(os, op->strides);
        os << "}";
        break;
      case OP_SOFTMAX:
      case OP_FLATTEN:
      case OP_CONCAT:
      case OP_GATHER: os << " {axis=" << op->axis << "}"; break;
      case OP_LEAKYRELU: os << " {alpha=" << op->alpha << "}"; break;
      case OP_MATMUL_BIAS: if (op->mode == 7) os << " {gelu}"; break;
      case OP_ATTENTION: os << " {heads=" << op->group << ", scale=" << op->alpha << (op->axis ? ", packed" : "") << "}"; break;
      case OP_SQUEEZE:
      case OP_UNSQUEEZE: os << " {axes="; print_shape(os, op->perm); os << "}"; break;
      case OP_TRANSPOSE: os << " {perm="; print_shape(os, op->perm); os << "}"; break;
      case OP_MATMUL2D:
        os << " {alpha=" << op->alpha << ", beta=" << op->beta << ", transA=" << op->trans_a
           << ", transB=" << op->trans_b;
        if (op->operands.size() == 4) { os << ", dimC="; print_shape(os, op->kernel); }
        os << "}";
        break;
      case OP_CLIP: os << " {min=" << op->lo << ", max=" << op->hi << "}"; break;
      case OP_LAYERNORM: os << " {eps=" << op->eps << "}"; break;
      default: break;
    }
    if (op->result) {
      os << " : " << dtype_name(op->result->dtype);
      print_shape(os, op->result->shape);
    }
    os << "\n";
  }
  return os.str();
}

}  // namespace dnnc
