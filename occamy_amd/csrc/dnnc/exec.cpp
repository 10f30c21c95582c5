// Executor: walks a compiled DNN program and issues one runtime call per
// operation, which is what the reference's DNN-to-LLVM lowering turns the
// program into (src/Conversion/DNNToLLVM/Ops/** build the dims arrays, pass
// raw device pointers and call the row of DNNAPISpecs.inc).  The runtime is
// bound at run time from a shared object that exports include/dnnrt.h.
//
// Two ways of running a program:
//   occamy   - the reference's semantics per inference: create the pool,
//              upload every constant into its pool slot, run, copy results
//              back, wait, release the pool
//              (src/Transform/DNN/mallocPoolOpt.hpp:239-265,
//               src/Conversion/ONNXToDNN/Ops/Constant.cpp:86-90).
//   resident - the pool and a second arena holding all constants are created
//              once; an inference is input copy + kernels + output copy, and
//              the kernels can be replayed from a captured graph.
#include "exec.h"

#include <dlfcn.h>

#include <algorithm>
#include <cstring>

namespace dnnc {

#define LOAD(name)                                                            \
  do {                                                                         \
    *(void **)(&rt.name) = dlsym(rt.dl, #name);                                \
    if (!rt.name) { err = std::string("runtime library lacks ") + #name; return false; } \
  } while (0)

bool load_runtime(const std::string &path, RuntimeApi &rt, std::string &err) {
  rt.dl = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (!rt.dl) { err = std::string("cannot load runtime library: ") + dlerror(); return false; }
  LOAD(dnnrtCreate); LOAD(dnnrtDestroy); LOAD(dnnrtDeviceMemoryStats); LOAD(dnnrtStreamCreate); LOAD(dnnrtStreamDestroy);
  LOAD(dnnrtSetStream); LOAD(dnnrtSetTensorFormat); LOAD(dnnrtSetFilterLayout); LOAD(dnnrtSetActivationCoef); LOAD(dnnrtSetConvTile); LOAD(dnnrtListConvTiles); LOAD(dnnrtMemFill); LOAD(dnnrtMatmulNdBias); LOAD(dnnrtAttention); LOAD(dnnrtSync); LOAD(dnnrtLastError);
  LOAD(dnnrtIsHostBackend); LOAD(dnnrtGraphBegin); LOAD(dnnrtGraphEnd); LOAD(dnnrtGraphLaunch);
  LOAD(dnnrtGraphDestroy); LOAD(dnnrtEventCreate); LOAD(dnnrtEventRecord); LOAD(dnnrtEventElapsedMs);
  LOAD(dnnrtEventDestroy); LOAD(dnnrtMemPoolInit); LOAD(dnnrtMemOffset); LOAD(dnnrtMemcpy);
  LOAD(dnnrtMalloc); LOAD(dnnrtDealloc); LOAD(dnnrtHostAlloc); LOAD(dnnrtHostFree);
  LOAD(dnnrtConv); LOAD(dnnrtConvBiasActiv); LOAD(dnnrtConvBiasAddActiv); LOAD(dnnrtConvBiasActivMaxPool); LOAD(dnnrtConvBiasAddConvBiasActiv); LOAD(dnnrtActive); LOAD(dnnrtTensorOp); LOAD(dnnrtClip);
  LOAD(dnnrtErf); LOAD(dnnrtNegative); LOAD(dnnrtReciprocal); LOAD(dnnrtPow); LOAD(dnnrtCastI64toFloat);
  LOAD(dnnrtGelu); LOAD(dnnrtReduce); LOAD(dnnrtSoftmax); LOAD(dnnrtLayerNorm); LOAD(dnnrtMaxPool);
  LOAD(dnnrtAveragePool); LOAD(dnnrtMatmul2d); LOAD(dnnrtMatmulNd); LOAD(dnnrtFlatten);
  LOAD(dnnrtReshape); LOAD(dnnrtTranspose); LOAD(dnnrtGather);
  LOAD(dnnrtLeakyRelu); LOAD(dnnrtPRelu); LOAD(dnnrtConcat); LOAD(dnnrtSqueeze); LOAD(dnnrtUnsqueeze); LOAD(dnnrtExpand);
  return true;
}
#undef LOAD

static int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

void Session::drop_graphs() {
  if (graph) rt.dnnrtGraphDestroy(graph);
  graph = nullptr;
  for (auto &g : parked_graphs) rt.dnnrtGraphDestroy(g.second);
  parked_graphs.clear();
}

Session::~Session() {
  if (!rt.dl) return;
  drop_graphs();
  if (handle) rt.dnnrtSync(handle);
  if (pool) rt.dnnrtDealloc(pool);
  if (weights) rt.dnnrtDealloc(weights);
  for (auto &kv : staged_out) rt.dnnrtDealloc(kv.second);
  for (auto &kv : host_const) rt.dnnrtHostFree(kv.second);
  for (void *p : host_out) rt.dnnrtHostFree(p);
  for (void *p : host_in) rt.dnnrtHostFree(p);
  if (handle) rt.dnnrtDestroy(handle);
  if (stream) rt.dnnrtStreamDestroy(stream);
}

std::string Session::rt_error(const char *what) const {
  return std::string(what) + ": " + rt.dnnrtLastError();
}

// KCRS -> KRSC, element size es
static void permute_kcrs_to_krsc(const uint8_t *src, uint8_t *dst, const Shape &w, int64_t es) {
  const int64_t K = w[0], C = w[1], R = w[2], S = w[3];
  for (int64_t k = 0; k < K; k++)
    for (int64_t c = 0; c < C; c++)
      for (int64_t r = 0; r < R; r++)
        for (int64_t s = 0; s < S; s++)
          std::memcpy(dst + (((k * R + r) * S + s) * C + c) * es, src + (((k * C + c) * R + r) * S + s) * es, (size_t)es);
}

// KCRS -> CRSK, element size es
static void permute_kcrs_to_crsk(const uint8_t *src, uint8_t *dst, const Shape &w, int64_t es) {
  const int64_t K = w[0], CRS = w[1] * w[2] * w[3];
  for (int64_t k = 0; k < K; k++)
    for (int64_t j = 0; j < CRS; j++)
      std::memcpy(dst + (j * K + k) * es, src + (k * CRS + j) * es, (size_t)es);
}

static bool is_compute(OpKind k) { return k >= OP_CONVFWD && k < OP_RETURN; }

bool Session::init(const Program *p,const std::string &runtime_path, int mode_, std::string &err) {
  prog = p;
  mode = mode_;
  if (prog->pool_bytes < 0) { err = "the program was compiled without the pool pass"; return false; }
  if (!load_runtime(runtime_path, rt, err)) return false;
  host_backend = rt.dnnrtIsHostBackend() != 0;
  if (prog->channels_last && host_backend) { err = "channels-last programs need the GPU runtime"; return false; }
  if (rt.dnnrtCreate(&handle)) { err = rt_error("dnnrtCreate"); return false; }
  if (rt.dnnrtStreamCreate(&stream)) { err = rt_error("dnnrtStreamCreate"); return false; }
  if (rt.dnnrtSetStream(handle, stream)) { err = rt_error("dnnrtSetStream"); return false; }
  ptr.assign(prog->value_store.size(), nullptr);

  // Which constants are convolution filters and nothing else.  They are
  // re-laid once, in the pinned host copy: K,R,S,C for a channels-last (fp16)
  // program, C,R,S,K for fp32 programs on the GPU runtime.
  std::map<std::string, bool> is_filter;
  std::map<const Value *, std::string> device_copy_of;  // device tensor -> the constant uploaded into it
  for (const Op *op : prog->ops) {
    if (op->kind != OP_MEMCPY || op->mode != 1) continue;
    const Value *src = op->operands[1];
    if (!src->def || src->def->kind != OP_HOST_CONST) continue;
    const std::string &name = src->def->const_name;
    bool only_filter = true, any = false;
    for (const auto &u : op->operands[0]->uses) {
      if (u.first == op) continue;
      const bool conv = u.first->kind == OP_CONVFWD || u.first->kind == OP_CONV_BIAS_ACTIV ||
                        u.first->kind == OP_CONV_BIAS_ADD_ACTIV || u.first->kind == OP_CONV_BIAS_ACTIV_MAXPOOL ||
                        u.first->kind == OP_CONV_ADD_CONV_ACTIV;
      if (conv && (u.second == 1 || (u.first->kind == OP_CONV_ADD_CONV_ACTIV && u.second == 5))) any = true;
      else if (is_compute(u.first->kind)) only_filter = false;
    }
    const bool f = any && only_filter;
    auto it = is_filter.find(name);
    if (it == is_filter.end()) is_filter[name] = f;
    else it->second = it->second && f;
    device_copy_of[op->operands[0]] = name;
  }
  // The two filters of a fused shortcut pair go to one kernel, which takes one layout: if one of them has to
  // stay as it is (another operator reads the same constant), so does the other.
  for (bool changed = true; changed;) {
    changed = false;
    for (const Op *op : prog->ops) {
      if (op->kind != OP_CONV_ADD_CONV_ACTIV) continue;
      const auto a = device_copy_of.find(op->operands[1]), b = device_copy_of.find(op->operands[5]);
      if (a == device_copy_of.end() || b == device_copy_of.end()) continue;
      bool &fa = is_filter[a->second], &fb = is_filter[b->second];
      if (fa != fb) { fa = fb = false; changed = true; }
    }
  }

  // Constants: one pinned host copy each (the reference keeps them as globals
  // of the model library); function results: one pinned buffer each.
  int64_t weight_bytes = 0;
  for (const Op *op : prog->ops) {
    if (op->kind == OP_HOST_CONST) {
      const GTensor &t = prog->graph->tensors.at(op->const_name);
      void *h = nullptr;
      if (rt.dnnrtHostAlloc(&h, (int64_t)t.data.size())) { err = rt_error("dnnrtHostAlloc"); return false; }
      const auto fit = is_filter.find(op->const_name);
      const bool filter = fit != is_filter.end() && fit->second && t.shape.size() == 4;
      if (filter && prog->channels_last) {
        permute_kcrs_to_krsc(t.data.data(), (uint8_t *)h, t.shape, dtype_bytes(t.dtype));
      } else if (filter && !host_backend && t.dtype == F32) {
        permute_kcrs_to_crsk(t.data.data(), (uint8_t *)h, t.shape, dtype_bytes(t.dtype));
        crsk_const[op->const_name] = true;
      } else {
        std::memcpy(h, t.data.data(), t.data.size());
      }
      host_const[op->const_name] = h;
      ptr[(size_t)op->result->id] = h;
      weight_bytes += align_up((int64_t)t.data.size(), 256);
    } else if (op->kind == OP_HOST_ALLOC) {
      void *h = nullptr;
      if (rt.dnnrtHostAlloc(&h, op->bytes)) { err = rt_error("dnnrtHostAlloc"); return false; }
      if ((size_t)op->out_index >= host_out.size()) host_out.resize((size_t)op->out_index + 1, nullptr);
      host_out[(size_t)op->out_index] = h;
      ptr[(size_t)op->result->id] = h;
    }
  }
  filter_crsk.assign(prog->value_store.size(), 0);
  for (const Op *op : prog->ops) {
    if (op->kind != OP_MEMCPY || op->mode != 1) continue;
    const Value *src = op->operands[1];
    if (src->def && src->def->kind == OP_HOST_CONST && crsk_const.count(src->def->const_name))
      filter_crsk[(size_t)op->operands[0]->id] = 1;
  }
  for (const Value *a : prog->args) {
    void *h = nullptr;
    if (rt.dnnrtHostAlloc(&h, shape_numel(a->shape) * dtype_bytes(a->dtype))) { err = rt_error("dnnrtHostAlloc"); return false; }
    host_in.push_back(h);
  }
  weights_bytes = weight_bytes;

  if (mode == MODE_RESIDENT) {
    if (rt.dnnrtMemPoolInit(&pool, std::max(prog->pool_bytes, prog->pool_extent))) { err = rt_error("dnnrtMemPoolInit"); return false; }
    if (rt.dnnrtMalloc(&weights, weight_bytes)) { err = rt_error("dnnrtMalloc(weights)"); return false; }
    // Upload every constant once, into the weights arena; the pool slot the
    // planner gave it stays unused.
    int64_t woff = 0;
    for (const Op *op : prog->ops) {
      if (op->kind == OP_MEMPOOL_INIT) ptr[(size_t)op->result->id] = pool;
      else if (op->kind == OP_MEM_OFFSET) ptr[(size_t)op->result->id] = (char *)pool + op->offset;
    }
    for (const Op *op : prog->ops) {
      if (op->kind != OP_MEMCPY || op->mode != 1) continue;
      const Value *src = op->operands[1];
      if (!src->def || src->def->kind != OP_HOST_CONST) continue;
      void *dev = (char *)weights + woff;
      woff += align_up(op->bytes, 256);
      if (rt.dnnrtMemcpy(dev, ptr[(size_t)src->id], op->bytes, 1, stream)) { err = rt_error("dnnrtMemcpy(constant)"); return false; }
      ptr[(size_t)op->operands[0]->id] = dev;
    }
    if (rt.dnnrtSync(handle)) { err = rt_error("dnnrtSync"); return false; }
    // a result that is copied out before the last compute operation
    bool compute_later = false;
    for (auto it = prog->ops.rbegin(); it != prog->ops.rend(); ++it) {
      const Op *op = *it;
      if (is_compute(op->kind)) compute_later = true;
      if (op->kind != OP_MEMCPY || op->mode != 2 || !compute_later) continue;
      void *stage = nullptr;
      if (rt.dnnrtMalloc(&stage, op->bytes)) { err = rt_error("dnnrtMalloc(result staging)"); return false; }
      staged_out[op] = stage;
    }
  }
  return true;
}

int Session::format_for(const Op *op) const {
  if (!prog->channels_last) return 0;  // NCHW
  if (op->kind == OP_CONVFWD || op->kind == OP_CONV_BIAS_ACTIV || op->kind == OP_CONV_BIAS_ADD_ACTIV || op->kind == OP_CONV_BIAS_ACTIV_MAXPOOL ||
      op->kind == OP_CONV_ADD_CONV_ACTIV) {
    const Value *x = op->operands[0];
    // the function argument's slot holds what the host sent: NCHW
    const bool from_arg = x->def && x->def->kind == OP_MEM_OFFSET;
    return from_arg ? 2 : 1;
  }
  return 1;
}

// One compute operation -> one runtime call.
bool Session::issue(const Op *op, std::string &err) {
  auto P = [&](size_t i) { return ptr[(size_t)op->operands[i]->id]; };
  void *out = op->operands.empty() ? nullptr : P(op->operands.size() - 1);
  const Value *ov = op->operands.empty() ? nullptr : op->operands.back();
  const int dt = ov ? (int)ov->dtype : 0;
  if (prog->channels_last || cur_format != 0) {
    const int f = format_for(op);
    if (f != cur_format) {
      if (rt.dnnrtSetTensorFormat(handle, f)) { err = rt_error("dnnrtSetTensorFormat"); return false; }
      cur_format = f;
    }
  }
  if (op->kind == OP_CONVFWD || op->kind == OP_CONV_BIAS_ACTIV || op->kind == OP_CONV_BIAS_ADD_ACTIV || op->kind == OP_CONV_BIAS_ACTIV_MAXPOOL ||
      op->kind == OP_CONV_ADD_CONV_ACTIV) {
    const int lay = filter_crsk[(size_t)op->operands[1]->id] ? DNNRT_FILTER_CRSK : DNNRT_FILTER_KCRS;
    if (op->kind == OP_CONV_ADD_CONV_ACTIV && filter_crsk[(size_t)op->operands[5]->id] != filter_crsk[(size_t)op->operands[1]->id]) {
      err = "executor: the two filters of a fused shortcut pair were uploaded in different layouts";
      return false;
    }
    if (lay != cur_filter_layout) {
      if (rt.dnnrtSetFilterLayout(handle, lay)) { err = rt_error("dnnrtSetFilterLayout"); return false; }
      cur_filter_layout = lay;
    }
    if ((op->mode == 3 || op->mode == 6) && op->kind != OP_CONVFWD && op->coef != cur_act_coef) {
      if (rt.dnnrtSetActivationCoef(handle, op->coef)) { err = rt_error("dnnrtSetActivationCoef"); return false; }
      cur_act_coef = op->coef;
    }
  }
  // a copy whose output buffer is its input's (the alias_copies pass): nothing to do
  if ((op->kind == OP_FLATTEN || op->kind == OP_RESHAPE || op->kind == OP_SQUEEZE || op->kind == OP_UNSQUEEZE) &&
      op->operands.size() == 2 && P(0) == out) {
    ptr[(size_t)op->result->id] = out;
    return true;
  }
  void *r = nullptr;
  auto pad4 =[](const Shape &s) { Shape o = s; while (o.size() < 4) o.push_back(1); return o; };
  switch (op->kind) {
    case OP_CONVFWD:
      r = rt.dnnrtConv(handle, P(0), op->dimA.data(), P(1), op->dimB.data(), P(2), 0, algo_operand(op, 0, op->algo), op->group,
                       op->pads.data(), op->strides.data(), out, dt);
      break;
    case OP_CONV_BIAS_ACTIV: {
      const int64_t dimB[4] = {1, op->dimB[0], 1, 1};
      r = rt.dnnrtConvBiasActiv(handle, P(0), op->dimA.data(), P(1), op->dimB.data(), P(2), dimB, P(3), 0, algo_operand(op, 0, 1),
                                op->group, op->pads.data(), op->strides.data(), op->mode, out, dt);
      break;
    }
    case OP_CONV_BIAS_ADD_ACTIV: {  // operands: x, w, bias, workspace, z, out
      const int64_t dimB[4] = {1, op->dimB[0], 1, 1};
      r = rt.dnnrtConvBiasAddActiv(handle, P(0), op->dimA.data(), P(1), op->dimB.data(), P(2), dimB, P(4), P(3), 0, algo_operand(op, 0, 1),
                                   op->group, op->pads.data(), op->strides.data(), op->mode, out, dt);
      break;
    }
    case OP_CONV_BIAS_ACTIV_MAXPOOL: {  // operands: x, w, bias, workspace, out
      const int64_t dimB[4] = {1, op->dimB[0], 1, 1};
      r = rt.dnnrtConvBiasActivMaxPool(handle, P(0), op->dimA.data(), P(1), op->dimB.data(), P(2), dimB, op->group, op->pads.data(),
                                       op->strides.data(), op->mode, op->kernel.data(), op->pool_pads.data(), op->pool_strides.data(),
                                       out, op->dimOut.data(), dt);
      break;
    }
    case OP_CONV_ADD_CONV_ACTIV:  // operands: x, w, bias, workspace, x2, w2, bias2, workspace2, out
      r = rt.dnnrtConvBiasAddConvBiasActiv(handle, P(0), op->dimA.data(), P(1), op->dimB.data(), P(2), op->pads.data(), op->strides.data(),
                                           P(4), op->dimA2.data(), P(5), op->dimB2.data(), P(6), op->pads2.data(), op->strides2.data(),
                                           op->mode, algo_operand(op, 0, 1), algo_operand(op, 1, 1), out, dt);
      break;
    case OP_ACTIVATION: {
      const Shape d = pad4(op->dimA);  // the lowering pads the dims to 4 with trailing ones
      if (d.size() > 4) {
        const int64_t flat[4] = {shape_numel(op->dimA), 1, 1, 1};
        r = rt.dnnrtActive(handle, P(0), flat, (int32_t)op->mode, out, dt);
      } else {
        r = rt.dnnrtActive(handle, P(0), d.data(), (int32_t)op->mode, out, dt);
      }
      break;
    }
    case OP_ADD:
    case OP_MUL: {
      const int32_t rank = (int32_t)op->dimA.size();
      r = rt.dnnrtTensorOp(handle, op->kind == OP_ADD ? 0 : 1, P(0), op->dimA.data(), rank, P(1), op->dimB.data(),
                           rank, out, op->dimA.data(), rank, op->coef, dt);
      break;
    }
    case OP_SQRT: {
      const int32_t rank = (int32_t)op->dimA.size();
      r = rt.dnnrtTensorOp(handle, 4, P(0), op->dimA.data(), rank, nullptr, op->dimA.data(), rank, out,
                           op->dimA.data(), rank, 1.f, dt);
      break;
    }
    case OP_NEGATIVE: r = rt.dnnrtNegative(handle, P(0), out, op->dimA.data(), (int64_t)op->dimA.size(), dt); break;
    case OP_RECIPROCAL: r = rt.dnnrtReciprocal(handle, P(0), out, op->dimA.data(), (int64_t)op->dimA.size(), dt); break;
    case OP_ERF: r = rt.dnnrtErf(handle, P(0), out, op->dimA.data(), (int64_t)op->dimA.size(), dt); break;
    case OP_GELU: r = rt.dnnrtGelu(handle, P(0), out, op->dimA.data(), (int64_t)op->dimA.size(), dt); break;
    case OP_POW: r = rt.dnnrtPow(handle, P(0), P(1), out, op->dimA.data(), (int64_t)op->dimA.size(), dt); break;
    case OP_CLIP: r = rt.dnnrtClip(handle, P(0), out, op->dimA.data(), op->lo, op->hi, (int64_t)op->dimA.size(), dt); break;
    case OP_LEAKYRELU:
      r = rt.dnnrtLeakyRelu(handle, P(0), out, op->dimA.data(), op->alpha, (int64_t)op->dimA.size(), dt);
      break;
    case OP_PRELU:
      r = rt.dnnrtPRelu(handle, P(0), out, op->dimA.data(), P(1), op->dimB.data(), (int64_t)op->dimA.size(), dt);
      break;
    case OP_CONCAT: {
      const size_t n_in = op->operands.size() - 1;
      const void *xs[16];
      const int64_t *ds[16];
      for (size_t i = 0; i < n_in; i++) { xs[i] = P(i); ds[i] = op->operands[i]->shape.data(); }
      r = rt.dnnrtConcat(handle, xs, ds, out, op->dimOut.data(), op->axis, (int64_t)n_in, (int32_t)op->dimOut.size(), dt);
      break;
    }
    case OP_SQUEEZE:
      r = rt.dnnrtSqueeze(handle, P(0), op->dimA.data(), (int64_t)op->dimA.size(), out, op->dimOut.data(),
                          (int64_t)op->dimOut.size(), dt);
      break;
    case OP_UNSQUEEZE:
      r = rt.dnnrtUnsqueeze(handle, P(0), op->dimA.data(), (int64_t)op->dimA.size(), out, op->dimOut.data(),
                            (int64_t)op->dimOut.size(), dt);
      break;
    case OP_EXPAND:  // operands: input, shape (device copy, not read), output
      r = rt.dnnrtExpand(handle, P(0), op->dimA.data(), (int64_t)op->dimA.size(), out, op->dimOut.data(),
                         (int64_t)op->dimOut.size(), dt);
      break;
    case OP_CAST:
      r = rt.dnnrtCastI64toFloat(handle, (const int64_t *)P(0), out, op->dimA.data(), (int64_t)op->dimA.size(), dt);
      break;
    case OP_REDUCE:
      r = rt.dnnrtReduce(handle, (int32_t)op->dimA.size(), P(0), op->dimA.data(), out, op->dimOut.data(),
                         (int32_t)op->mode, dt);
      break;
    case OP_MAXPOOL:
      r = rt.dnnrtMaxPool(handle, P(0), op->dimA.data(), out, op->dimOut.data(), op->kernel.data(), op->pads.data(),
                          op->strides.data(), dt);
      break;
    case OP_AVGPOOL:
      r = rt.dnnrtAveragePool(handle, P(0), op->dimA.data(), out, op->dimOut.data(), op->kernel.data(),
                              op->pads.data(), op->strides.data(), dt);
      break;
    case OP_SOFTMAX:
      r = rt.dnnrtSoftmax(handle, P(0), op->dimA.data(), out, op->dimA.data(), op->axis, (int64_t)op->dimA.size(), dt);
      break;
    case OP_LAYERNORM:
      r = rt.dnnrtLayerNorm(handle, P(0), op->dimA.data(), (int64_t)op->dimA.size(), P(1), P(2), op->eps, out, dt);
      break;
    case OP_FLATTEN:
      r = rt.dnnrtFlatten(handle, P(0), op->dimA.data(), out, op->dimOut.data(), (int32_t)op->axis,
                          (int64_t)op->dimA.size(), dt);
      break;
    case OP_RESHAPE: r = rt.dnnrtReshape(handle, P(0), op->dimA.data(), (int64_t)op->dimA.size(), out, dt); break;
    case OP_TRANSPOSE:
      r = rt.dnnrtTranspose(handle, P(0), op->dimA.data(), out, op->dimOut.data(), op->perm.data(),
                            (int64_t)op->dimA.size(), dt);
      break;
    case OP_GATHER:
      r = rt.dnnrtGather(handle, P(0), op->dimA.data(), (int64_t)op->dimA.size(), out, op->dimOut.data(),
                         (int64_t)op->dimOut.size(), (const int64_t *)P(1), op->dimB.data(), (int64_t)op->dimB.size(),
                         op->axis, dt);
      break;
    case OP_MATMUL2D:
      if (op->operands.size() == 4)  // a, b, c, out: C folded in by the matmul + bias fusion
        r = rt.dnnrtMatmul2d(handle, 2, P(0), op->dimA.data(), P(1), op->dimB.data(), P(2), op->kernel.data(), out,
                             op->dimOut.data(), op->alpha, op->beta, op->trans_a, op->trans_b, dt);
      else
        r = rt.dnnrtMatmul2d(handle, 2, P(0), op->dimA.data(), P(1), op->dimB.data(), out, op->dimOut.data(), out,
                             op->dimOut.data(), op->alpha, op->beta, op->trans_a, op->trans_b, dt);
      break;
    case OP_MATMULND:
      r = rt.dnnrtMatmulNd(handle, P(0), op->dimA.data(), (int32_t)op->dimA.size(), P(1), op->dimB.data(),
                           (int32_t)op->dimB.size(), out, op->dimOut.data(), (int32_t)op->dimOut.size(), dt);
      break;
    case OP_ATTENTION:  // operands: q, k, v, out
      if (op->axis) {  // one tensor holds [Q | K | V] per row
        const int64_t hidden = op->dimA[2];
        char *base = (char *)P(0);
        const int64_t es = dt == DNNRT_F16 ? 2 : 4;  // bytes per element
        r = rt.dnnrtAttention(handle, base, base + hidden * es, base + 2 * hidden * es, out, op->dimA[0], op->dimA[1], op->dimB[1],
                              op->group, hidden / op->group, 3 * hidden, op->alpha, dt);
      } else {
        r = rt.dnnrtAttention(handle, P(0), P(1), P(2), out, op->dimA[0], op->dimA[1], op->dimB[1], op->group,
                              op->dimA[2] / op->group, 0, op->alpha, dt);
      }
      break;
    case OP_MATMUL_BIAS:  // operands: a, b, bias, [residual,] out
      r = rt.dnnrtMatmulNdBias(handle, P(0), op->dimA.data(), (int32_t)op->dimA.size(), P(1), op->dimB.data(),
                               (int32_t)op->dimB.size(), P(2), op->operands.size() == 5 ? P(3) : nullptr, op->mode == 7,
                               out, op->dimOut.data(), (int32_t)op->dimOut.size(), dt);
      break;
    default: err = std::string("executor: unexpected op ") + op_name(op->kind); return false;
  }
  if (!r) { err = std::string(op_name(op->kind)) + ": " + rt.dnnrtLastError(); return false; }
  ptr[(size_t)op->result->id] = r;
  return true;
}

// The reference's per-inference sequence, call for call.
bool Session::run_occamy(const void *const *inputs, void *const *outputs, std::string &err) {
  void *run_pool = nullptr;
  for (size_t i = 0; i < prog->args.size(); i++) {
    std::memcpy(host_in[i], inputs[i], (size_t)(shape_numel(prog->args[i]->shape) * dtype_bytes(prog->args[i]->dtype)));
    ptr[(size_t)prog->args[i]->id] = host_in[i];
  }
  bool ok = true;
  for (const Op *op : prog->ops) {
    switch (op->kind) {
      case OP_MEMPOOL_INIT:
        if (rt.dnnrtMemPoolInit(&run_pool, op->bytes)) { err = rt_error("dnnrtMemPoolInit"); ok = false; }
        ptr[(size_t)op->result->id] = run_pool;
        last_pool_bytes = op->bytes;
        if (ok && debug_fill >= 0 && rt.dnnrtMemFill(run_pool, debug_fill, op->bytes, stream)) { err = rt_error("dnnrtMemFill"); ok = false; }
        break;
      case OP_MEM_OFFSET: {
        void *q = nullptr;
        if (rt.dnnrtMemOffset(&q, ptr[(size_t)op->operands[0]->id], op->offset, op->bytes)) { err = rt_error("dnnrtMemOffset"); ok = false; }
        ptr[(size_t)op->result->id] = q;
        if (ok && debug_fill >= 0 && rt.dnnrtMemFill(q, debug_fill, op->bytes, stream)) { err = rt_error("dnnrtMemFill"); ok = false; }
        break;
      }
      case OP_MEMCPY:
        if (rt.dnnrtMemcpy(ptr[(size_t)op->operands[0]->id], ptr[(size_t)op->operands[1]->id], op->bytes, (int32_t)op->mode, stream)) {
          err = rt_error("dnnrtMemcpy"); ok = false;
        }
        break;
      case OP_DEALLOC:  // only the pool's own release survives the pool pass
        if (rt.dnnrtSync(handle)) { err = rt_error("dnnrtSync"); ok = false; }
        if (rt.dnnrtDealloc(ptr[(size_t)op->operands[0]->id])) { err = rt_error("dnnrtDealloc"); ok = false; }
        run_pool = nullptr;
        break;
      case OP_HOST_CONST: case OP_HOST_ALLOC: case OP_RETURN: break;
      default: ok = issue(op, err); break;
    }
    if (!ok) break;
  }
  if (!ok) {
    rt.dnnrtSync(handle);
    if (run_pool) rt.dnnrtDealloc(run_pool);
    return false;
  }
  const Op *ret = prog->ops.back();
  for (size_t i = 0; i < ret->operands.size(); i++) {
    const Value *v = ret->operands[i];
    std::memcpy(outputs[i], ptr[(size_t)v->id], (size_t)(shape_numel(v->shape) * dtype_bytes(v->dtype)));
  }
  return true;
}

bool Session::issue_all_compute(std::string &err) {
  for (const Op *op : prog->ops) {
    if (is_compute(op->kind)) {
      if (!issue(op, err)) return false;
    } else if (op->kind == OP_MEMCPY && op->mode == 2) {
      auto st = staged_out.find(op);
      if (st == staged_out.end()) continue;
      // a copy kernel, so that a captured graph holds it too
      const Value *v = op->operands[1];
      const int64_t n = shape_numel(v->shape);
      if (!rt.dnnrtReshape(handle, ptr[(size_t)v->id], &n, 1, st->second, (int32_t)v->dtype)) {
        err = rt_error("dnnrtReshape(result staging)");
        return false;
      }
    }
  }
  return true;
}

// Resident inference.  `on_device` != 0: inputs/outputs are device pointers and
// the call returns without waiting (sync() does).
bool Session::run_resident(const void *const *inputs, void *const *outputs, int on_device, int use_graph, std::string &err) {
  const bool borrow = on_device == 2 && !host_backend;
  auto other_slot = [&](const Op *op) -> size_t {  // the pool tensor behind a result copy (see below)
    const Value *v = op->operands[1];
    if (v->def && v->def->kind == OP_MEM_OFFSET) return (size_t)v->id;
    return (size_t)v->def->operands.back()->id;
  };
  // The pool reuses the inputs' slots for later tensors, so every pass over
  // the kernels must be preceded by a fresh copy of the inputs.
  auto copy_inputs = [&]() -> bool {
    if (borrow) return true;
    for (const Op *op : prog->ops) {
      if (op->kind != OP_MEMCPY || op->mode != 1) continue;
      const Value *src = op->operands[1];
      if (src->arg_index < 0) continue;
      const size_t ai = (size_t)src->arg_index;
      const void *from = inputs[ai];
      if (!on_device) { std::memcpy(host_in[ai], inputs[ai], (size_t)op->bytes); from = host_in[ai]; }
      if (rt.dnnrtMemcpy(ptr[(size_t)op->operands[0]->id], const_cast<void *>(from), op->bytes, on_device ? 3 : 1, stream)) {
        err = rt_error("dnnrtMemcpy(input)"); return false;
      }
    }
    return true;
  };
  // on_device == 2: the kernels read the caller's input buffers where they are (no copy into the pool slots).  The
  // argument slots' values point at those buffers for as long as the caller keeps passing the same addresses; a
  // recorded graph holds them, so a change of address drops it.
  {
    bool moved = false;
    for (const Op *op : prog->ops) {
      if (op->kind != OP_MEMCPY || op->mode != 1 || op->operands[1]->arg_index < 0) continue;
      const size_t slot = (size_t)op->operands[0]->id;
      if (!arg_home.count(slot)) arg_home[slot] = ptr[slot];
      void *want = borrow ? const_cast<void *>(inputs[(size_t)op->operands[1]->arg_index]) : arg_home[slot];
      if (ptr[slot] != want) { ptr[slot] = want; moved = true; }
    }
    // The same for the results: the pool tensor a result is computed into (the output operand of the operation
    // that produces it) points at the caller's result buffer, so the last kernel writes there and no copy
    // follows.  Only that one tensor value moves: whatever else the planner put at the same pool offset at other
    // times stays in the pool, and a copy-type operation that would have aliased it copies instead.
    direct_out.clear();
    for (const Op *op : prog->ops) {
      if (op->kind != OP_MEMCPY || op->mode != 2 || staged_out.count(op)) continue;
      const Value *v = op->operands[1], *bv = nullptr;
      if (v->def && v->def->kind == OP_MEM_OFFSET) bv = v;
      else if (v->def && is_compute(v->def->kind) && !v->def->operands.empty()) {
        const Value *o = v->def->operands.back();
        if (o->def && o->def->kind == OP_MEM_OFFSET) bv = o;
      }
      if (!bv) continue;
      const size_t slot = (size_t)bv->id;
      // A second result out of one tensor, or a tensor that is also an argument's slot, is copied after the
      // kernels as before, from wherever the first result or the argument put the tensor for this run.
      bool shared = arg_home.count(slot) != 0;
      for (const Op *other : direct_out) shared = shared || other_slot(other) == slot;
      if (shared) continue;
      if (!out_home.count(slot)) out_home[slot] = ptr[slot];
      void *want = borrow ? outputs[(size_t)op->operands[0]->def->out_index] : out_home[slot];
      if (ptr[slot] != want) { ptr[slot] = want; moved = true; }
      if (borrow) direct_out.push_back(op);
    }
    // the addresses this run's kernels see: the key of its graph
    std::vector<void *> key;
    for (const auto &h : arg_home) key.push_back(ptr[h.first]);
    for (const auto &h : out_home) key.push_back(ptr[h.first]);
    if (moved || key != graph_key) {
      if (graph) {  // park the current one, take back the one recorded with these addresses if there is one
        parked_graphs.emplace_back(graph_key, graph);
        graph = nullptr;
        if (parked_graphs.size() > 4) { rt.dnnrtGraphDestroy(parked_graphs.front().second); parked_graphs.erase(parked_graphs.begin()); }
      }
      for (size_t i = 0; i < parked_graphs.size(); i++)
        if (parked_graphs[i].first == key) { graph = parked_graphs[i].second; parked_graphs.erase(parked_graphs.begin() + (long)i); break; }
      graph_key = key;
    }
  }
  // A graph launch costs the host about as much as half a dozen kernel launches: a program of up to three kernels
  // (the single convolution block: 19 us per pass replayed, 8 us launched directly) is issued as it is.
  int launching = 0;
  for (const Op *op : prog->ops) launching += launches(op) ? 1 : 0;
  const bool graphed = use_graph && !host_backend && launching > 3;
  if (graphed && !graph) {
    // One eager pass on real data first: it validates every call outside of
    // capture.  Then the same call sequence is recorded (nothing runs).
    if (!copy_inputs() || !issue_all_compute(err)) return false;
    if (rt.dnnrtSync(handle)) { err = rt_error("dnnrtSync"); return false; }
    if (rt.dnnrtGraphBegin(handle)) { err = rt_error("dnnrtGraphBegin"); return false; }
    const bool ok = issue_all_compute(err);
    void *g = nullptr;
    if (rt.dnnrtGraphEnd(handle, &g)) { if (ok) err = rt_error("dnnrtGraphEnd"); return false; }
    if (!ok) { rt.dnnrtGraphDestroy(g); return false; }
    graph = g;
  }
  // 1. inputs into their pool slots  2. kernels
  if (!copy_inputs()) return false;
  if (graphed) {
    if (rt.dnnrtGraphLaunch(handle, graph)) { err = rt_error("dnnrtGraphLaunch"); return false; }
  } else {
    if (!issue_all_compute(err)) return false;
  }
  // 3. outputs
  for (const Op *op : prog->ops) {
    if (op->kind != OP_MEMCPY || op->mode != 2) continue;
    if (std::find(direct_out.begin(), direct_out.end(), op) != direct_out.end()) continue;  // written in place
    const Op *ha = op->operands[0]->def;
    const size_t oi = (size_t)ha->out_index;
    void *dst = on_device ? outputs[oi] : host_out[oi];
    auto st = staged_out.find(op);
    void *src = st != staged_out.end() ? st->second : ptr[(size_t)op->operands[1]->id];
    if (rt.dnnrtMemcpy(dst, src, op->bytes, on_device ? 3 : 2, stream)) {
      err = rt_error("dnnrtMemcpy(output)"); return false;
    }
  }
  if (!on_device) {
    if (rt.dnnrtSync(handle)) { err = rt_error("dnnrtSync"); return false; }
    for (const Op *op : prog->ops)
      if (op->kind == OP_HOST_ALLOC) std::memcpy(outputs[(size_t)op->out_index], host_out[(size_t)op->out_index], (size_t)op->bytes);
  }
  return true;
}

bool Session::profile_resident(const void *const *inputs, int on_device, bool by_class, std::vector<float> &ms, std::string &err) {
  if (mode != MODE_RESIDENT) { err = "profiling needs a resident session"; return false; }
  // profiling copies the inputs into their pool slots: argument values that point at a caller's buffers go home
  for (const auto &h : arg_home) ptr[h.first] = h.second;
  for (const auto &h : out_home) ptr[h.first] = h.second;
  direct_out.clear();
  // the operations that launch something, in program order (an aliased copy only hands its input's address on;
  // a first eager pass has set those)
  std::vector<const Op *> compute;
  for (const Op *op : prog->ops)
    if (launches(op)) compute.push_back(op);
  for (const Op *op : prog->ops)
    if (is_compute(op->kind) && !launches(op) && !ptr[(size_t)op->result->id]) {
      std::string e2;
      if (!issue_all_compute(e2)) { err = e2; return false; }
      break;
    }
  if (by_class) return profile_classes(inputs, on_device, compute, ms, err);
  std::vector<void *> ev(compute.size() + 1, nullptr);
  bool ok = true;
  for (void *&e : ev)
    if (rt.dnnrtEventCreate(&e)) { err = rt_error("dnnrtEventCreate"); ok = false; break; }
  if (ok) {
    for (const Op *op : prog->ops) {  // inputs into their pool slots
      if (op->kind != OP_MEMCPY || op->mode != 1 || op->operands[1]->arg_index < 0) continue;
      const size_t ai = (size_t)op->operands[1]->arg_index;
      const void *from = inputs[ai];
      if (!on_device) { std::memcpy(host_in[ai], inputs[ai], (size_t)op->bytes); from = host_in[ai]; }
      if (rt.dnnrtMemcpy(ptr[(size_t)op->operands[0]->id], const_cast<void *>(from), op->bytes, on_device ? 3 : 1, stream)) {
        err = rt_error("dnnrtMemcpy(input)"); ok = false; break;
      }
    }
  }
  if (ok && rt.dnnrtEventRecord(ev[0], stream)) { err = rt_error("dnnrtEventRecord"); ok = false; }
  for (size_t i = 0; ok && i < compute.size(); i++) {
    ok = issue(compute[i], err);
    if (ok && rt.dnnrtEventRecord(ev[i + 1], stream)) { err = rt_error("dnnrtEventRecord"); ok = false; }
  }
  if (rt.dnnrtSync(handle) && ok) { err = rt_error("dnnrtSync"); ok = false; }
  ms.assign(compute.size(), 0.f);
  for (size_t i = 0; ok && i < compute.size(); i++)
    if (rt.dnnrtEventElapsedMs(ev[i], ev[i + 1], &ms[i])) { err = rt_error("dnnrtEventElapsedMs"); ok = false; }
  for (void *e : ev) rt.dnnrtEventDestroy(e);
  return ok;
}

// One pair of timestamps per operation class, around all of the class's
// launches issued back to back (in program order, on whatever the buffers
// hold: only the durations matter).  A timestamp between two kernels of a few
// microseconds costs about as much as the kernels; this way the class average
// is the kernels' own duration plus the gap between consecutive dispatches
// (a repeated launch finds its operands in the caches, so a small class reads
// a little faster here than inside the whole program).
bool Session::profile_classes(const void *const *inputs, int on_device, const std::vector<const Op *> &compute,
                              std::vector<float> &ms, std::string &err) {
  std::vector<std::string> classes;
  for (const Op *op : compute) {
    const std::string c = op_class(op);
    if (std::find(classes.begin(), classes.end(), c) == classes.end()) classes.push_back(c);
  }
  bool ok = true;
  for (const Op *op : prog->ops) {  // inputs into their pool slots
    if (op->kind != OP_MEMCPY || op->mode != 1 || op->operands[1]->arg_index < 0) continue;
    const size_t ai = (size_t)op->operands[1]->arg_index;
    const void *from = inputs[ai];
    if (!on_device) { std::memcpy(host_in[ai], inputs[ai], (size_t)op->bytes); from = host_in[ai]; }
    if (rt.dnnrtMemcpy(ptr[(size_t)op->operands[0]->id], const_cast<void *>(from), op->bytes, on_device ? 3 : 1, stream)) {
      err = rt_error("dnnrtMemcpy(input)"); return false;
    }
  }
  void *e0 = nullptr, *e1 = nullptr;
  if (rt.dnnrtEventCreate(&e0) || rt.dnnrtEventCreate(&e1)) { err = rt_error("dnnrtEventCreate"); return false; }
  ms.assign(compute.size(), 0.f);
  for (size_t i = 0; ok && i < compute.size(); i++) ok = issue(compute[i], err);  // one whole pass first: real values everywhere
  for (const std::string &c : classes) {
    if (!ok) break;
    // a class of one or two launches is repeated: behind an idle stream the first dispatch alone takes
    // longer to reach the GPU than such a kernel runs
    size_t members = 0, n = 0;
    for (const Op *op : compute) members += c == op_class(op);
    const size_t reps = members >= 32 ? 1 : (32 + members - 1) / members;
    if (rt.dnnrtEventRecord(e0, stream)) { err = rt_error("dnnrtEventRecord"); ok = false; break; }
    for (size_t r = 0; ok && r < reps; r++)
      for (size_t i = 0; ok && i < compute.size(); i++)
        if (c == op_class(compute[i])) { ok = issue(compute[i], err); n++; }
    if (ok && rt.dnnrtEventRecord(e1, stream)) { err = rt_error("dnnrtEventRecord"); ok = false; }
    if (ok && rt.dnnrtSync(handle)) { err = rt_error("dnnrtSync"); ok = false; }
    float total = 0.f;
    if (ok && rt.dnnrtEventElapsedMs(e0, e1, &total)) { err = rt_error("dnnrtEventElapsedMs"); ok = false; }
    for (size_t i = 0; ok && i < compute.size(); i++)
      if (c == op_class(compute[i])) ms[i] = total / (float)n;
  }
  rt.dnnrtEventDestroy(e0);
  rt.dnnrtEventDestroy(e1);
  return ok;
}

int64_t Session::algo_operand(const Op *op, int which, int64_t reference_value) const {
  const auto it = tuned.find(op);
  const int64_t id = it == tuned.end() ? 0 : (which ? it->second.second : it->second.first);
  return id > 0 ? DNNRT_CONV_ALGO_BASE + id : reference_value;
}

static bool tunable(const Op *op) {
  return (op->kind == OP_CONVFWD || op->kind == OP_CONV_BIAS_ACTIV || op->kind == OP_CONV_BIAS_ADD_ACTIV || op->kind == OP_CONV_ADD_CONV_ACTIV) &&
         !op->operands.empty() && op->operands.back()->dtype == F16;
}

std::vector<int64_t> Session::algos() const {
  std::vector<int64_t> out;
  for (const Op *op : prog->ops) {
    if (!launches(op)) continue;
    const auto it = tuned.find(op);
    out.push_back(it == tuned.end() ? 0 : it->second.first);
    out.push_back(it == tuned.end() ? 0 : it->second.second);
  }
  return out;
}

bool Session::set_algos(const int64_t *a, int64_t n, std::string &err) {
  std::vector<const Op *> compute;
  for (const Op *op : prog->ops)
    if (launches(op)) compute.push_back(op);
  if (!a || n != 2 * (int64_t)compute.size()) { err = "set_algos: two values per operation that launches are expected"; return false; }
  tuned.clear();
  for (size_t i = 0; i < compute.size(); i++) {
    if (a[2 * i] < 0 || a[2 * i + 1] < 0 || a[2 * i] >= 1000 || a[2 * i + 1] >= 1000) { err = "set_algos: a variant id is 0 .. 999"; return false; }
    if ((a[2 * i] || a[2 * i + 1]) && tunable(compute[i])) tuned[compute[i]] = {a[2 * i], a[2 * i + 1]};
  }
  drop_graphs();
  return true;
}

bool Session::tune(const void *const *inputs, int on_device, int reps, int64_t &changed, std::string &err) {
  changed = 0;
  if (mode != MODE_RESIDENT) { err = "tuning needs a resident session"; return false; }
  std::vector<const Op *> compute;
  for (const Op *op : prog->ops)
    if (launches(op)) compute.push_back(op);
  bool any = false;
  for (const Op *op : compute) any = any || tunable(op);
  if (host_backend || !prog->channels_last || !any) return true;
  std::vector<int32_t> ids((size_t)std::max(rt.dnnrtListConvTiles(nullptr, 0), 0));
  rt.dnnrtListConvTiles(ids.data(), (int32_t)ids.size());
  reps = std::max(reps, 3);
  const std::map<const Op *, std::pair<int64_t, int64_t>> before = tuned;
  // median per operation over `reps` profiled passes with the current choices
  auto measure = [&](std::vector<float> &med) -> bool {
    std::vector<std::vector<float>> runs;
    std::vector<float> ms;
    if (!profile_resident(inputs, on_device, false, ms, err)) return false;  // one pass to settle (code, caches)
    for (int r = 0; r < reps; r++) {
      if (!profile_resident(inputs, on_device, false, ms, err)) return false;
      runs.push_back(ms);
    }
    med.assign(compute.size(), 0.f);
    for (size_t i = 0; i < compute.size(); i++) {
      std::vector<float> v;
      for (const auto &r : runs) v.push_back(r[i]);
      std::sort(v.begin(), v.end());
      med[i] = v[v.size() / 2];
    }
    return true;
  };
  bool ok = true;
  for (int which = 0; which < 2 && ok; which++) {  // 0: every operation's (first) convolution; 1: the second one of the pairs
    std::vector<const Op *> targets;
    for (const Op *op : compute)
      if (tunable(op) && (which == 0 || op->kind == OP_CONV_ADD_CONV_ACTIV)) targets.push_back(op);
    if (targets.empty()) break;
    const auto chosen = tuned;  // what this round starts from
    auto with = [&](int64_t id) {
      tuned = chosen;
      for (const Op *op : targets) {
        auto &t = tuned[op];
        (which ? t.second : t.first) = id;
      }
    };
    std::vector<float> base;
    with(0);
    ok = measure(base);
    std::vector<float> best = base;
    std::vector<int64_t> best_id(compute.size(), 0);
    for (size_t c = 0; ok && c < ids.size(); c++) {
      std::vector<float> t;
      with(ids[c]);
      ok = measure(t);
      for (size_t i = 0; ok && i < compute.size(); i++)
        if (t[i] < best[i]) { best[i] = t[i]; best_id[i] = ids[c]; }
    }
    tuned = chosen;
    for (size_t i = 0; ok && i < compute.size(); i++) {
      if (std::find(targets.begin(), targets.end(), compute[i]) == targets.end()) continue;
      auto &t = tuned[compute[i]];
      (which ? t.second : t.first) = best[i] < 0.97f * base[i] ? best_id[i] : 0;
    }
  }
  if (!ok) { tuned = before; drop_graphs(); return false; }
  for (auto it = tuned.begin(); it != tuned.end();) {
    if (!it->second.first && !it->second.second) it = tuned.erase(it);
    else { changed++; ++it; }
  }
  drop_graphs();
  return true;
}

bool Session::set_conv_tile(int tile, std::string &err) {
  if (rt.dnnrtSetConvTile(handle, tile)) { err = rt_error("dnnrtSetConvTile"); return false; }
  drop_graphs();
  return true;
}

bool Session::sync(std::string &err) {
  if (rt.dnnrtSync(handle)) { err = rt_error("dnnrtSync"); return false; }
  return true;
}

}  // namespace dnnc
