#include "../../../include/dnnc.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <sstream>

#include "exec.h"
#include "ir.h"
#include "planner.h"

using namespace dnnc;

struct dnncGraph { Graph g; bool compiled = false; };
struct dnncProgram { Program p; std::string text; };
struct dnncSession { Session s; };

static thread_local std::string g_err;
static int32_t fail(const std::string &m) { g_err = m; return 1; }

extern "C" {

const char *dnncLastError(void) { return g_err.c_str(); }

dnncGraph *dnncGraphCreate(void) { return new dnncGraph(); }
void dnncGraphDestroy(dnncGraph *g) { delete g; }

dnncGraph *dnncGraphFromOnnx(const void *bytes, int64_t nbytes) {
  if (!bytes || nbytes <= 0) { g_err = "dnncGraphFromOnnx: empty buffer"; return nullptr; }
  dnncGraph *g = new dnncGraph();
  std::string err;
  if (!graph_from_onnx((const uint8_t *)bytes, (size_t)nbytes, g->g, err)) {
    g_err = "dnncGraphFromOnnx: " + err;
    delete g;
    return nullptr;
  }
  return g;
}
int32_t dnncGraphNumInputs(const dnncGraph *g) { return g ? (int32_t)g->g.inputs.size() : 0; }
int32_t dnncGraphNumOutputs(const dnncGraph *g) { return g ? (int32_t)g->g.outputs.size() : 0; }
const char *dnncGraphInputName(const dnncGraph *g, int32_t i) {
  return (g && i >= 0 && (size_t)i < g->g.inputs.size()) ? g->g.inputs[(size_t)i].c_str() : nullptr;
}
const char *dnncGraphOutputName(const dnncGraph *g, int32_t i) {
  return (g && i >= 0 && (size_t)i < g->g.outputs.size()) ? g->g.outputs[(size_t)i].c_str() : nullptr;
}
int32_t dnncGraphInputInfo(const dnncGraph *g, int32_t i, int32_t *dtype, int32_t *rank, int64_t *dims, int32_t cap) {
  if (!g || i < 0 || (size_t)i >= g->g.inputs.size()) return fail("dnncGraphInputInfo: no such input");
  const GTensor &t = g->g.tensors.at(g->g.inputs[(size_t)i]);
  if (dtype) *dtype = (int32_t)t.dtype;
  if (rank) *rank = (int32_t)t.shape.size();
  if (dims) for (int32_t d = 0; d < cap && (size_t)d < t.shape.size(); d++) dims[d] = t.shape[(size_t)d];
  return 0;
}

static bool valid_dtype(int32_t dt) { return dt >= 0 && dt <= 2; }

int32_t dnncGraphAddInput(dnncGraph *g, const char *name, int32_t dtype, int32_t rank, const int64_t *dims) {
  if (!g || !name || !valid_dtype(dtype) || rank < 0 || (rank > 0 && !dims)) return fail("dnncGraphAddInput: bad arguments");
  if (g->g.tensors.count(name)) return fail(std::string("tensor '") + name + "' already defined");
  GTensor t;
  t.name = name; t.dtype = (DType)dtype; t.shape.assign(dims, dims + rank); t.is_input = true;
  for (int64_t d : t.shape) if (d <= 0) return fail("dnncGraphAddInput: dims must be positive");
  g->g.tensors[name] = t;
  g->g.inputs.push_back(name);
  return 0;
}

int32_t dnncGraphAddConstant(dnncGraph *g, const char *name, int32_t dtype, int32_t rank, const int64_t *dims, const void *data) {
  if (!g || !name || !valid_dtype(dtype) || rank < 0 || (rank > 0 && !dims) || !data) return fail("dnncGraphAddConstant: bad arguments");
  if (g->g.tensors.count(name)) return fail(std::string("tensor '") + name + "' already defined");
  GTensor t;
  t.name = name; t.dtype = (DType)dtype; t.shape.assign(dims, dims + rank); t.is_const = true;
  for (int64_t d : t.shape) if (d < 0) return fail("dnncGraphAddConstant: negative dim");
  const size_t bytes = (size_t)(shape_numel(t.shape) * dtype_bytes(t.dtype));
  t.data.assign((const uint8_t *)data, (const uint8_t *)data + bytes);
  g->g.tensors[name] = std::move(t);
  GNode n;
  n.op_type = "Constant";
  n.output = name;
  g->g.nodes.push_back(n);
  return 0;
}

int32_t dnncGraphAddNode(dnncGraph *g, const char *op_type, int32_t n_inputs, const char *const *inputs, const char *output, const char *attrs) {
  if (!g || !op_type || !output || n_inputs < 0 || (n_inputs > 0 && !inputs)) return fail("dnncGraphAddNode: bad arguments");
  GNode n;
  n.op_type = op_type;
  n.output = output;
  for (int i = 0; i < n_inputs; i++) n.inputs.push_back(inputs[i] ? inputs[i] : "");
  if (attrs && *attrs) {
    std::stringstream ss(attrs);
    std::string item;
    while (std::getline(ss, item, ';')) {
      if (item.empty()) continue;
      const size_t eq = item.find('=');
      if (eq == std::string::npos) return fail("dnncGraphAddNode: attribute without '=': " + item);
      const std::string key = item.substr(0, eq), val = item.substr(eq + 1);
      if (val.find_first_of(".eEn") != std::string::npos && val.find(',') == std::string::npos) {
        n.floats[key] = std::strtod(val.c_str(), nullptr);
      } else {
        std::vector<int64_t> v;
        std::stringstream vs(val);
        std::string tok;
        while (std::getline(vs, tok, ',')) if (!tok.empty()) v.push_back(std::strtoll(tok.c_str(), nullptr, 10));
        n.ints[key] = v;
      }
    }
  }
  g->g.nodes.push_back(n);
  return 0;
}

int32_t dnncGraphAddOutput(dnncGraph *g, const char *name) {
  if (!g || !name) return fail("dnncGraphAddOutput: bad arguments");
  g->g.outputs.push_back(name);
  return 0;
}

dnncProgram *dnncCompile(dnncGraph *g, const dnncOptions *opt) {
  if (!g || !opt) { g_err = "dnncCompile: bad arguments"; return nullptr; }
  if (g->compiled) { g_err = "dnncCompile: a graph can be compiled once"; return nullptr; }
  std::string err;
  if (!infer_shapes(g->g, opt->recompose != 0, opt->fuse_attention != 0, err)) { g_err = err; return nullptr; }
  if (opt->const_at_use) constant_at_use(g->g);
  g->compiled = true;
  dnncProgram *pp = new dnncProgram();
  Program &p = pp->p;
  if (!emit_program(g->g, p, err)) { g_err = err; delete pp; return nullptr; }
  func_args_to_device(p);
  erase_dummy_constants(p);
  p.channels_last_requested = opt->channels_last != 0;
  if (opt->fusion) fuse_conv_bias_activ(p);
  if (opt->fusion && opt->fuse_activations) fuse_conv_activations(p);
  if (opt->fusion && opt->fuse_matmul_bias) fuse_matmul_bias(p);
  if (opt->fusion && opt->fuse_residual) fuse_residual_add(p);
  if (opt->fusion && opt->fuse_first_layer_maxpool) fuse_first_layer_maxpool(p);
  if (opt->fusion && opt->fuse_residual && opt->fuse_projection_shortcut) fuse_projection_shortcut(p);
  if (opt->alias_copies) alias_copies(p);
  if (opt->fusion && opt->fuse_residual && opt->inplace_residual) inplace_residual(p);
  if (opt->dealloc_opt) dealloc_opt(p);
  if (opt->channels_last) {
    // Only fp16 programs whose rank-4 tensors flow through layout-aware calls
    // can be kept channels-last.
    for (const Op *op : p.ops) {
      if (!op->result || op->kind == OP_HOST_CONST) continue;
      const bool r4 = op->result->shape.size() == 4 && op->result->shape[2] * op->result->shape[3] > 1;
      if (!r4) continue;
      if (op->result->dtype != F16) { g_err = "channels_last needs an fp16 graph"; delete pp; return nullptr; }
      switch (op->kind) {
        case OP_MALLOC: case OP_HOST_ALLOC: case OP_CONVFWD: case OP_CONV_BIAS_ACTIV: case OP_CONV_BIAS_ADD_ACTIV: case OP_CONV_BIAS_ACTIV_MAXPOOL:
        case OP_CONV_ADD_CONV_ACTIV: case OP_ACTIVATION: case OP_ADD:
        case OP_MUL: case OP_MAXPOOL: case OP_AVGPOOL: case OP_CLIP: case OP_REDUCE: case OP_LEAKYRELU: case OP_PRELU:
        case OP_CONCAT: break;
        default: g_err = std::string("channels_last: ") + op_name(op->kind) + " has no channels-last form"; delete pp; return nullptr;
      }
      if (op->kind == OP_HOST_ALLOC) { g_err = "channels_last: a returned rank-4 tensor would come back in NHWC order"; delete pp; return nullptr; }
    }
    // Operands: a rank-4 tensor with spatial extent may be read only by a call that has a channels-last form
    // (a Flatten or Reshape of it would copy NHWC bytes under an NCHW shape), and a constant of that kind is
    // uploaded as the graph holds it, N,C,H,W: only convolution filters are re-laid (K,R,S,C) at upload.
    auto spatial4 = [](const Value *v) { return v->shape.size() == 4 && v->shape[2] * v->shape[3] > 1; };
    auto holds_constant = [](const Value *v) {
      for (const auto &u : v->uses)
        if (u.first->kind == OP_MEMCPY && u.first->mode == 1 && u.second == 0 && u.first->operands[1]->def &&
            u.first->operands[1]->def->kind == OP_HOST_CONST)
          return true;
      return false;
    };
    for (const Op *op : p.ops) {
      bool layout_aware = false, conv = false;
      switch (op->kind) {
        case OP_CONVFWD: case OP_CONV_BIAS_ACTIV: case OP_CONV_BIAS_ADD_ACTIV: case OP_CONV_BIAS_ACTIV_MAXPOOL: case OP_CONV_ADD_CONV_ACTIV:
          conv = true; layout_aware = true; break;
        case OP_ACTIVATION: case OP_ADD: case OP_MUL: case OP_MAXPOOL: case OP_AVGPOOL: case OP_CLIP: case OP_REDUCE:
        case OP_LEAKYRELU: case OP_PRELU: case OP_CONCAT: layout_aware = true; break;
        case OP_MALLOC: case OP_DEALLOC: case OP_MEMCPY: case OP_HOST_CONST: case OP_HOST_ALLOC: case OP_RETURN: continue;
        default: break;
      }
      for (size_t i = 0; i + 1 < op->operands.size(); i++) {  // the last operand is the output buffer (checked above)
        const Value *v = op->operands[i];
        if (!spatial4(v)) continue;
        if (!layout_aware) {
          g_err = std::string("channels_last: ") + op_name(op->kind) + " reads a rank-4 tensor with spatial extent and has no channels-last form";
          delete pp; return nullptr;
        }
        if (holds_constant(v) && !(conv && (i == 1 || (op->kind == OP_CONV_ADD_CONV_ACTIV && i == 5)))) {
          g_err = std::string("channels_last: a rank-4 constant with spatial extent feeds ") + op_name(op->kind) +
                  ", which would read its N,C,H,W bytes as N,H,W,C";
          delete pp; return nullptr;
        }
      }
    }
    // the NCHW function arguments may feed convolutions only
    for (const Op *op : p.ops)
      if (op->kind == OP_MEMCPY && op->mode == 1 && op->operands[1]->arg_index >= 0 && op->operands[0]->shape.size() == 4)
        for (const auto &u : op->operands[0]->uses)
          if (u.first->kind != OP_MEMCPY && u.first->kind != OP_DEALLOC && u.first->kind != OP_CONVFWD && u.first->kind != OP_CONV_BIAS_ACTIV &&
              !(u.first->kind == OP_CONV_BIAS_ACTIV_MAXPOOL && u.second == 0) &&
              !(u.first->kind == OP_CONV_BIAS_ADD_ACTIV && u.second == 0)) {
            g_err = "channels_last: a rank-4 function argument may only feed convolutions"; delete pp; return nullptr;
          }
    p.channels_last = true;
  }
  if (opt->pool_opt && !malloc_pool_opt(p, err, opt->compact_pool != 0)) { g_err = err; delete pp; return nullptr; }
  return pp;
}

void dnncProgramDestroy(dnncProgram *p) { delete p; }

const char *dnncProgramText(dnncProgram *p) {
  if (!p) return "";
  p->text = p->p.to_text();
  return p->text.c_str();
}

int64_t dnncProgramPoolBytes(const dnncProgram *p) { return p ? p->p.pool_bytes : -1; }
int64_t dnncProgramPoolExtent(const dnncProgram *p) { return p ? p->p.pool_extent : -1; }

int64_t dnncProgramEvents(const dnncProgram *p, int32_t *kind, int64_t *id, int64_t *bytes, int64_t *offset, int64_t cap) {
  if (!p) return -1;
  int64_t n = 0;
  auto put = [&](int32_t k, int64_t i, int64_t b, int64_t o) {
    if (n < cap && kind && id && bytes && offset) { kind[n] = k; id[n] = i; bytes[n] = b; offset[n] = o; }
    n++;
  };
  if (p->p.pool_bytes >= 0) {
    for (const PoolEvent &e : p->p.trace) put(e.kind, e.id, e.bytes, e.offset);
  } else {
    for (const PoolEvent &e : pool_events(p->p)) put(e.kind, e.id, e.bytes, e.offset);
  }
  return n;
}

int32_t dnncProgramNumInputs(const dnncProgram *p) { return p ? (int32_t)p->p.args.size() : -1; }
int32_t dnncProgramNumOutputs(const dnncProgram *p) { return p ? (int32_t)p->p.out_names.size() : -1; }

int32_t dnncProgramOutputInfo(const dnncProgram *p, int32_t i, int32_t *dtype, int32_t *rank, int64_t *dims) {
  if (!p || i < 0 || (size_t)i >= p->p.out_names.size()) return fail("dnncProgramOutputInfo: bad index");
  const Value *v = p->p.ops.back()->operands[(size_t)i];
  if (v->shape.size() > 8) return fail("dnncProgramOutputInfo: rank above 8");
  *dtype = (int32_t)v->dtype;
  *rank = (int32_t)v->shape.size();
  for (size_t d = 0; d < v->shape.size(); d++) dims[d] = v->shape[d];
  return 0;
}

int64_t dnncProgramNumOps(const dnncProgram *p, int32_t compute_only) {
  if (!p) return -1;
  int64_t n = 0;
  for (const Op *op : p->p.ops)
    if (!compute_only || launches(op)) n++;
  return n;
}

int32_t dnncProgramComputeOp(const dnncProgram *p, int64_t i, const char **name, const char **work_class, double *flops, double *bytes) {
  if (!p || !name || !work_class || !flops || !bytes) return fail("dnncProgramComputeOp: bad arguments");
  int64_t n = 0;
  for (const Op *op : p->p.ops) {
    if (!launches(op)) continue;
    if (n++ != i) continue;
    *name = op_name(op->kind);
    *work_class = op_class(op);
    op_work(op, *flops, *bytes);
    return 0;
  }
  return fail("dnncProgramComputeOp: index out of range");
}

int64_t dnncPlanPool(int64_t n, const int32_t *kind, const int64_t *id, const int64_t *bytes, int64_t *offset) {
  PoolSimulator sim;
  for (int64_t i = 0; i < n; i++) {
    if (kind[i] == 0) {
      offset[i] = sim.reserve(id[i], PoolSimulator::round_size(bytes[i]));
      if (offset[i] < 0) return -1;
    } else {
      offset[i] = -1;
      if (!sim.release(id[i])) return -1;
    }
  }
  return sim.peak();
}

int64_t dnncPlanFreeList(int64_t n, const int32_t *kind, const int64_t *id, const int64_t *bytes, int64_t upto, int64_t *out, int64_t cap) {
  PoolSimulator sim;
  for (int64_t i = 0; i <= upto && i < n; i++) {
    if (kind[i] == 0) sim.reserve(id[i], PoolSimulator::round_size(bytes[i]));
    else sim.release(id[i]);
  }
  const auto fl = sim.free_list();
  for (size_t i = 0; i < fl.size() && (int64_t)i < cap; i++) { out[2 * i] = fl[i].first; out[2 * i + 1] = fl[i].second; }
  return (int64_t)fl.size();
}

dnncSession *dnncSessionCreate(dnncProgram *p, const char *runtime_library, int32_t mode) {
  if (!p || !runtime_library || (mode != DNNC_MODE_OCCAMY && mode != DNNC_MODE_RESIDENT)) { g_err = "dnncSessionCreate: bad arguments"; return nullptr; }
  dnncSession *s = new dnncSession();
  std::string err;
  if (!s->s.init(&p->p, runtime_library, mode, err)) { g_err = err; delete s; return nullptr; }
  return s;
}

void dnncSessionDestroy(dnncSession *s) { delete s; }

int32_t dnncSessionRun(dnncSession *s, const void *const *inputs, void *const *outputs) {
  if (!s || !inputs || !outputs) return fail("dnncSessionRun: bad arguments");
  std::string err;
  const bool ok = s->s.mode == MODE_OCCAMY ? s->s.run_occamy(inputs, outputs, err) : s->s.run_resident(inputs, outputs, 0, 0, err);
  return ok ? 0 : fail(err);
}

int32_t dnncSessionRunResident(dnncSession *s, const void *const *inputs, void *const *outputs, int32_t on_device, int32_t use_graph) {
  if (!s || !inputs || !outputs) return fail("dnncSessionRunResident: bad arguments");
  if (s->s.mode != MODE_RESIDENT) return fail("dnncSessionRunResident: the session was created in occamy mode");
  std::string err;
  return s->s.run_resident(inputs, outputs, on_device, use_graph, err) ? 0 : fail(err);
}

int32_t dnncSessionSync(dnncSession *s) {
  if (!s) return fail("dnncSessionSync: null session");
  std::string err;
  return s->s.sync(err) ? 0 : fail(err);
}

int32_t dnncSessionSetDebugFill(dnncSession *s, int32_t byte) {
  if (!s || byte < -1 || byte > 255) return fail("dnncSessionSetDebugFill: bad arguments");
  s->s.debug_fill = byte;
  return 0;
}

int32_t dnncSessionSetConvTile(dnncSession *s, int32_t tile) {
  if (!s) return fail("dnncSessionSetConvTile: null session");
  std::string err;
  return s->s.set_conv_tile(tile, err) ? 0 : fail(err);
}

int64_t dnncSessionTune(dnncSession *s, const void *const *inputs, int32_t on_device, int32_t reps) {
  if (!s || !inputs) { fail("dnncSessionTune: bad arguments"); return -1; }
  std::string err;
  int64_t changed = 0;
  if (!s->s.tune(inputs, on_device, reps, changed, err)) { fail(err); return -1; }
  return changed;
}

int64_t dnncSessionGetAlgos(const dnncSession *s, int64_t *algos, int64_t cap) {
  if (!s) { fail("dnncSessionGetAlgos: null session"); return -1; }
  const std::vector<int64_t> a = s->s.algos();
  for (size_t i = 0; algos && i < a.size() && (int64_t)i < cap; i++) algos[i] = a[i];
  return (int64_t)a.size();
}

int32_t dnncSessionSetAlgos(dnncSession *s, const int64_t *algos, int64_t n) {
  if (!s) return fail("dnncSessionSetAlgos: null session");
  std::string err;
  return s->s.set_algos(algos, n, err) ? 0 : fail(err);
}

int64_t dnncSessionProfile(dnncSession *s, const void *const *inputs, int32_t on_device, float *ms, int64_t cap) {
  if (!s || !inputs) { fail("dnncSessionProfile: bad arguments"); return -1; }
  std::vector<float> t;
  std::string err;
  if (!s->s.profile_resident(inputs, on_device & 1, (on_device & 2) != 0, t, err)) { fail(err); return -1; }
  for (size_t i = 0; i < t.size() && (int64_t)i < cap && ms; i++) ms[i] = t[i];
  return (int64_t)t.size();
}

int64_t dnncSessionWeightsBytes(const dnncSession *s) { return s ? s->s.weights_bytes : -1; }
int64_t dnncSessionLastPoolBytes(const dnncSession *s) { return s ? s->s.last_pool_bytes : -1; }
int32_t dnncSessionDeviceBytes(const dnncSession *s, int64_t *allocated_now, int64_t *allocated_peak, int64_t *static_bytes, int32_t reset_peak) {
  if (!s) { g_err = "dnncSessionDeviceBytes: no session"; return 1; }
  return s->s.device_bytes(allocated_now, allocated_peak, static_bytes, reset_peak);
}

}  // extern "C"
