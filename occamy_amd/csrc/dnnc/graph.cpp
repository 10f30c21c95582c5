// ONNX-level graph: shape inference for the operator subset the DNN dialect
// covers, and the ONNX-level rewrites that shape the event trace:
// GlobalAveragePool -> ReduceMean over (H, W), Identity / inference-mode
// Dropout removal and inference-mode BatchNormalization folded into the
// preceding convolution or turned into Mul + Add (all done by onnx-mlir's
// canonicalisation ahead of the reference's own passes), and "constant at
// use" (src/Transform/ONNX/ONNXConstantAtUsePass.cpp:29-58).
#include <algorithm>
#include <cmath>
#include <cstring>

#include "ir.h"

namespace dnnc {

static bool get_ints(const GNode &n, const char *key, std::vector<int64_t> &out) {
  auto it = n.ints.find(key);
  if (it == n.ints.end()) return false;
  out = it->second;
  return true;
}
static int64_t get_int(const GNode &n, const char *key, int64_t dflt) {
  auto it = n.ints.find(key);
  return (it == n.ints.end() || it->second.empty()) ? dflt : it->second[0];
}

static bool broadcast_shape(const Shape &a, const Shape &b, Shape &out) {
  const size_t r = std::max(a.size(), b.size());
  out.assign(r, 1);
  for (size_t i = 0; i < r; i++) {
    const int64_t da = i < r - a.size() ? 1 : a[i - (r - a.size())];
    const int64_t db = i < r - b.size() ? 1 : b[i - (r - b.size())];
    if (da != db && da != 1 && db != 1) return false;
    out[i] = std::max(da, db);
  }
  return true;
}

// ---- float <-> stored element, for constants rewritten at compile time
static float half_to_float(uint16_t h) {
  const int s = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  const float v = e == 0 ? std::ldexp((float)m, -24) : e == 31 ? (m ? NAN : INFINITY) : std::ldexp((float)(m + 1024), e - 25);
  return s ? -v : v;
}
static uint16_t float_to_half(float f) {  // round to nearest even
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7FFFFFFFu;
  if (x >= 0x7F800000u) return (uint16_t)(sign | (x > 0x7F800000u ? 0x7E00u : 0x7C00u));
  if (x >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);  // rounds to >= 65520: infinity
  if (x < 0x33000001u) return (uint16_t)sign;                // below half of the smallest subnormal
  const int e = (int)(x >> 23) - 127;
  uint32_t m = (x & 0x7FFFFFu) | 0x800000u;
  int shift = e < -14 ? 13 + (-14 - e) : 13;
  uint32_t q = m >> shift;
  const uint32_t rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1))) q++;
  // q carries the implicit one for normals; adding the exponent field lets a carry ripple into it
  const uint32_t h = e < -14 ? q : ((uint32_t)(e + 15 - 1) << 10) + q;
  return (uint16_t)(sign | h);
}
static double load_elem(const GTensor &t, int64_t i) {
  if (t.dtype == F32) { float v; std::memcpy(&v, t.data.data() + i * 4, 4); return v; }
  if (t.dtype == F16) { uint16_t h; std::memcpy(&h, t.data.data() + i * 2, 2); return half_to_float(h); }
  int64_t v; std::memcpy(&v, t.data.data() + i * 8, 8); return (double)v;
}
static void store_elem(GTensor &t, int64_t i, double v) {
  if (t.dtype == F32) { const float f = (float)v; std::memcpy(t.data.data() + i * 4, &f, 4); }
  else if (t.dtype == F16) { const uint16_t h = float_to_half((float)v); std::memcpy(t.data.data() + i * 2, &h, 2); }
  else { const int64_t q = (int64_t)v; std::memcpy(t.data.data() + i * 8, &q, 8); }
}

static int count_uses(const Graph &g, const std::string &name) {
  int n = 0;
  for (const GNode &m : g.nodes)
    for (const std::string &i : m.inputs) n += i == name;
  for (const std::string &o : g.outputs) n += o == name;
  return n;
}

// Identity and inference-mode Dropout forward their input: later nodes read
// the input directly.  One that produces a graph output stays, as a copy.
static void forward_aliases(Graph &g) {
  std::map<std::string, std::string> alias;
  std::vector<GNode> kept;
  for (GNode &n : g.nodes) {
    for (std::string &i : n.inputs) {
      auto it = alias.find(i);
      if (it != alias.end()) i = it->second;
    }
    bool fwd = (n.op_type == "Identity" || n.op_type == "Dropout") && !n.inputs.empty() && !n.inputs[0].empty();
    if (n.op_type == "Pad" && n.inputs.size() >= 2 && !n.inputs[0].empty()) {
      // Ops/cuda/Pad.cpp:33-55: a Pad whose constant pads are zero is its input; any other Pad is refused
      auto it = g.tensors.find(n.inputs[1]);
      if (it != g.tensors.end() && it->second.is_const && it->second.dtype == I64) {
        const int64_t *p = reinterpret_cast<const int64_t *>(it->second.data.data());
        fwd = true;
        for (size_t k = 0; k < it->second.data.size() / 8; k++) fwd = fwd && p[k] == 0;
      }
    }
    if (fwd && std::find(g.outputs.begin(), g.outputs.end(), n.output) == g.outputs.end()) {
      alias[n.output] = n.inputs[0];
      continue;
    }
    if (fwd) { n.op_type = "Identity"; n.inputs.resize(1); }
    kept.push_back(n);
  }
  g.nodes.swap(kept);
}

// BatchNormalization with constant statistics at g.nodes[at] (shapes are
// known):  y = x * s[c] + t[c],  s = scale / sqrt(var + eps),  t = bias - mean * s.
// Folded into the producing Conv when x has no other reader (w' = w * s[k],
// b' = b * s + t), else replaced by Mul and Add with [C,1,..] constants.
static bool rewrite_batchnorm(Graph &g, size_t at, std::string &err) {
  const GNode bn = g.nodes[at];
  auto fail = [&](const std::string &m) { err = "BatchNormalization '" + bn.output + "': " + m; return false; };
  if (bn.inputs.size() < 5) return fail("needs X, scale, B, mean and var");
  const GTensor *c[4];
  for (int i = 0; i < 4; i++) {
    auto it = g.tensors.find(bn.inputs[(size_t)i + 1]);
    if (it == g.tensors.end() || !it->second.is_const) return fail("scale, B, mean and var must be constants (inference mode)");
    c[i] = &it->second;
  }
  const GTensor x = g.tensors.at(bn.inputs[0]);
  if (x.shape.size() < 2) return fail("input rank < 2");
  const int64_t C = x.shape[1];
  for (int i = 0; i < 4; i++)
    if (shape_numel(c[i]->shape) != C || c[i]->dtype == I64) return fail("statistics must be float tensors with one entry per channel");
  auto ef = bn.floats.find("epsilon");
  const double eps = ef == bn.floats.end() ? 1e-5 : ef->second;
  std::vector<double> s((size_t)C), t((size_t)C);
  for (int64_t k = 0; k < C; k++) {
    s[(size_t)k] = load_elem(*c[0], k) / std::sqrt(load_elem(*c[3], k) + eps);
    t[(size_t)k] = load_elem(*c[1], k) - load_elem(*c[2], k) * s[(size_t)k];
  }
  auto new_const = [&](const std::string &name, DType dt, const Shape &shape) -> GTensor & {
    GTensor ct;
    ct.name = name; ct.dtype = dt; ct.shape = shape; ct.is_const = true;
    ct.data.assign((size_t)(shape_numel(shape) * dtype_bytes(dt)), 0);
    return g.tensors[name] = ct;
  };
  auto const_node = [](const std::string &name) { GNode cn; cn.op_type = "Constant"; cn.output = name; return cn; };
  size_t prod = at;  // the producer of x
  for (size_t i = 0; i < at; i++)
    if (g.nodes[i].output == bn.inputs[0]) prod = i;
  bool fold = prod != at && g.nodes[prod].op_type == "Conv" && count_uses(g, bn.inputs[0]) == 1;
  if (fold) {
    const GNode &cv = g.nodes[prod];
    auto wt = g.tensors.find(cv.inputs[1]);
    fold = wt != g.tensors.end() && wt->second.is_const && wt->second.dtype != I64 && wt->second.shape.size() == 4 && wt->second.shape[0] == C;
    if (fold && cv.inputs.size() > 2 && !cv.inputs[2].empty()) {
      auto bt = g.tensors.find(cv.inputs[2]);
      fold = bt != g.tensors.end() && bt->second.is_const && shape_numel(bt->second.shape) == C;
    }
  }
  std::vector<std::string> maybe_dead{bn.inputs[1], bn.inputs[2], bn.inputs[3], bn.inputs[4]};
  std::vector<GNode> fresh;  // what replaces the BN node (and, when folding, precedes the conv)
  if (fold) {
    const GNode cv = g.nodes[prod];
    const GTensor w = g.tensors.at(cv.inputs[1]);
    const bool has_b = cv.inputs.size() > 2 && !cv.inputs[2].empty();
    const GTensor b = has_b ? g.tensors.at(cv.inputs[2]) : GTensor();
    const std::string wn = bn.output + "_folded_w", bname = bn.output + "_folded_b";
    if (g.tensors.count(wn) || g.tensors.count(bname)) return fail("name clash with a folded constant");
    GTensor &nw = new_const(wn, w.dtype, w.shape);
    const int64_t per_k = shape_numel(w.shape) / C;
    for (int64_t k = 0; k < C; k++)
      for (int64_t j = 0; j < per_k; j++) store_elem(nw, k * per_k + j, load_elem(w, k * per_k + j) * s[(size_t)k]);
    GTensor &nb = new_const(bname, w.dtype, {C});
    for (int64_t k = 0; k < C; k++) store_elem(nb, k, (has_b ? load_elem(b, k) : 0.0) * s[(size_t)k] + t[(size_t)k]);
    maybe_dead.push_back(cv.inputs[1]);
    if (has_b) maybe_dead.push_back(cv.inputs[2]);
    g.nodes.erase(g.nodes.begin() + (long)at);
    GNode &conv = g.nodes[prod];
    conv.inputs.resize(3);
    conv.inputs[1] = wn;
    conv.inputs[2] = bname;
    conv.output = bn.output;
    g.nodes.insert(g.nodes.begin() + (long)prod, const_node(bname));
    g.nodes.insert(g.nodes.begin() + (long)prod, const_node(wn));
  } else {
    Shape cs(x.shape.size() - 1, 1);
    cs[0] = C;
    const std::string sn = bn.output + "_bn_scale", tn = bn.output + "_bn_shift", mid = bn.output + "_bn_scaled";
    if (g.tensors.count(sn) || g.tensors.count(tn) || g.tensors.count(mid)) return fail("name clash with a derived constant");
    GTensor &st = new_const(sn, x.dtype, cs);
    for (int64_t k = 0; k < C; k++) store_elem(st, k, s[(size_t)k]);
    GTensor &tt = new_const(tn, x.dtype, cs);
    for (int64_t k = 0; k < C; k++) store_elem(tt, k, t[(size_t)k]);
    GNode mul, add;
    mul.op_type = "Mul"; mul.inputs = {bn.inputs[0], sn}; mul.output = mid;
    add.op_type = "Add"; add.inputs = {mid, tn}; add.output = bn.output;
    g.nodes[at] = add;
    g.nodes.insert(g.nodes.begin() + (long)at, mul);
    g.nodes.insert(g.nodes.begin() + (long)at, const_node(tn));
    g.nodes.insert(g.nodes.begin() + (long)at, const_node(sn));
  }
  // constants that fed only the replaced nodes go away with them
  for (const std::string &d : maybe_dead) {
    if (count_uses(g, d) != 0) continue;
    for (size_t j = 0; j < g.nodes.size(); j++)
      if (g.nodes[j].op_type == "Constant" && g.nodes[j].output == d) { g.nodes.erase(g.nodes.begin() + (long)j); break; }
    g.tensors.erase(d);
  }
  return true;
}

// ---- recomposition of LayerNormalization and Gelu from the primitive
// operators exporters write them as (what onnx-mlir's recompose patterns do
// at the ONNX level; the DNN dialect of the reference never sees the fused
// forms, so this runs only when asked for).  Shapes are known.
namespace {
struct Matcher {
  Graph &g;
  std::map<std::string, size_t> producer;
  explicit Matcher(Graph &g_) : g(g_) {
    for (size_t i = 0; i < g.nodes.size(); i++) producer[g.nodes[i].output] = i;
  }
  const GNode *def(const std::string &name, const char *op) const {
    auto it = producer.find(name);
    if (it == producer.end() || g.nodes[it->second].op_type != op) return nullptr;
    return &g.nodes[it->second];
  }
  bool scalar(const std::string &name, double &v) const {
    auto it = g.tensors.find(name);
    if (it == g.tensors.end() || !it->second.is_const || it->second.dtype == I64 || shape_numel(it->second.shape) != 1) return false;
    v = load_elem(it->second, 0);
    return true;
  }
  bool single_use(const std::string &name) const { return count_uses(g, name) == 1; }
  // n is a binary node with one operand produced by `op` and the other anything: returns the pair
  bool split(const GNode &n, const char *op, const GNode *&inner, std::string &other) const {
    if (n.inputs.size() != 2) return false;
    for (int k = 0; k < 2; k++)
      if ((inner = def(n.inputs[(size_t)k], op)) != nullptr) { other = n.inputs[(size_t)(1 - k)]; return true; }
    return false;
  }
  bool last_axis_mean(const GNode &n) const {
    auto ax = n.ints.find("axes");
    auto kd = n.ints.find("keepdims");
    if (ax == n.ints.end() || ax->second.size() != 1 || n.inputs.empty()) return false;
    if (kd != n.ints.end() && !kd->second.empty() && kd->second[0] != 1) return false;
    const int64_t rank = (int64_t)g.tensors.at(n.inputs[0]).shape.size();
    return ax->second[0] == -1 || ax->second[0] == rank - 1;
  }
};
}  // namespace

// out = Add(Mul(Div(d, Sqrt(Add(ReduceMean(Pow(d, 2)), eps))), gamma), beta), d = Sub(x, ReduceMean(x))
static bool match_layernorm(const Matcher &m, const GNode &root, GNode &fused, std::vector<std::string> &dead) {
  if (root.op_type != "Add") return false;
  const GNode *mul, *div, *sub, *sqrt_, *add_eps, *mean2, *pow_, *mean1;
  std::string beta, gamma, eps_name, two_name;
  if (!m.split(root, "Mul", mul, beta) || !m.split(*mul, "Div", div, gamma)) return false;
  if (div->inputs.size() != 2 || !(sub = m.def(div->inputs[0], "Sub")) || !(sqrt_ = m.def(div->inputs[1], "Sqrt"))) return false;
  if (!(add_eps = m.def(sqrt_->inputs[0], "Add")) || !m.split(*add_eps, "ReduceMean", mean2, eps_name)) return false;
  if (!(pow_ = m.def(mean2->inputs[0], "Pow")) || pow_->inputs.size() != 2 || pow_->inputs[0] != sub->output) return false;
  two_name = pow_->inputs[1];
  if (sub->inputs.size() != 2 || !(mean1 = m.def(sub->inputs[1], "ReduceMean")) || mean1->inputs[0] != sub->inputs[0]) return false;
  double eps, two;
  if (!m.scalar(eps_name, eps) || !m.scalar(two_name, two) || two != 2.0 || !(eps >= 0.0)) return false;  // (1e-12 stored as fp16 is 0)
  if (!m.last_axis_mean(*mean1) || !m.last_axis_mean(*mean2)) return false;
  const GTensor &x = m.g.tensors.at(sub->inputs[0]);
  auto vec_const = [&](const std::string &n) {
    auto it = m.g.tensors.find(n);
    return it != m.g.tensors.end() && it->second.is_const && it->second.dtype == x.dtype &&
           shape_numel(it->second.shape) == x.shape.back() && !it->second.shape.empty() && it->second.shape.back() == x.shape.back();
  };
  if (x.shape.empty() || !vec_const(gamma) || !vec_const(beta)) return false;
  // nothing else may read the intermediates
  if (!m.single_use(mean1->output) || m.g.tensors.count(sub->output) == 0 || count_uses(m.g, sub->output) != 2) return false;
  for (const GNode *n : {pow_, mean2, add_eps, sqrt_, div, mul})
    if (!m.single_use(n->output)) return false;
  fused = GNode();
  fused.op_type = "LayerNormalization";
  fused.inputs = {sub->inputs[0], gamma, beta};
  fused.output = root.output;
  fused.ints["axis"] = {-1};
  fused.floats["epsilon"] = eps;
  dead = {mean1->output, sub->output, pow_->output, mean2->output, add_eps->output, sqrt_->output, div->output, mul->output};
  return true;
}

// out = Mul(Mul(x, Add(Erf(Div(x, sqrt 2)), 1)), 0.5)
static bool match_gelu(const Matcher &m, const GNode &root, GNode &fused, std::vector<std::string> &dead) {
  if (root.op_type != "Mul") return false;
  const GNode *inner, *add1, *erf, *div;
  std::string half_name, x, one_name;
  double half, one, c;
  if (!m.split(root, "Mul", inner, half_name) || !m.scalar(half_name, half) || half != 0.5) return false;
  if (inner->inputs.size() != 2) return false;
  bool ok = false;
  for (int k = 0; k < 2 && !ok; k++) {  // x itself may come from an Add: try both operand orders
    x = inner->inputs[(size_t)(1 - k)];
    if (!(add1 = m.def(inner->inputs[(size_t)k], "Add"))) continue;
    if (!m.split(*add1, "Erf", erf, one_name) || !m.scalar(one_name, one) || one != 1.0) continue;
    if (!(div = m.def(erf->inputs[0], "Div")) || div->inputs.size() != 2 || div->inputs[0] != x) continue;
    if (!m.scalar(div->inputs[1], c) || std::fabs(c - 1.4142135623730951) > 1e-3) continue;
    ok = true;
  }
  if (!ok) return false;
  for (const GNode *n : {div, erf, add1, inner})
    if (!m.single_use(n->output)) return false;
  fused = GNode();
  fused.op_type = "Gelu";
  fused.inputs = {x};
  fused.output = root.output;
  dead = {div->output, erf->output, add1->output, inner->output};
  return true;
}

// Div(x, c) with a one-element constant c becomes Mul(x, 1/c): the reference
// lowers Div to reciprocal + mul (Ops/cudnn/Div.cpp), so only the reciprocal
// moves from run time to compile time (1.0f / c in the tensor's type, as the
// device computes it).
static bool fold_constant_divisors(Graph &g) {
  bool any = false;
  for (size_t i = 0; i < g.nodes.size(); i++) {
    GNode &n = g.nodes[i];
    if (n.op_type != "Div" || n.inputs.size() != 2) continue;
    auto it = g.tensors.find(n.inputs[1]);
    if (it == g.tensors.end() || !it->second.is_const || it->second.dtype == I64 || shape_numel(it->second.shape) != 1) continue;
    const std::string name = n.output + "_recip", old = n.inputs[1];
    if (g.tensors.count(name)) continue;
    GTensor r = it->second;
    r.name = name;
    store_elem(r, 0, (double)(1.0f / (float)load_elem(it->second, 0)));
    g.tensors[name] = r;
    n.op_type = "Mul";
    n.inputs[1] = name;
    GNode cn;
    cn.op_type = "Constant";
    cn.output = name;
    g.nodes.insert(g.nodes.begin() + (long)i, cn);
    i++;
    if (count_uses(g, old) == 0) {
      for (size_t j = 0; j < g.nodes.size(); j++)
        if (g.nodes[j].op_type == "Constant" && g.nodes[j].output == old) {
          g.nodes.erase(g.nodes.begin() + (long)j);
          if (j < i) i--;
          break;
        }
      g.tensors.erase(old);
    }
    any = true;
  }
  return any;
}

// out = Reshape(Transpose(MatMul(Softmax(scale * MatMul(q, k)), v), [0,2,1,3]), [B, S, H*D]) with
// q, v = Transpose(Reshape(Q | V, [B, S, H, D]), [0,2,1,3]) and k = Transpose(Reshape(K, [B, S, H, D]), [0,2,3,1]):
// the attention core of an exported transformer encoder, heads split and merged by data movement.
static bool match_attention(const Matcher &m, const GNode &root, GNode &fused, std::vector<std::string> &dead) {
  if (root.op_type != "Reshape" || root.inputs.empty()) return false;
  auto perm_is = [](const GNode *n, std::initializer_list<int64_t> want) {
    auto it = n->ints.find("perm");
    return it != n->ints.end() && it->second == std::vector<int64_t>(want);
  };
  const GNode *merge, *mm2, *soft, *mm1, *scl = nullptr, *t[3], *r[3];
  if (!(merge = m.def(root.inputs[0], "Transpose")) || !perm_is(merge, {0, 2, 1, 3})) return false;
  if (!(mm2 = m.def(merge->inputs[0], "MatMul")) || mm2->inputs.size() != 2) return false;
  if (!(soft = m.def(mm2->inputs[0], "Softmax"))) return false;
  auto ax = soft->ints.find("axis");
  const int64_t axis = ax == soft->ints.end() || ax->second.empty() ? -1 : ax->second[0];
  if (axis != -1 && axis != 3) return false;
  double scale = 1.0, c;
  std::string other;
  if ((mm1 = m.def(soft->inputs[0], "MatMul")) == nullptr) {
    if ((scl = m.def(soft->inputs[0], "Div")) != nullptr) {
      if (scl->inputs.size() != 2 || !(mm1 = m.def(scl->inputs[0], "MatMul")) || !m.scalar(scl->inputs[1], c) || c == 0.0) return false;
      scale = (double)(1.0f / (float)c);
    } else if ((scl = m.def(soft->inputs[0], "Mul")) != nullptr) {
      if (!m.split(*scl, "MatMul", mm1, other) || !m.scalar(other, c)) return false;
      scale = c;
    } else {
      return false;
    }
  }
  if (mm1->inputs.size() != 2) return false;
  const std::string tn[3] = {mm1->inputs[0], mm1->inputs[1], mm2->inputs[1]};
  for (int i = 0; i < 3; i++) {
    if (!(t[i] = m.def(tn[i], "Transpose")) || !(r[i] = m.def(t[i]->inputs[0], "Reshape"))) return false;
    if (i == 1 ? !perm_is(t[i], {0, 2, 3, 1}) : !perm_is(t[i], {0, 2, 1, 3})) return false;
  }
  const GTensor &q = m.g.tensors.at(r[0]->inputs[0]), &k = m.g.tensors.at(r[1]->inputs[0]), &v = m.g.tensors.at(r[2]->inputs[0]);
  const Shape &qs = m.g.tensors.at(r[0]->output).shape, &ks = m.g.tensors.at(r[1]->output).shape, &vs = m.g.tensors.at(r[2]->output).shape;
  if ((q.dtype != F32 && q.dtype != F16) || k.dtype != q.dtype || v.dtype != q.dtype || q.shape.size() != 3 || k.shape.size() != 3 || v.shape != k.shape || qs.size() != 4 || ks.size() != 4 || vs != ks) return false;
  const int64_t B = qs[0], Sq = qs[1], H = qs[2], D = qs[3], Sk = ks[1];
  if (ks[0] != B || ks[2] != H || ks[3] != D || (D != 32 && D != 64 && D != 128)) return false;
  if (q.shape != Shape{B, Sq, H * D} || k.shape != Shape{B, Sk, H * D} || m.g.tensors.at(root.output).shape != q.shape) return false;
  std::vector<const GNode *> inner{merge, mm2, soft, mm1, t[0], t[1], t[2], r[0], r[1], r[2]};
  if (scl) inner.push_back(scl);
  for (const GNode *n : inner)
    if (!m.single_use(n->output)) return false;
  fused = GNode();
  fused.op_type = "FusedAttention";
  fused.inputs = {r[0]->inputs[0], r[1]->inputs[0], r[2]->inputs[0]};
  fused.output = root.output;
  fused.ints["heads"] = {H};
  fused.floats["scale"] = scale;
  dead.clear();
  for (const GNode *n : inner) dead.push_back(n->output);
  return true;
}

// Q, K and V of a matched attention block that are three Linear layers of the
// same input, Add(bias, MatMul(x, W)) with constant W [in, hidden] and bias
// [hidden], read by nothing else: one product with the three weight matrices
// side by side gives a [B, S, 3*hidden] tensor whose rows hold Q | K | V, and
// the attention call reads its operands out of that tensor.
static void pack_qkv(const Matcher &m, GNode &fused, std::vector<std::string> &dead, std::vector<GNode> &pre) {
  Graph &g = m.g;
  const GNode *add[3], *mm[3];
  std::string bias[3];
  for (int i = 0; i < 3; i++) {
    if (!(add[i] = m.def(fused.inputs[(size_t)i], "Add")) || !m.split(*add[i], "MatMul", mm[i], bias[i])) return;
    if (!m.single_use(add[i]->output) || !m.single_use(mm[i]->output) || mm[i]->inputs.size() != 2) return;
    if (mm[i]->inputs[0] != mm[0]->inputs[0]) return;
  }
  const GTensor *w[3], *b[3];
  for (int i = 0; i < 3; i++) {
    auto wi = g.tensors.find(mm[i]->inputs[1]), bi = g.tensors.find(bias[i]);
    if (wi == g.tensors.end() || bi == g.tensors.end() || !wi->second.is_const || !bi->second.is_const) return;
    w[i] = &wi->second; b[i] = &bi->second;
    if ((w[i]->dtype != F32 && w[i]->dtype != F16) || w[i]->dtype != w[0]->dtype || b[i]->dtype != w[0]->dtype || w[i]->shape.size() != 2 ||
        w[i]->shape != w[0]->shape ||
        b[i]->shape != Shape{w[i]->shape[1]})
      return;
  }
  const int64_t in = w[0]->shape[0], hid = w[0]->shape[1];
  const std::string base = fused.output + "_qkv", wn = base + "_w", bn = base + "_b", mn = base + "_mm";
  if (g.tensors.count(base) || g.tensors.count(wn) || g.tensors.count(bn) || g.tensors.count(mn)) return;
  GTensor wt, bt;
  const int64_t es = w[0]->dtype == F32 ? 4 : 2;  // bytes per element
  wt.name = wn; wt.dtype = w[0]->dtype; wt.shape = {in, 3 * hid}; wt.is_const = true; wt.data.resize((size_t)(in * 3 * hid * es));
  bt.name = bn; bt.dtype = w[0]->dtype; bt.shape = {3 * hid}; bt.is_const = true; bt.data.resize((size_t)(3 * hid * es));
  for (int i = 0; i < 3; i++) {
    for (int64_t r = 0; r < in; r++)
      std::memcpy(wt.data.data() + ((r * 3 + i) * hid) * es, w[i]->data.data() + r * hid * es, (size_t)(hid * es));
    std::memcpy(bt.data.data() + (int64_t)i * hid * es, b[i]->data.data(), (size_t)(hid * es));
  }
  g.tensors[wn] = std::move(wt);
  g.tensors[bn] = std::move(bt);
  GNode cw, cb, nm, na;
  cw.op_type = "Constant"; cw.output = wn;
  cb.op_type = "Constant"; cb.output = bn;
  nm.op_type = "MatMul"; nm.inputs = {mm[0]->inputs[0], wn}; nm.output = mn;
  na.op_type = "Add"; na.inputs = {bn, mn}; na.output = base;  // bias first, as exporters write it
  pre = {cw, cb, nm, na};
  for (int i = 0; i < 3; i++) { dead.push_back(add[i]->output); dead.push_back(mm[i]->output); }
  fused.inputs = {base, base, base};
  fused.ints["packed"] = {1};
}

static bool recompose(Graph &g, bool norms, bool attention) {
  bool any = false;
  for (size_t i = 0; i < g.nodes.size(); i++) {
    Matcher m(g);
    GNode fused;
    std::vector<std::string> dead;
    std::vector<GNode> pre;  // nodes to put in front of the fused one
    bool hit = attention && match_attention(m, g.nodes[i], fused, dead);
    if (hit) pack_qkv(m, fused, dead, pre);
    else hit = norms && (match_layernorm(m, g.nodes[i], fused, dead) || match_gelu(m, g.nodes[i], fused, dead));
    if (!hit) continue;
    // constants read by the matched nodes only go with them
    std::vector<std::string> consts;
    for (const std::string &d : dead)
      for (const std::string &in : g.nodes[m.producer.at(d)].inputs) {
        auto t = g.tensors.find(in);
        if (t != g.tensors.end() && t->second.is_const) consts.push_back(in);
      }
    for (const std::string &in : g.nodes[i].inputs) {
      auto t = g.tensors.find(in);
      if (t != g.tensors.end() && t->second.is_const) consts.push_back(in);
    }
    g.nodes[i] = fused;
    g.nodes.insert(g.nodes.begin() + (long)i, pre.begin(), pre.end());
    std::vector<GNode> kept;
    for (GNode &n : g.nodes)
      if (std::find(dead.begin(), dead.end(), n.output) == dead.end()) kept.push_back(n);
    g.nodes.swap(kept);
    for (const std::string &d : dead) g.tensors.erase(d);
    for (const std::string &c : consts) {
      if (!g.tensors.count(c) || count_uses(g, c) != 0) continue;
      for (size_t j = 0; j < g.nodes.size(); j++)
        if (g.nodes[j].op_type == "Constant" && g.nodes[j].output == c) { g.nodes.erase(g.nodes.begin() + (long)j); break; }
      g.tensors.erase(c);
    }
    any = true;
    i = (size_t)-1;  // positions moved: rescan
  }
  // after the matchers: Gelu's own Div by sqrt(2) must still be there for them
  return (norms && fold_constant_divisors(g)) || any;
}

static bool infer_pass(Graph &g, std::string &err) {
  for (GNode &n : g.nodes) {
    if (n.op_type == "Constant") continue;
    // onnx-mlir rewrites GlobalAveragePool to ReduceMean(axes = spatial dims, keepdims = 1)
    if (n.op_type == "GlobalAveragePool") {
      n.op_type = "ReduceMean";
      n.ints["axes"] = {2, 3};
      n.ints["keepdims"] = {1};
    }
    std::vector<const GTensor *> in;
    for (const std::string &name : n.inputs) {
      if (name.empty()) { in.push_back(nullptr); continue; }
      auto it = g.tensors.find(name);
      if (it == g.tensors.end()) {
        err = n.op_type + ": input '" + name + "' is not defined before use";
        return false;
      }
      in.push_back(&it->second);
    }
    if (in.empty() || !in[0]) { err = n.op_type + ": missing first input"; return false; }
    GTensor out;
    out.name = n.output;
    out.dtype = in[0]->dtype;
    const Shape &x = in[0]->shape;
    const std::string &t = n.op_type;
    auto fail = [&](const std::string &m) { err = t + " '" + n.output + "': " + m; return false; };

    if (t == "Conv") {
      if (in.size() < 2 || !in[1] || x.size() != 4 || in[1]->shape.size() != 4) return fail("needs 4-D X and W");
      const Shape &w = in[1]->shape;
      std::vector<int64_t> pads{0, 0, 0, 0}, strides{1, 1}, dil;
      get_ints(n, "pads", pads);
      get_ints(n, "strides", strides);
      if (get_ints(n, "dilations", dil))
        for (int64_t d : dil) if (d != 1) return fail("dilation must be 1");
      if (pads.size() != 4 || strides.size() != 2) return fail("pads must have 4 and strides 2 entries");
      // the reference reads pads[0] and pads[2] as the (symmetric) h and w pads
      // (src/Conversion/ONNXToDNN/Ops/cudnn/Conv.cpp:40-44); asymmetric pads are out of its reach
      if (pads[0] != pads[2] || pads[1] != pads[3]) return fail("asymmetric pads are not supported");
      const int64_t group = get_int(n, "group", 1);
      if (group < 1 || x[1] != w[1] * group || w[0] % group) return fail("channel/group mismatch");
      const int64_t P = (x[2] + pads[0] + pads[2] - w[2]) / strides[0] + 1;
      const int64_t Q = (x[3] + pads[1] + pads[3] - w[3]) / strides[1] + 1;
      if (P < 1 || Q < 1) return fail("empty output");
      out.shape = {x[0], w[0], P, Q};
    } else if (t == "Relu" || t == "Sigmoid" || t == "Tanh" || t == "Sqrt" || t == "Erf" || t == "Clip" ||
               t == "Gelu" || t == "Pow" || t == "Softmax" || t == "LayerNormalization" || t == "LeakyRelu" ||
               t == "Identity" || t == "BatchNormalization") {
      if (t == "Softmax" && g.opset > 0 && g.opset < 13) {
        // before opset 13: axis defaults to 1 and the input is flattened to [prod(d[:axis]), prod(d[axis:])];
        // that is the per-axis operator only when the axis is the last one
        int64_t ax = get_int(n, "axis", 1);
        if (ax < 0) ax += (int64_t)x.size();
        if (ax != (int64_t)x.size() - 1) return fail("Softmax of opset " + std::to_string(g.opset) + " over flattened trailing dims is not supported (axis must be the last)");
        n.ints["axis"] = {ax};
      }
      out.shape = x;
    } else if (t == "FusedAttention") {  // produced by the recomposition only
      if (in.size() != 3 || !in[1] || !in[2] || x.size() != 3) return fail("needs Q, K and V of rank 3");
      out.shape = x;
      if (get_int(n, "packed", 0)) out.shape[2] = x[2] / 3;
    } else if (t == "PRelu") {
      if (in.size() < 2 || !in[1]) return fail("needs a slope");
      Shape b;
      if (!broadcast_shape(x, in[1]->shape, b) || b != x) return fail("the slope does not broadcast to X");
      out.shape = x;
    } else if (t == "Concat") {
      int64_t axis = get_int(n, "axis", 0);
      if (axis < 0) axis += (int64_t)x.size();
      if (axis < 0 || axis >= (int64_t)x.size()) return fail("axis out of range");
      out.shape = x;
      for (size_t i = 1; i < in.size(); i++) {
        if (!in[i] || in[i]->shape.size() != x.size() || in[i]->dtype != out.dtype) return fail("inputs differ in rank or type");
        for (size_t d = 0; d < x.size(); d++)
          if ((int64_t)d != axis && in[i]->shape[d] != x[d]) return fail("inputs differ off the axis");
        out.shape[(size_t)axis] += in[i]->shape[(size_t)axis];
      }
      n.ints["axis"] = {axis};
    } else if (t == "Squeeze" || t == "Unsqueeze") {
      // axes: an attribute up to opset 12, a constant input from opset 13 on
      std::vector<int64_t> axes;
      bool have = get_ints(n, "axes", axes);
      if (!have && in.size() > 1 && in[1]) {
        if (!in[1]->is_const || in[1]->dtype != I64) return fail("axes must be an int64 constant");
        const int64_t *a = reinterpret_cast<const int64_t *>(in[1]->data.data());
        axes.assign(a, a + in[1]->data.size() / 8);
        have = true;
      }
      const int64_t rank_out = t == "Squeeze" ? (int64_t)x.size() : (int64_t)(x.size() + axes.size());
      const int64_t rank_ref = t == "Squeeze" ? (int64_t)x.size() : rank_out;
      std::vector<bool> mark((size_t)rank_ref, false);
      if (t == "Unsqueeze" && !have) return fail("needs axes");
      for (int64_t &a : axes) {
        if (a < 0) a += rank_ref;
        if (a < 0 || a >= rank_ref || mark[(size_t)a]) return fail("axis out of range or repeated");
        mark[(size_t)a] = true;
      }
      if (t == "Squeeze") {
        for (size_t d = 0; d < x.size(); d++) {
          if (have ? mark[d] : x[d] == 1) {
            if (x[d] != 1) return fail("squeezed dim is not 1");
            if (!have) axes.push_back((int64_t)d);
          } else {
            out.shape.push_back(x[d]);
          }
        }
      } else {
        size_t src = 0;
        for (int64_t d = 0; d < rank_out; d++) out.shape.push_back(mark[(size_t)d] ? 1 : x[src++]);
      }
      n.ints["axes"] = axes;
    } else if (t == "Add" || t == "Sub" || t == "Mul" || t == "Div") {
      if (in.size() < 2 || !in[1]) return fail("needs two inputs");
      if (!broadcast_shape(x, in[1]->shape, out.shape)) return fail("operands do not broadcast");
    } else if (t == "ReduceMean") {
      std::vector<int64_t> axes;
      const int64_t rank = (int64_t)x.size(), keep = get_int(n, "keepdims", 1);
      if (!get_ints(n, "axes", axes)) for (int64_t i = 0; i < rank; i++) axes.push_back(i);
      std::vector<bool> red((size_t)rank, false);
      for (int64_t a : axes) {
        if (a < 0) a += rank;
        if (a < 0 || a >= rank) return fail("axis out of range");
        red[(size_t)a] = true;
      }
      for (int64_t i = 0; i < rank; i++) {
        if (!red[(size_t)i]) out.shape.push_back(x[(size_t)i]);
        else if (keep) out.shape.push_back(1);
      }
    } else if (t == "MaxPool" || t == "AveragePool") {
      std::vector<int64_t> k, pads{0, 0, 0, 0}, strides{1, 1};
      if (!get_ints(n, "kernel_shape", k) || k.size() != 2 || x.size() != 4) return fail("needs 4-D X and kernel_shape[2]");
      get_ints(n, "pads", pads);
      get_ints(n, "strides", strides);
      if (pads.size() != 4 || strides.size() != 2) return fail("pads must have 4 and strides 2 entries");
      if (get_int(n, "ceil_mode", 0) != 0) return fail("ceil_mode is not supported");
      // the kernels divide by the full window, the reference's cuDNN mode (count include padding); the operator's
      // default leaves the padding out of the count
      if (t == "AveragePool" && (pads[0] || pads[1] || pads[2] || pads[3]) && get_int(n, "count_include_pad", 0) == 0)
        return fail("padded AveragePool needs count_include_pad = 1 (windows are divided by their full size)");
      const int64_t P = (x[2] + pads[0] + pads[2] - k[0]) / strides[0] + 1;
      const int64_t Q = (x[3] + pads[1] + pads[3] - k[1]) / strides[1] + 1;
      if (P < 1 || Q < 1) return fail("empty output");
      out.shape = {x[0], x[1], P, Q};
    } else if (t == "Gemm") {
      if (in.size() < 2 || !in[1] || x.size() != 2 || in[1]->shape.size() != 2) return fail("needs 2-D A and B");
      const int64_t ta = get_int(n, "transA", 0), tb = get_int(n, "transB", 0);
      const Shape &b = in[1]->shape;
      const int64_t M = ta ? x[1] : x[0], K = ta ? x[0] : x[1], Kb = tb ? b[1] : b[0], N = tb ? b[0] : b[1];
      if (K != Kb) return fail("inner dims differ");
      out.shape = {M, N};
    } else if (t == "MatMul") {
      if (in.size() < 2 || !in[1] || x.size() < 2 || in[1]->shape.size() < 2) return fail("needs two inputs of rank >= 2");
      const Shape &b = in[1]->shape;
      if (x.back() != b[b.size() - 2]) return fail("inner dims differ");
      Shape ba(x.begin(), x.end() - 2), bb(b.begin(), b.end() - 2), bo;
      if (!broadcast_shape(ba, bb, bo)) return fail("batch dims do not broadcast");
      out.shape = bo;
      out.shape.push_back(x[x.size() - 2]);
      out.shape.push_back(b.back());
    } else if (t == "Cast") {
      out.shape = x;
      out.dtype = (DType)get_int(n, "to", F32);
    } else if (t == "Gather") {
      if (in.size() < 2 || !in[1]) return fail("needs indices");
      int64_t axis = get_int(n, "axis", 0);
      if (axis < 0) axis += (int64_t)x.size();
      if (axis < 0 || axis >= (int64_t)x.size()) return fail("axis out of range");
      out.shape.assign(x.begin(), x.begin() + axis);
      out.shape.insert(out.shape.end(), in[1]->shape.begin(), in[1]->shape.end());
      out.shape.insert(out.shape.end(), x.begin() + axis + 1, x.end());
    } else if (t == "Expand") {
      if (in.size() < 2 || !in[1] || !in[1]->is_const || in[1]->dtype != I64) return fail("shape must be an int64 constant");
      const int64_t *s = reinterpret_cast<const int64_t *>(in[1]->data.data());
      const Shape want(s, s + in[1]->data.size() / 8);
      if (!broadcast_shape(x, want, out.shape)) return fail("input does not broadcast to shape");
      if (out.shape.size() > 8) return fail("rank above 8");
    } else if (t == "Reshape") {
      if (in.size() < 2 || !in[1] || !in[1]->is_const || in[1]->dtype != I64) return fail("shape must be an int64 constant");
      const int64_t *s = reinterpret_cast<const int64_t *>(in[1]->data.data());
      const size_t r = in[1]->data.size() / 8;
      int64_t known = 1, infer_at = -1;
      for (size_t i = 0; i < r; i++) {
        int64_t d = s[i];
        if (d == 0) { if (i >= x.size()) return fail("0 in shape beyond input rank"); d = x[i]; }
        if (d == -1) { if (infer_at >= 0) return fail("two -1 in shape"); infer_at = (int64_t)i; d = 1; }
        out.shape.push_back(d);
        known *= d;
      }
      if (infer_at >= 0) out.shape[(size_t)infer_at] = shape_numel(x) / known;
      if (shape_numel(out.shape) != shape_numel(x)) return fail("element count changes");
    } else if (t == "Flatten") {
      int64_t axis = get_int(n, "axis", 1);
      if (axis < 0) axis += (int64_t)x.size();
      int64_t a = 1, b = 1;
      for (int64_t i = 0; i < (int64_t)x.size(); i++) (i < axis ? a : b) *= x[(size_t)i];
      out.shape = {a, b};
    } else if (t == "Transpose") {
      std::vector<int64_t> perm;
      if (!get_ints(n, "perm", perm)) for (int64_t i = (int64_t)x.size() - 1; i >= 0; i--) perm.push_back(i);
      if (perm.size() != x.size()) return fail("perm rank");
      for (int64_t p : perm) {
        if (p < 0 || p >= (int64_t)x.size()) return fail("perm entry out of range");
        out.shape.push_back(x[(size_t)p]);
      }
      n.ints["perm"] = perm;
    } else {
      return fail("operator is not in the DNN dialect's coverage");
    }
    if (g.tensors.count(n.output)) return fail("output name already defined");
    g.tensors[n.output] = out;
  }
  for (const std::string &o : g.outputs)
    if (!g.tensors.count(o)) { err = "graph output '" + o + "' is never produced"; return false; }
  return true;
}

bool infer_shapes(Graph &g, bool recompose_norms, bool fuse_attention, std::string &err) {
  forward_aliases(g);
  if (!infer_pass(g, err)) return false;
  bool rewritten = (recompose_norms || fuse_attention) && recompose(g, recompose_norms, fuse_attention);
  for (size_t i = 0; i < g.nodes.size();) {
    if (g.nodes[i].op_type != "BatchNormalization") { i++; continue; }
    if (!rewrite_batchnorm(g, i, err)) return false;
    rewritten = true;
    i = 0;
  }
  if (!rewritten) return true;
  for (auto it = g.tensors.begin(); it != g.tensors.end();)  // derived shapes: inferred again
    it = (it->second.is_input || it->second.is_const) ? std::next(it) : g.tensors.erase(it);
  return infer_pass(g, err);
}

// Each constant is moved to just before its first user; constants sharing a
// first user keep their original relative order.
void constant_at_use(Graph &g) {
  struct Move { size_t cst, user; };
  std::vector<Move> moves;
  for (size_t i = 0; i < g.nodes.size(); i++) {
    if (g.nodes[i].op_type != "Constant") continue;
    for (size_t j = i + 1; j < g.nodes.size(); j++) {
      const auto &in = g.nodes[j].inputs;
      if (std::find(in.begin(), in.end(), g.nodes[i].output) != in.end()) {
        moves.push_back({i, j});
        break;
      }
    }
  }
  // Rebuild the node list: walk the users in order and emit, before each, the
  // constants that were scheduled for it (in original constant order).
  std::vector<bool> moved(g.nodes.size(), false);
  std::vector<std::vector<size_t>> before(g.nodes.size());
  for (const Move &m : moves) { moved[m.cst] = true; before[m.user].push_back(m.cst); }
  std::vector<GNode> out;
  out.reserve(g.nodes.size());
  for (size_t j = 0; j < g.nodes.size(); j++) {
    if (moved[j]) continue;
    for (size_t c : before[j]) out.push_back(g.nodes[c]);
    out.push_back(g.nodes[j]);
  }
  g.nodes.swap(out);
}

}  // namespace dnnc
