// ONNX-level graph: shape inference for the operator subset the DNN dialect
// covers, and the two ONNX-level rewrites that shape the event trace:
// GlobalAveragePool -> ReduceMean over (H, W) (done by onnx-mlir ahead of the
// reference's own passes) and "constant at use"
// (src/Transform/ONNX/ONNXConstantAtUsePass.cpp:29-58).
#include <algorithm>
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

bool infer_shapes(Graph &g, std::string &err) {
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
               t == "Gelu" || t == "Pow" || t == "Softmax" || t == "LayerNormalization") {
      out.shape = x;
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
