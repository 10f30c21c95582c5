// ONNX model file -> Graph.
//
// The reference takes an .onnx file on its command line
// (`core-dnn --EmitLib ... model.onnx`, test/models/*/run.py) and imports it
// with onnx-mlir's front end (third_party/onnx-mlir, absent from the
// reference tree) which links protobuf and the `onnx` package.  Neither is
// available here, so this is a reader for the protobuf wire format restricted
// to the messages and fields of onnx.proto3 that an inference graph of the
// operators in ir.h needs (field numbers below are those of the published
// onnx/onnx.proto3; unknown fields are skipped, as protobuf requires):
//
//   ModelProto      7 graph
//   GraphProto      1 node*  5 initializer*  11 input*  12 output*
//   NodeProto       1 input*  2 output*  4 op_type  5 attribute*  7 domain
//   AttributeProto  1 name  2 f  3 i  4 s  5 t  7 floats*  8 ints*  20 type
//   TensorProto     1 dims*  2 data_type  4 float_data*  5 int32_data*
//                   7 int64_data*  8 name  9 raw_data  13 external_data*  14 data_location
//   ValueInfoProto  1 name  2 type -> TypeProto 1 tensor_type -> 1 elem_type,
//                   2 shape -> TensorShapeProto 1 dim* -> 1 dim_value | 2 dim_param
//
// Initializers become constants in file order ahead of the nodes (the
// constant-at-use pass then moves each before its first user, as in the
// reference); graph inputs that are initializers (IR version < 4 files list
// them) are not inputs; Constant nodes with a tensor value become constants
// in place.  Shapes must be static.
#include <cstring>

#include "ir.h"

namespace dnnc {

namespace {

struct Reader {
  const uint8_t *p, *end;
  bool ok = true;
  bool done() const { return p >= end || !ok; }
  uint64_t varint() {
    uint64_t v = 0;
    for (int shift = 0; shift < 64; shift += 7) {
      if (p >= end) { ok = false; return 0; }
      const uint8_t b = *p++;
      v |= (uint64_t)(b & 0x7f) << shift;
      if (!(b & 0x80)) return v;
    }
    ok = false;  // more than 10 bytes
    return 0;
  }
  // next field: number and wire type
  bool tag(uint32_t &field, uint32_t &wire) {
    if (done()) return false;
    const uint64_t t = varint();
    field = (uint32_t)(t >> 3);
    wire = (uint32_t)(t & 7);
    return ok && field != 0;
  }
  Reader bytes() {  // length-delimited payload
    const uint64_t n = varint();
    if (!ok || n > (uint64_t)(end - p)) { ok = false; return Reader{p, p}; }
    Reader r{p, p + n};
    p += n;
    return r;
  }
  uint32_t fixed32() {
    if (end - p < 4) { ok = false; return 0; }
    uint32_t v; std::memcpy(&v, p, 4); p += 4; return v;
  }
  uint64_t fixed64() {
    if (end - p < 8) { ok = false; return 0; }
    uint64_t v; std::memcpy(&v, p, 8); p += 8; return v;
  }
  void skip(uint32_t wire) {
    switch (wire) {
      case 0: varint(); break;
      case 1: fixed64(); break;
      case 2: bytes(); break;
      case 5: fixed32(); break;
      default: ok = false;  // groups (3, 4) do not occur in onnx.proto3
    }
  }
  std::string str() { Reader r = bytes(); return std::string((const char *)r.p, (size_t)(r.end - r.p)); }
};

// repeated scalar: packed (wire 2) or one element per tag
template <typename F>
void repeated(Reader &r, uint32_t wire, uint32_t elem_wire, F &&one) {
  if (wire == 2) {
    Reader q = r.bytes();
    while (!q.done()) one(q);
    if (!q.ok) r.ok = false;
  } else if (wire == elem_wire) {
    one(r);
  } else {
    r.skip(wire);
  }
}

struct OnnxTensor {
  std::string name;
  std::vector<int64_t> dims;
  int32_t data_type = 0;
  std::vector<float> float_data;
  std::vector<int32_t> int32_data;
  std::vector<int64_t> int64_data;
  const uint8_t *raw = nullptr;
  size_t raw_bytes = 0;
  bool has_raw = false, external = false;
};

bool parse_tensor(Reader r, OnnxTensor &t) {
  uint32_t f, w;
  while (r.tag(f, w)) {
    switch (f) {
      case 1: repeated(r, w, 0, [&](Reader &q) { t.dims.push_back((int64_t)q.varint()); }); break;
      case 2: if (w == 0) t.data_type = (int32_t)r.varint(); else r.skip(w); break;
      case 4: repeated(r, w, 5, [&](Reader &q) { uint32_t u = q.fixed32(); float v; std::memcpy(&v, &u, 4); t.float_data.push_back(v); }); break;
      case 5: repeated(r, w, 0, [&](Reader &q) { t.int32_data.push_back((int32_t)q.varint()); }); break;
      case 7: repeated(r, w, 0, [&](Reader &q) { t.int64_data.push_back((int64_t)q.varint()); }); break;
      case 8: if (w == 2) t.name = r.str(); else r.skip(w); break;
      case 9:
        if (w == 2) { Reader q = r.bytes(); t.raw = q.p; t.raw_bytes = (size_t)(q.end - q.p); t.has_raw = true; }
        else r.skip(w);
        break;
      case 13: t.external = true; r.skip(w); break;
      case 14: if (w == 0) { if (r.varint() == 1) t.external = true; } else r.skip(w); break;
      default: r.skip(w);
    }
  }
  return r.ok;
}

// TensorProto.DataType -> DType; only what the runtime computes in
bool map_dtype(int32_t onnx_type, DType &dt) {
  switch (onnx_type) {
    case 1: dt = F32; return true;
    case 10: dt = F16; return true;
    case 7: dt = I64; return true;
    default: return false;
  }
}

bool tensor_to_constant(const OnnxTensor &t, GTensor &out, std::string &err) {
  if (t.external) { err = "tensor '" + t.name + "' keeps its data in an external file"; return false; }
  DType dt;
  if (!map_dtype(t.data_type, dt)) { err = "tensor '" + t.name + "': data type " + std::to_string(t.data_type) + " (float, float16 and int64 are supported)"; return false; }
  out.name = t.name; out.dtype = dt; out.shape = t.dims; out.is_const = true;
  for (int64_t d : out.shape) if (d < 0) { err = "tensor '" + t.name + "': negative dim"; return false; }
  const int64_t n = shape_numel(out.shape);
  const size_t bytes = (size_t)(n * dtype_bytes(dt));
  out.data.resize(bytes);
  if (t.has_raw) {  // little-endian fixed-width, which is what this machine stores
    if (t.raw_bytes != bytes) { err = "tensor '" + t.name + "': raw_data holds " + std::to_string(t.raw_bytes) + " bytes, dims need " + std::to_string(bytes); return false; }
    std::memcpy(out.data.data(), t.raw, bytes);
    return true;
  }
  if (dt == F32) {
    if ((int64_t)t.float_data.size() != n) { err = "tensor '" + t.name + "': float_data count does not match dims"; return false; }
    std::memcpy(out.data.data(), t.float_data.data(), bytes);
  } else if (dt == I64) {
    if ((int64_t)t.int64_data.size() != n) { err = "tensor '" + t.name + "': int64_data count does not match dims"; return false; }
    std::memcpy(out.data.data(), t.int64_data.data(), bytes);
  } else {  // float16: one value per int32_data element, bits in the low half
    if ((int64_t)t.int32_data.size() != n) { err = "tensor '" + t.name + "': int32_data count does not match dims"; return false; }
    for (int64_t i = 0; i < n; i++) {
      const uint16_t h = (uint16_t)t.int32_data[(size_t)i];
      std::memcpy(out.data.data() + 2 * i, &h, 2);
    }
  }
  return true;
}

struct OnnxValueInfo {
  std::string name;
  int32_t elem_type = 0;
  std::vector<int64_t> dims;
  bool has_shape = false, dynamic = false;
};

bool parse_value_info(Reader r, OnnxValueInfo &v) {
  uint32_t f, w;
  while (r.tag(f, w)) {
    if (f == 1 && w == 2) v.name = r.str();
    else if (f == 2 && w == 2) {  // TypeProto
      Reader ty = r.bytes();
      uint32_t f2, w2;
      while (ty.tag(f2, w2)) {
        if (f2 == 1 && w2 == 2) {  // tensor_type
          Reader tt = ty.bytes();
          uint32_t f3, w3;
          while (tt.tag(f3, w3)) {
            if (f3 == 1 && w3 == 0) v.elem_type = (int32_t)tt.varint();
            else if (f3 == 2 && w3 == 2) {  // TensorShapeProto
              v.has_shape = true;
              Reader sh = tt.bytes();
              uint32_t f4, w4;
              while (sh.tag(f4, w4)) {
                if (f4 == 1 && w4 == 2) {  // Dimension
                  Reader dm = sh.bytes();
                  uint32_t f5, w5;
                  bool have = false;
                  while (dm.tag(f5, w5)) {
                    if (f5 == 1 && w5 == 0) { v.dims.push_back((int64_t)dm.varint()); have = true; }
                    else { if (f5 == 2) v.dynamic = true; dm.skip(w5); }
                  }
                  if (!have) { v.dynamic = true; v.dims.push_back(-1); }
                  if (!dm.ok) sh.ok = false;
                } else sh.skip(w4);
              }
              if (!sh.ok) tt.ok = false;
            } else tt.skip(w3);
          }
          if (!tt.ok) ty.ok = false;
        } else ty.skip(w2);
      }
      if (!ty.ok) r.ok = false;
    } else r.skip(w);
  }
  return r.ok;
}

bool parse_node(Reader r, Graph &g, std::string &err) {
  GNode n;
  std::vector<std::string> outputs;
  std::string domain;
  OnnxTensor value;
  bool has_value = false;
  uint32_t f, w;
  while (r.tag(f, w)) {
    if (f == 1 && w == 2) n.inputs.push_back(r.str());
    else if (f == 2 && w == 2) outputs.push_back(r.str());
    else if (f == 4 && w == 2) n.op_type = r.str();
    else if (f == 7 && w == 2) domain = r.str();
    else if (f == 5 && w == 2) {  // AttributeProto
      Reader at = r.bytes();
      std::string name, sval;
      std::vector<int64_t> ints;
      std::vector<double> floats;
      bool has_i = false, has_f = false, has_t = false, other = false;
      int64_t iv = 0;
      double fv = 0;
      uint32_t f2, w2;
      while (at.tag(f2, w2)) {
        switch (f2) {
          case 1: if (w2 == 2) name = at.str(); else at.skip(w2); break;
          case 2: if (w2 == 5) { uint32_t u = at.fixed32(); float x; std::memcpy(&x, &u, 4); fv = x; has_f = true; } else at.skip(w2); break;
          case 3: if (w2 == 0) { iv = (int64_t)at.varint(); has_i = true; } else at.skip(w2); break;
          case 5: if (w2 == 2) { has_t = parse_tensor(at.bytes(), value); if (!has_t) at.ok = false; } else at.skip(w2); break;
          case 7: repeated(at, w2, 5, [&](Reader &q) { uint32_t u = q.fixed32(); float x; std::memcpy(&x, &u, 4); floats.push_back(x); }); break;
          case 8: repeated(at, w2, 0, [&](Reader &q) { ints.push_back((int64_t)q.varint()); }); break;
          case 4: if (w2 == 2) { sval = at.str(); other = true; } else at.skip(w2); break;
          case 6: case 9: case 10: case 11: other = true; at.skip(w2); break;  // g, strings, tensors, graphs
          default: at.skip(w2);  // type (20), doc_string, ...
        }
      }
      if (!at.ok) { r.ok = false; break; }
      if (has_t && name == "value") has_value = true;
      else if (!ints.empty()) n.ints[name] = ints;
      else if (has_i) n.ints[name] = {iv};
      else if (has_f) n.floats[name] = fv;
      else if (!floats.empty()) { err = "node attribute '" + name + "': float lists are not used by any supported operator"; return false; }
      else if (name == "auto_pad" && sval != "NOTSET") { err = "auto_pad=" + sval + " is not supported (export with explicit pads)"; return false; }
      else if (other) { /* other strings and sub-graphs carry nothing the supported operators read */ }
    } else r.skip(w);
  }
  if (!r.ok) { err = "malformed NodeProto"; return false; }
  if (!domain.empty() && domain != "ai.onnx") { err = "operator '" + n.op_type + "' of domain '" + domain + "'"; return false; }
  if (outputs.empty() || outputs[0].empty()) { err = "node '" + n.op_type + "' has no output"; return false; }
  // Dropout's mask and BatchNormalization's running statistics are training
  // outputs: they stay undefined, so a node that reads one is refused later
  const bool extra_ok = n.op_type == "Dropout" || n.op_type == "BatchNormalization";
  for (size_t i = 1; i < outputs.size() && !extra_ok; i++)
    if (!outputs[i].empty()) { err = "node '" + n.op_type + "' has more than one output ('" + outputs[i] + "')"; return false; }
  n.output = outputs[0];
  if (n.op_type == "Constant") {
    if (!has_value) { err = "Constant node '" + n.output + "' without a tensor value"; return false; }
    GTensor t;
    value.name = n.output;
    if (!tensor_to_constant(value, t, err)) return false;
    if (g.tensors.count(t.name)) { err = "tensor '" + t.name + "' defined twice"; return false; }
    g.tensors[t.name] = std::move(t);
    GNode c;
    c.op_type = "Constant";
    c.output = n.output;
    g.nodes.push_back(c);
    return true;
  }
  if (n.op_type == "BatchNormalization") {
    auto tm = n.ints.find("training_mode");
    if (tm != n.ints.end() && !tm->second.empty() && tm->second[0] != 0) { err = "BatchNormalization in training mode"; return false; }
  }
  if (n.op_type == "Cast") {  // attribute `to` is a TensorProto.DataType
    auto it = n.ints.find("to");
    DType dt;
    if (it == n.ints.end() || it->second.size() != 1 || !map_dtype((int32_t)it->second[0], dt)) { err = "Cast: unsupported target type"; return false; }
    it->second[0] = (int64_t)dt;
  }
  // while trailing optional inputs are absent ONNX may spell them as ""
  while (!n.inputs.empty() && n.inputs.back().empty()) n.inputs.pop_back();
  g.nodes.push_back(std::move(n));
  return true;
}

}  // namespace

bool graph_from_onnx(const uint8_t *data, size_t nbytes, Graph &g, std::string &err) {
  Reader model{data, data + nbytes};
  const uint8_t *graph_p = nullptr, *graph_end = nullptr;
  uint32_t f, w;
  while (model.tag(f, w)) {
    if (f == 7 && w == 2) { Reader r = model.bytes(); graph_p = r.p; graph_end = r.end; }
    else if (f == 8 && w == 2) {  // opset_import: OperatorSetIdProto { 1: domain, 2: version }
      Reader r = model.bytes();
      std::string domain;
      int64_t version = 0;
      uint32_t f2, w2;
      while (r.tag(f2, w2)) {
        if (f2 == 1 && w2 == 2) domain = r.str();
        else if (f2 == 2 && w2 == 0) version = (int64_t)r.varint();
        else r.skip(w2);
      }
      if (!r.ok) { err = "malformed opset_import"; return false; }
      if (domain.empty() || domain == "ai.onnx") g.opset = version;
    }
    else model.skip(w);
  }
  if (!model.ok) { err = "not an ONNX ModelProto (malformed protobuf)"; return false; }
  if (!graph_p) { err = "the ONNX model has no graph"; return false; }

  // first pass: initializers and value infos (inputs may precede or follow them in the file)
  std::vector<OnnxValueInfo> inputs, outputs;
  std::vector<std::pair<const uint8_t *, const uint8_t *>> node_spans;
  Reader gr{graph_p, graph_end};
  while (gr.tag(f, w)) {
    if (f == 5 && w == 2) {
      OnnxTensor t;
      if (!parse_tensor(gr.bytes(), t)) { err = "malformed initializer"; return false; }
      if (t.name.empty()) { err = "initializer without a name"; return false; }
      GTensor c;
      if (!tensor_to_constant(t, c, err)) return false;
      if (g.tensors.count(c.name)) { err = "tensor '" + c.name + "' defined twice"; return false; }
      GNode n;
      n.op_type = "Constant";
      n.output = c.name;
      g.tensors[c.name] = std::move(c);
      g.nodes.push_back(n);
    } else if ((f == 11 || f == 12) && w == 2) {
      OnnxValueInfo v;
      if (!parse_value_info(gr.bytes(), v)) { err = "malformed ValueInfoProto"; return false; }
      (f == 11 ? inputs : outputs).push_back(v);
    } else if (f == 1 && w == 2) {
      Reader r = gr.bytes();
      node_spans.push_back({r.p, r.end});
    } else gr.skip(w);
  }
  if (!gr.ok) { err = "malformed GraphProto"; return false; }

  for (const OnnxValueInfo &v : inputs) {
    if (g.tensors.count(v.name)) continue;  // an initializer listed among the inputs
    GTensor t;
    t.name = v.name; t.is_input = true;
    if (!map_dtype(v.elem_type, t.dtype)) { err = "input '" + v.name + "': element type " + std::to_string(v.elem_type) + " (float, float16 and int64 are supported)"; return false; }
    if (!v.has_shape || v.dynamic) { err = "input '" + v.name + "' has no static shape"; return false; }
    for (int64_t d : v.dims) if (d <= 0) { err = "input '" + v.name + "': dims must be positive"; return false; }
    t.shape = v.dims;
    g.tensors[t.name] = t;
    g.inputs.push_back(t.name);
  }
  for (const auto &span : node_spans)
    if (!parse_node(Reader{span.first, span.second}, g, err)) return false;
  if (outputs.empty()) { err = "the ONNX graph has no output"; return false; }
  for (const OnnxValueInfo &v : outputs) g.outputs.push_back(v.name);
  return true;
}

}  // namespace dnnc
