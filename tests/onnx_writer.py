"""Serialises a compiler.Graph's Python-side mirror as an ONNX ModelProto, byte
by byte from the published onnx.proto3 (no `onnx` / protobuf package exists
here).  Test infrastructure for the ONNX reader: it can lay the same model out
in the several ways real exporters do (raw_data or typed data fields, packed or
unpacked repeated fields, initializers also listed as graph inputs, constants
as Constant nodes, shuffled field order)."""
import struct

import numpy as np

ONNX_DTYPE = {np.dtype(np.float32): 1, np.dtype(np.float16): 10, np.dtype(np.int64): 7}


def varint(v):
    v &= (1 << 64) - 1  # negative int64 -> ten-byte two's complement, as protobuf does
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def tag(field, wire):
    return varint((field << 3) | wire)


def f_varint(field, v):
    return tag(field, 0) + varint(v)


def f_bytes(field, payload):
    return tag(field, 2) + varint(len(payload)) + payload


def f_string(field, s):
    return f_bytes(field, s.encode())


def f_float(field, x):
    return tag(field, 5) + struct.pack("<f", x)


def tensor_proto(name, a, typed_fields=False, packed=True):
    a = np.ascontiguousarray(a)
    out = b""
    if packed:
        out += f_bytes(1, b"".join(varint(d) for d in a.shape)) if a.ndim else b""
    else:
        out += b"".join(f_varint(1, d) for d in a.shape)
    out += f_varint(2, ONNX_DTYPE[a.dtype])
    if typed_fields:
        if a.dtype == np.float32:
            out += f_bytes(4, a.tobytes()) if packed else b"".join(f_float(4, float(x)) for x in a.ravel())
        elif a.dtype == np.int64:
            vals = [varint(int(x)) for x in a.ravel()]
            out += f_bytes(7, b"".join(vals)) if packed else b"".join(tag(7, 0) + v for v in vals)
        else:  # float16 travels as int32_data holding the bit patterns
            vals = [varint(int(x)) for x in a.view(np.uint16).ravel()]
            out += f_bytes(5, b"".join(vals)) if packed else b"".join(tag(5, 0) + v for v in vals)
        out += f_string(8, name)
    else:
        out += f_string(8, name) + f_bytes(9, a.tobytes())
    return out


def value_info(name, shape, dtype, dim_param=None):
    dims = b""
    for i, d in enumerate(shape):
        if dim_param is not None and i == 0:
            dims += f_bytes(1, f_string(2, dim_param))
        else:
            dims += f_bytes(1, f_varint(1, d))
    tensor_type = f_varint(1, ONNX_DTYPE[np.dtype(dtype)]) + f_bytes(2, dims)
    return f_string(1, name) + f_bytes(2, f_bytes(1, tensor_type))


def attribute(name, v, packed=True):
    out = f_string(1, name)
    if isinstance(v, float):
        return out + f_float(2, v) + f_varint(20, 1)
    if isinstance(v, str):
        return out + f_bytes(4, v.encode()) + f_varint(20, 3)
    if isinstance(v, np.ndarray):
        return out + f_bytes(5, tensor_proto("", v)) + f_varint(20, 4)
    if isinstance(v, (list, tuple)):
        vals = [varint(int(x)) for x in v]
        body = f_bytes(8, b"".join(vals)) if packed else b"".join(tag(8, 0) + x for x in vals)
        return out + body + f_varint(20, 7)
    return out + f_varint(3, int(v)) + f_varint(20, 2)


ONNX_CAST_TO = {0: 1, 1: 10, 2: 7}  # the graph's dtype codes -> TensorProto.DataType


def node_proto(op_type, inputs, output, attrs, packed=True, extra_attrs=()):
    out = b"".join(f_string(1, i or "") for i in inputs) + f_string(2, output)
    out += f_string(3, output + "_node") + f_string(4, op_type)
    for k, v in attrs.items():
        if op_type == "Cast" and k == "to":
            v = ONNX_CAST_TO[int(v)]
        out += f_bytes(5, attribute(k, v, packed))
    for k, v in extra_attrs:
        out += f_bytes(5, attribute(k, v, packed))
    return out


def model_bytes(g, typed_fields=False, packed=True, initializers_as_inputs=False, constants_as_nodes=False,
                dynamic_batch=None, auto_pad=None, opset=13):
    """g: a compiler.Graph built through its Python methods (the mirror is read, not the C++ object)."""
    graph = b""
    nodes = b""
    if constants_as_nodes:
        for name, a in g.constants.items():
            nodes += f_bytes(1, f_string(2, name) + f_string(4, "Constant") + f_bytes(5, attribute("value", np.asarray(a))))
    for op_type, inputs, output, attrs in g.nodes:
        extra = [("auto_pad", auto_pad)] if (auto_pad and op_type == "Conv") else []
        nodes += f_bytes(1, node_proto(op_type, inputs, output, attrs, packed, extra))
    graph += nodes + f_string(2, "main_graph")
    if not constants_as_nodes:
        for name, a in g.constants.items():
            graph += f_bytes(5, tensor_proto(name, a, typed_fields, packed))
    for name, (shape, dt) in g.input_shapes.items():
        graph += f_bytes(11, value_info(name, shape, dt, dynamic_batch))
    if initializers_as_inputs and not constants_as_nodes:
        for name, a in g.constants.items():
            graph += f_bytes(11, value_info(name, a.shape, a.dtype))
    for name in g.outputs:
        graph += f_bytes(12, value_info(name, (), np.float32))  # the reader takes output names only
    opset_id = f_string(1, "") + f_varint(2, opset)
    return f_varint(1, 8) + f_string(2, "tests/onnx_writer.py") + f_bytes(8, opset_id) + f_bytes(7, graph)
