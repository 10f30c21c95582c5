"""The ONNX reader (the reference's input format, `core-dnn ... model.onnx`).

No `onnx` package or exporter exists offline, so the files come from
tests/onnx_writer.py, written from the same published onnx.proto3 as the reader
but independently of it (Python, emitting; the reader is C++, parsing), plus one
model assembled by hand below.  A graph that went through a file must compile to
the very same DNN program (text, pool layout) as the graph built in memory."""
import os

import numpy as np
import pytest

import onnx_writer as ow
from helpers import ORACLE_PATH
from occamy_amd import compiler, models

SMALL = {
    "single_conv": models.single_conv,
    "resnet50": lambda: models.resnet50(image=32, classes=10),
    "mobilenet_v2": lambda: models.mobilenet_v2(image=32, classes=10),
    "bert": lambda: models.bert_encoder(layers=2, hidden=64, heads=4, ffn=128, seq=16, vocab=100),
    "bert_fused": lambda: models.bert_encoder(layers=1, hidden=64, heads=4, ffn=128, seq=16, vocab=100, fused=True),
    "resnet50_fp16": lambda: models.resnet50(2, np.float16, image=32, classes=10),
    "alexnet": lambda: models.alexnet(image=96, classes=10, hidden=64),
    "yolo_v1": lambda: models.yolo_v1(batch=1, image=64, width=0.0625, fc=32),
    "srgan": lambda: models.srgan_generator(height=8, width=6, feats=16, blocks=2),
}

# x: float[1,2] -> Relu -> y, by hand from onnx.proto3:
#   ModelProto  08 08            ir_version = 8
#               3A 28            graph (field 7), 40 bytes
#   GraphProto  0A 0C            node (field 1), 12 bytes
#     NodeProto 0A 01 78           input "x"
#               12 01 79           output "y"
#               22 04 52 65 6C 75  op_type "Relu"
#               5A 13            input (field 11), 19 bytes
#     ValueInfo 0A 01 78           name "x"
#               12 0E              type, 14 bytes
#       Type    0A 0C                tensor_type, 12 bytes
#         Tensor 08 01                 elem_type = FLOAT
#                12 08                 shape, 8 bytes
#                   0A 02 08 01          dim { dim_value: 1 }
#                   0A 02 08 02          dim { dim_value: 2 }
#               62 03            output (field 12), 3 bytes
#     ValueInfo 0A 01 79           name "y"
HAND_MADE_RELU = bytes.fromhex(
    "0808" "3A28"
    "0A0C" "0A0178" "120179" "220452656C75"
    "5A13" "0A0178" "120E" "0A0C" "0801" "1208" "0A020801" "0A020802"
    "6203" "0A0179")


def test_hand_assembled_model():
    g = compiler.load_onnx(HAND_MADE_RELU)
    assert g.input_shapes == {"x": ((1, 2), np.dtype(np.float32))} and g.outputs == ["y"]
    p = g.compile()
    assert "dnn.activationfwd" in p.text and p.text.count("dnn.malloc") == 0  # pooled
    s = p.session(runtime_library=ORACLE_PATH)
    np.testing.assert_array_equal(s.run(np.array([[-1.5, 2.0]], np.float32))[0], [[0.0, 2.0]])
    s.close()


LAYOUTS = [
    dict(),                                            # raw_data, packed repeated fields
    dict(typed_fields=True),                           # float_data / int64_data / int32_data
    dict(typed_fields=True, packed=False),             # one element per tag
    dict(initializers_as_inputs=True),                 # IR < 4 style
    dict(constants_as_nodes=True),                     # Constant nodes instead of initializers
]


def tiny_fp16():
    g = compiler.Graph()
    r = np.random.default_rng(3)
    x = g.input("x", (1, 8, 6, 6), np.float16)
    w = g.constant((r.standard_normal((4, 8, 3, 3)) * 0.2).astype(np.float16), "w")
    b = g.constant(r.uniform(-0.1, 0.1, 4).astype(np.float16), "b")
    g.output(g.node("Relu", [g.node("Conv", [x, w, b], "c", kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1])], "y"))
    return g, [r.standard_normal((1, 8, 6, 6)).astype(np.float16)]


SMALL["tiny_fp16"] = tiny_fp16
BIG = {"resnet50", "mobilenet_v2", "resnet50_fp16"}  # millions of weights: per-element encodings are left to the small ones


@pytest.mark.parametrize("layout", range(len(LAYOUTS)))
@pytest.mark.parametrize("name", list(SMALL))
def test_file_round_trip_gives_the_same_program(name, layout):
    if name in BIG and LAYOUTS[layout].get("typed_fields"):
        pytest.skip("typed data fields are exercised on the small models")
    g0, inputs = SMALL[name]()
    data = ow.model_bytes(g0, **LAYOUTS[layout])
    g1 = compiler.load_onnx(data)
    assert g1.input_shapes == g0.input_shapes and g1.outputs == g0.outputs
    flags = dict(fusion=True) if "bert" not in name else {}
    p0, p1 = g0.compile(**flags), g1.compile(**flags)
    assert p1.text == p0.text
    assert p1.pool_bytes == p0.pool_bytes and p1.events() == p0.events()
    if layout == 0:  # the tensors themselves arrived intact: same numbers out
        s0, s1 = p0.session(runtime_library=ORACLE_PATH), p1.session(runtime_library=ORACLE_PATH)
        for a, b in zip(s0.run(*inputs), s1.run(*inputs)):
            np.testing.assert_array_equal(a, b)
        s0.close(); s1.close()


def test_file_on_disk(tmp_path):
    g0, inputs = models.single_conv()
    path = tmp_path / "single_conv.onnx"
    path.write_bytes(ow.model_bytes(g0))
    p = compiler.load_onnx(str(path)).compile()
    assert p.pool_bytes == 1753344  # the single-conv configuration's planned pool


def test_negative_and_large_integers_survive():
    g = compiler.Graph()
    x = g.input("x", (2, 3, 4), np.float32)
    idx = g.constant(np.array([-1, 0, 2 ** 40 % 3], np.int64), "idx")   # -1: ten-byte varint
    y = g.node("Gather", [x, idx], "y", axis=1)
    g.output(y)
    for layout in (dict(), dict(typed_fields=True), dict(typed_fields=True, packed=False)):
        g1 = compiler.load_onnx(ow.model_bytes(g, **layout))
        s = g1.compile().session(runtime_library=ORACLE_PATH)
        xv = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
        np.testing.assert_array_equal(s.run(xv)[0], xv[:, [-1, 0, 1], :])
        s.close()


def _single(op, **attrs):
    g = compiler.Graph()
    x = g.input("x", (1, 4, 8, 8), np.float32)
    g.output(g.node(op, [x], "y", **attrs))
    return g


def test_what_the_reader_refuses():
    g0, _ = models.single_conv()
    good = ow.model_bytes(g0)
    with pytest.raises(RuntimeError, match="static shape"):
        compiler.load_onnx(ow.model_bytes(g0, dynamic_batch="N"))
    with pytest.raises(RuntimeError, match="auto_pad"):
        compiler.load_onnx(ow.model_bytes(g0, auto_pad="SAME_UPPER"))
    compiler.load_onnx(ow.model_bytes(g0, auto_pad="NOTSET"))           # the default spelled out is fine
    for cut in (1, 7, len(good) // 2, len(good) - 1):                   # truncated files
        with pytest.raises(RuntimeError):
            compiler.load_onnx(good[:cut]).compile()
    with pytest.raises(RuntimeError):
        compiler.load_onnx(b"")
    with pytest.raises(RuntimeError, match="no graph"):
        compiler.load_onnx(ow.f_varint(1, 8))
    # a double tensor
    t = ow.f_bytes(1, ow.varint(1)) + ow.f_varint(2, 11) + ow.f_string(8, "w") + ow.f_bytes(9, b"\0" * 8)
    with pytest.raises(RuntimeError, match="data type 11"):
        compiler.load_onnx(ow.f_bytes(7, ow.f_bytes(5, t)))
    # raw_data of the wrong length
    t = ow.f_bytes(1, ow.varint(3)) + ow.f_varint(2, 1) + ow.f_string(8, "w") + ow.f_bytes(9, b"\0" * 8)
    with pytest.raises(RuntimeError, match="raw_data"):
        compiler.load_onnx(ow.f_bytes(7, ow.f_bytes(5, t)))
    # an operator the DNN dialect has no lowering for is reported by name at compile time
    with pytest.raises(RuntimeError, match="Selu"):
        compiler.load_onnx(ow.model_bytes(_single("Selu"))).compile()
    # Softmax before opset 13 flattens the trailing dims: only the last axis means the same thing
    def soft(axis_attr):
        g = compiler.Graph()
        g.input("x", (2, 3, 4))
        g.output(g.node("Softmax", ["x"], **axis_attr))
        return g
    with pytest.raises(RuntimeError, match="opset 11"):
        compiler.load_onnx(ow.model_bytes(soft({}), opset=11)).compile()          # default axis 1 of a rank-3 input
    assert "axis=2" in compiler.load_onnx(ow.model_bytes(soft({"axis": -1}), opset=11)).compile().text
    assert "axis=-1" in compiler.load_onnx(ow.model_bytes(soft({}), opset=13)).compile().text  # opset 13: last axis
    # a padded AveragePool that leaves the padding out of the count
    def avg(**extra):
        g = compiler.Graph()
        g.input("x", (1, 2, 6, 6))
        g.output(g.node("AveragePool", ["x"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1], **extra))
        return g
    with pytest.raises(RuntimeError, match="count_include_pad"):
        avg().compile()
    assert avg(count_include_pad=1).compile().pool_bytes > 0
    # two outputs on one node
    n = ow.f_string(1, "x") + ow.f_string(2, "y") + ow.f_string(2, "mask") + ow.f_string(4, "MaxPool")
    vi = ow.value_info("x", (1, 1, 4, 4), np.float32)
    with pytest.raises(RuntimeError, match="more than one output"):
        compiler.load_onnx(ow.f_bytes(7, ow.f_bytes(1, n) + ow.f_bytes(11, vi) + ow.f_bytes(12, ow.f_string(1, "y"))))


def test_training_outputs_of_dropout_and_batchnorm_are_tolerated():
    # exporters list Dropout's mask and BatchNormalization's running statistics as further outputs
    r = np.random.default_rng(8)
    c = 3
    stats = [r.uniform(0.5, 1.5, c), r.uniform(-0.2, 0.2, c), r.standard_normal(c) * 0.1, r.uniform(0.5, 1.5, c)]
    names = ["scale", "bias", "mean", "var"]
    graph = b""
    bn = ow.f_string(1, "x") + b"".join(ow.f_string(1, n) for n in names) + ow.f_string(2, "n") + ow.f_string(2, "run_mean") + \
        ow.f_string(2, "run_var") + ow.f_string(4, "BatchNormalization") + ow.f_bytes(5, ow.attribute("epsilon", 1e-3))
    dr = ow.f_string(1, "n") + ow.f_string(2, "d") + ow.f_string(2, "mask") + ow.f_string(4, "Dropout")
    rl = ow.f_string(1, "d") + ow.f_string(2, "y") + ow.f_string(4, "Relu")
    graph += ow.f_bytes(1, bn) + ow.f_bytes(1, dr) + ow.f_bytes(1, rl)
    for n, a in zip(names, stats):
        graph += ow.f_bytes(5, ow.tensor_proto(n, a.astype(np.float32)))
    graph += ow.f_bytes(11, ow.value_info("x", (2, c, 4, 4), np.float32)) + ow.f_bytes(12, ow.f_string(1, "y"))
    g = compiler.load_onnx(ow.f_varint(1, 8) + ow.f_bytes(7, graph))
    p = g.compile()
    assert [n for n, *_ in p.compute_ops()] == ["dnn.mul", "dnn.add", "dnn.activationfwd"]
    x = r.standard_normal((2, c, 4, 4)).astype(np.float32)
    s = p.session(runtime_library=ORACLE_PATH)
    sc, bi, mu, va = (a.reshape(1, c, 1, 1) for a in stats)
    want = np.maximum((x - mu) / np.sqrt(va + 1e-3) * sc + bi, 0)
    np.testing.assert_allclose(s.run(x)[0], want, rtol=1e-5, atol=1e-6)
    s.close()
    # training mode is refused, and so is a reader of a training output
    bad = bn + ow.f_bytes(5, ow.attribute("training_mode", 1))
    with pytest.raises(RuntimeError, match="training mode"):
        compiler.load_onnx(ow.f_varint(1, 8) + ow.f_bytes(7, graph.replace(ow.f_bytes(1, bn), ow.f_bytes(1, bad))))
    rl2 = ow.f_string(1, "mask") + ow.f_string(2, "y") + ow.f_string(4, "Relu")
    with pytest.raises(RuntimeError, match="not defined"):
        compiler.load_onnx(ow.f_varint(1, 8) + ow.f_bytes(7, graph.replace(ow.f_bytes(1, rl), ow.f_bytes(1, rl2)))).compile()


def test_unknown_fields_are_skipped():
    g0, _ = models.single_conv()
    data = ow.model_bytes(g0)
    # doc_string (6), model_version (5), metadata_props (14) and a 64-bit field in front
    junk = ow.f_string(6, "doc") + ow.f_varint(5, 3) + ow.f_bytes(14, ow.f_string(1, "k") + ow.f_string(2, "v")) + \
        ow.tag(31, 1) + b"\1\2\3\4\5\6\7\x08"
    p = compiler.load_onnx(junk + data).compile()
    assert p.pool_bytes == 1753344


def test_command_line_tune_and_algos(tmp_path):
    """python -m occamy_amd model.onnx --resident --tune FILE / --algos FILE: on the host build of the ABI there is
    nothing to tune (no variant is chosen), the file holds two entries per runtime call, and it is accepted back."""
    import json
    import subprocess
    import sys
    g0, _ = models.single_conv()
    model, saved = tmp_path / "m.onnx", tmp_path / "algos.json"
    model.write_bytes(ow.model_bytes(g0))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    base = [sys.executable, "-m", "occamy_amd", str(model), "--runtime", ORACLE_PATH, "--iterations", "1"]
    r = subprocess.run(base + ["--resident", "--tune", str(saved)], capture_output=True, text=True, cwd=root)
    assert r.returncode == 0 and "tuned: 0 operation(s)" in r.stdout, r.stderr
    assert json.loads(saved.read_text()) == {"program_ops": 3, "algos": [[0, 0]] * 3}
    r = subprocess.run(base + ["--resident", "--algos", str(saved)], capture_output=True, text=True, cwd=root)
    assert r.returncode == 0, r.stderr
    r = subprocess.run(base + ["--tune", str(saved)], capture_output=True, text=True, cwd=root)
    assert r.returncode != 0 and "--resident" in r.stderr
