"""Whole programs on the CPU: compiler + executor + oracle runtime against an
independent torch evaluation of the same ONNX-level graph (graph_eval.py).
This pins the emission rules' arithmetic meaning (operand order, broadcast
dims, fusion, pool aliasing): a wrong offset or an early dealloc corrupts a
tensor and shows up as a numeric mismatch."""
import numpy as np
import pytest

import graph_eval
from helpers import ORACLE_PATH
from occamy_amd import compiler, models

RTOL, ATOL = 1e-4, 1e-5


def run_oracle(builder, mode=compiler.MODE_OCCAMY, **flags):
    g, inputs = builder()
    p = g.compile(**flags)
    s = p.session(mode, runtime_library=ORACLE_PATH)
    out = s.run(*inputs)
    if mode == compiler.MODE_OCCAMY:
        assert s.last_pool_bytes == p.pool_bytes  # the arena the runtime is asked for is the planned pool
    s.close()
    return g, inputs, out


def check(builder, rtol=RTOL, atol=ATOL, **flags):
    g, inputs, out = run_oracle(builder, **flags)
    ref = graph_eval.evaluate(g, inputs)
    for o, r in zip(out, ref):
        scale = max(1.0, float(np.abs(r).max()))
        np.testing.assert_allclose(o, r, rtol=rtol, atol=atol * scale)
    return out


def test_single_conv():
    a = check(models.single_conv)
    b = check(models.single_conv, fusion=True)
    np.testing.assert_allclose(a[0], b[0], rtol=1e-5, atol=1e-6)  # fused rounds once, unfused twice
    assert a[0].shape == (1, 64, 56, 56) and (a[0] >= 0).all()


def test_modes_and_flags_agree():
    small = lambda: models.resnet50(image=32, classes=10)  # noqa: E731
    base = check(small)
    for flags in [dict(fusion=True), dict(dealloc_opt=False), dict(const_at_use=False), dict(fusion=True, dealloc_opt=False)]:
        _, _, out = run_oracle(small, **flags)
        if flags.get("fusion"):  # the fused op rounds once where conv + add round twice
            np.testing.assert_allclose(out[0], base[0], rtol=1e-4, atol=1e-3)
        else:                    # scheduling flags must not change a single bit
            np.testing.assert_array_equal(out[0], base[0])
    _, _, out = run_oracle(small, mode=compiler.MODE_RESIDENT)
    np.testing.assert_array_equal(out[0], base[0])
    _, _, out = run_oracle(small, mode=compiler.MODE_RESIDENT, fusion=True)
    np.testing.assert_allclose(out[0], base[0], rtol=1e-4, atol=1e-3)


def test_resnet50_small_image():
    check(lambda: models.resnet50(image=64, classes=100))
    check(lambda: models.resnet50(batch=2, image=32, classes=10), fusion=True)


def test_mobilenet_small_image():
    check(lambda: models.mobilenet_v2(image=64, classes=100))
    check(lambda: models.mobilenet_v2(image=32, classes=10), fusion=True)


def test_bert_small():
    small = dict(layers=2, hidden=64, heads=4, ffn=128, seq=16, vocab=100)
    a = check(lambda: models.bert_encoder(**small), rtol=1e-4, atol=1e-4)
    b = check(lambda: models.bert_encoder(fused=True, **small), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(a[0], b[0], rtol=1e-4, atol=1e-4)


def test_every_emission_rule_once():
    """A graph that touches the operators the models above do not."""
    def build():
        g = compiler.Graph()
        x = np.random.default_rng(0).standard_normal((2, 4, 9, 9)).astype(np.float32)
        g.input("x", x.shape)
        idx = np.array([[3, 0], [1, 1]], np.int64)
        g.input("idx", idx.shape, np.int64)
        w = g.constant(np.random.default_rng(1).standard_normal((6, 4, 3, 3)).astype(np.float32) * 0.2)
        c = g.node("Conv", ["x", w], pads=[0, 0, 0, 0], strides=[2, 2])          # no bias, stride 2
        t = g.node("Tanh", [g.node("Sigmoid", [c])])
        a = g.node("AveragePool", [t], kernel_shape=[2, 2], strides=[2, 2])
        m = g.node("Mul", [a, g.constant(np.full((1, 6, 1, 1), 1.5, np.float32))])
        s = g.node("Sub", [m, g.constant(np.full((6, 1, 1), 0.25, np.float32))])
        d = g.node("Div", [s, g.constant(np.array(2.0, np.float32))])
        q = g.node("Sqrt", [g.node("Pow", [d, g.constant(np.array(2.0, np.float32))])])
        f = g.node("Flatten", [q], axis=1)
        r = g.node("Reshape", [f, g.constant(np.array([2, 6, -1], np.int64))])
        tr = g.node("Transpose", [r], perm=[0, 2, 1])
        sm = g.node("Softmax", [tr], axis=1)
        gt = g.node("Gather", [sm, "idx"], axis=2)
        e = g.node("Erf", [gt])
        rm = g.node("ReduceMean", [e], axes=[1], keepdims=0)
        g.output(rm)
        g.output(g.node("Clip", [c, g.constant(np.array(-0.5, np.float32)), g.constant(np.array(0.5, np.float32))]))
        return g, [x, idx]
    out = check(build)
    assert out[0].shape == (2, 2, 2) and out[1].shape == (2, 6, 4, 4)


def test_executor_errors():
    g, inputs = models.single_conv()
    p = g.compile(pool_opt=False)
    with pytest.raises(RuntimeError, match="pool pass"):
        p.session(runtime_library=ORACLE_PATH)
    g, inputs = models.single_conv()
    p = g.compile()
    with pytest.raises(RuntimeError, match="cannot load"):
        p.session(runtime_library="/nonexistent/libdnnrt.so")
    s = p.session(runtime_library=ORACLE_PATH)
    with pytest.raises(RuntimeError, match="occamy mode"):
        s.run_device([0], [0])


def test_residual_fusion_matches_unfused_chain():
    # The oracle runs the fused closer of a residual block as the reference's
    # three calls, so the flag must not change a single bit on the CPU.
    small = lambda: models.resnet50(batch=2, image=32, classes=10)  # noqa: E731
    _, _, a = run_oracle(small, fusion=True)
    _, _, b = run_oracle(small, fusion=True, fuse_residual=True)
    np.testing.assert_array_equal(a[0], b[0])
    check(small, fusion=True, fuse_residual=True)
    mb = lambda: models.mobilenet_v2(image=32, classes=10)  # noqa: E731
    _, _, a = run_oracle(mb, fusion=True)
    _, _, b = run_oracle(mb, fusion=True, fuse_residual=True)
    np.testing.assert_array_equal(a[0], b[0])
