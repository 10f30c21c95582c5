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


def test_device_memory_accounting_of_the_executor():
    # what the executor takes from the runtime's allocator per inference is the planned pool and nothing else
    # (the host build of the ABI counts its heap blocks the way the GPU build counts hipMalloc)
    g, inputs = models.resnet50(image=32, classes=10)
    p = g.compile()
    s = p.session(compiler.MODE_OCCAMY, runtime_library=ORACLE_PATH)
    base, _, static = s.device_bytes(reset_peak=True)
    assert static == 0
    s.run(*inputs)
    now, peak, _ = s.device_bytes()
    assert now == base and peak - base == p.pool_bytes
    s.close()


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


def test_poisoned_pool_changes_nothing():
    """The executor's debug fill: the pool, and then every tensor's slot as it is carved out, is filled with 0xFF
    bytes (NaN in fp32 and fp16) before use.  A kernel that left part of its output unwritten, or an operator placed
    before its producer, would carry NaNs into the result; the result must be the unpoisoned run's, bit for bit."""
    for builder, flags in [(lambda: models.resnet50(image=32, classes=10), dict(fusion=True)),
                           (lambda: models.mobilenet_v2(image=32, classes=10), dict()),
                           (lambda: models.bert_encoder(layers=1, hidden=64, heads=2, ffn=128, seq=16, vocab=50), dict())]:
        g, inputs = builder()
        p = g.compile(**flags)
        s = p.session(compiler.MODE_OCCAMY, runtime_library=ORACLE_PATH)
        plain = s.run(*inputs)
        s.set_debug_fill(0xFF)
        poisoned = s.run(*inputs)
        s.set_debug_fill(-1)
        s.close()
        for a, b in zip(plain, poisoned):
            assert np.isfinite(b).all()
            np.testing.assert_array_equal(a, b)


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


ALEX = lambda: models.alexnet(image=96, classes=10, hidden=64)                    # noqa: E731
YOLO = lambda: models.yolo_v1(batch=2, image=64, width=0.0625, fc=32)             # noqa: E731
SRGAN = lambda: models.srgan_generator(height=8, width=6, feats=16, blocks=2)     # noqa: E731


@pytest.mark.parametrize("builder", [ALEX, YOLO, SRGAN], ids=["alexnet", "yolo_v1", "srgan"])
def test_reference_test_models_small(builder):
    a = check(builder)
    b = check(builder, fusion=True)
    for x, y in zip(a, b):
        np.testing.assert_allclose(x, y, rtol=1e-4, atol=1e-5 * max(1.0, float(np.abs(x).max())))
    _, _, c = run_oracle(builder, mode=compiler.MODE_RESIDENT)
    for x, y in zip(a, c):
        np.testing.assert_array_equal(x, y)


def test_returned_tensor_that_is_read_again_stays_alive():
    # SRGAN returns the feature map and keeps reading it; freeing it at the
    # copy to the host (what the reference's dealloc placement does) lets the
    # pool hand its bytes to a later tensor.  Every flag combination must agree.
    base = check(SRGAN)
    for flags in [dict(dealloc_opt=False), dict(const_at_use=False), dict(pool_opt=True, dealloc_opt=True)]:
        _, _, out = run_oracle(SRGAN, **flags)
        for x, y in zip(base, out):
            np.testing.assert_array_equal(x, y)


def test_widened_operator_surface():
    """LeakyRelu, PRelu (shared and per-channel slope), Concat, Squeeze,
    Unsqueeze, Identity, Dropout, and BatchNormalization in its three shapes:
    folded into the convolution before it, kept apart because the
    convolution's result has a second reader, and on a non-convolution."""
    def build():
        r = np.random.default_rng(5)
        g = compiler.Graph()
        x = r.standard_normal((2, 4, 6, 6)).astype(np.float32)
        g.input("x", x.shape)

        def bn(v, c):
            return g.node("BatchNormalization", [v] + [g.constant(a.astype(np.float32)) for a in (
                r.uniform(0.5, 1.5, c), r.uniform(-0.2, 0.2, c), r.standard_normal(c) * 0.1, r.uniform(0.5, 1.5, c))],
                epsilon=1e-3)

        w1 = g.constant((r.standard_normal((8, 4, 3, 3)) * 0.2).astype(np.float32))
        b1 = g.constant((r.standard_normal(8) * 0.1).astype(np.float32))
        c1 = g.node("Conv", ["x", w1, b1], pads=[1, 1, 1, 1])
        f1 = g.node("LeakyRelu", [bn(c1, 8)], alpha=0.2)                       # folds (bias present)
        w2 = g.constant((r.standard_normal((8, 8, 1, 1)) * 0.3).astype(np.float32))
        c2 = g.node("Conv", [f1, w2])
        n2 = bn(c2, 8)                                                         # c2 has two readers: Mul + Add
        cat = g.node("Concat", [n2, g.node("Identity", [c2]), f1], axis=1)     # 24 channels
        pr = g.node("PRelu", [cat, g.constant(r.uniform(0.1, 0.4, (24, 1, 1)).astype(np.float32))])
        pool = g.node("GlobalAveragePool", [pr])                               # [2,24,1,1]
        sq = g.node("Squeeze", [pool, g.constant(np.array([2, 3], np.int64))])  # [2,24]
        d = g.node("Dropout", [bn(sq, 24)])                                    # BN on a rank-2 tensor
        un = g.node("Unsqueeze", [d], axes=[0, 3])                             # [1,2,24,1]
        sh = g.node("PRelu", [un, g.constant(np.array([0.3], np.float32))])
        g.output(g.node("Squeeze", [sh]))                                      # every 1 goes: [2,24]
        g.output(g.node("Identity", [pr]))                                     # a returned Identity is a copy
        g.output(g.node("Concat", [sq, sq], axis=-1))
        return g, [x]
    out = check(build)
    assert out[0].shape == (2, 24) and out[1].shape == (2, 24, 6, 6) and out[2].shape == (2, 48)
    g, _ = build()
    text = g.compile().text
    assert "BatchNormalization" not in text and text.count("dnn.convfwd") == 2
    assert text.count("dnn.concat") == 2 and text.count("dnn.squeeze") == 2 and text.count("dnn.unsqueeze") == 1
    assert text.count("dnn.prelu") == 2 and text.count("dnn.leakyrelu") == 1


def expand_pad_graph():
    r = np.random.default_rng(6)
    g = compiler.Graph()
    x = r.standard_normal((2, 1, 5)).astype(np.float32)
    g.input("x", x.shape)
    p = g.node("Pad", ["x", g.constant(np.zeros(6, np.int64))])                     # zero pads: the input itself
    e = g.node("Expand", [p, g.constant(np.array([3, 2, 4, 5], np.int64))])         # [3,2,4,5]
    m = g.node("Mul", [e, g.constant(r.standard_normal((4, 1)).astype(np.float32))])
    g.output(g.node("Relu", [m]))
    g.output(g.node("Expand", ["x", g.constant(np.array([1, 1, 1], np.int64))]))    # shape of ones: a copy
    return g, [x]


def test_expand_and_zero_pad():
    """Expand broadcasts (the shape constant stays a device operand, as in
    Ops/cuda/Expand.cpp:40-47); a Pad with zero pads is its input
    (Ops/cuda/Pad.cpp:48-52) and any other Pad is refused."""
    out = check(expand_pad_graph)
    assert out[0].shape == (3, 2, 4, 5) and out[1].shape == (2, 1, 5)
    g, _ = expand_pad_graph()
    text = g.compile().text
    assert text.count("dnn.expand") == 2 and "Pad" not in text
    # the expanded tensor outlives the call: its buffer is released after the Mul that reads it
    lines = expand_pad_graph()[0].compile(pool_opt=False).text.splitlines()
    first = next(i for i, l in enumerate(lines) if "dnn.expand" in l)
    mul = next(i for i, l in enumerate(lines) if "dnn.mul" in l)
    buf = lines[first].split("dnn.expand")[1].split(" :")[0].split(",")[-1].strip()
    freed = next(i for i, l in enumerate(lines) if "dnn.dealloc" in l and l.split("dnn.dealloc")[1].split()[0] == buf)
    assert freed > mul
    g = compiler.Graph()
    g.input("x", (1, 3, 4, 4))
    g.output(g.node("Pad", ["x", g.constant(np.array([0, 0, 1, 1, 0, 0, 1, 1], np.int64))]))
    with pytest.raises(RuntimeError, match="Pad"):
        g.compile()


@pytest.mark.parametrize("builder", [lambda: models.mobilenet_v2(image=32, classes=10), YOLO, SRGAN,
                                     lambda: models.resnet50(image=32, classes=10)],
                         ids=["mobilenet_v2", "yolo_v1", "srgan", "resnet50"])
def test_activation_fusion_matches_unfused_chain(builder):
    # The oracle runs a fused conv + clipped / leaky ReLU as the reference's
    # separate calls, so the flags must not change a single bit on the CPU.
    _, _, a = run_oracle(builder, fusion=True)
    _, _, b = run_oracle(builder, fusion=True, fuse_activations=True, fuse_residual=True)
    for x, y in zip(a, b):
        np.testing.assert_array_equal(x, y)
    check(builder, fusion=True, fuse_activations=True, fuse_residual=True)
    _, _, c = run_oracle(builder, mode=compiler.MODE_RESIDENT, fusion=True, fuse_activations=True, fuse_residual=True)
    for x, y in zip(a, c):
        np.testing.assert_array_equal(x, y)


def test_projection_shortcut_fusion_matches_unfused_chain():
    """The oracle runs the fused shortcut + closer call as the chain of the two calls: not a bit may change, per
    inference (with the debug fill), without the dealloc pass, and resident; four launches fewer."""
    small = lambda: models.resnet50(image=32, classes=10)  # noqa: E731
    flags = dict(fusion=True, fuse_residual=True)
    _, _, a = run_oracle(small, **flags)
    assert small()[0].compile(fuse_projection_shortcut=True, **flags).text.count("add-conv") == 4
    for more in (dict(), dict(dealloc_opt=False)):
        _, _, b = run_oracle(small, fuse_projection_shortcut=True, **flags, **more)
        np.testing.assert_array_equal(a[0], b[0])
    _, _, c = run_oracle(small, mode=compiler.MODE_RESIDENT, fuse_projection_shortcut=True, **flags)
    np.testing.assert_array_equal(a[0], c[0])
    check(small, fuse_projection_shortcut=True, **flags)
    g, inputs = small()
    s = g.compile(fuse_projection_shortcut=True, **flags).session(compiler.MODE_OCCAMY, runtime_library=ORACLE_PATH)
    s.set_debug_fill(0xFF)
    np.testing.assert_array_equal(s.run(*inputs)[0], a[0])
    s.close()


def test_inplace_residual_changes_nothing():
    """A closing convolution that writes over its residual operand: the oracle (which takes Z == Y like
    cudnnConvolutionBiasActivationForward does) gives the same bits per inference with a poisoned pool, without the
    dealloc pass and resident, for ResNet-50 with and without the fused shortcut pairs and for MobileNetV2; the
    pool never holds the sixteen (ten) buffers the pass removes."""
    for small, flags in ((lambda: models.resnet50(image=32, classes=10), dict(fusion=True, fuse_residual=True)),
                         (lambda: models.resnet50(image=32, classes=10), dict(fusion=True, fuse_residual=True, fuse_projection_shortcut=True, alias_copies=True)),
                         (lambda: models.mobilenet_v2(image=32, classes=10), dict(fusion=True, fuse_residual=True, fuse_activations=True))):
        _, _, a = run_oracle(small, **flags)
        for more in (dict(), dict(dealloc_opt=False)):
            _, _, b = run_oracle(small, inplace_residual=True, **flags, **more)
            np.testing.assert_array_equal(a[0], b[0])
        _, _, c = run_oracle(small, mode=compiler.MODE_RESIDENT, inplace_residual=True, **flags)
        np.testing.assert_array_equal(a[0], c[0])
        check(small, inplace_residual=True, **flags)
        g, inputs = small()
        p = g.compile(inplace_residual=True, **flags)
        mallocs = lambda prog: sum(1 for k, _, _, _ in prog.events() if k == 0)  # noqa: E731
        assert mallocs(p) < mallocs(small()[0].compile(**flags))
        s = p.session(compiler.MODE_OCCAMY, runtime_library=ORACLE_PATH)
        s.set_debug_fill(0xFF)
        np.testing.assert_array_equal(s.run(*inputs)[0], a[0])
        s.close()


def test_bert_fp16_fused_paths_on_the_oracle():
    """A small fp16 BERT through the oracle: the program with the recomposed LayerNorm / GELU, the fused
    matmul-bias and the fused attention call (packed Q | K | V, whose three views are offsets in elements of the
    tensors' type) stays within the fp16 chain's rounding of the unfused program, and both of the fp32 network on
    the same weights."""
    small = lambda dt: models.bert_encoder(layers=2, hidden=64, heads=2, seq=16, vocab=50, ffn=128, dtype=dt)  # noqa: E731
    g16, inputs = small(np.float16)
    g32 = compiler.Graph()
    for name, (shape, dt) in g16.input_shapes.items():
        g32.input(name, shape, dt if np.dtype(dt).kind == "i" else np.float32)
    for name, arr in g16.constants.items():
        g32.constant(arr if arr.dtype.kind == "i" else arr.astype(np.float32), name)
    for op, ins, out, at in g16.nodes:
        g32.node(op, ins, out, **at)
    for o in g16.outputs:
        g32.output(o)
    want = g32.compile().session(runtime_library=ORACLE_PATH).run(*inputs)[0]
    _, _, plain = run_oracle(lambda: small(np.float16))
    np.testing.assert_allclose(plain[0].astype(np.float32), want, rtol=2e-2, atol=3e-2)
    flags = dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True, alias_copies=True)
    assert "attention" in small(np.float16)[0].compile(**flags).text
    _, _, fused = run_oracle(lambda: small(np.float16), **flags)
    np.testing.assert_allclose(fused[0].astype(np.float32), want, rtol=2e-2, atol=3e-2)


def test_ssd_resnet50_program():
    """SSD300 on ResNet-50 as the reference's test exports it (the network only: decoding and non-maximum
    suppression are Python in test/models/ssd-resnet50/run.py): 8732 boxes at 300 x 300, two results; the fused
    program (residual blocks, shortcut pairs, first layer with its pooling, in-place sums) gives the oracle's
    unfused result to the fp32 tolerance."""
    build = lambda: models.ssd_resnet50(1, labels=7)  # noqa: E731
    g, inputs = build()
    plain = g.compile()
    assert [shape for shape, _ in plain.output_info()] == [(1, 4, 8732), (1, 7, 8732)]
    flags = dict(fusion=True, fuse_residual=True, fuse_first_layer_maxpool=True, fuse_projection_shortcut=True, inplace_residual=True, compact_pool=True)
    fused = build()[0].compile(**flags)
    assert fused.num_ops(compute_only=True) < plain.num_ops(compute_only=True) // 2
    assert fused.text.count("add-conv") == 3 and "maxpoolfwd" in fused.text
    a = plain.session(runtime_library=ORACLE_PATH).run(*inputs)
    b = fused.session(runtime_library=ORACLE_PATH).run(*inputs)
    for x, y in zip(a, b):
        np.testing.assert_allclose(y, x, rtol=1e-4, atol=1e-4 * float(np.abs(x).max()))


def test_compact_pool_changes_nothing():
    """Offsets from the planner that knows every lifetime: the same bits from the oracle, per inference with a
    poisoned pool and resident, for ResNet-50 with every fusion, MobileNetV2, BERT and YOLOv1."""
    cases = [(lambda: models.resnet50(image=32, classes=10), dict(fusion=True, fuse_residual=True, fuse_projection_shortcut=True, alias_copies=True, inplace_residual=True)),
             (lambda: models.mobilenet_v2(image=32, classes=10), dict(fusion=True, fuse_residual=True, fuse_activations=True)),
             (lambda: models.bert_encoder(layers=2, hidden=64, heads=2, seq=16, vocab=50, ffn=128), dict(recompose=True, fusion=True)),
             (YOLO, dict(fusion=True, fuse_activations=True))]
    for small, flags in cases:
        _, _, a = run_oracle(small, **flags)
        _, _, b = run_oracle(small, compact_pool=True, **flags)
        _, _, c = run_oracle(small, mode=compiler.MODE_RESIDENT, compact_pool=True, **flags)
        for x, y, z in zip(a, b, c):
            np.testing.assert_array_equal(x, y)
            np.testing.assert_array_equal(x, z)
        g, inputs = small()
        p = g.compile(compact_pool=True, **flags)
        s = p.session(compiler.MODE_OCCAMY, runtime_library=ORACLE_PATH)
        s.set_debug_fill(0xFF)
        for x, y in zip(s.run(*inputs), a):
            np.testing.assert_array_equal(x, y)
        assert s.last_pool_bytes == p.pool_bytes
        s.close()


@pytest.mark.parametrize("builder,copies", [(lambda: models.resnet50(image=32, classes=10), 1), (ALEX, 1),
                                            (lambda: models.bert_encoder(layers=2, hidden=64, heads=2, seq=16, vocab=50, ffn=128), None),
                                            (YOLO, None)],
                         ids=["resnet50", "alexnet", "bert", "yolo_v1"])
def test_aliased_copies_change_nothing(builder, copies):
    """Flatten / Reshape / Squeeze / Unsqueeze on their input's buffer: every copy leaves the launch count and its
    buffer leaves the pool's event trace, the results keep every bit (per inference, with the dealloc pass on and
    off, and resident), and no tensor is read after its buffer was released (the debug fill would turn that
    into NaN)."""
    _, _, a = run_oracle(builder, fusion=True)
    plain = builder()[0].compile(fusion=True)
    aliased = builder()[0].compile(fusion=True, alias_copies=True)
    n = sum(plain.text.count(k) for k in ("dnn.flatten", "dnn.reshape", "dnn.squeeze", "dnn.unsqueeze"))
    assert n >= 1 and (copies is None or n == copies)
    gone = plain.num_ops(compute_only=True) - aliased.num_ops(compute_only=True)
    assert 1 <= gone <= n and (copies is None or gone == copies)
    assert len(aliased.events()) == len(plain.events()) - 2 * gone
    assert aliased.pool_bytes <= plain.pool_bytes
    for flags in (dict(), dict(dealloc_opt=False)):
        _, _, b = run_oracle(builder, fusion=True, alias_copies=True, **flags)
        for x, y in zip(a, b):
            np.testing.assert_array_equal(x, y)
    _, _, c = run_oracle(builder, mode=compiler.MODE_RESIDENT, fusion=True, alias_copies=True)
    for x, y in zip(a, c):
        np.testing.assert_array_equal(x, y)
    g, inputs = builder()
    s = g.compile(fusion=True, alias_copies=True).session(compiler.MODE_OCCAMY, runtime_library=ORACLE_PATH)
    s.set_debug_fill(0xFF)
    for x, y in zip(a, s.run(*inputs)):
        np.testing.assert_array_equal(x, y)
    s.close()


def test_aliased_copy_that_is_returned():
    """A Flatten whose result the function returns: the copy to the host reads the copy's own buffer, so the copy
    cannot share its input's (it stays a copy); one that also feeds the classifier among them."""
    small = lambda: models.resnet50(2, image=32, classes=10, stage_means=True)  # noqa: E731
    want = check(small)
    assert len(want) == 5
    for flags in (dict(alias_copies=True), dict(fusion=True, alias_copies=True, dealloc_opt=False)):
        for mode in (compiler.MODE_OCCAMY, compiler.MODE_RESIDENT):
            _, _, got = run_oracle(small, mode=mode, **flags)
            for a, b in zip(got, want):
                if flags.get("fusion"):
                    np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-3)
                else:
                    np.testing.assert_array_equal(a, b)


def _residual_around_a_reshape():
    # t = Relu(x); y = Reshape(t); a chain of unary operators on y; out = Add(t, Reshape(chain)): t is read again
    # after the copy of it has had its last reader, the shape of a residual branch around a reshape
    g = compiler.Graph()
    x = g.input("x", (2, 8, 16))
    t = g.node("Relu", [x])
    y = g.node("Reshape", [t, g.constant(np.array([16, 16], np.int64))])
    for op in ("Sigmoid", "Tanh", "Sigmoid", "Tanh"):
        y = g.node(op, [y])
    back = g.node("Reshape", [y, g.constant(np.array([2, 8, 16], np.int64))])
    g.output(g.node("Add", [t, back]))
    rng = np.random.default_rng(11)
    return g, [rng.standard_normal((2, 8, 16)).astype(np.float32)]


def test_aliased_copy_whose_input_is_read_again_later():
    """A copy that shares its input's buffer is a second writer of that buffer; the buffer must outlive the readers
    of every writer's result, not only those of the last one."""
    check(_residual_around_a_reshape)
    _, _, a = run_oracle(_residual_around_a_reshape)
    for mode in (compiler.MODE_OCCAMY, compiler.MODE_RESIDENT):
        _, _, b = run_oracle(_residual_around_a_reshape, mode=mode, alias_copies=True)
        np.testing.assert_array_equal(a[0], b[0])
    g, inputs = _residual_around_a_reshape()
    p = g.compile(alias_copies=True)
    assert p.num_ops(compute_only=True) == _residual_around_a_reshape()[0].compile().num_ops(compute_only=True) - 2
    s = p.session(compiler.MODE_OCCAMY, runtime_library=ORACLE_PATH)
    s.set_debug_fill(0xFF)
    np.testing.assert_array_equal(a[0], s.run(*inputs)[0])
    s.close()


@pytest.mark.parametrize("builder", [lambda: models.resnet50(image=32, classes=10), ALEX,
                                     lambda: models.mobilenet_v2(image=32, classes=10)],
                         ids=["resnet50", "alexnet", "mobilenet_v2"])
def test_gemm_bias_fusion_matches_unfused_chain(builder):
    # Gemm is a product and an in-place bias add in the reference (Ops/cublas/Gemm.cpp:60-81); folded
    # into one call the oracle still runs the chain, so not a bit may change and one launch per Gemm goes
    _, _, a = run_oracle(builder, fusion=True)
    _, _, b = run_oracle(builder, fusion=True, fuse_matmul_bias=True)
    for x, y in zip(a, b):
        np.testing.assert_array_equal(x, y)
    ta, tb = builder()[0].compile(fusion=True).text, builder()[0].compile(fusion=True, fuse_matmul_bias=True).text
    gemms = ta.count("dnn.matmul2d")
    assert gemms >= 1 and tb.count("dnn.matmul2d") == gemms
    assert ta.count("dnn.add") - tb.count("dnn.add") == gemms and "dimC=[1," in tb
    check(builder, fusion=True, fuse_matmul_bias=True)


def test_recomposed_bert_matches_torch_and_the_decomposed_program():
    small = dict(layers=2, hidden=64, heads=4, ffn=128, seq=16, vocab=100)
    flags = dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True)
    a = check(lambda: models.bert_encoder(**small), rtol=1e-4, atol=1e-4)
    b = check(lambda: models.bert_encoder(**small), rtol=1e-4, atol=1e-4, **flags)
    np.testing.assert_allclose(a[0], b[0], rtol=1e-4, atol=1e-4)
    _, _, c = run_oracle(lambda: models.bert_encoder(**small), mode=compiler.MODE_RESIDENT, **flags)
    np.testing.assert_array_equal(b[0], c[0])


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
