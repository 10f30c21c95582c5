"""Whole programs on the MI355X: the same compiled DNN program is executed
through the C ABI against the gfx950 library and against the CPU oracle, on
the same seeded inputs.  Tolerances: rtol 1e-4 / atol 1e-5 (scaled by the
output's magnitude) for fp32; rtol 2e-2 with an absolute floor of 4e-3 of the largest reference value for fp16."""
import numpy as np
import pytest

from helpers import ORACLE_PATH
from occamy_amd import compiler, models
from test_e2e_cpu import expand_pad_graph

pytestmark = pytest.mark.gpu


def run(builder, runtime=None, mode=compiler.MODE_OCCAMY, **flags):
    g, inputs = builder()
    p = g.compile(**flags)
    s = p.session(mode, runtime_library=runtime)
    out = s.run(*inputs)
    info = dict(pool=p.pool_bytes, requested=s.last_pool_bytes, weights=s.weights_bytes)
    s.close()
    return out, info


def close(got, ref, rtol=1e-4, atol=1e-5):
    scale = max(1.0, float(np.abs(ref).max()))
    np.testing.assert_allclose(got, ref, rtol=rtol, atol=atol * scale)


CONFIGS = {
    "single_conv": models.single_conv,
    "resnet50": models.resnet50,
    "mobilenet_v2": models.mobilenet_v2,
    "bert_2_layers": lambda: models.bert_encoder(layers=2),
    # the reference's other test models (test/models/{alexnet,yolo,srgan}/run.py) at their own sizes
    "alexnet": models.alexnet,
    "yolo_v1": lambda: models.yolo_v1(batch=1),
    "srgan": lambda: models.srgan_generator(height=64, width=48),
    "expand_pad": expand_pad_graph,
}


@pytest.fixture(scope="module")
def oracle_outputs():
    return {k: run(b, ORACLE_PATH)[0] for k, b in CONFIGS.items()}


@pytest.mark.parametrize("name", list(CONFIGS))
def test_occamy_mode_matches_oracle(name, oracle_outputs):
    out, info = run(CONFIGS[name])
    assert info["requested"] == info["pool"]  # device arena == planned pool, byte for byte
    for o, r in zip(out, oracle_outputs[name]):
        close(o, r)


@pytest.mark.parametrize("name", ["single_conv", "resnet50", "mobilenet_v2", "bert_2_layers"])
def test_device_memory_is_the_planned_pool(name):
    """Every byte the runtime library takes from the device allocator is counted (dnnrtDeviceMemoryStats).  Per
    inference (the reference's semantics) the peak of a run is the planned pool, to the byte, and nothing is held
    before or after it: the handle's reduction scratch is the library's static array (8 MiB + 64 KiB, plus the
    1 MiB + 4 KiB of the entry point that allocates nothing), not an allocation.  Resident: pool + the constants'
    arena, held for the session's life."""
    g, inputs = CONFIGS[name]()
    p = g.compile()
    s = p.session(compiler.MODE_OCCAMY)
    base, _, static = s.device_bytes(reset_peak=True)
    assert static == (8 << 20) + (64 << 10) + (1 << 20) + (4 << 10)
    s.run(*inputs)
    now, peak, _ = s.device_bytes()
    assert now == base and peak - base == p.pool_bytes == s.last_pool_bytes
    s.close()
    s = p.session(compiler.MODE_RESIDENT)
    s.run(*inputs)
    now, peak, _ = s.device_bytes()
    assert now - base == peak - base == p.pool_bytes + s.weights_bytes
    s.close()


@pytest.mark.parametrize("name", list(CONFIGS))
def test_fused_program_matches_oracle(name, oracle_outputs):
    out, _ = run(CONFIGS[name], fusion=True)
    for o, r in zip(out, oracle_outputs[name]):
        close(o, r)


@pytest.mark.parametrize("name", ["single_conv", "resnet50", "bert_2_layers", "srgan"])
def test_resident_mode_and_graph_replay(name, oracle_outputs):
    import torch
    g, inputs = CONFIGS[name]()
    p = g.compile(fusion=True)
    s = p.session(compiler.MODE_RESIDENT)
    out = s.run(*inputs)
    for o, r in zip(out, oracle_outputs[name]):
        close(o, r)
    # device-resident inputs, captured graph, several replays with other work in between
    dev_in = [torch.from_numpy(a).cuda() for a in inputs]
    dev_out = [torch.empty(o.shape, dtype=torch.from_numpy(o).dtype, device="cuda") for o in out]
    torch.cuda.synchronize()
    for it in range(4):
        for t in dev_out:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        s.run_device([t.data_ptr() for t in dev_in], [t.data_ptr() for t in dev_out], use_graph=True)
        s.sync()
        for t, o in zip(dev_out, out):
            np.testing.assert_array_equal(t.cpu().numpy(), o)  # replay == eager, bit for bit
    s.run_device([t.data_ptr() for t in dev_in], [t.data_ptr() for t in dev_out], use_graph=False)
    s.sync()
    np.testing.assert_array_equal(dev_out[0].cpu().numpy(), out[0])
    s.close()


def test_poisoned_pool_changes_nothing_on_the_gpu():
    """Every kernel writes all of its output and no operator reads a slot before its producer ran: with the pool and
    every freshly carved slot filled with 0xFF bytes (NaN) the results are those of the plain run, bit for bit.
    fp32 networks with and without the fused calls, BERT with its fused paths, fp16 channels-last."""
    cases = [(lambda: models.resnet50(image=64, classes=100), dict()),
             (lambda: models.resnet50(image=64, classes=100), dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True)),
             (lambda: models.mobilenet_v2(image=64, classes=100), dict(fusion=True, fuse_residual=True, fuse_activations=True)),
             (lambda: models.bert_encoder(layers=2), dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True)),
             (lambda: models.resnet50(4, np.float16, seed=5, image=64), dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, channels_last=True)),
             (lambda: models.resnet50(4, np.float16, seed=5, image=64),
              dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, channels_last=True, fuse_first_layer_maxpool=True)),
             (lambda: models.resnet50(image=64, classes=100),
              dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, fuse_first_layer_maxpool=True, fuse_projection_shortcut=True)),
             (lambda: models.srgan_generator(1, np.float32, height=24, width=16), dict(fusion=True, fuse_activations=True))]
    for builder, flags in cases:
        g, inputs = builder()
        s = g.compile(**flags).session(compiler.MODE_OCCAMY)
        plain = s.run(*inputs)
        s.set_debug_fill(0xFF)
        poisoned = s.run(*inputs)
        s.close()
        for a, b in zip(plain, poisoned):
            assert np.isfinite(b.astype(np.float32)).all()
            np.testing.assert_array_equal(a, b)


def test_bert_fused_layernorm_gelu(oracle_outputs):
    out, _ = run(lambda: models.bert_encoder(layers=2, fused=True))
    close(out[0], oracle_outputs["bert_2_layers"][0], 1e-4, 1e-4)


def test_new_input_same_session():
    g, inputs = models.single_conv()
    p = g.compile()
    s = p.session()
    so = p.session(runtime_library=ORACLE_PATH)
    for seed in (7, 8):
        x = np.random.default_rng(seed).standard_normal(inputs[0].shape).astype(np.float32)
        close(s.run(x)[0], so.run(x)[0])
    s.close()
    so.close()


def as_fp32_graph(g16, inputs):
    """The same graph with every constant and input widened to fp32 (the values stay fp16-representable)."""
    g = compiler.Graph()
    for name, (shape, _) in g16.input_shapes.items():
        g.input(name, shape, np.float32)
    for name, arr in g16.constants.items():
        g.constant(arr.astype(np.float32), name)
    for op, ins, out, at in g16.nodes:
        g.node(op, ins, out, **at)
    for o in g16.outputs:
        g.output(o)
    return g, [a.astype(np.float32) for a in inputs]


def close16(got, want):
    """fp16 storage against the fp32 oracle on the same fp16-representable weights and input: rtol 2e-2 with an
    absolute floor of 4e-3 of the largest reference value (the networks measure 4e-4 .. 7e-4 of it: every
    activation is rounded to fp16 between layers), and the same arg-max along the last axis nearly everywhere."""
    got, want = got.astype(np.float32), want.astype(np.float32)
    assert np.isfinite(got).all()
    np.testing.assert_allclose(got, want, rtol=2e-2, atol=4e-3 * float(np.abs(want).max()))


def test_resnet50_fp16_batch_64_every_stage():
    """Batch 64 with the benchmark's flags, and the per-channel spatial mean of every residual stage's result
    returned beside the logits: each stage is compared at its own magnitude (rtol 2e-2 of values that are means
    of non-negative activations), so a wrong late layer cannot hide behind the size of the logits."""
    flags = dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, channels_last=True, fuse_first_layer_maxpool=True,
                 fuse_projection_shortcut=True, alias_copies=True, inplace_residual=True, compact_pool=True)
    build16 = lambda: models.resnet50(64, np.float16, seed=5, stage_means=True)  # noqa: E731
    out16, info = run(build16, **flags)
    assert info["requested"] == info["pool"]
    ref, _ = run(lambda: as_fp32_graph(*build16()), ORACLE_PATH, fusion=True)
    assert [o.shape for o in out16] == [(64, 1000), (64, 256), (64, 512), (64, 1024), (64, 2048)]
    for got, want in zip(out16, ref):
        close16(got, want)
    for got, want in zip(out16[1:], ref[1:]):  # means of ReLU outputs: compare where the mean is not nearly zero
        got, want = got.astype(np.float32), want
        big = want > 0.05 * want.max()
        assert big.mean() > 0.5
        np.testing.assert_allclose(got[big], want[big], rtol=2e-2)


def test_resnet50_fp16_batch_64_as_benchmarked():
    """The throughput configuration at its own size and with the benchmark's own flags (64 x 3 x 224 x 224,
    fp16 storage, fp32 accumulation, channels-last, every fusion bench.py switches on), against the fp32
    oracle on the same fp16-representable weights and input: rtol 2e-2, atol 4e-3 of the largest logit."""
    flags = dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, channels_last=True, fuse_first_layer_maxpool=True,
                 fuse_projection_shortcut=True, alias_copies=True, inplace_residual=True, compact_pool=True)
    build16 = lambda: models.resnet50(64, np.float16, seed=5)  # noqa: E731
    out16, info = run(build16, **flags)
    assert info["requested"] == info["pool"]
    ref, _ = run(lambda: as_fp32_graph(*build16()), ORACLE_PATH, fusion=True)
    got, want = out16[0].astype(np.float32), ref[0]
    assert got.shape == (64, 1000) and np.isfinite(got).all()
    close16(got, want)
    assert (got.argmax(1) == want.argmax(1)).mean() > 0.9
    # resident mode, replayed from a captured graph (what bench.py times): the same bits
    import torch
    g, inputs = build16()
    p = g.compile(**flags)
    s = p.session(compiler.MODE_RESIDENT)
    dev_in = [torch.from_numpy(a).cuda() for a in inputs]
    dev_out = torch.empty((64, 1000), dtype=torch.float16, device="cuda")
    for _ in range(3):
        dev_out.fill_(float("nan"))
        torch.cuda.synchronize()
        s.run_device([t.data_ptr() for t in dev_in], [dev_out.data_ptr()], use_graph=True)
        s.sync()
        np.testing.assert_array_equal(dev_out.cpu().numpy(), out16[0])
    s.close()


def test_measured_choice_of_convolution_variants():
    """Session.tune times the runtime's fp16 channels-last convolution variants on the program's own layers and
    keeps the winners as the calls' `algo` operands: the results stay within the fp16 tolerance of the fp32 oracle
    (variants may split a reduction differently), a second session given the same choices gives the first one's
    bits, eager and replayed from a graph, and an fp32 program has nothing to tune."""
    import torch
    flags = dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, channels_last=True, fuse_first_layer_maxpool=True,
                 fuse_projection_shortcut=True, alias_copies=True, inplace_residual=True, compact_pool=True)
    build16 = lambda: models.resnet50(8, np.float16, seed=5, image=96)  # noqa: E731
    ref, _ = run(lambda: as_fp32_graph(*build16()), ORACLE_PATH, fusion=True)
    g, inputs = build16()
    p = g.compile(**flags)
    s = p.session(compiler.MODE_RESIDENT)
    plain = s.run(*inputs)[0]
    close16(plain, ref[0])
    assert all(a == (0, 0) for a in s.algos()) and len(s.algos()) == p.num_ops(compute_only=True)
    changed = s.tune(inputs, reps=3)
    chosen = s.algos()
    assert changed == sum(1 for a in chosen if a != (0, 0))
    tuned = s.run(*inputs)[0]
    close16(tuned, ref[0])
    s.close()
    # every variant id on every convolution that can take it, through the algo operand: still the oracle's result
    s2 = p.session(compiler.MODE_RESIDENT)
    s2.set_algos(chosen)
    np.testing.assert_array_equal(s2.run(*inputs)[0], tuned)
    dev_in = [torch.from_numpy(a).cuda() for a in inputs]
    dev_out = torch.empty(tuned.shape, dtype=torch.float16, device="cuda")
    for _ in range(2):
        s2.run_device([t.data_ptr() for t in dev_in], [dev_out.data_ptr()], use_graph=True)
        s2.sync()
        np.testing.assert_array_equal(dev_out.cpu().numpy(), tuned)
    for vid in (3, 4, 12, 64, 66, 54):
        s2.set_algos([(vid, vid)] * len(chosen))
        close16(s2.run(*inputs)[0], ref[0])
    with pytest.raises(RuntimeError):
        s2.set_algos([(0, 0)])
    s2.close()
    g32, in32 = models.resnet50(image=64, classes=10)
    s32 = g32.compile(fusion=True).session(compiler.MODE_RESIDENT)
    assert s32.tune(in32, reps=3) == 0
    s32.close()


def test_bert_base_12_layers_as_benchmarked():
    """BERT-base at its full depth with the benchmark's flags, against the oracle running the unfused
    program (tolerance: rtol 1e-4, atol 1e-4 on outputs of order one after the final LayerNorm)."""
    flags = dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True, alias_copies=True)
    ref, _ = run(models.bert_encoder, ORACLE_PATH)
    out, info = run(models.bert_encoder, **flags)
    assert info["requested"] == info["pool"]
    close(out[0], ref[0], 1e-4, 1e-4)
    out, _ = run(models.bert_encoder, mode=compiler.MODE_RESIDENT, **flags)
    close(out[0], ref[0], 1e-4, 1e-4)


@pytest.mark.parametrize("batch,image", [(2, 64), (4, 224)])
def test_resnet50_fp16_channels_last(batch, image):
    """fp16 weights/activations, fp32 accumulation, NHWC on the device, against
    the fp32 oracle on the same (fp16-representable) weights and input."""
    build16 = lambda: models.resnet50(batch, np.float16, seed=5, image=image)  # noqa: E731
    out16, info = run(build16, fusion=True, channels_last=True)
    assert info["requested"] == info["pool"]

    ref, _ = run(lambda: as_fp32_graph(*build16()), ORACLE_PATH, fusion=True)
    got, want = out16[0].astype(np.float32), ref[0]
    assert np.isfinite(got).all()
    close16(got, want)
    # the classifier's bias folded into the product: one launch fewer, same tolerance
    fused, _ = run(build16, fusion=True, channels_last=True, fuse_residual=True, fuse_matmul_bias=True)
    close16(fused[0], want)
    assert "dimC=[1," in build16()[0].compile(fusion=True, channels_last=True, fuse_matmul_bias=True).text
    # resident + graph replay gives the same bits as the per-inference mode
    g, inputs = build16()
    p = g.compile(fusion=True, channels_last=True)
    s = p.session(compiler.MODE_RESIDENT)
    np.testing.assert_array_equal(s.run(*inputs)[0], out16[0])
    s.close()


@pytest.mark.parametrize("batch,image", [(3, 64), (2, 224), (1, 90)])
def test_first_layer_maxpool_fusion_fp16_channels_last(batch, image):
    """The first convolution and its max-pool as one call: the same bits as this library's own two calls (same
    products in the same order, an exact maximum), per inference and replayed from a captured graph, and the
    fp32 oracle's result to the fp16 tolerance.  90 x 90: strips and steps that hang over the edge."""
    build16 = lambda: models.resnet50(batch, np.float16, seed=5, image=image)  # noqa: E731
    flags = dict(fusion=True, channels_last=True, fuse_residual=True, fuse_matmul_bias=True)
    assert "maxpoolfwd" in build16()[0].compile(fuse_first_layer_maxpool=True, **flags).text
    two, _ = run(build16, **flags)
    one, info = run(build16, fuse_first_layer_maxpool=True, **flags)
    assert info["requested"] == info["pool"]
    np.testing.assert_array_equal(one[0], two[0])
    res, _ = run(build16, mode=compiler.MODE_RESIDENT, fuse_first_layer_maxpool=True, **flags)
    np.testing.assert_array_equal(res[0], one[0])
    ref, _ = run(lambda: as_fp32_graph(*build16()), ORACLE_PATH, fusion=True)
    close16(one[0], ref[0])


@pytest.mark.parametrize("batch,image", [(1, 224), (2, 75)])
def test_first_layer_maxpool_fusion_fp32(batch, image):
    """fp32 N,C,H,W programs: the first convolution and its max-pool as one call, per inference and replayed from a
    captured graph, against the oracle running the unfused program to the fp32 tolerance of every ResNet-50 test
    here; and against this library's own two calls bit for bit (the unfused first layer runs the same kernel's
    arithmetic, the maximum is exact)."""
    build = lambda: models.resnet50(batch, seed=6, image=image, classes=100)  # noqa: E731
    flags = dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, fuse_projection_shortcut=True, alias_copies=True)  # the benchmark's
    assert "maxpoolfwd" in build()[0].compile(fuse_first_layer_maxpool=True, **flags).text
    two, _ = run(build, **flags)
    one, info = run(build, fuse_first_layer_maxpool=True, **flags)
    assert info["requested"] == info["pool"]
    np.testing.assert_array_equal(one[0], two[0])
    res, _ = run(build, mode=compiler.MODE_RESIDENT, fuse_first_layer_maxpool=True, **flags)
    np.testing.assert_array_equal(res[0], one[0])
    ref, _ = run(build, ORACLE_PATH, fusion=True)
    close(one[0], ref[0], 1e-4, 1e-4)


@pytest.mark.parametrize("dtype,batch,image", [(np.float16, 4, 224), (np.float16, 3, 64), (np.float32, 1, 224), (np.float32, 2, 64)])
def test_inplace_residual_on_the_gpu(dtype, batch, image):
    """Closing convolutions that write over their residual operand: the same bits as with an output buffer of their
    own, per inference with a poisoned pool and replayed from a captured graph; a smaller set of buffers."""
    build = lambda: models.resnet50(batch, dtype, seed=7, image=image, classes=100)  # noqa: E731
    flags = dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, fuse_projection_shortcut=True, alias_copies=True)
    if dtype == np.float16:
        flags.update(channels_last=True, fuse_first_layer_maxpool=True)
    plain, _ = run(build, **flags)
    g, inputs = build()
    p = g.compile(inplace_residual=True, **flags)
    mallocs = lambda prog: sum(1 for k, _, _, _ in prog.events() if k == 0)  # noqa: E731
    assert mallocs(p) == mallocs(build()[0].compile(**flags)) - 12
    s = p.session(compiler.MODE_OCCAMY)
    s.set_debug_fill(0xFF)
    np.testing.assert_array_equal(s.run(*inputs)[0], plain[0])
    s.close()
    s = p.session(compiler.MODE_RESIDENT)
    for _ in range(2):
        np.testing.assert_array_equal(s.run(*inputs)[0], plain[0])
    s.close()


@pytest.mark.parametrize("batch,image", [(2, 64), (8, 224)])
def test_mobilenet_v2_fp16_channels_last(batch, image):
    """MobileNetV2 with fp16 weights and activations, channels-last on the device: its depthwise layers on the
    channels-last depthwise kernel, ReLU6 fused as a clipped ReLU, inverted-residual sums written in place; against
    the fp32 oracle on the same fp16-representable weights and input (rtol 2e-2, atol 4e-3 of the largest logit),
    per inference and replayed from a captured graph."""
    build16 = lambda: models.mobilenet_v2(batch, np.float16, seed=4, image=image, classes=100)  # noqa: E731
    flags = dict(fusion=True, fuse_residual=True, fuse_activations=True, fuse_matmul_bias=True, channels_last=True, alias_copies=True,
                 inplace_residual=True, compact_pool=True)
    out16, info = run(build16, **flags)
    assert info["requested"] == info["pool"]
    ref, _ = run(lambda: as_fp32_graph(*build16()), ORACLE_PATH, fusion=True)
    got, want = out16[0].astype(np.float32), ref[0]
    assert np.isfinite(got).all()
    close16(got, want)
    res, _ = run(build16, mode=compiler.MODE_RESIDENT, **flags)
    np.testing.assert_array_equal(res[0], out16[0])


def test_bert_fp16():
    """A two-layer BERT-base encoder with fp16 weights and activations: the products on the generic fp16 kernel
    (batched, bias + residual + GELU fused with `fuse_matmul_bias`), soft-max, LayerNorm, GELU, gathers and
    transposes in their fp16 forms; against the fp32 oracle on the same fp16-representable weights (LayerNorm
    outputs are O(1): rtol 2e-2, atol 3e-2), unfused and with the fused paths, the fused attention call among
    them."""
    build16 = lambda: models.bert_encoder(layers=2, dtype=np.float16)  # noqa: E731
    ref, _ = run(lambda: models.bert_encoder(layers=2, dtype=np.float16), ORACLE_PATH)
    ref32 = None
    g16, in16 = build16()
    g32 = compiler.Graph()
    for name, (shape, dt) in g16.input_shapes.items():
        g32.input(name, shape, dt if np.dtype(dt).kind == "i" else np.float32)
    for name, arr in g16.constants.items():
        g32.constant(arr if arr.dtype.kind == "i" else arr.astype(np.float32), name)
    for op, ins, out, at in g16.nodes:
        g32.node(op, ins, out, **at)
    for o in g16.outputs:
        g32.output(o)
    s32 = g32.compile().session(runtime_library=ORACLE_PATH)
    ref32 = s32.run(*in16)[0]
    s32.close()
    for flags in (dict(), dict(recompose=True, fusion=True, fuse_matmul_bias=True, alias_copies=True, compact_pool=True),
                  dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True, alias_copies=True)):
        out, info = run(build16, **flags)
        got = out[0].astype(np.float32)
        assert np.isfinite(got).all()
        np.testing.assert_allclose(got, ref32, rtol=2e-2, atol=3e-2)
        np.testing.assert_allclose(got, ref[0].astype(np.float32), rtol=2e-2, atol=3e-2)
        res, _ = run(build16, mode=compiler.MODE_RESIDENT, **flags)
        np.testing.assert_array_equal(res[0], out[0])


@pytest.mark.parametrize("batch", [1, 3])
def test_ssd_resnet50(batch):
    """SSD300 on ResNet-50 (the reference's test/models/ssd-resnet50 network: 300 x 300 images, 8732 boxes, box and
    class tensors; three images there) against the oracle running the unfused program, with the reference's flags
    and with every fusion, per inference and resident."""
    build = lambda: models.ssd_resnet50(batch, labels=21)  # noqa: E731
    ref, _ = run(build, ORACLE_PATH)
    for flags in (dict(), dict(fusion=True, fuse_residual=True, fuse_first_layer_maxpool=True, fuse_projection_shortcut=True,
                               inplace_residual=True, compact_pool=True)):
        out, info = run(build, **flags)
        assert info["requested"] == info["pool"]
        assert [o.shape for o in out] == [(batch, 4, 8732), (batch, 21, 8732)]
        for a, b in zip(out, ref):
            close(a, b, 1e-4, 1e-4)
        res, _ = run(build, mode=compiler.MODE_RESIDENT, **flags)
        for a, b in zip(res, out):
            np.testing.assert_array_equal(a, b)


def test_resident_run_reads_device_inputs_in_place():
    """run_device(in_place=True): the kernels read the caller's input buffer instead of a copy in the pool and write
    the result into the caller's result buffer instead of copying it there; the same bits as with the copies, eager
    and replayed; the input buffer is left as it was; another input address and another result address (the graph is
    recorded again), then the copying mode and the profiler on the same session."""
    import torch
    for builder, flags in ((lambda: models.resnet50(4, np.float16, seed=5, image=64),
                            dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, channels_last=True, fuse_first_layer_maxpool=True,
                                 fuse_projection_shortcut=True, alias_copies=True, inplace_residual=True, compact_pool=True)),
                           (lambda: models.resnet50(2, seed=6, image=64, classes=100), dict(fusion=True, fuse_residual=True, fuse_first_layer_maxpool=True)),
                           (lambda: models.bert_encoder(layers=2), dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True))):
        want, _ = run(builder, **flags)
        g, inputs = builder()
        p = g.compile(**flags)
        s = p.session(compiler.MODE_RESIDENT)
        (shape, dt), = p.output_info()[:1]
        out = torch.empty(shape, dtype=torch.from_numpy(np.empty(0, dt)).dtype, device="cuda")
        a = [torch.from_numpy(x).cuda() for x in inputs]
        b = [torch.from_numpy(x).cuda() for x in inputs]   # the same values at other addresses
        for dev, graph in ((a, False), (a, True), (a, True), (b, True), (b, False)):
            out.zero_()
            torch.cuda.synchronize()
            s.run_device([t.data_ptr() for t in dev], [out.data_ptr()], use_graph=graph, in_place=True)
            s.sync()
            np.testing.assert_array_equal(out.cpu().numpy(), want[0])
            for t, x in zip(dev, inputs):
                np.testing.assert_array_equal(t.cpu().numpy(), x)
        out.zero_()
        torch.cuda.synchronize()
        s.run_device([t.data_ptr() for t in a], [out.data_ptr()], use_graph=True)   # copying again
        s.sync()
        np.testing.assert_array_equal(out.cpu().numpy(), want[0])
        s.run_device([t.data_ptr() for t in a], [out.data_ptr()], use_graph=True, in_place=True)
        s.sync()
        assert len(s.profile(inputs)) == p.num_ops(compute_only=True)
        out.zero_()
        torch.cuda.synchronize()
        s.run_device([t.data_ptr() for t in b], [out.data_ptr()], use_graph=True, in_place=True)
        s.sync()
        np.testing.assert_array_equal(out.cpu().numpy(), want[0])
        # the result is written where the caller wants it as well: another result address (the graph is recorded
        # again), and the first one is left alone by that run
        out2 = torch.zeros_like(out)
        out.fill_(7)
        torch.cuda.synchronize()
        s.run_device([t.data_ptr() for t in b], [out2.data_ptr()], use_graph=True, in_place=True)
        s.run_device([t.data_ptr() for t in b], [out2.data_ptr()], use_graph=True, in_place=True)
        s.sync()
        np.testing.assert_array_equal(out2.cpu().numpy(), want[0])
        assert bool((out == 7).all())
        s.close()


def test_resident_run_in_place_with_two_results():
    """Two results, the first of them produced before the last operation and read again by it: with
    run_device(in_place=True) both land in the caller's buffers with the bits of the copying mode, eager and
    replayed, also after the result addresses change."""
    import torch
    from occamy_amd.compiler import Graph

    def builder():
        r = np.random.default_rng(12)
        g = Graph()
        x = r.standard_normal((2, 16, 12, 12)).astype(np.float32)
        g.input("X", x.shape, np.float32)
        w1 = g.constant((r.standard_normal((24, 16, 3, 3)) * 0.1).astype(np.float32))
        b1 = g.constant(r.uniform(-0.1, 0.1, 24).astype(np.float32))
        a = g.node("Relu", [g.node("Conv", ["X", w1, b1], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1], group=1)])
        w2 = g.constant((r.standard_normal((8, 24, 1, 1)) * 0.1).astype(np.float32))
        b2 = g.constant(r.uniform(-0.1, 0.1, 8).astype(np.float32))
        c = g.node("Conv", [a, w2, b2], kernel_shape=[1, 1], pads=[0, 0, 0, 0], strides=[1, 1], group=1)
        g.output(a)
        g.output(c)
        return g, [x]

    want, _ = run(builder, fusion=True)
    g, inputs = builder()
    p = g.compile(fusion=True)
    s = p.session(compiler.MODE_RESIDENT)
    x = torch.from_numpy(inputs[0]).cuda()
    outs = [[torch.zeros(tuple(w.shape), device="cuda") for w in want] for _ in range(2)]
    for o, graph in ((outs[0], False), (outs[0], True), (outs[0], True), (outs[1], True), (outs[0], True)):
        for t in o:
            t.zero_()
        torch.cuda.synchronize()
        s.run_device([x.data_ptr()], [t.data_ptr() for t in o], use_graph=graph, in_place=True)
        s.sync()
        for t, w in zip(o, want):
            np.testing.assert_array_equal(t.cpu().numpy(), w)
    s.run_device([x.data_ptr()], [t.data_ptr() for t in outs[1]], use_graph=True)   # the copying mode again
    s.sync()
    for t, w in zip(outs[1], want):
        np.testing.assert_array_equal(t.cpu().numpy(), w)
    s.close()


def test_resident_run_in_place_with_one_tensor_returned_twice():
    """The same tensor listed as a result twice (two device-to-host copies of one pool tensor behind the last
    operation): in place, the first lands in the caller's buffer directly and the second is copied from there;
    eager, replayed, and after the result addresses change."""
    import torch
    from occamy_amd.compiler import Graph

    def builder():
        r = np.random.default_rng(13)
        g = Graph()
        x = r.standard_normal((2, 16, 12, 12)).astype(np.float32)
        g.input("X", x.shape, np.float32)
        w1 = g.constant((r.standard_normal((24, 16, 3, 3)) * 0.1).astype(np.float32))
        b1 = g.constant(r.uniform(-0.1, 0.1, 24).astype(np.float32))
        a = g.node("Relu", [g.node("Conv", ["X", w1, b1], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1], group=1)])
        g.output(a)
        g.output(a)
        return g, [x]

    want, _ = run(builder, fusion=True)
    assert len(want) == 2
    np.testing.assert_array_equal(want[0], want[1])
    g, inputs = builder()
    s = g.compile(fusion=True).session(compiler.MODE_RESIDENT)
    x = torch.from_numpy(inputs[0]).cuda()
    outs = [[torch.zeros(tuple(w.shape), device="cuda") for w in want] for _ in range(2)]
    for o, graph in ((outs[0], False), (outs[0], True), (outs[1], True), (outs[0], True)):
        for t in o:
            t.zero_()
        torch.cuda.synchronize()
        s.run_device([x.data_ptr()], [t.data_ptr() for t in o], use_graph=graph, in_place=True)
        s.sync()
        for t, w in zip(o, want):
            np.testing.assert_array_equal(t.cpu().numpy(), w)
    s.close()


def test_compact_pool_on_the_gpu():
    """Offsets from the planner that knows every lifetime: the same bits as with the reference's first fit, per
    inference with a poisoned pool (what a tensor placed over a live one would show) and replayed from a captured
    graph; fp16 channels-last and fp32 ResNet-50, MobileNetV2, a two-layer BERT with its fused paths, SRGAN (two
    results, one of them read again after it was copied out), YOLOv1, AlexNet."""
    cases = [(lambda: models.resnet50(4, np.float16, seed=5, image=64),
              dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, channels_last=True, fuse_first_layer_maxpool=True,
                   fuse_projection_shortcut=True, alias_copies=True, inplace_residual=True)),
             (lambda: models.resnet50(image=64, classes=100), dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, fuse_projection_shortcut=True)),
             (lambda: models.mobilenet_v2(image=64, classes=100), dict(fusion=True, fuse_residual=True, fuse_activations=True)),
             (lambda: models.bert_encoder(layers=2), dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True)),
             (lambda: models.srgan_generator(1, np.float32, height=24, width=16), dict(fusion=True, fuse_residual=True, fuse_activations=True, inplace_residual=True)),
             (lambda: models.yolo_v1(2, image=128, width=0.125, fc=64), dict(fusion=True, fuse_activations=True, fuse_matmul_bias=True)),
             (lambda: models.alexnet(1, image=96, classes=10, hidden=64), dict(fusion=True, fuse_matmul_bias=True, alias_copies=True))]
    for builder, flags in cases:
        plain, _ = run(builder, **flags)
        g, inputs = builder()
        p = g.compile(compact_pool=True, **flags)
        n = sum(1 for k, _, _, _ in p.events() if k == 0)  # every tensor is rounded to 256 bytes, the reference rounds to 32
        assert p.pool_bytes <= builder()[0].compile(**flags).pool_bytes + 256 * n
        s = p.session(compiler.MODE_OCCAMY)
        s.set_debug_fill(0xFF)
        for a, b in zip(s.run(*inputs), plain):
            np.testing.assert_array_equal(a, b)
        assert s.last_pool_bytes == p.pool_bytes
        s.close()
        s = p.session(compiler.MODE_RESIDENT)
        for _ in range(2):
            for a, b in zip(s.run(*inputs), plain):
                np.testing.assert_array_equal(a, b)
        s.close()


def test_aliased_copies_change_nothing_on_the_gpu():
    """Flatten / Reshape on their input's buffer: one launch fewer per copy and the same bits, per inference, with
    a poisoned pool, and replayed from a captured graph; fp32 ResNet-50, a BERT whose reshapes survive the
    attention fusion's absence, fp16 channels-last ResNet-50."""
    cases = [(lambda: models.resnet50(image=64, classes=100), dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True)),
             (lambda: models.bert_encoder(layers=2), dict(recompose=True, fusion=True, fuse_matmul_bias=True)),
             (lambda: models.resnet50(4, np.float16, seed=5, image=64), dict(fusion=True, fuse_residual=True, channels_last=True))]
    for builder, flags in cases:
        plain, _ = run(builder, **flags)
        g, inputs = builder()
        p = g.compile(alias_copies=True, **flags)
        assert p.num_ops(compute_only=True) < builder()[0].compile(**flags).num_ops(compute_only=True)
        s = p.session(compiler.MODE_OCCAMY)
        s.set_debug_fill(0xFF)
        np.testing.assert_array_equal(s.run(*inputs)[0], plain[0])
        s.close()
        s = p.session(compiler.MODE_RESIDENT)
        for _ in range(2):
            np.testing.assert_array_equal(s.run(*inputs)[0], plain[0])
        assert len(s.profile(inputs)) == p.num_ops(compute_only=True)
        s.close()


@pytest.mark.parametrize("batch,image", [(3, 64), (2, 224)])
def test_projection_shortcut_fusion_fp16_channels_last(batch, image):
    """Every block's projection shortcut and last convolution as one call (the first two stages' pairs give the two
    calls' bits, the last two are one reduction rounded once): the fp32 oracle's result to the fp16 tolerance, the
    two-call program's closely, and the same bits per inference and replayed from a captured graph."""
    build16 = lambda: models.resnet50(batch, np.float16, seed=5, image=image)  # noqa: E731
    flags = dict(fusion=True, channels_last=True, fuse_residual=True, fuse_matmul_bias=True)
    assert "add-conv" in build16()[0].compile(fuse_projection_shortcut=True, **flags).text
    two, _ = run(build16, **flags)
    one, info = run(build16, fuse_projection_shortcut=True, **flags)
    assert info["requested"] == info["pool"]
    ref, _ = run(lambda: as_fp32_graph(*build16()), ORACLE_PATH, fusion=True)
    close16(one[0], ref[0])
    close16(one[0], two[0])
    res, _ = run(build16, mode=compiler.MODE_RESIDENT, fuse_projection_shortcut=True, **flags)
    np.testing.assert_array_equal(res[0], one[0])


def test_projection_shortcut_fusion_fp32(oracle_outputs):
    """fp32 ResNet-50 at batch 1 with every shortcut pair as one call (four launches fewer; the pairs' sums are rounded
    once instead of three times): the oracle's result to the usual fp32 tolerance, per inference and resident."""
    flags = dict(fusion=True, fuse_residual=True, fuse_projection_shortcut=True)
    assert CONFIGS["resnet50"]()[0].compile(**flags).text.count("add-conv") == 4
    out, info = run(CONFIGS["resnet50"], **flags)
    assert info["requested"] == info["pool"]
    close(out[0], oracle_outputs["resnet50"][0])
    res, _ = run(CONFIGS["resnet50"], mode=compiler.MODE_RESIDENT, **flags)
    np.testing.assert_array_equal(res[0], out[0])


def test_projection_shortcut_pair_whose_filters_cannot_share_a_layout():
    """A fused shortcut pair takes both filters in one layout.  Here the shortcut's filter constant is also read by
    an operator that is no convolution, so it stays K,C,R,S on the device, and the closing filter has to stay with
    it: the pair runs and gives the oracle's result, per inference and resident."""
    from occamy_amd.compiler import Graph

    def builder():
        r = np.random.default_rng(14)
        g = Graph()
        x = r.standard_normal((1, 32, 14, 14)).astype(np.float32)
        g.input("X", x.shape, np.float32)
        conv = lambda src, w, b, **kw: g.node("Conv", [src, w, b], kernel_shape=[1, 1], pads=[0, 0, 0, 0], strides=[1, 1], group=1, **kw)  # noqa: E731
        w1 = g.constant((r.standard_normal((16, 32, 1, 1)) * 0.2).astype(np.float32))
        b1 = g.constant(r.uniform(-0.1, 0.1, 16).astype(np.float32))
        w2 = g.constant((r.standard_normal((64, 16, 1, 1)) * 0.2).astype(np.float32))
        b2 = g.constant(r.uniform(-0.1, 0.1, 64).astype(np.float32))
        wsc = g.constant((r.standard_normal((64, 32, 1, 1)) * 0.2).astype(np.float32))
        bsc = g.constant(r.uniform(-0.1, 0.1, 64).astype(np.float32))
        main = conv(g.node("Relu", [conv("X", w1, b1)]), w2, b2)
        g.output(g.node("Relu", [g.node("Add", [main, conv("X", wsc, bsc)])]))
        g.output(g.node("Relu", [wsc]))  # the second reader of the shortcut's filter
        return g, [x]

    flags = dict(fusion=True, fuse_residual=True, fuse_projection_shortcut=True)
    assert "add-conv" in builder()[0].compile(**flags).text
    want, _ = run(builder, ORACLE_PATH)
    for mode in (compiler.MODE_OCCAMY, compiler.MODE_RESIDENT):
        got, _ = run(builder, mode=mode, **flags)
        for a, b in zip(got, want):
            close(a, b)


@pytest.mark.parametrize("name", ["resnet50", "mobilenet_v2"])
def test_residual_fusion_fp32(name, oracle_outputs):
    """conv+bias -> add -> relu as one call: against the oracle, and bit for
    bit against this library's own three-call chain (same sums, same order)."""
    fused, _ = run(CONFIGS[name], fusion=True, fuse_residual=True)
    close(fused[0], oracle_outputs[name][0])
    chain, _ = run(CONFIGS[name], fusion=True)
    np.testing.assert_array_equal(fused[0], chain[0])
    res, _ = run(CONFIGS[name], mode=compiler.MODE_RESIDENT, fusion=True, fuse_residual=True)
    np.testing.assert_array_equal(res[0], fused[0])


def test_residual_fusion_fp16_channels_last():
    build16 = lambda: models.resnet50(2, np.float16, seed=5, image=64)  # noqa: E731
    chain, _ = run(build16, fusion=True, channels_last=True)
    fused, _ = run(build16, fusion=True, channels_last=True, fuse_residual=True)
    # the fused closer rounds conv+bias to fp16 exactly where the chain stores
    # it, so only the final fp32->fp16 rounding of the sum can differ (the chain
    # adds in fp16 arithmetic): a few fp16 ulps after 16 blocks
    close16(fused[0], chain[0])


@pytest.mark.parametrize("name", ["mobilenet_v2", "yolo_v1", "srgan"])
def test_activation_fusion_fp32(name, oracle_outputs):
    out, _ = run(CONFIGS[name], fusion=True, fuse_residual=True, fuse_activations=True)
    for o, r in zip(out, oracle_outputs[name]):
        close(o, r)
    out, _ = run(CONFIGS[name], mode=compiler.MODE_RESIDENT, fusion=True, fuse_residual=True, fuse_activations=True)
    for o, r in zip(out, oracle_outputs[name]):
        close(o, r)


@pytest.mark.parametrize("name", ["resnet50", "alexnet", "mobilenet_v2"])
def test_gemm_bias_folded_into_the_product(name, oracle_outputs):
    for mode in (compiler.MODE_OCCAMY, compiler.MODE_RESIDENT):
        out, _ = run(CONFIGS[name], mode=mode, fusion=True, fuse_matmul_bias=True)
        for o, r in zip(out, oracle_outputs[name]):
            close(o, r)


def test_bert_recomposed_with_fused_linear_layers(oracle_outputs):
    flags = dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True)
    out, _ = run(CONFIGS["bert_2_layers"], **flags)
    close(out[0], oracle_outputs["bert_2_layers"][0], 1e-4, 1e-4)
    out, _ = run(CONFIGS["bert_2_layers"], mode=compiler.MODE_RESIDENT, **flags)
    close(out[0], oracle_outputs["bert_2_layers"][0], 1e-4, 1e-4)


def test_model_from_an_onnx_file_runs_like_the_built_graph(tmp_path):
    """ResNet-50 through a file: ONNX bytes -> reader -> compiler -> gfx950."""
    import onnx_writer
    g0, inputs = models.resnet50()
    path = tmp_path / "resnet50.onnx"
    path.write_bytes(onnx_writer.model_bytes(g0))
    g1 = compiler.load_onnx(str(path))
    p0, p1 = g0.compile(fusion=True), g1.compile(fusion=True)
    assert p1.text == p0.text and p1.pool_bytes == p0.pool_bytes
    s0, s1 = p0.session(), p1.session()
    np.testing.assert_array_equal(s1.run(*inputs)[0], s0.run(*inputs)[0])
    s0.close()
    s1.close()
