"""The pass pipeline: emission order, dealloc placement, fusion and the pool
layout of the benchmark graphs.

The single-conv trace is checked against the recording of the reference
(tests/golden/planner_single_conv.json).  For the big graphs, which the
reference's tests hold no recording of, the checks are structural: every
tensor is allocated before and released after each of its uses (in both the
direct and the aliased-result sense), the program's offsets equal what the
planner ORACLE computes from the program's own event trace, and planned pool
size equals the highest planned byte."""
import json
import os
import re

import numpy as np
import pytest

from occamy_amd import compiler, models
from test_planner import oracle_plan

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_single_conv_trace_matches_reference_recording():
    gold = json.load(open(os.path.join(GOLDEN, "planner_single_conv.json")))
    g, _ = models.single_conv()
    p = g.compile(fusion=False, dealloc_opt=True, pool_opt=True)
    ev = p.events()
    want = [(0 if e["op"] == "malloc" else 1, e.get("bytes", 0), e.get("offset", -1)) for e in gold["events"]]
    assert [(k, b, o) for k, _, b, o in ev] == want
    # same tensor is freed as the recording names: X, ws, W, B, then Y, R
    ids = {}
    for e, (k, i, b, o) in zip(gold["events"], ev):
        if k == 0:
            ids[e["id"]] = i
        else:
            assert ids[e["id"]] == i
    assert p.pool_bytes == gold["peak"] == p.pool_extent
    # op order of the recording
    seq = [name for _, name, _ in parse(p.text) if name in ("dnn.convfwd", "dnn.add", "dnn.activationfwd")]
    assert seq == ["dnn.convfwd", "dnn.add", "dnn.activationfwd"]


def test_single_conv_fused():
    gold = json.load(open(os.path.join(GOLDEN, "planner_single_conv.json")))["fused"]
    g, _ = models.single_conv()
    p = g.compile(fusion=True)
    assert p.pool_bytes == gold["peak"]
    assert "dnn.conv-bias-relufwd" in p.text and "dnn.convfwd" not in p.text and "dnn.activationfwd" not in p.text
    mallocs = [e for e in p.events() if e[0] == 0]
    assert len(mallocs) == 5 and mallocs[-1][3] == gold["R_offset"]  # X W B ws R: the conv's own Y is gone


def parse(text):
    """[(result or None, op name, [operands])] of a program's text form."""
    out = []
    for ln in text.splitlines():
        m = re.match(r"(?:(%\w+) = )?([\w.\-]+)((?: ?%\w+,?)*)", ln)
        res, name, ops = m.group(1), m.group(2), re.findall(r"%\w+", m.group(3))
        out.append((res, name, ops))
    return out


def check_lifetimes(graph_builder, **flags):
    """Compile without the pool pass and replay: no op may touch a tensor
    before its malloc or after its dealloc, where 'touch' follows results back
    to the buffer they alias (a compute op's result is its last operand)."""
    g, _ = graph_builder()
    p = g.compile(pool_opt=False, **flags)
    alias, live, freed = {}, set(), set()
    n_malloc = n_free = 0
    for res, name, ops in parse(p.text):
        bufs = [alias.get(o, o) for o in ops]
        if name == "dnn.malloc":
            live.add(res)
            alias[res] = res
            n_malloc += 1
        elif name == "dnn.dealloc":
            assert bufs[0] in live, f"double free / free before malloc: {bufs[0]}"
            live.discard(bufs[0])
            freed.add(bufs[0])
            n_free += 1
        elif name.startswith("host.") or name == "return":
            if res:
                alias[res] = res
        else:
            for b in bufs:
                if b.startswith("%arg"):
                    continue
                assert b not in freed, f"{name} uses {b} after its dealloc"
                assert b in live or not b.startswith("%") or alias.get(b) == b, f"{name} uses {b} before malloc"
            if res:
                alias[res] = bufs[-1]
    assert n_malloc == n_free and not live
    return p


SMALL = dict(image=64, classes=10)


@pytest.mark.parametrize("fusion", [False, True])
def test_lifetimes_resnet(fusion):
    check_lifetimes(lambda: models.resnet50(**SMALL), fusion=fusion)


@pytest.mark.parametrize("fusion", [False, True])
def test_lifetimes_mobilenet(fusion):
    check_lifetimes(lambda: models.mobilenet_v2(**SMALL), fusion=fusion)


@pytest.mark.parametrize("fused", [False, True])
def test_lifetimes_bert(fused):
    check_lifetimes(lambda: models.bert_encoder(layers=2, hidden=64, heads=4, ffn=128, seq=16, vocab=100, fused=fused))


@pytest.mark.parametrize("fusion", [False, True])
def test_lifetimes_alexnet_yolo_srgan(fusion):
    check_lifetimes(lambda: models.alexnet(image=96, classes=10, hidden=64), fusion=fusion)
    check_lifetimes(lambda: models.yolo_v1(batch=1, image=64, width=0.0625, fc=32), fusion=fusion)
    # the generator returns its feature map and goes on reading it
    check_lifetimes(lambda: models.srgan_generator(height=8, width=6, feats=16, blocks=2), fusion=fusion)


def test_batchnorm_folds_into_the_convolution_before_it():
    g, _ = models.yolo_v1(batch=1, image=64, width=0.0625, fc=32)
    n_conv = sum(1 for op, *_ in g.nodes if op == "Conv")
    ops = [name for name, *_ in g.compile().compute_ops()]
    # every block is conv, bias add (the folded shift), leaky relu: no Mul is left over
    assert ops.count("dnn.convfwd") == n_conv == 24 and ops.count("dnn.add") == n_conv + 2 and "dnn.mul" not in ops
    g, _ = models.yolo_v1(batch=1, image=64, width=0.0625, fc=32)
    ops = [name for name, *_ in g.compile(fusion=True).compute_ops()]
    assert ops.count("dnn.conv-bias-relufwd") == n_conv and "dnn.convfwd" not in ops


def test_activation_fusion_flag():
    count = lambda p: {n: [m for m, *_ in p.compute_ops()].count(n) for n in  # noqa: E731
                       ("dnn.clip", "dnn.leakyrelu", "dnn.prelu", "dnn.add", "dnn.conv-bias-relufwd", "dnn.conv-bias-add-relufwd")}
    flags = dict(fusion=True, fuse_activations=True, fuse_residual=True)
    g, _ = models.mobilenet_v2(**SMALL)
    c = count(check_lifetimes(lambda: models.mobilenet_v2(**SMALL), **flags))
    # every ReLU6 and every residual sum is gone; the one add left is the classifier's bias
    assert c["dnn.clip"] == 0 and c["dnn.add"] == 1 and c["dnn.conv-bias-add-relufwd"] == 10 and c["dnn.conv-bias-relufwd"] == 42
    p = g.compile(**flags)
    assert "activMode=3, activCoef=6" in p.text
    c = count(check_lifetimes(lambda: models.yolo_v1(batch=1, image=64, width=0.0625, fc=32), **flags))
    assert c["dnn.leakyrelu"] == 1 and c["dnn.conv-bias-relufwd"] == 24            # the one left follows a Gemm
    c = count(check_lifetimes(lambda: models.srgan_generator(height=8, width=6, feats=16, blocks=2), **flags))
    assert c["dnn.prelu"] == 2 and c["dnn.add"] == 0 and c["dnn.conv-bias-add-relufwd"] == 3   # two PRelu follow a pixel shuffle
    # without `fusion` the flag does nothing
    g, _ = models.mobilenet_v2(**SMALL)
    assert count(g.compile(fuse_activations=True))["dnn.clip"] == 35


def test_recompose_flag():
    small = dict(layers=2, hidden=64, heads=4, ffn=128, seq=16, vocab=100)
    names = lambda p: [n for n, *_ in p.compute_ops()]  # noqa: E731
    g, _ = models.bert_encoder(**small)
    plain = names(g.compile())
    assert "dnn.layernorm" not in plain and "dnn.gelu" not in plain and plain.count("dnn.reciprocal") == 9
    p = check_lifetimes(lambda: models.bert_encoder(**small), recompose=True)
    got = names(p)
    # 1 + 2 per layer LayerNorms, one Gelu per layer, no reciprocal of a constant left at run time
    assert got.count("dnn.layernorm") == 5 and got.count("dnn.gelu") == 2 and "dnn.reciprocal" not in got
    assert not {"dnn.pow", "dnn.sqrt", "dnn.erf", "dnn.reduce", "dnn.negative"} & set(got)
    # what the builder's own fused graph compiles to, but for the folded divisors
    g, _ = models.bert_encoder(fused=True, **small)
    ref = names(g.compile())
    assert [n for n in ref if n != "dnn.reciprocal"] == got
    p = check_lifetimes(lambda: models.bert_encoder(**small), recompose=True, fusion=True, fuse_matmul_bias=True)
    got = names(p)
    # the residual sums and the Gelu of every layer ride on their Linear layer: what is left are the
    # two embedding sums
    assert got.count("dnn.matmulnd-bias") == 12 and got.count("dnn.matmulnd") == 4 and got.count("dnn.add") == 2
    two_heads = dict(small, heads=2)   # head size 32: the attention kernel takes it
    p = check_lifetimes(lambda: models.bert_encoder(**two_heads), recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True)
    assert len(names(p)) == 2 * 7 + 4   # per layer: qkv, attention, projection, LayerNorm, two feed-forward layers, LayerNorm
    assert "dnn.gelu" not in got and p.text.count("{gelu}") == 2


def test_attention_fusion_flag():
    small = dict(layers=2, hidden=64, heads=2, ffn=128, seq=16, vocab=100)
    names = lambda p: [n for n, *_ in p.compute_ops()]  # noqa: E731
    p = check_lifetimes(lambda: models.bert_encoder(**small), fuse_attention=True)
    got = names(p)
    # per layer: 3 head splits (Reshape + Transpose), two MatMuls, the scaling, Softmax and the head merge go
    assert got.count("dnn.attention") == 2 and "dnn.softmax" not in got and "dnn.transpose" not in got and "dnn.reshape" not in got
    assert "heads=2, scale=0.176777, packed" in p.text          # Q, K, V come out of one product
    assert got.count("dnn.matmulnd") == 2 * 4                    # qkv, output projection, two feed-forward layers
    # head size 16 has no kernel: the graph is left as it is
    g, _ = models.bert_encoder(layers=1, hidden=64, heads=4, ffn=128, seq=16, vocab=100)
    assert "dnn.attention" not in names(g.compile(fuse_attention=True))


def test_recompose_leaves_near_misses_alone():
    def ln_graph(eps_node="eps", power=2.0, extra_reader=False, axes=(-1,)):
        g = compiler.Graph()
        x = g.input("x", (2, 5, 8))
        c = lambda v, n: g.constant(np.array(v, np.float32), n)  # noqa: E731
        mu = g.node("ReduceMean", [x], "mu", axes=list(axes), keepdims=1)
        d = g.node("Sub", [x, mu], "d")
        var = g.node("ReduceMean", [g.node("Pow", [d, c(power, "two")], "sq")], "var", axes=list(axes), keepdims=1)
        sd = g.node("Sqrt", [g.node("Add", [var, c(1e-5, eps_node)], "ve")], "sd")
        y = g.node("Add", [g.node("Mul", [g.node("Div", [d, sd], "n"), g.constant(np.ones(8, np.float32), "gamma")], "sc"),
                           g.constant(np.zeros(8, np.float32), "beta")], "y")
        g.output(y)
        if extra_reader:
            g.output(g.node("Relu", ["sd"], "also"))
        return g
    count = lambda g: [n for n, *_ in g.compile(recompose=True).compute_ops()].count("dnn.layernorm")  # noqa: E731
    assert count(ln_graph()) == 1
    assert count(ln_graph(power=3.0)) == 0            # not a variance
    assert count(ln_graph(extra_reader=True)) == 0    # the standard deviation is read elsewhere
    assert count(ln_graph(axes=(1,))) == 0            # not the last axis


def planned_vs_oracle(p):
    ev = p.events()
    off, peak = oracle_plan([(k, i, b) for k, i, b, _ in ev])
    assert [o for _, _, _, o in ev] == off
    assert p.pool_bytes == peak == p.pool_extent
    return ev


def test_pool_resnet50_full_size():
    g, _ = models.resnet50()
    p = g.compile()
    ev = planned_vs_oracle(p)
    mallocs = [e for e in ev if e[0] == 0]
    # 53 convolutions x (W, B, ws, Y) + 49 relu + 16 add + maxpool + reduce + flatten + gemm (W, bias, Y) + input
    assert len(mallocs) == 53 * 4 + 49 + 16 + 1 + 1 + 1 + 3 + 1
    assert len(ev) == 2 * len(mallocs)
    # weights live in the pool only while their layer runs: the pool is far smaller than the weights
    weights = sum(b for k, _, b, _ in ev if k == 0)
    assert p.pool_bytes < 0.5 * weights
    g, _ = models.resnet50()
    pf = g.compile(fusion=True)
    planned_vs_oracle(pf)
    assert pf.num_ops(compute_only=True) < p.num_ops(compute_only=True)
    txt = pf.text
    assert txt.count("dnn.conv-bias-relufwd") == 53 and "dnn.convfwd" not in txt
    assert txt.count("activMode=1") == 33 and txt.count("activMode=5") == 20  # 16 x 2 + stem; 16 x conv3 + 4 downsample


def test_pool_mobilenet_and_bert():
    g, _ = models.mobilenet_v2()
    p = g.compile()
    planned_vs_oracle(p)
    assert p.text.count("group=") == 52 and p.text.count("dnn.clip") == 35
    # Clip bounds are folded to attributes and their constant uploads removed
    assert "min=0, max=6" in p.text
    g, _ = models.bert_encoder(layers=2)
    p = g.compile()
    planned_vs_oracle(p)
    assert p.text.count("dnn.softmax") == 2 and p.text.count("dnn.matmulnd") == 2 * 8
    g, _ = models.bert_encoder(layers=2, fused=True)
    pf = g.compile()
    planned_vs_oracle(pf)
    assert pf.text.count("dnn.layernorm") == 5 and pf.text.count("dnn.gelu") == 2


def test_fp16_channels_last_flag():
    g, _ = models.resnet50(dtype=np.float16, **SMALL)
    p = g.compile(fusion=True, channels_last=True)
    g32, _ = models.resnet50(dtype=np.float32, **SMALL)
    p32 = g32.compile(fusion=True)
    # same event structure, half the bytes per tensor
    e16, e32 = p.events(), p32.events()
    assert [(k, b * 2) for k, _, b, _ in e16] == [(k, b) for k, _, b, _ in e32]
    g, _ = models.resnet50(dtype=np.float32, **SMALL)
    with pytest.raises(RuntimeError):
        g.compile(channels_last=True)  # fp32 graphs stay NCHW


def test_first_layer_maxpool_fusion():
    """conv 7x7/2 over the 3-channel argument + ReLU + max-pool 3x3/2 -> one call, in channels-last fp16 programs with
    an even image width and in fp32 programs; the convolution's buffer (the largest activation of the network) is
    never allocated."""
    flags = dict(fusion=True, fuse_residual=True, channels_last=True)
    g, _ = models.resnet50(dtype=np.float16, **SMALL)
    plain = g.compile(**flags)
    g, _ = models.resnet50(dtype=np.float16, **SMALL)
    fused = g.compile(fuse_first_layer_maxpool=True, **flags)
    assert plain.text.count("dnn.maxpool") == 1 and "maxpoolfwd" not in plain.text
    assert fused.text.count("dnn.conv-bias-relu-maxpoolfwd") == 1 and "dnn.maxpool " not in fused.text
    line = next(l for l in fused.text.splitlines() if "maxpoolfwd" in l)
    assert "pads=[3,3], strides=[2,2], group=1, activMode=1, poolKernel=[3,3], poolPads=[1,1,1,1], poolStrides=[2,2]" in line
    assert fused.num_ops(compute_only=True) == plain.num_ops(compute_only=True) - 1
    assert fused.pool_bytes <= plain.pool_bytes
    conv_bytes = 1 * 64 * 32 * 32 * 2  # the convolution's result at a 64 x 64 image, batch 1
    sizes = lambda prog: sorted(b for k, _, b, _ in prog.events() if k == 0)
    gone = list(sizes(plain))
    gone.remove(conv_bytes)
    assert sizes(fused) == gone
    check_lifetimes(lambda: models.resnet50(dtype=np.float16, **SMALL), fuse_first_layer_maxpool=True, **flags)
    # fp16: not without channels-last (the kernel writes N,H,W,C), not for an odd width
    g, _ = models.resnet50(dtype=np.float16, **SMALL)
    assert "maxpoolfwd" not in g.compile(fusion=True, fuse_first_layer_maxpool=True).text
    # fp32 N,C,H,W programs: any width
    for shape in (SMALL, dict(SMALL, image=SMALL.get("image", 32) + 1)):
        g, _ = models.resnet50(dtype=np.float32, **shape)
        plain32 = g.compile(fusion=True)
        g, _ = models.resnet50(dtype=np.float32, **shape)
        fused32 = g.compile(fusion=True, fuse_first_layer_maxpool=True)
        assert fused32.text.count("dnn.conv-bias-relu-maxpoolfwd") == 1 and "dnn.maxpool " not in fused32.text
        assert fused32.num_ops(compute_only=True) == plain32.num_ops(compute_only=True) - 1
    check_lifetimes(lambda: models.resnet50(dtype=np.float32, **SMALL), fusion=True, fuse_residual=True, fuse_first_layer_maxpool=True)
    odd = dict(SMALL, image=SMALL.get("image", 32) + 1)
    g, _ = models.resnet50(dtype=np.float16, **odd)
    assert "maxpoolfwd" not in g.compile(fuse_first_layer_maxpool=True, **flags).text
    # nor when something else reads the convolution's result
    g, _ = models.resnet50(dtype=np.float16, **SMALL)
    assert "maxpoolfwd" not in g.compile(fuse_first_layer_maxpool=True, channels_last=True).text  # no fusion flag: conv, add, relu apart


def test_inplace_residual():
    """A fused conv + add + activation whose residual operand nothing reads afterwards names that operand's buffer
    as its output: ResNet-50's twelve identity blocks (and, without the shortcut fusion, its four projection blocks)
    lose their output buffers, chains of blocks walk down one buffer, and every tensor is still alive when read."""
    for dt, flags in ((np.float32, dict(fusion=True, fuse_residual=True)), (np.float16, dict(fusion=True, fuse_residual=True, channels_last=True))):
        g, _ = models.resnet50(dtype=dt, **SMALL)
        plain = g.compile(**flags)
        g, _ = models.resnet50(dtype=dt, **SMALL)
        inpl = g.compile(inplace_residual=True, **flags)
        mallocs = lambda prog: sum(1 for k, _, _, _ in prog.events() if k == 0)  # noqa: E731
        assert mallocs(inpl) == mallocs(plain) - 16
        assert inpl.num_ops(compute_only=True) == plain.num_ops(compute_only=True)
        closers = [l for l in inpl.text.splitlines() if "conv-bias-add-relufwd" in l]
        assert len(closers) == 16
        for l in closers:  # operands: x, w, bias, workspace, z, out; z is a result, out the buffer it lives in
            ops = l.split("conv-bias-add-relufwd")[1].split("{")[0].replace(" ", "").split(",")
            assert len(ops) == 6 and ops[4] != ops[5]
        g, _ = models.resnet50(dtype=dt, **SMALL)
        with_pairs = g.compile(inplace_residual=True, fuse_projection_shortcut=True, **flags)
        assert mallocs(with_pairs) == mallocs(plain) - 16  # four shortcut results, twelve identity blocks' outputs
        check_lifetimes(lambda: models.resnet50(dtype=dt, **SMALL), inplace_residual=True, **flags)
        check_lifetimes(lambda: models.resnet50(dtype=dt, **SMALL), inplace_residual=True, fuse_projection_shortcut=True, alias_copies=True, **flags)
        # nothing without the residual fusion
        g, _ = models.resnet50(dtype=dt, **SMALL)
        assert mallocs(g.compile(fusion=True, inplace_residual=True)) == mallocs(models.resnet50(dtype=dt, **SMALL)[0].compile(fusion=True))
    # a residual operand that is read again later keeps its buffer
    def again():
        g = compiler.Graph()
        g.input("x", (1, 8, 6, 6), np.float32)
        r = np.random.default_rng(0)
        g.constant(r.standard_normal((8, 8, 1, 1)).astype(np.float32), "w")
        g.constant(r.standard_normal(8).astype(np.float32), "b")
        g.node("Conv", ["x", "w", "b"], "c", kernel_shape=[1, 1])
        g.node("Relu", ["c"], "z")
        g.node("Conv", ["z", "w", "b"], "d", kernel_shape=[1, 1])
        g.node("Add", ["d", "z"], "s")
        g.node("Relu", ["s"], "y")
        g.node("Add", ["y", "z"], "t")  # z again
        g.output("t")
        return g
    flags = dict(fusion=True, fuse_residual=True)
    mallocs = lambda prog: sum(1 for k, _, _, _ in prog.events() if k == 0)  # noqa: E731
    p2 = again().compile(inplace_residual=True, **flags)
    assert "conv-bias-add-relufwd" in p2.text
    assert mallocs(p2) == mallocs(again().compile(**flags))


def test_compact_pool():
    """The planner that knows every lifetime before it places anything: no two tensors alive together overlap, the
    pool is not larger than the reference's first fit on these programs (up to its rounding of every tensor to 256
    bytes where the reference rounds to 32) and reaches the bytes alive at once on ResNet-50; the events (ids,
    sizes, order) are those of the first-fit program."""
    def peak_and_overlap(prog):
        live, cur, peak = {}, 0, 0
        for k, i, b, off in prog.events():
            if k == 0:
                assert off >= 0 and off % 32 == 0
                for bb, oo in live.values():
                    assert not (b and bb and off < oo + bb and oo < off + b), "two live tensors overlap"
                live[i] = (b, off)
                cur += b
                peak = max(peak, cur)
                assert off + b <= prog.pool_bytes
            else:
                cur -= live.pop(i)[0]
        return peak
    cases = [(lambda: models.resnet50(dtype=np.float32, **SMALL), dict(fusion=True, fuse_residual=True)),
             (lambda: models.resnet50(dtype=np.float16, **SMALL), dict(fusion=True, fuse_residual=True, channels_last=True, inplace_residual=True, fuse_projection_shortcut=True)),
             (lambda: models.mobilenet_v2(image=32, classes=10), dict(fusion=True, fuse_residual=True, fuse_activations=True)),
             (lambda: models.bert_encoder(layers=2, hidden=64, heads=2, seq=16, vocab=50, ffn=128), dict()),
             (lambda: models.single_conv(), dict())]
    for build, flags in cases:
        first = build()[0].compile(**flags)
        tight = build()[0].compile(compact_pool=True, **flags)
        assert [(k, i, b) for k, i, b, _ in first.events()] == [(k, i, b) for k, i, b, _ in tight.events()]
        peak = peak_and_overlap(tight)
        peak_and_overlap(first)
        n = sum(1 for k, _, _, _ in tight.events() if k == 0)
        assert peak <= tight.pool_bytes <= first.pool_bytes + 256 * n
        assert first.text.count("dnn.mem-offset") == tight.text.count("dnn.mem-offset")
    g, _ = models.resnet50(dtype=np.float32, **SMALL)
    tight = g.compile(compact_pool=True, fusion=True, fuse_residual=True)
    assert tight.pool_bytes <= 1.02 * peak_and_overlap(tight)  # the bytes alive at once, up to the rounding of each tensor to 256 bytes
    # without the pool pass the flag does nothing
    g, _ = models.single_conv()
    assert "dnn.malloc" in g.compile(pool_opt=False, compact_pool=True).text


def test_projection_shortcut_fusion():
    """Every projection shortcut of ResNet-50 (conv + bias) and the last convolution (+ add + ReLU) of its block become
    one call; the shortcuts' buffers are never allocated.  fp32 programs and channels-last fp16 programs."""
    for dt, flags in ((np.float16, dict(fusion=True, fuse_residual=True, channels_last=True)), (np.float32, dict(fusion=True, fuse_residual=True))):
        g, _ = models.resnet50(dtype=dt, **SMALL)
        plain = g.compile(**flags)
        g, _ = models.resnet50(dtype=dt, **SMALL)
        fused = g.compile(fuse_projection_shortcut=True, **flags)
        assert "add-conv" not in plain.text and fused.text.count("dnn.conv-bias-add-conv-bias-relufwd") == 4
        lines = [l for l in fused.text.splitlines() if "add-conv" in l]
        name = "f16" if dt == np.float16 else "f32"
        assert "pads=[0,0], strides=[1,1], pads2=[0,0], strides2=[1,1], activMode=1" in lines[0] and lines[0].rstrip().endswith(f"{name}[1,256,16,16]")
        assert "pads=[0,0], strides=[1,1], pads2=[0,0], strides2=[2,2], activMode=1" in lines[1] and lines[1].rstrip().endswith(f"{name}[1,512,8,8]")
        assert fused.num_ops(compute_only=True) == plain.num_ops(compute_only=True) - 4
        assert fused.text.count("dnn.conv-bias-add-relufwd") == plain.text.count("dnn.conv-bias-add-relufwd") - 4
        es = 2 if dt == np.float16 else 4
        sizes = lambda prog: sorted(b for k, _, b, _ in prog.events() if k == 0)
        gone = list(sizes(plain))
        for shortcut_bytes in (256 * 16 * 16 * es, 512 * 8 * 8 * es, 1024 * 4 * 4 * es, 2048 * 2 * 2 * es):
            gone.remove(shortcut_bytes)
        assert sizes(fused) == gone  # (first fit is not monotonic: the pool itself may come out a little larger)
        check_lifetimes(lambda: models.resnet50(dtype=dt, **SMALL), fuse_projection_shortcut=True, **flags)
    # needs the residual fusion (it extends that call); fp16 programs must be channels-last
    g, _ = models.resnet50(dtype=np.float16, **SMALL)
    assert "add-conv" not in g.compile(fusion=True, channels_last=True, fuse_projection_shortcut=True).text
    g, _ = models.resnet50(dtype=np.float16, **SMALL)
    assert "add-conv" not in g.compile(fusion=True, fuse_residual=True, fuse_projection_shortcut=True).text


def test_channels_last_refuses_what_it_cannot_lay_out():
    """A rank-4 constant with spatial extent reaches the device N,C,H,W (only convolution filters are re-laid at
    upload), and Flatten / Reshape copy bytes: channels_last must refuse both at compile time, not at run time."""
    def conv_graph():
        g = compiler.Graph()
        g.input("x", (1, 8, 8, 8), np.float16)
        w = g.constant(np.ones((64, 8, 3, 3), np.float16))
        return g, g.node("Conv", ["x", w], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1], group=1)
    g, c = conv_graph()
    k = g.constant(np.ones((1, 64, 8, 8), np.float16))
    a = g.node("Add", [c, k])
    g.output(g.node("ReduceMean", [a], axes=[2, 3], keepdims=1))
    with pytest.raises(RuntimeError, match="constant"):
        g.compile(channels_last=True)
    g, c = conv_graph()
    g.output(g.node("Flatten", [c], axis=1))
    with pytest.raises(RuntimeError, match="no channels-last form"):
        g.compile(channels_last=True)
    # a per-channel constant and a flatten of a 1x1 map are fine
    g, c = conv_graph()
    k = g.constant(np.ones((1, 64, 1, 1), np.float16))
    m = g.node("ReduceMean", [g.node("Add", [c, k])], axes=[2, 3], keepdims=1)
    g.output(g.node("Flatten", [m], axis=1))
    assert g.compile(channels_last=True).pool_bytes > 0


def test_compile_errors():
    g = compiler.Graph()
    g.input("x", (1, 3, 8, 8))
    with pytest.raises(RuntimeError):
        g.node("Conv", ["x", "nope"])
        g.compile()
    g = compiler.Graph()
    g.input("x", (1, 3, 8, 8))
    y = g.node("Relu", ["x"])
    g.node("NoSuchOp", [y], "z")
    g.output("z")
    with pytest.raises(RuntimeError, match="not in the DNN dialect"):
        g.compile()
    g = compiler.Graph()
    g.input("x", (1, 3, 8, 8))
    w = g.constant(np.zeros((4, 3, 3, 3), np.float32))
    g.output(g.node("Conv", ["x", w], pads=[1, 0, 0, 1]))
    with pytest.raises(RuntimeError, match="asymmetric"):
        g.compile()


def test_residual_fusion_flag():
    g, _ = models.resnet50()
    pf = g.compile(fusion=True)
    g2, _ = models.resnet50()
    pr = g2.compile(fusion=True, fuse_residual=True)
    planned_vs_oracle(pr)
    txt = pr.text
    # every bottleneck ends conv3 (+ shortcut) -> add -> relu: 16 blocks, 16 fused closers
    assert txt.count("dnn.conv-bias-add-relufwd") == 16
    assert txt.count("dnn.conv-bias-relufwd") == 53 - 16
    assert "dnn.add" in txt and txt.count("dnn.add") == 1             # the classifier's bias add stays
    assert txt.count("dnn.activationfwd") == 0
    assert pr.num_ops(compute_only=True) == pf.num_ops(compute_only=True) - 32
    # two intermediate tensors per block are never allocated
    assert len(pr.events()) == len(pf.events()) - 2 * 2 * 16
    # (first fit is not monotonic: fewer tensors need not mean a smaller pool)
    # the flag alone (without conv+bias fusion) changes nothing
    g3, _ = models.resnet50(**SMALL)
    g4, _ = models.resnet50(**SMALL)
    assert g3.compile(fuse_residual=True).text == g4.compile().text
    check_lifetimes(lambda: models.resnet50(**SMALL), fusion=True, fuse_residual=True)
    check_lifetimes(lambda: models.mobilenet_v2(**SMALL), fusion=True, fuse_residual=True)
