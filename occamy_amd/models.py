"""Graph builders for the benchmark configurations: the ONNX graphs a PyTorch
export of these models gives (node vocabulary and order as in the reference's
test/models/*/run.py flows), with seeded synthetic weights.

Each builder returns ``(Graph, [input arrays])``.  In ResNet-50, MobileNetV2
and BERT BatchNorm is already folded into the convolution bias, as onnx-mlir's
ONNX-level rewrites leave it before the reference's own passes run; AlexNet,
YOLOv1 and the SRGAN generator (test/models/{alexnet,yolo,srgan}/run.py of the
reference) keep the exporter's BatchNormalization / Dropout nodes, which the
compiler folds or forwards itself.
"""
import numpy as np

from . import rng
from .compiler import Graph


class _Init:
    """Hands out seeded tensors; every tensor gets its own stream number."""

    def __init__(self, seed, dtype):
        self.seed, self.dtype, self.stream = seed, dtype, 0

    def _next(self):
        self.stream += 1
        return self.stream

    def he_normal(self, shape):
        fan_in = int(np.prod(shape[1:]))
        return rng.normal(self.seed, self._next(), shape, std=np.sqrt(2.0 / fan_in)).astype(self.dtype)

    def normal(self, shape, std):
        return rng.normal(self.seed, self._next(), shape, std=std).astype(self.dtype)

    def uniform(self, shape, lo, hi):
        return rng.uniform(self.seed, self._next(), shape, lo, hi).astype(self.dtype)


def single_conv(dtype=np.float32, seed=1):
    """Conv2d(3x3, 64->64, stride 1, pad 1) + bias + ReLU on 1x64x56x56."""
    init = _Init(seed, dtype)
    g = Graph()
    x = rng.normal(seed, 0, (1, 64, 56, 56)).astype(dtype)
    bound = float(np.sqrt(6.0 / (64 * 9)))  # Kaiming-uniform
    g.input("X", x.shape, dtype)
    w = g.constant(init.uniform((64, 64, 3, 3), -bound, bound), "W")
    b = g.constant(init.uniform((64,), -0.1, 0.1), "B")
    c = g.node("Conv", ["X", w, b], "conv", kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1], group=1)
    r = g.node("Relu", [c], "relu")
    g.output(r)
    return g, [x]


def _conv(g, init, x, cin, cout, k, stride, pad, group=1, bias=True):
    w = g.constant(init.he_normal((cout, cin // group, k, k)))
    ins = [x, w]
    if bias:
        ins.append(g.constant(init.uniform((cout,), -0.1, 0.1)))
    return g.node("Conv", ins, kernel_shape=[k, k], pads=[pad] * 4, strides=[stride, stride], group=group)


def resnet50(batch=1, dtype=np.float32, seed=2, image=224, classes=1000, stage_means=False):
    """ResNet-50 v1.5: bottlenecks [3,4,6,3], stride on the 3x3, folded BN.
    stage_means: the per-channel spatial mean of each of the four stages' results is returned after the logits
    ([batch, 256], [batch, 512], [batch, 1024], [batch, 2048]), so that a comparison sees every stage at its own
    magnitude and not only through the classifier."""
    init = _Init(seed, dtype)
    g = Graph()
    x_np = rng.normal(seed, 0, (batch, 3, image, image)).astype(dtype)
    g.input("input", x_np.shape, dtype)
    x = _conv(g, init, "input", 3, 64, 7, 2, 3)
    x = g.node("Relu", [x])
    x = g.node("MaxPool", [x], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[2, 2])
    cin = 64
    taps = []
    for planes, blocks, stride in [(64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)]:
        for b in range(blocks):
            s = stride if b == 0 else 1
            identity = x
            o = g.node("Relu", [_conv(g, init, x, cin, planes, 1, 1, 0)])
            o = g.node("Relu", [_conv(g, init, o, planes, planes, 3, s, 1)])
            o = _conv(g, init, o, planes, planes * 4, 1, 1, 0)
            if b == 0:
                identity = _conv(g, init, x, cin, planes * 4, 1, s, 0)
            x = g.node("Relu", [g.node("Add", [o, identity])])
            cin = planes * 4
        if stage_means and planes != 512:
            taps.append(g.node("Flatten", [g.node("GlobalAveragePool", [x])], axis=1))
    x = g.node("GlobalAveragePool", [x])
    x = g.node("Flatten", [x], axis=1)
    w = g.constant(init.he_normal((classes, cin)))
    bias = g.constant(np.zeros((classes,), dtype))
    y = g.node("Gemm", [x, w, bias], "logits", alpha=1.0, beta=1.0, transB=1)
    g.output(y)
    for t in taps + ([x] if stage_means else []):
        g.output(t)
    return g, [x_np]


def ssd_resnet50(batch=1, dtype=np.float32, seed=8, image=300, labels=81):
    """SSD300 on a ResNet-50 backbone as the reference's test exports it
    (test/models/ssd-resnet50/run.py: NVIDIA's `nvidia_ssd`, whose forward pass ends at the box and class
    tensors; decoding and non-maximum suppression happen in Python afterwards and are not part of the
    network): ResNet-50 up to its third stage with that stage's stride removed (1024 channels at 38 x 38 for
    a 300 x 300 image), five extra blocks of 1x1 -> 3x3 convolutions (BatchNorm folded, ReLU) down to 1 x 1,
    a 3x3 location head and a 3x3 class head on each of the six feature maps (4, 6, 6, 6, 4, 4 boxes per
    cell), every head's result viewed as [N, 4 or labels, boxes] and concatenated: two results,
    [N, 4, 8732] and [N, labels, 8732]."""
    init = _Init(seed, dtype)
    g = Graph()
    x_np = rng.normal(seed, 0, (batch, 3, image, image)).astype(dtype)
    g.input("input", x_np.shape, dtype)
    x = g.node("Relu", [_conv(g, init, "input", 3, 64, 7, 2, 3)])
    x = g.node("MaxPool", [x], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[2, 2])
    size = ((image + 6 - 7) // 2 + 1 + 2 - 3) // 2 + 1
    cin = 64
    for planes, blocks, stride in [(64, 3, 1), (128, 4, 2), (256, 6, 1)]:  # the third stage keeps its input's size
        for b in range(blocks):
            s = stride if b == 0 else 1
            identity = x
            o = g.node("Relu", [_conv(g, init, x, cin, planes, 1, 1, 0)])
            o = g.node("Relu", [_conv(g, init, o, planes, planes, 3, s, 1)])
            o = _conv(g, init, o, planes, planes * 4, 1, 1, 0)
            if b == 0:
                identity = _conv(g, init, x, cin, planes * 4, 1, s, 0)
            x = g.node("Relu", [g.node("Add", [o, identity])])
            cin = planes * 4
        size = (size - 1) // stride + 1
    feeds = [(x, cin, size)]
    for i, (cout, mid) in enumerate(zip([512, 512, 256, 256, 256], [256, 256, 128, 128, 128])):
        o = g.node("Relu", [_conv(g, init, x, cin, mid, 1, 1, 0)])
        if i < 3:
            x = g.node("Relu", [_conv(g, init, o, mid, cout, 3, 2, 1)])
            size = (size + 2 - 3) // 2 + 1
        else:
            x = g.node("Relu", [_conv(g, init, o, mid, cout, 3, 1, 0)])
            size = size - 2
        cin = cout
        feeds.append((x, cin, size))
    locs, confs = [], []
    for (f, c, sz), boxes in zip(feeds, [4, 6, 6, 6, 4, 4]):
        n = boxes * sz * sz
        loc = _conv(g, init, f, c, boxes * 4, 3, 1, 1)
        conf = _conv(g, init, f, c, boxes * labels, 3, 1, 1)
        locs.append(g.node("Reshape", [loc, g.constant(np.array([batch, 4, n], np.int64))]))
        confs.append(g.node("Reshape", [conf, g.constant(np.array([batch, labels, n], np.int64))]))
    g.output(g.node("Concat", locs, "locs", axis=2))
    g.output(g.node("Concat", confs, "confs", axis=2))
    return g, [x_np]


def mobilenet_v2(batch=1, dtype=np.float32, seed=3, image=224, classes=1000):
    """MobileNetV2 width 1.0; ReLU6 is Clip(0, 6) with constant bounds."""
    init = _Init(seed, dtype)
    g = Graph()
    x_np = rng.normal(seed, 0, (batch, 3, image, image)).astype(dtype)
    g.input("input", x_np.shape, dtype)

    def relu6(v):
        lo = g.constant(np.array(0.0, dtype))
        hi = g.constant(np.array(6.0, dtype))
        return g.node("Clip", [v, lo, hi])

    x = relu6(_conv(g, init, "input", 3, 32, 3, 2, 1))
    cin = 32
    for t, c, n, s in [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]:
        for i in range(n):
            stride = s if i == 0 else 1
            hidden = cin * t
            o = x
            if t != 1:
                o = relu6(_conv(g, init, o, cin, hidden, 1, 1, 0))
            o = relu6(_conv(g, init, o, hidden, hidden, 3, stride, 1, group=hidden))
            o = _conv(g, init, o, hidden, c, 1, 1, 0)
            x = g.node("Add", [x, o]) if (stride == 1 and cin == c) else o
            cin = c
    x = relu6(_conv(g, init, x, cin, 1280, 1, 1, 0))
    x = g.node("GlobalAveragePool", [x])
    x = g.node("Flatten", [x], axis=1)
    w = g.constant(init.he_normal((classes, 1280)))
    bias = g.constant(np.zeros((classes,), dtype))
    y = g.node("Gemm", [x, w, bias], "logits", alpha=1.0, beta=1.0, transB=1)
    g.output(y)
    return g, [x_np]


def _batchnorm(g, init, x, c):
    scale = g.constant(init.uniform((c,), 0.5, 1.5))
    bias = g.constant(init.uniform((c,), -0.1, 0.1))
    mean = g.constant(init.normal((c,), 0.1))
    var = g.constant(init.uniform((c,), 0.5, 1.5))
    return g.node("BatchNormalization", [x, scale, bias, mean, var], epsilon=1e-5, momentum=0.9)


def _linear(g, init, x, nin, nout, name=None):
    w = g.constant(init.he_normal((nout, nin)))
    b = g.constant(init.uniform((nout,), -0.1, 0.1))
    return g.node("Gemm", [x, w, b], name, alpha=1.0, beta=1.0, transB=1)


def alexnet(batch=1, dtype=np.float32, seed=5, image=224, classes=1000, hidden=4096):
    """torchvision AlexNet as torch.onnx.export writes it: the adaptive 6x6
    average pool of a 224x224 image is an AveragePool with a 1x1 window, the
    classifier's Dropout nodes are kept (inference: they forward their input)."""
    init = _Init(seed, dtype)
    g = Graph()
    x_np = rng.normal(seed, 0, (batch, 3, image, image)).astype(dtype)
    g.input("input", x_np.shape, dtype)
    pool = dict(kernel_shape=[3, 3], pads=[0, 0, 0, 0], strides=[2, 2])
    x = g.node("Relu", [_conv(g, init, "input", 3, 64, 11, 4, 2)])
    x = g.node("MaxPool", [x], **pool)
    x = g.node("Relu", [_conv(g, init, x, 64, 192, 5, 1, 2)])
    x = g.node("MaxPool", [x], **pool)
    x = g.node("Relu", [_conv(g, init, x, 192, 384, 3, 1, 1)])
    x = g.node("Relu", [_conv(g, init, x, 384, 256, 3, 1, 1)])
    x = g.node("Relu", [_conv(g, init, x, 256, 256, 3, 1, 1)])
    x = g.node("MaxPool", [x], **pool)
    side = (((image + 4 - 11) // 4 + 1 - 3) // 2 + 1 - 3) // 2 + 1
    side = (side - 3) // 2 + 1
    x = g.node("AveragePool", [x], kernel_shape=[1, 1], pads=[0, 0, 0, 0], strides=[1, 1])
    x = g.node("Flatten", [x], axis=1)
    x = g.node("Dropout", [x])
    x = g.node("Relu", [_linear(g, init, x, 256 * side * side, hidden)])
    x = g.node("Dropout", [x])
    x = g.node("Relu", [_linear(g, init, x, hidden, hidden)])
    y = _linear(g, init, x, hidden, classes, "logits")
    g.output(y)
    return g, [x_np]


YOLO_V1_LAYERS = [(7, 64, 2, 3), "M", (3, 192, 1, 1), "M", (1, 128, 1, 0), (3, 256, 1, 1), (1, 256, 1, 0),
                  (3, 512, 1, 1), "M", [(1, 256, 1, 0), (3, 512, 1, 1), 4], (1, 512, 1, 0), (3, 1024, 1, 1), "M",
                  [(1, 512, 1, 0), (3, 1024, 1, 1), 2], (3, 1024, 1, 1), (3, 1024, 2, 1), (3, 1024, 1, 1),
                  (3, 1024, 1, 1)]


def yolo_v1(batch=2, dtype=np.float32, seed=6, image=448, width=1.0, boxes=2, classes=20, fc=496):
    """YOLOv1 with BatchNorm (test/models/yolo/run.py of the reference):
    bias-free Conv -> BatchNormalization -> LeakyRelu(0.1) blocks, 2x2 max
    pools, Flatten, two Linear layers.  `image` must be a multiple of 64;
    `width` scales the channel counts (tests use a narrow copy)."""
    init = _Init(seed, dtype)
    g = Graph()
    x_np = rng.normal(seed, 0, (batch, 3, image, image)).astype(dtype)
    g.input("input", x_np.shape, dtype)
    x, cin = "input", 3

    def block(x, cin, k, cout, stride, pad):
        cout = max(8, int(cout * width))
        c = _conv(g, init, x, cin, cout, k, stride, pad, bias=False)
        return g.node("LeakyRelu", [_batchnorm(g, init, c, cout)], alpha=0.1), cout

    for item in YOLO_V1_LAYERS:
        if item == "M":
            x = g.node("MaxPool", [x], kernel_shape=[2, 2], pads=[0, 0, 0, 0], strides=[2, 2])
        elif isinstance(item, tuple):
            x, cin = block(x, cin, *item)
        else:
            for _ in range(item[2]):
                x, cin = block(x, cin, *item[0])
                x, cin = block(x, cin, *item[1])
    split = image // 64
    x = g.node("Flatten", [x], axis=1)
    x = g.node("LeakyRelu", [_linear(g, init, x, cin * split * split, fc)], alpha=0.1)
    y = _linear(g, init, x, fc, split * split * (classes + boxes * 5), "cells")
    g.output(y)
    return g, [x_np]


def srgan_generator(batch=1, dtype=np.float32, seed=7, height=24, width=24, feats=64, blocks=16):
    """SRGAN generator, 4x upscaling (test/models/srgan/srgan_model.py of the
    reference): 9x9 conv, residual blocks of conv-BN-PReLU-conv-BN, two
    conv + PixelShuffle(2) + PReLU stages, 3x3 conv + Tanh.  One PReLU
    parameter is shared by every activation, as nn.PReLU() gives.  PixelShuffle
    is Reshape -> Transpose(0,1,4,2,5,3) -> Reshape.  Two results: the image
    and the feature map before upsampling."""
    init = _Init(seed, dtype)
    g = Graph()
    x_np = rng.normal(seed, 0, (batch, 3, height, width)).astype(dtype)
    g.input("lr", x_np.shape, dtype)
    slope = g.constant(np.full((1,), 0.25, dtype), "prelu_slope")

    def conv(x, cin, cout, k):
        w = g.constant(init.normal((cout, cin, k, k), 0.02))  # the reference's own initialisation (srgan/ops.py)
        b = g.constant(init.uniform((cout,), -0.05, 0.05))
        return g.node("Conv", [x, w, b], kernel_shape=[k, k], pads=[k // 2] * 4, strides=[1, 1], group=1)

    x = g.node("PRelu", [conv("lr", 3, feats, 9), slope])
    skip = x
    for _ in range(blocks):
        r = g.node("PRelu", [_batchnorm(g, init, conv(x, feats, feats, 3), feats), slope])
        r = _batchnorm(g, init, conv(r, feats, feats, 3), feats)
        x = g.node("Add", [r, x])
    x = _batchnorm(g, init, conv(x, feats, feats, 3), feats)
    feat = g.node("Add", [x, skip], "feat")
    x, h, w = feat, height, width
    for _ in range(2):
        x = conv(x, feats, feats * 4, 3)
        x = g.node("Reshape", [x, g.constant(np.array([batch, feats, 2, 2, h, w], np.int64))])
        x = g.node("Transpose", [x], perm=[0, 1, 4, 2, 5, 3])
        h, w = h * 2, w * 2
        x = g.node("Reshape", [x, g.constant(np.array([batch, feats, h, w], np.int64))])
        x = g.node("PRelu", [x, slope])
    y = g.node("Tanh", [conv(x, feats, 3, 3)], "sr")
    g.output(y)
    g.output(feat)
    return g, [x_np]


def bert_encoder(layers=12, hidden=768, heads=12, ffn=3072, seq=128, vocab=30522, dtype=np.float32, seed=4,
                 fused=False):
    """BERT-base-shaped encoder (post-LayerNorm, GELU(erf)), batch 1.

    With ``fused=False`` LayerNorm and GELU appear as the primitive chains a
    PyTorch export produces (and the reference lowers op by op); with
    ``fused=True`` they are single LayerNormalization / Gelu nodes.
    """
    init = _Init(seed, dtype)
    g = Graph()
    ids = rng.integers(seed, 0, (1, seq), 0, vocab)
    g.input("input_ids", ids.shape, np.int64)
    dh = hidden // heads
    eps = 1e-12

    def scalar(v):
        return g.constant(np.array(v, dtype))

    def layernorm(x):
        gamma, beta = g.constant(np.ones((hidden,), dtype)), g.constant(np.zeros((hidden,), dtype))
        if fused:
            return g.node("LayerNormalization", [x, gamma, beta], axis=-1, epsilon=eps)
        mu = g.node("ReduceMean", [x], axes=[-1], keepdims=1)
        d = g.node("Sub", [x, mu])
        var = g.node("ReduceMean", [g.node("Pow", [d, scalar(2.0)])], axes=[-1], keepdims=1)
        std = g.node("Sqrt", [g.node("Add", [var, scalar(eps)])])
        return g.node("Add", [g.node("Mul", [g.node("Div", [d, std]), gamma]), beta])

    def linear(x, nin, nout):
        w = g.constant(init.normal((nin, nout), 0.02))
        b = g.constant(init.normal((nout,), 0.02))
        return g.node("Add", [b, g.node("MatMul", [x, w])])  # bias first, as the exporter writes it

    def gelu(x):
        if fused:
            return g.node("Gelu", [x])
        e = g.node("Erf", [g.node("Div", [x, scalar(float(np.sqrt(2.0)))])])
        return g.node("Mul", [g.node("Mul", [x, g.node("Add", [e, scalar(1.0)])]), scalar(0.5)])

    word = g.constant(init.normal((vocab, hidden), 0.02), "word_embeddings")
    pos = g.constant(init.normal((1, seq, hidden), 0.02), "position_embeddings")
    tok = g.constant(init.normal((hidden,), 0.02), "token_type_embedding")
    x = g.node("Gather", [word, "input_ids"], axis=0)
    x = g.node("Add", [g.node("Add", [x, pos]), tok])
    x = layernorm(x)
    for _ in range(layers):
        def split(v, perm):
            shp = g.constant(np.array([1, seq, heads, dh], np.int64))
            return g.node("Transpose", [g.node("Reshape", [v, shp])], perm=perm)
        q = split(linear(x, hidden, hidden), [0, 2, 1, 3])
        k = split(linear(x, hidden, hidden), [0, 2, 3, 1])
        v = split(linear(x, hidden, hidden), [0, 2, 1, 3])
        s = g.node("Div", [g.node("MatMul", [q, k]), scalar(float(np.sqrt(dh)))])
        p = g.node("Softmax", [s], axis=-1)
        c = g.node("Transpose", [g.node("MatMul", [p, v])], perm=[0, 2, 1, 3])
        c = g.node("Reshape", [c, g.constant(np.array([1, seq, hidden], np.int64))])
        x = layernorm(g.node("Add", [linear(c, hidden, hidden), x]))
        h = linear(gelu(linear(x, hidden, ffn)), ffn, hidden)
        x = layernorm(g.node("Add", [h, x]))
    g.output(x)
    return g, [ids]
