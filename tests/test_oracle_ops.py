"""Pins the CPU oracle (oracle/dnnrt_oracle.c).

The reference holds no golden vectors for these operators and its arithmetic
(cuDNN / cuBLASLt / CUDA kernels) cannot run here, so each oracle function is
checked against what fixes it independently: an independent library (torch
CPU / numpy in float64), closed forms, and brute force on tiny shapes -- with
cases chosen so that a dropped term, a wrong sign or index, or a transposed
operand fails.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import opcases as oc
from helpers import OracleBackend, rng
from occamy_amd import _abi


@pytest.fixture(scope="module")
def be():
    return OracleBackend()


def t64(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float64))


# ---- convolution -----------------------------------------------------------

def brute_conv(x, w, b, pads, strides, group):
    """7-loop definition in Python floats (float64), tiny shapes only."""
    N, C, H, W = x.shape
    K, Cg, R, S = w.shape
    P, Q = oc.conv_out_hw(H, W, R, S, pads, strides)
    y = np.zeros((N, K, P, Q))
    Kg = K // group
    for n in range(N):
        for k in range(K):
            g = k // Kg
            for p in range(P):
                for q in range(Q):
                    acc = 0.0 if b is None else float(b[k])
                    for c in range(Cg):
                        for r in range(R):
                            for s in range(S):
                                ih, iw = p * strides[0] - pads[0] + r, q * strides[1] - pads[1] + s
                                if 0 <= ih < H and 0 <= iw < W:
                                    acc += float(x[n, g * Cg + c, ih, iw]) * float(w[k, c, r, s])
                    y[n, k, p, q] = acc
    return y


@pytest.mark.parametrize("R,S", [(1, 1), (3, 3), (2, 3)])
@pytest.mark.parametrize("stride", [(1, 1), (2, 2), (1, 2)])
@pytest.mark.parametrize("pad", [(0, 0), (1, 1), (2, 1)])
@pytest.mark.parametrize("group", [1, 2, 4])
def test_conv_bruteforce_tiny(be, R, S, stride, pad, group):
    r = rng(R * 100 + S * 10 + stride[0] + pad[0] * 7 + group)
    x = r.standard_normal((2, 4, 6, 5)).astype(np.float32)
    w = r.standard_normal((4, 4 // group, R, S)).astype(np.float32)
    b = r.standard_normal(4).astype(np.float32)
    if 6 + 2 * pad[0] < R or 5 + 2 * pad[1] < S:
        pytest.skip("empty output")
    ref = brute_conv(x, w, b, pad, stride, group)
    got = oc.conv(be, x, w, b, pad, stride, group, _abi.ACT_IDENTITY)
    np.testing.assert_allclose(got, ref, rtol=1e-6, atol=1e-6)
    got_nb = oc.conv(be, x, w, None, pad, stride, group)
    np.testing.assert_allclose(got_nb, brute_conv(x, w, None, pad, stride, group), rtol=1e-6, atol=1e-6)
    relu = oc.conv(be, x, w, b, pad, stride, group, _abi.ACT_RELU)
    np.testing.assert_array_equal(relu, np.maximum(got, 0))


@pytest.mark.parametrize("shape", [
    # (N, C, H, W, K, R, stride, pad, group)
    (1, 64, 56, 56, 64, 3, 1, 1, 1),     # the single-conv configuration
    (2, 3, 33, 35, 16, 7, 2, 3, 1),      # stem-like, odd sizes
    (1, 32, 14, 14, 32, 3, 2, 1, 32),    # depthwise stride 2
    (1, 24, 9, 9, 48, 1, 2, 0, 1),       # strided 1x1
])
def test_conv_vs_torch_float64(be, shape):
    N, C, H, W, K, R, st, pd, g = shape
    r = rng(sum(shape))
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = (r.standard_normal((K, C // g, R, R)) * 0.1).astype(np.float32)
    b = r.uniform(-0.1, 0.1, K).astype(np.float32)
    ref = F.conv2d(t64(x), t64(w), t64(b), stride=st, padding=pd, groups=g).numpy()
    got = oc.conv(be, x, w, b, (pd, pd), (st, st), g, _abi.ACT_IDENTITY)
    np.testing.assert_allclose(got, ref, rtol=2e-6, atol=2e-6)
    # with a residual tensor: relu(conv + b + z), and exactly the three-call chain
    z = r.standard_normal(ref.shape).astype(np.float32)
    fused = oc.conv(be, x, w, b, (pd, pd), (st, st), g, _abi.ACT_RELU, z=z)
    np.testing.assert_allclose(fused, np.maximum(ref + z.astype(np.float64), 0), rtol=2e-6, atol=2e-6)
    chain = oc.unary(be, "relu", oc.tensor_op(be, _abi.OP_ADD, got, z))
    np.testing.assert_array_equal(fused, chain)
    lin = oc.conv(be, x, w, b, (pd, pd), (st, st), g, _abi.ACT_IDENTITY, z=z)
    np.testing.assert_array_equal(lin, oc.tensor_op(be, _abi.OP_ADD, got, z))


def test_conv_closed_forms(be):
    r = rng(5)
    x = r.standard_normal((1, 3, 8, 8)).astype(np.float32)
    # identity filter: centre tap 1 on the matching channel -> Y == X
    w = np.zeros((3, 3, 3, 3), np.float32)
    for c in range(3):
        w[c, c, 1, 1] = 1
    np.testing.assert_array_equal(oc.conv(be, x, w, None, (1, 1), (1, 1)), x)
    # all-ones input and filter: each output counts its in-range taps times C
    ones = np.ones((1, 2, 5, 5), np.float32)
    y = oc.conv(be, ones, np.ones((1, 2, 3, 3), np.float32), None, (1, 1), (1, 1))
    cnt = np.array([[(min(i + 1, 4) - max(i - 1, 0) + 1) * (min(j + 1, 4) - max(j - 1, 0) + 1)
                     for j in range(5)] for i in range(5)], np.float32)
    np.testing.assert_array_equal(y[0, 0], 2 * cnt)
    # a filter with a single off-centre tap shifts the image (catches r/s or
    # sign mix-ups): tap (r=0, s=2) reads X[p-1, q+1]
    w = np.zeros((1, 1, 3, 3), np.float32)
    w[0, 0, 0, 2] = 1
    xi = np.arange(36, dtype=np.float32).reshape(1, 1, 6, 6)
    y = oc.conv(be, xi, w, None, (1, 1), (1, 1))[0, 0]
    exp = np.zeros((6, 6), np.float32)
    exp[1:, :-1] = xi[0, 0, :-1, 1:]
    np.testing.assert_array_equal(y, exp)
    # 1x1 stride-1 convolution is W[K,C] @ X[C,HW]
    w1 = r.standard_normal((5, 3, 1, 1)).astype(np.float32)
    y = oc.conv(be, x, w1, None, (0, 0), (1, 1))
    ref = (w1.reshape(5, 3).astype(np.float64) @ x.reshape(3, 64).astype(np.float64)).reshape(1, 5, 8, 8)
    np.testing.assert_allclose(y, ref, rtol=1e-6, atol=1e-6)


def test_conv_errors(be):
    x = np.zeros((1, 4, 4, 4), np.float32)
    with pytest.raises(RuntimeError):
        oc.conv(be, x, np.zeros((4, 3, 1, 1), np.float32))      # C/g mismatch
    with pytest.raises(RuntimeError):
        oc.conv(be, x, np.zeros((4, 4, 7, 7), np.float32))      # empty output


def test_conv_fp16_storage(be):
    r = rng(11)
    x = r.standard_normal((1, 8, 6, 6)).astype(np.float16)
    w = (r.standard_normal((4, 8, 3, 3)) * 0.2).astype(np.float16)
    b = r.uniform(-0.1, 0.1, 4).astype(np.float16)
    got = oc.conv(be, x, w, b, (1, 1), (1, 1), 1, _abi.ACT_RELU)
    ref = F.relu(F.conv2d(t64(x), t64(w), t64(b), padding=1)).numpy()
    assert got.dtype == np.float16
    # one rounding to fp16 of the exact value
    np.testing.assert_array_equal(got, ref.astype(np.float32).astype(np.float16))


# ---- fp16 conversion -----------------------------------------------------------

def test_fp16_round_trip_all_values(be):
    """Every finite fp16 value must survive widen -> negate -> negate -> narrow, and
    float32 -> fp16 rounding must agree with numpy on a sweep incl. subnormals/ties."""
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    fin = allh[np.isfinite(allh)]
    np.testing.assert_array_equal(oc.unary(be, "negative", oc.unary(be, "negative", fin)).view(np.uint16),
                                  fin.view(np.uint16))
    r = rng(3)
    f = np.concatenate([r.standard_normal(20000) * 10.0 ** r.integers(-9, 5, 20000),
                        np.array([65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8,
                                  6.1035156e-5, 6.0975552e-5, 0.0, -0.0])]).astype(np.float32)
    with np.errstate(over="ignore"):
        expect = f.astype(np.float16)
    got = oc.cast(be, f.astype(np.int64), np.float16)  # integers only; separate path below
    np.testing.assert_array_equal(got, f.astype(np.int64).astype(np.float32).astype(np.float16))
    # float path: x * 1 through tensor_op MUL keeps the value, narrowing does the rounding
    xs = expect  # representable inputs stay fixed
    np.testing.assert_array_equal(oc.tensor_op(be, _abi.OP_MUL, xs, np.ones_like(xs)).view(np.uint16)[np.isfinite(xs)],
                                  xs.view(np.uint16)[np.isfinite(xs)])
    # products that need rounding: compare against numpy's float32 -> float16
    a = (r.standard_normal(5000)).astype(np.float16)
    b = (r.standard_normal(5000)).astype(np.float16)
    prod = (a.astype(np.float32) * b.astype(np.float32)).astype(np.float16)
    np.testing.assert_array_equal(oc.tensor_op(be, _abi.OP_MUL, a, b).view(np.uint16), prod.view(np.uint16))


# ---- elementwise -------------------------------------------------------------------

def test_unary_ops(be):
    x = np.concatenate([rng(1).standard_normal(1000) * 3, [0.0, -0.0, 7.5, -7.5]]).astype(np.float32)
    np.testing.assert_array_equal(oc.unary(be, "relu", x), np.where(x < 0, np.float32(0), x))
    np.testing.assert_array_equal(oc.unary(be, "negative", x), -x)
    np.testing.assert_array_equal(oc.unary(be, "clip", x, lo=0.0, hi=6.0), np.clip(x, 0, 6))
    nz = x[x != 0]
    np.testing.assert_array_equal(oc.unary(be, "reciprocal", nz), (np.float32(1) / nz))
    np.testing.assert_array_equal(oc.unary(be, "sqrt", np.abs(x)), np.sqrt(np.abs(x)))
    ref_erf = np.array([math.erf(float(v)) for v in x])
    np.testing.assert_allclose(oc.unary(be, "erf", x), ref_erf, rtol=1e-6, atol=1e-7)
    ref_gelu = np.array([0.5 * float(v) * (1 + math.erf(float(v) / math.sqrt(2))) for v in x])
    np.testing.assert_allclose(oc.unary(be, "gelu", x), ref_gelu, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(oc.unary(be, "sigmoid", x), 1 / (1 + np.exp(-x.astype(np.float64))), rtol=1e-6)
    np.testing.assert_allclose(oc.unary(be, "tanh", x), np.tanh(x.astype(np.float64)), rtol=1e-6, atol=1e-7)
    # NaN goes through ReLU, as with CUDNN_PROPAGATE_NAN
    assert np.isnan(oc.unary(be, "relu", np.array([np.nan], np.float32))[0])
    np.testing.assert_array_equal(oc.pow_(be, x, 2.0), x * x)
    np.testing.assert_allclose(oc.pow_(be, np.abs(x) + 0.5, 1.5), (np.abs(x.astype(np.float64)) + 0.5) ** 1.5, rtol=1e-6)
    i = rng(2).integers(-2 ** 40, 2 ** 40, 500)
    np.testing.assert_array_equal(oc.cast(be, i), i.astype(np.float32))


def test_tensor_op_broadcast(be):
    r = rng(7)
    a = r.standard_normal((2, 5, 3, 4)).astype(np.float32)
    for bshape in [(2, 5, 3, 4), (1, 5, 1, 1), (1, 1, 1, 4), (2, 1, 3, 1), (1, 1, 1, 1), (1, 5, 3, 1)]:
        b = r.standard_normal(bshape).astype(np.float32)
        np.testing.assert_array_equal(oc.tensor_op(be, _abi.OP_ADD, a, b), a + b)
        np.testing.assert_array_equal(oc.tensor_op(be, _abi.OP_MUL, a, b), a * b)
        np.testing.assert_array_equal(oc.tensor_op(be, _abi.OP_ADD, a, b, coef=-2.0), a + np.float32(-2) * b)
        np.testing.assert_array_equal(oc.tensor_op(be, _abi.OP_ADD, a, b, inplace=True), a + b)
    with pytest.raises(RuntimeError):
        oc.tensor_op(be, _abi.OP_ADD, a, np.zeros((2, 5, 3, 2), np.float32))
    # rank 2 and 3 (Gemm bias, LayerNorm scale)
    a2 = r.standard_normal((3, 7)).astype(np.float32)
    b2 = r.standard_normal((1, 7)).astype(np.float32)
    np.testing.assert_array_equal(oc.tensor_op(be, _abi.OP_ADD, a2, b2), a2 + b2)


# ---- reductions ---------------------------------------------------------------------

def test_reduce_mean(be):
    r = rng(9)
    x = r.standard_normal((2, 6, 7, 7)).astype(np.float32)
    ref = x.astype(np.float64)
    np.testing.assert_allclose(oc.reduce_mean(be, x, (2, 6, 1, 1)), ref.mean((2, 3), keepdims=True), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(oc.reduce_mean(be, x, (2, 1, 7, 7)), ref.mean(1, keepdims=True), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(oc.reduce_mean(be, x, (1, 6, 7, 7)), ref.mean(0, keepdims=True), rtol=1e-6, atol=1e-7)
    x3 = r.standard_normal((2, 5, 33)).astype(np.float32)
    np.testing.assert_allclose(oc.reduce_mean(be, x3, (2, 5, 1)), x3.astype(np.float64).mean(2, keepdims=True), rtol=1e-6, atol=1e-7)
    # constant tensor: mean is the constant exactly
    c = np.full((1, 3, 4, 4), 2.5, np.float32)
    np.testing.assert_array_equal(oc.reduce_mean(be, c, (1, 3, 1, 1)), np.full((1, 3, 1, 1), 2.5, np.float32))


def test_softmax(be):
    r = rng(10)
    x = (r.standard_normal((2, 3, 5, 16)) * 4).astype(np.float32)
    for axis in (3, -1, 1, 0):
        got = oc.softmax(be, x, axis)
        ref = torch.softmax(t64(x), dim=axis).numpy()
        np.testing.assert_allclose(got, ref, rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(got.sum(axis), 1.0, rtol=1e-6)
    # shift invariance and the closed form of a constant row
    np.testing.assert_allclose(oc.softmax(be, x + 100.0, 3), oc.softmax(be, x, 3), rtol=1e-4)
    np.testing.assert_allclose(oc.softmax(be, np.full((2, 8), 3.0, np.float32), 1), 1 / 8, rtol=1e-7)
    # large magnitudes must not overflow
    big = np.array([[1000.0, 1000.0, -1000.0]], np.float32)
    np.testing.assert_allclose(oc.softmax(be, big, 1), [[0.5, 0.5, 0.0]], atol=1e-7)


def test_layernorm(be):
    r = rng(12)
    x = (r.standard_normal((2, 7, 48)) * 3 + 1).astype(np.float32)
    g = r.standard_normal(48).astype(np.float32)
    b = r.standard_normal(48).astype(np.float32)
    got = oc.layernorm(be, x, g, b, 1e-5)
    ref = F.layer_norm(t64(x), (48,), t64(g), t64(b), 1e-5).numpy()
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-6)
    # gamma 1, beta 0: rows have zero mean and unit (biased) variance
    y = oc.layernorm(be, x, np.ones(48, np.float32), np.zeros(48, np.float32), 0.0).astype(np.float64)
    np.testing.assert_allclose(y.mean(-1), 0, atol=1e-6)
    np.testing.assert_allclose(y.var(-1), 1, rtol=1e-5)
    # equals the decomposed chain the reference emits, built from the oracle's primitives
    mu = oc.reduce_mean(be, x, (2, 7, 1))
    d = oc.tensor_op(be, _abi.OP_ADD, x, oc.unary(be, "negative", mu))
    var = oc.reduce_mean(be, oc.pow_(be, d, 2.0), (2, 7, 1))
    std = oc.unary(be, "sqrt", oc.tensor_op(be, _abi.OP_ADD, var, np.full((1, 1, 1), 1e-5, np.float32)))
    chain = oc.tensor_op(be, _abi.OP_MUL, d, oc.unary(be, "reciprocal", std))
    chain = oc.tensor_op(be, _abi.OP_ADD, oc.tensor_op(be, _abi.OP_MUL, chain, g.reshape(1, 1, 48)), b.reshape(1, 1, 48))
    np.testing.assert_allclose(got, chain, rtol=1e-5, atol=2e-6)


# ---- pooling -----------------------------------------------------------------------------

def test_conv_bias_activ_max_pool_is_the_chain_of_its_two_calls(be):
    """The oracle's dnnrtConvBiasActivMaxPool against torch (fp64 convolution rounded to the tensor's type, then
    max_pool2d: an independent statement of the chain) and against the oracle's own two calls, fp32 and fp16,
    ReLU and identity, on a first-layer shape and on one that is not (the oracle takes any)."""
    r = rng(21)
    for dt, (N, C, H, W, K, R, st, pd), (pk, pp, ps) in [(np.float32, (2, 3, 33, 36, 64, 7, 2, 3), (3, 1, 2)),
                                                        (np.float16, (2, 3, 33, 36, 64, 7, 2, 3), (3, 1, 2)),
                                                        (np.float16, (1, 5, 12, 11, 7, 3, 1, 1), (2, 0, 2))]:
        x = r.standard_normal((N, C, H, W)).astype(dt)
        w = (r.standard_normal((K, C, R, R)) * 0.2).astype(dt)
        b = r.uniform(-0.5, 0.5, K).astype(dt)
        for act in (_abi.ACT_RELU, _abi.ACT_IDENTITY):
            conv = oc.conv(be, x, w, b, (pd, pd), (st, st), 1, act)
            chain = oc.pool(be, "max", conv, (pk, pk), (pp, pp), (ps, ps))
            X, Wt, B = be.put(x), be.put(w), be.put(b)
            Y = be.empty(chain.shape, dt)
            be.ops.conv_bias_activ_max_pool(be.ptr(X), x.shape, be.ptr(Wt), w.shape, be.ptr(B), (pd, pd), (st, st), act, (pk, pk),
                                            (pp, pp, pp, pp), (ps, ps), be.ptr(Y), chain.shape, dtype=oc.DT[np.dtype(dt)])
            got = be.get(Y)
            np.testing.assert_array_equal(got, chain)
            c64 = F.conv2d(t64(x), t64(w), t64(b), st, pd)
            if act == _abi.ACT_RELU:
                c64 = c64.relu()
            ref = F.max_pool2d(torch.from_numpy(c64.numpy().astype(dt).astype(np.float32)), pk, ps, pp).numpy()
            np.testing.assert_allclose(got.astype(np.float32), ref, rtol=2e-3 if dt == np.float16 else 1e-5, atol=2e-3 if dt == np.float16 else 1e-5)
    with pytest.raises(RuntimeError, match="dimY"):
        be.ops.conv_bias_activ_max_pool(be.ptr(X), x.shape, be.ptr(Wt), w.shape, be.ptr(B), (pd, pd), (st, st), act, (pk, pk),
                                        (pp, pp, pp, pp), (ps, ps), be.ptr(Y), (1, 7, 5, 5), dtype=_abi.F16)


def test_pooling(be):
    r = rng(13)
    x = r.standard_normal((2, 3, 13, 12)).astype(np.float32)
    for k, p, s in [(3, 1, 2), (2, 0, 2), (3, 0, 1), (3, 1, 1)]:
        got = oc.pool(be, "max", x, (k, k), (p, p), (s, s))
        ref = F.max_pool2d(torch.from_numpy(x), k, s, p).numpy()
        np.testing.assert_array_equal(got, ref)
        got = oc.pool(be, "avg", x, (k, k), (p, p), (s, s))
        ref = F.avg_pool2d(t64(x), k, s, p, count_include_pad=True).numpy()
        np.testing.assert_allclose(got, ref, rtol=1e-6, atol=1e-7)
    # negative inputs: padding must not win the max
    neg = -np.abs(x) - 1
    assert (oc.pool(be, "max", neg, (3, 3), (1, 1), (2, 2)) < 0).all()


# ---- matrix products -------------------------------------------------------------------------

def test_matmul2d(be):
    r = rng(14)
    a = r.standard_normal((5, 9)).astype(np.float32)
    b = r.standard_normal((9, 7)).astype(np.float32)
    c = r.standard_normal((5, 7)).astype(np.float32)
    A, B = a.astype(np.float64), b.astype(np.float64)
    np.testing.assert_allclose(oc.matmul2d(be, a, b), A @ B, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(oc.matmul2d(be, a.T.copy(), b, transA=1), A @ B, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(oc.matmul2d(be, a, b.T.copy(), transB=1), A @ B, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(oc.matmul2d(be, a.T.copy(), b.T.copy(), transA=1, transB=1), A @ B, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(oc.matmul2d(be, a, b, c.copy(), alpha=0.5, beta=-2.0), 0.5 * (A @ B) - 2.0 * c, rtol=1e-6, atol=1e-6)
    # C as one row: the Gemm bias.  With alpha = beta = 1 it is the product followed by the bias add, bit for bit
    row = c[0].copy()
    np.testing.assert_allclose(oc.matmul2d_row(be, a, b, row, alpha=0.5, beta=-2.0), 0.5 * (A @ B) - 2.0 * row, rtol=1e-6, atol=1e-6)
    np.testing.assert_array_equal(oc.matmul2d_row(be, a, b, row), oc.tensor_op(be, _abi.OP_ADD, oc.matmul2d(be, a, b), row.reshape(1, -1)))
    np.testing.assert_array_equal(oc.matmul2d_row(be, a[:1], b, row), oc.matmul2d(be, a[:1], b, row.reshape(1, -1).copy(), beta=1.0))
    # permutation matrix: rows of b reordered exactly
    perm = np.eye(9, dtype=np.float32)[r.permutation(9)]
    np.testing.assert_array_equal(oc.matmul2d(be, perm, b), perm @ b)
    with pytest.raises(RuntimeError):
        oc.matmul2d(be, a, b, transB=1)


def test_matmul_nd(be):
    r = rng(15)
    cases = [((4, 6), (6, 3)), ((2, 4, 6), (6, 3)), ((2, 3, 4, 6), (2, 3, 6, 5)), ((1, 3, 4, 6), (1, 3, 6, 4)),
             ((2, 4, 6), (2, 6, 3)), ((4, 6), (3, 6, 2))]
    for sa, sb in cases:
        a = r.standard_normal(sa).astype(np.float32)
        b = r.standard_normal(sb).astype(np.float32)
        np.testing.assert_allclose(oc.matmul_nd(be, a, b), np.matmul(a.astype(np.float64), b.astype(np.float64)), rtol=1e-6, atol=1e-6)


def test_matmul_nd_bias(be):
    r = rng(34)
    for sa, sb in [((5, 7), (7, 3)), ((2, 4, 6, 5), (5, 8)), ((3, 6, 5), (3, 5, 4))]:
        a = r.standard_normal(sa).astype(np.float32)
        b = r.standard_normal(sb).astype(np.float32)
        bias = r.standard_normal(sb[-1]).astype(np.float32)
        ref = np.matmul(a.astype(np.float64), b.astype(np.float64)) + bias
        np.testing.assert_allclose(oc.matmul_nd_bias(be, a, b, bias), ref, rtol=1e-5, atol=1e-5)
        z = r.standard_normal(ref.shape).astype(np.float32)
        np.testing.assert_allclose(oc.matmul_nd_bias(be, a, b, bias, z=z), ref + z, rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(oc.matmul_nd_bias(be, a, b, bias, gelu=True), F.gelu(torch.from_numpy(ref)).numpy(), rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(oc.matmul_nd_bias(be, a, b, bias, z=z, gelu=True), F.gelu(torch.from_numpy(ref + z)).numpy(),
                                   rtol=1e-5, atol=1e-5)


def attention_ref(q, k, v, heads, scale):
    B, Sq, hidden = q.shape
    D = hidden // heads
    qh = t64(q).reshape(B, Sq, heads, D).permute(0, 2, 1, 3)
    kh = t64(k).reshape(B, -1, heads, D).permute(0, 2, 1, 3)
    vh = t64(v).reshape(B, -1, heads, D).permute(0, 2, 1, 3)
    p = torch.softmax(qh @ kh.transpose(-1, -2) * scale, -1)
    return (p @ vh).permute(0, 2, 1, 3).reshape(B, Sq, hidden).numpy()


def test_attention(be):
    r = rng(35)
    for B, Sq, Sk, H, D in [(1, 16, 16, 4, 64), (2, 5, 9, 3, 32), (1, 7, 1, 2, 128)]:
        q, k, v = (r.standard_normal((B, S, H * D)).astype(np.float32) for S in (Sq, Sk, Sk))
        got = oc.attention(be, q, k, v, H, 1.0 / math.sqrt(D))
        np.testing.assert_allclose(got, attention_ref(q, k, v, H, 1.0 / math.sqrt(D)), rtol=1e-5, atol=1e-6)
    # one key: the soft-max is 1 and the output is that key's value row, whatever the scores
    np.testing.assert_allclose(got, np.broadcast_to(v, got.shape), rtol=1e-6, atol=1e-6)
    # Q, K, V as column blocks of one wider tensor
    qkv = r.standard_normal((2, 9, 3 * 96)).astype(np.float32)
    np.testing.assert_allclose(oc.attention_packed(be, qkv, 3, 0.2),
                               attention_ref(qkv[:, :, :96], qkv[:, :, 96:192], qkv[:, :, 192:], 3, 0.2), rtol=1e-5, atol=1e-6)
    # heads do not mix: changing head 1's keys leaves head 0's output alone
    q, k, v = (r.standard_normal((1, 6, 128)).astype(np.float32) for _ in range(3))
    a = oc.attention(be, q, k, v, 2, 0.125)
    k2 = k.copy(); k2[:, :, 64:] *= 2.0
    b = oc.attention(be, q, k2, v, 2, 0.125)
    np.testing.assert_array_equal(a[:, :, :64], b[:, :, :64])
    assert np.abs(a[:, :, 64:] - b[:, :, 64:]).max() > 1e-3


# ---- data movement --------------------------------------------------------------------------------

def test_data_movement(be):
    r = rng(16)
    x = r.standard_normal((2, 3, 4, 5)).astype(np.float32)
    np.testing.assert_array_equal(oc.flatten(be, x, 1), x.reshape(2, 60))
    np.testing.assert_array_equal(oc.reshape(be, x, (6, 20)), x.reshape(6, 20))
    for perm in [(0, 2, 1, 3), (0, 2, 3, 1), (3, 2, 1, 0), (1, 0, 2, 3)]:
        np.testing.assert_array_equal(oc.transpose(be, x, perm), x.transpose(perm))
    np.testing.assert_array_equal(oc.transpose(be, x[0], (1, 0, 2)), x[0].transpose(1, 0, 2))
    np.testing.assert_array_equal(oc.transpose(be, x[0, 0], (1, 0)), x[0, 0].T)
    xi = r.integers(-5, 5, (3, 4)).astype(np.int64)
    np.testing.assert_array_equal(oc.transpose(be, xi, (1, 0)), xi.T)
    table = r.standard_normal((11, 6)).astype(np.float32)
    idx = r.integers(0, 11, (2, 5))
    np.testing.assert_array_equal(oc.gather(be, table, idx, 0), np.take(table, idx, 0))
    np.testing.assert_array_equal(oc.gather(be, table, np.array([-1, 0]), 0), np.take(table, [-1, 0], 0))
    np.testing.assert_array_equal(oc.gather(be, x, np.array([2, 0]), 2), np.take(x, [2, 0], 2))
    ti = r.integers(-1000, 1000, (7, 3, 2)).astype(np.int64)     # CUDAGatherInt64Func: same walk on 8-byte elements
    np.testing.assert_array_equal(oc.gather(be, ti, np.array([[6, 0], [3, -2]]), 0), np.take(ti, [[6, 0], [3, -2]], 0))
    np.testing.assert_array_equal(oc.gather(be, ti, np.array([1]), 2), np.take(ti, [1], 2))
    with pytest.raises(RuntimeError):
        oc.gather(be, table, np.array([11]), 0)


def test_conv_with_clipped_and_leaky_relu(be):
    # modes 3 and 6 of the fused call against torch's operators applied to torch's convolution
    r = rng(33)
    x = r.standard_normal((2, 6, 9, 9)).astype(np.float32)
    w = (r.standard_normal((8, 6, 3, 3)) * 0.5).astype(np.float32)
    b = r.standard_normal(8).astype(np.float32)
    z = r.standard_normal((2, 8, 9, 9)).astype(np.float32)
    y = F.conv2d(t64(x), t64(w), t64(b), padding=1)
    got = oc.conv(be, x, w, b, pads=(1, 1), activ=_abi.ACT_CLIPPED_RELU, coef=1.5)
    np.testing.assert_allclose(got, torch.clamp(y, 0, 1.5).numpy(), rtol=1e-5, atol=1e-5)
    assert got.max() == 1.5 and got.min() == 0.0            # both bounds bite on this input
    got = oc.conv(be, x, w, b, pads=(1, 1), activ=_abi.ACT_LEAKY_RELU, coef=0.1)
    np.testing.assert_allclose(got, F.leaky_relu(y, 0.1).numpy(), rtol=1e-5, atol=1e-5)
    got = oc.conv(be, x, w, b, pads=(1, 1), activ=_abi.ACT_LEAKY_RELU, coef=0.1, z=z)
    np.testing.assert_allclose(got, F.leaky_relu(y + t64(z), 0.1).numpy(), rtol=1e-5, atol=1e-5)
    got = oc.conv(be, x, w, b, pads=(1, 1), activ=_abi.ACT_CLIPPED_RELU, coef=6.0, z=z)
    np.testing.assert_allclose(got, torch.clamp(y + t64(z), 0, 6).numpy(), rtol=1e-5, atol=1e-5)
    # the coefficient is sticky and does not touch ReLU
    np.testing.assert_allclose(oc.conv(be, x, w, b, pads=(1, 1), activ=_abi.ACT_RELU), F.relu(y).numpy(), rtol=1e-5, atol=1e-5)
    # the same through the stand-alone activation call
    X, Y = be.put(x), be.empty(x.shape, x.dtype)
    be.ops.set_activation_coef(0.25)
    be.ops.active(be.ptr(X), x.shape, _abi.ACT_LEAKY_RELU, be.ptr(Y), _abi.F32)
    np.testing.assert_array_equal(be.get(Y), np.where(x < 0, np.float32(0.25) * x, x))
    be.ops.active(be.ptr(X), x.shape, _abi.ACT_CLIPPED_RELU, be.ptr(Y), _abi.F32)
    np.testing.assert_array_equal(be.get(Y), np.clip(x, 0, 0.25))
    with pytest.raises(RuntimeError):
        oc.conv(be, x, w, b, pads=(1, 1), activ=4)             # ELU: not a mode of this runtime


def test_leaky_relu_and_prelu(be):
    # pinned by the defining formula on hand-picked values and by torch's operators
    x = np.array([-2.0, -0.5, 0.0, 0.5, 3.0], np.float32)
    np.testing.assert_array_equal(oc.leaky_relu(be, x, 0.25), np.array([-0.5, -0.125, 0.0, 0.5, 3.0], np.float32))
    np.testing.assert_array_equal(oc.leaky_relu(be, x, 0.0), np.maximum(x, 0))      # alpha 0 is relu
    np.testing.assert_array_equal(oc.leaky_relu(be, x, 1.0), x)                     # alpha 1 is the identity
    r = rng(31)
    t = r.standard_normal((2, 5, 3, 4)).astype(np.float32)
    np.testing.assert_array_equal(oc.leaky_relu(be, t, 0.1), F.leaky_relu(torch.from_numpy(t), 0.1).numpy())
    # one shared slope: what the reference kernel computes (it reads slope[0])
    np.testing.assert_array_equal(oc.prelu(be, t, np.array([0.3], np.float32)),
                                  F.prelu(torch.from_numpy(t), torch.tensor([0.3])).numpy())
    # per-channel slope, ONNX shape [C,1,1]: a transposed broadcast (over W or N) fails here
    sl = r.standard_normal((5, 1, 1)).astype(np.float32)
    np.testing.assert_array_equal(oc.prelu(be, t, sl), F.prelu(torch.from_numpy(t), torch.from_numpy(sl.reshape(5))).numpy())
    full = r.standard_normal(t.shape).astype(np.float32)
    np.testing.assert_array_equal(oc.prelu(be, t, full), np.where(t < 0, full * t, t))
    h = t.astype(np.float16)
    np.testing.assert_array_equal(oc.leaky_relu(be, h, 0.1), np.where(h < 0, (np.float32(0.1) * h.astype(np.float32)), h).astype(np.float16))
    with pytest.raises(RuntimeError):
        oc.prelu(be, t, np.ones((4, 1, 1), np.float32))


def test_concat_squeeze_unsqueeze(be):
    r = rng(32)
    a = r.standard_normal((2, 3, 4, 5)).astype(np.float32)
    for axis in range(4):
        shapes = [list(a.shape) for _ in range(3)]
        shapes[1][axis], shapes[2][axis] = 1, 7
        xs = [r.standard_normal(s).astype(np.float32) for s in shapes]
        np.testing.assert_array_equal(oc.concat(be, xs, axis), np.concatenate(xs, axis))
    np.testing.assert_array_equal(oc.concat(be, [a], 1), a)
    np.testing.assert_array_equal(oc.concat(be, [a, a], -1), np.concatenate([a, a], -1))
    xi = [r.integers(-9, 9, (3, k)).astype(np.int64) for k in (1, 4, 2)]
    np.testing.assert_array_equal(oc.concat(be, xi, 1), np.concatenate(xi, 1))
    xh = [r.standard_normal((2, k, 3)).astype(np.float16) for k in (3, 5)]
    np.testing.assert_array_equal(oc.concat(be, xh, 1), np.concatenate(xh, 1))
    many = [r.standard_normal((1, 2)).astype(np.float32) for _ in range(16)]
    np.testing.assert_array_equal(oc.concat(be, many, 0), np.concatenate(many, 0))
    with pytest.raises(RuntimeError):
        oc.concat(be, many + [many[0]], 0)                 # 17 inputs
    with pytest.raises(RuntimeError):
        oc.concat(be, [a, a[:, :, :3]], 1)                 # differ off the axis
    s = r.standard_normal((2, 1, 4, 1)).astype(np.float32)
    np.testing.assert_array_equal(oc.squeeze(be, s, (2, 4)), s.reshape(2, 4))
    np.testing.assert_array_equal(oc.squeeze(be, s, (2, 4, 1)), s.reshape(2, 4, 1))
    np.testing.assert_array_equal(oc.squeeze(be, s.reshape(2, 4), (1, 2, 1, 4), un=True), s.reshape(1, 2, 1, 4))
    with pytest.raises(RuntimeError):
        oc.squeeze(be, s, (4, 2))


def test_expand_broadcasts_like_numpy(be):
    # the reference's copy (CUDAExpandInt64Func.cu:10-15) is the case out == in
    r = rng(33)
    xi = r.integers(-9, 9, (3, 1, 5)).astype(np.int64)
    np.testing.assert_array_equal(oc.expand(be, xi, (3, 1, 5)), xi)
    for shape, out in [((3, 1, 5), (3, 4, 5)), ((3, 1, 5), (2, 3, 4, 5)), ((1,), (7,)), ((4, 1), (4, 6)),
                       ((1, 1, 1), (2, 3, 4)), ((5,), (2, 5)), ((2, 1, 3, 1, 2), (2, 4, 3, 5, 2))]:
        for dtype in (np.int64, np.float32, np.float16):
            x = (r.integers(-99, 99, shape).astype(dtype))
            np.testing.assert_array_equal(oc.expand(be, x, out), np.broadcast_to(x, out))
    with pytest.raises(RuntimeError):
        oc.expand(be, xi, (3, 4, 6))          # 5 does not broadcast to 6
    with pytest.raises(RuntimeError):
        oc.expand(be, xi, (4, 5))             # output rank below the input's


def test_nonzero_lists_flat_indices_in_order(be):
    # CUDANonZeroFloatFunc.cu:4-17: indices as values of the input's type, front of the output only
    r = rng(34)
    for dtype in (np.float32, np.int64, np.float16):
        x = (r.integers(-2, 3, (3, 5, 7)) * (r.random((3, 5, 7)) < 0.4)).astype(dtype)
        want = np.flatnonzero(x.reshape(-1))
        out = oc.nonzero(be, x, (1, x.size), -7)
        np.testing.assert_array_equal(out.reshape(-1)[: want.size], want.astype(dtype))
        np.testing.assert_array_equal(out.reshape(-1)[want.size:], np.full(x.size - want.size, -7, dtype))
        # an output smaller than the count holds the first indices only
        small = oc.nonzero(be, x, (3,), -7)
        np.testing.assert_array_equal(small, want[:3].astype(dtype))
    z = np.array([0.0, -0.0, np.nan, 1e-45, 0.0], np.float32)   # -0 is zero, NaN and denormals are not
    np.testing.assert_array_equal(oc.nonzero(be, z, (5,), -1.0), np.array([2, 3, -1, -1, -1], np.float32))
    np.testing.assert_array_equal(oc.nonzero(be, np.zeros((4, 4), np.float32), (16,), 5.0), np.full(16, 5.0, np.float32))


def test_empty_tensors_are_no_ops(be):
    # The reference's wrappers launch zero blocks for an empty tensor and return: no work, no error.
    got = oc.empty_tensor_behaviour(be)
    assert len(got) >= 30 and set(got.values()) == {"untouched"}, got


def test_layouts_the_oracle_lacks_are_refused(be):
    # The oracle restates the reference, which knows N,C,H,W tensors and
    # K,C,R,S filters only; asking it for anything else must fail, not drift.
    with pytest.raises(RuntimeError):
        be.ops.set_format(_abi.NHWC)
    with pytest.raises(RuntimeError):
        be.ops.set_filter_layout(_abi.FILTER_CRSK)
    be.ops.set_format(_abi.NCHW)
    be.ops.set_filter_layout(_abi.FILTER_KCRS)
