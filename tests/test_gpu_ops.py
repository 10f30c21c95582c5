"""Parity of the gfx950 library with the CPU oracle, operator by operator,
through the C ABI on the same seeded inputs.

Bars: bit-exact for copies, index work, max, clip, negate, ReLU, two-operand
add/mul, reciprocal and sqrt (no reassociation is involved); fp32 reductions
and transcendental functions within rtol 1e-4 / atol 1e-5 of the oracle
(which accumulates in double); fp16 storage within rtol 2e-2.
"""
import numpy as np
import pytest

import opcases as oc
from helpers import GpuBackend, OracleBackend, rng
from occamy_amd import _abi

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


@pytest.fixture(scope="module")
def gpu():
    return GpuBackend()


@pytest.fixture(scope="module")
def cpu():
    return OracleBackend()


def close(got, ref, rtol=RTOL, atol=ATOL):
    np.testing.assert_allclose(got, ref, rtol=rtol, atol=atol)


# ---- convolution ----------------------------------------------------------------

CONV_CASES = [
    # N, C, H, W, K, R, S, stride, pad, group
    (1, 64, 56, 56, 64, 3, 3, 1, 1, 1),     # the single-conv configuration (Kaiming-uniform below)
    (1, 3, 224, 224, 64, 7, 7, 2, 3, 1),    # ResNet stem
    (1, 64, 56, 56, 256, 1, 1, 1, 0, 1),
    (1, 256, 56, 56, 512, 1, 1, 2, 0, 1),   # strided 1x1 downsample
    (1, 128, 56, 56, 128, 3, 3, 2, 1, 1),
    (1, 512, 7, 7, 512, 3, 3, 1, 1, 1),     # 49 pixels: ragged column tile
    (1, 2048, 7, 7, 512, 1, 1, 1, 0, 1),
    (2, 16, 9, 11, 24, 3, 3, 1, 1, 1),      # batch > 1, ragged everything
    (3, 5, 8, 8, 7, 2, 3, 1, 0, 1),         # generic filter size, odd channels
    (1, 8, 12, 12, 16, 5, 5, 1, 2, 1),
    (1, 16, 10, 10, 32, 3, 3, 1, 1, 4),     # grouped
    (1, 32, 112, 112, 32, 3, 3, 1, 1, 32),  # MobileNetV2 depthwise
    (1, 96, 112, 112, 96, 3, 3, 2, 1, 96),  # depthwise stride 2
    (2, 6, 7, 7, 12, 3, 3, 1, 1, 6),        # depthwise with channel multiplier 2
    (1, 1, 5, 5, 1, 3, 3, 1, 1, 1),         # smallest
    (1, 64, 96, 80, 3, 3, 3, 1, 1, 1),      # image-producing last layer: three output channels
    (2, 16, 21, 17, 4, 3, 3, 2, 1, 1),      # four output channels, stride 2
    (2, 24, 9, 9, 2, 1, 1, 1, 0, 1),        # two output channels, 1x1
    # 3x3 layers that fill the chip (the LDS-tiled 3x3 kernel): 128x128 tiles with an odd channel count and
    # ragged rows; 64x64 tiles, stride 2, no padding; groups
    (1, 5, 190, 180, 130, 3, 3, 1, 1, 1),
    (2, 8, 260, 130, 64, 3, 3, 2, 0, 1),
    (1, 8, 182, 182, 256, 3, 3, 1, 1, 2),
]


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(map(str, c)))
def test_conv_f32(gpu, cpu, case):
    N, C, H, W, K, R, S, st, pd, g = case
    r = rng(hash(case) % (2 ** 31))
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    bound = np.sqrt(6.0 / (C // g * R * S))
    w = r.uniform(-bound, bound, (K, C // g, R, S)).astype(np.float32)
    b = r.uniform(-0.1, 0.1, K).astype(np.float32)
    args = ((pd, pd), (st, st), g)
    close(oc.conv(gpu, x, w, None, *args), oc.conv(cpu, x, w, None, *args))
    ref = oc.conv(cpu, x, w, b, *args, _abi.ACT_RELU)
    got = oc.conv(gpu, x, w, b, *args, _abi.ACT_RELU)
    close(got, ref)
    assert (got >= 0).all()
    close(oc.conv(gpu, x, w, b, *args, _abi.ACT_IDENTITY), oc.conv(cpu, x, w, b, *args, _abi.ACT_IDENTITY))
    # the same filter handed over C,R,S,K: same kernels' K,C,R,S result up to
    # the summation order of the tile shapes each layout selects
    close(oc.conv(gpu, x, w, b, *args, _abi.ACT_RELU, crsk=True), ref)
    close(oc.conv(gpu, x, w, None, *args, crsk=True), oc.conv(cpu, x, w, None, *args))
    # residual operand: relu((conv + b) + z); bit-equal to this library's own
    # conv -> add -> relu chain, which forms the same sums in the same order
    z = r.standard_normal(ref.shape).astype(np.float32)
    fused = oc.conv(gpu, x, w, b, *args, _abi.ACT_RELU, z=z)
    close(fused, oc.conv(cpu, x, w, b, *args, _abi.ACT_RELU, z=z))
    lin = oc.conv(gpu, x, w, b, *args, _abi.ACT_IDENTITY)
    np.testing.assert_array_equal(fused, oc.unary(gpu, "relu", oc.tensor_op(gpu, _abi.OP_ADD, lin, z)))
    close(oc.conv(gpu, x, w, b, *args, _abi.ACT_RELU, crsk=True, z=z), fused)
    # the result written over the residual operand (Z == Y): the same bits, from the kernels of either filter layout
    np.testing.assert_array_equal(oc.conv(gpu, x, w, b, *args, _abi.ACT_RELU, z=z, inplace=True), fused)
    np.testing.assert_array_equal(oc.conv(gpu, x, w, b, *args, _abi.ACT_RELU, crsk=True, z=z, inplace=True),
                                  oc.conv(gpu, x, w, b, *args, _abi.ACT_RELU, crsk=True, z=z))
    np.testing.assert_array_equal(oc.conv(cpu, x, w, b, *args, _abi.ACT_RELU, z=z, inplace=True), oc.conv(cpu, x, w, b, *args, _abi.ACT_RELU, z=z))


def random_conv_cases(seed, count, f16):
    """Seeded shapes around the kernels' boundaries: channel counts on both sides of the multiples of 8, 32 and
    64 the fast paths ask for, filter sizes 1 / 2 / 3 / 5 / 7, strides 1-3 (different along the two axes now and
    then), padding up to the filter's half and beyond, a few hundred to a few thousand output pixels."""
    r = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        R, S = (int(v) for v in r.choice([1, 1, 2, 3, 3, 3, 5, 7], 2)) if r.random() < 0.3 else (int(r.choice([1, 3, 3, 5])),) * 2
        grp = int(r.choice([1, 1, 1, 1, 2, 4])) if not f16 or r.random() < 0.3 else 1
        cg = int(r.choice([1, 3, 8, 16, 31, 32, 33, 64, 96, 128, 160, 192, 256])) if f16 else int(r.choice([1, 2, 3, 5, 8, 16, 24, 33, 64, 100]))
        kg = int(r.choice([1, 2, 8, 24, 40, 64, 72, 128, 136, 200, 256])) if f16 else int(r.choice([1, 2, 3, 4, 7, 16, 33, 64, 130]))
        if grp > 1:
            cg, kg = min(cg, 32), min(kg, 40)
        N, H, W = int(r.integers(1, 5)), int(r.integers(1, 30)), int(r.integers(1, 30))
        sh, sw = (int(r.integers(1, 4)),) * 2 if r.random() < 0.8 else (int(r.integers(1, 4)), int(r.integers(1, 4)))
        ph, pw = int(r.integers(0, R // 2 + 2)), int(r.integers(0, S // 2 + 2))
        P, Q = (H + 2 * ph - R) // sh + 1, (W + 2 * pw - S) // sw + 1
        if P < 1 or Q < 1 or H + 2 * ph < R or W + 2 * pw < S or N * cg * grp * H * W > 2_000_000 or N * kg * grp * P * Q > 2_000_000:
            continue
        cases.append((N, cg * grp, H, W, kg * grp, R, S, sh, sw, ph, pw, grp))
    return cases


def test_conv_f32_random_shapes(gpu, cpu):
    """120 seeded shapes through dnnrtConvBiasActiv / dnnrtConvBiasAddActiv on fp32 N,C,H,W tensors against the
    oracle (rtol 1e-4, atol 1e-5), with both filter layouts, each activation mode once in a while, and the residual
    form also written over its residual operand."""
    for i, (N, C, H, W, K, R, S, sh, sw, ph, pw, grp) in enumerate(random_conv_cases(2024, 120, False)):
        r = rng(1000 + i)
        x = r.standard_normal((N, C, H, W)).astype(np.float32)
        w = (r.standard_normal((K, C // grp, R, S)) * np.sqrt(2.0 / (C // grp * R * S))).astype(np.float32)
        b = r.uniform(-0.3, 0.3, K).astype(np.float32)
        activ, coef = [(_abi.ACT_RELU, None), (_abi.ACT_IDENTITY, None), (_abi.ACT_CLIPPED_RELU, 0.7), (_abi.ACT_LEAKY_RELU, 0.1)][i % 4]
        what = f"case {i}: x {x.shape} w {w.shape} strides {(sh, sw)} pads {(ph, pw)} group {grp} act {activ}"
        ref = oc.conv(cpu, x, w, b, (ph, pw), (sh, sw), grp, activ, coef=coef)
        for crsk in (False, True):
            got = oc.conv(gpu, x, w, b, (ph, pw), (sh, sw), grp, activ, crsk=crsk, coef=coef)
            np.testing.assert_allclose(got, ref, rtol=RTOL, atol=ATOL, err_msg=what)
        z = r.standard_normal(ref.shape).astype(np.float32)
        refz = oc.conv(cpu, x, w, b, (ph, pw), (sh, sw), grp, activ, z=z, coef=coef)
        gotz = oc.conv(gpu, x, w, b, (ph, pw), (sh, sw), grp, activ, z=z, coef=coef)
        np.testing.assert_allclose(gotz, refz, rtol=RTOL, atol=ATOL, err_msg=what + " + z")
        np.testing.assert_array_equal(oc.conv(gpu, x, w, b, (ph, pw), (sh, sw), grp, activ, z=z, coef=coef, inplace=True), gotz, err_msg=what + " in place")


def test_conv_f16_random_shapes(gpu, cpu):
    """120 seeded shapes through the fp16 convolution, channels-last (every fast path's boundary: channel counts
    around the multiples of 8 / 32 / 64, a few steps or many, padded or not, grouped and depthwise) and, every
    third case, N,C,H,W; against the oracle to one fp16 rounding (rtol 2e-3, atol 2e-3; 4e-3 with a residual),
    the residual form also in place."""
    for i, (N, C, H, W, K, R, S, sh, sw, ph, pw, grp) in enumerate(random_conv_cases(4048, 120, True)):
        if R != S or sh != sw or ph != pw:  # the fp16 helper takes square geometry
            S, sw, pw = R, sh, ph
            if (W + 2 * pw - S) // sw + 1 < 1 or W + 2 * pw < S:
                continue
        r = rng(3000 + i)
        x = r.standard_normal((N, C, H, W)).astype(np.float16)
        w = (r.standard_normal((K, C // grp, R, R)) * np.sqrt(2.0 / (C // grp * R * R))).astype(np.float16)
        b = r.uniform(-0.3, 0.3, K).astype(np.float16)
        fmt = _abi.NCHW if i % 3 == 2 else _abi.NHWC
        what = f"case {i}: x {x.shape} w {w.shape} stride {sh} pad {ph} group {grp} format {fmt}"
        ref = oc.conv(cpu, x, w, b, (ph, ph), (sh, sh), grp, _abi.ACT_RELU)
        got = conv_f16(gpu, x, w, b, (ph, ph), (sh, sh), grp, _abi.ACT_RELU, fmt)
        np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=2e-3, atol=2e-3, err_msg=what)
        z = r.standard_normal(ref.shape).astype(np.float16)
        refz = oc.conv(cpu, x, w, b, (ph, ph), (sh, sh), grp, _abi.ACT_RELU, z=z)
        gotz = conv_f16(gpu, x, w, b, (ph, ph), (sh, sh), grp, _abi.ACT_RELU, fmt, z=z)
        np.testing.assert_allclose(gotz.astype(np.float32), refz.astype(np.float32), rtol=4e-3, atol=4e-3, err_msg=what + " + z")
        np.testing.assert_array_equal(conv_f16(gpu, x, w, b, (ph, ph), (sh, sh), grp, _abi.ACT_RELU, fmt, z=z, inplace=True), gotz,
                                      err_msg=what + " in place")


def test_conv_f16_pointwise_and_depthwise_random_shapes(gpu, cpu):
    """Seeded channels-last fp16 shapes aimed at the two kernels without a workgroup tile: 1x1 stride-1 layers over
    a multiple of 8 channels up to 256 that is not a multiple of 64 (one to sixteen 16-channel steps, the last one
    half empty every other time; few and many filters, so that results leave both through the staging tile and
    straight from the accumulators; ragged last wavefronts; few pixels, so that the filter blocks are dealt over the
    grid) and 3x3 depthwise layers with stride 1 and 2 and padding 0 to 2; each activation mode in turn, with and
    without a residual, which is also written in place.  Against the oracle to one fp16 rounding."""
    r = np.random.default_rng(909)
    acts = [(_abi.ACT_RELU, None), (_abi.ACT_IDENTITY, None), (_abi.ACT_CLIPPED_RELU, 0.7), (_abi.ACT_LEAKY_RELU, 0.1)]
    for i in range(60):
        N, H, W = int(r.integers(1, 5)), int(r.integers(1, 25)), int(r.integers(1, 25))
        if i % 2 == 0:  # pointwise
            C = 8 * int(r.integers(1, 33))
            if C % 64 == 0:
                C += 8
            K = 8 * int(r.choice([1, 2, 3, 4, 5, 8, 9, 12, 18, 40]))
            R, st, pd, grp = 1, 1, 0, 1
        else:           # depthwise
            C = K = 8 * int(r.integers(1, 40))
            R, st, pd, grp = 3, int(r.integers(1, 3)), int(r.integers(0, 3)), C
            if H + 2 * pd < 3 or W + 2 * pd < 3:
                H, W = H + 3, W + 3
        activ, coef = acts[(i // 2) % 4]
        q = rng(5000 + i)
        x = q.standard_normal((N, C, H, W)).astype(np.float16)
        w = (q.standard_normal((K, C // grp, R, R)) * np.sqrt(2.0 / (C // grp * R * R))).astype(np.float16)
        b = q.uniform(-0.3, 0.3, K).astype(np.float16)
        what = f"case {i}: x {x.shape} w {w.shape} stride {st} pad {pd} group {grp} act {activ}"
        if coef is not None:
            gpu.ops.set_activation_coef(coef)
        ref = oc.conv(cpu, x, w, b, (pd, pd), (st, st), grp, activ, coef=coef)
        got = conv_f16(gpu, x, w, b, (pd, pd), (st, st), grp, activ, _abi.NHWC)
        np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=2e-3, atol=2e-3, err_msg=what)
        z = q.standard_normal(ref.shape).astype(np.float16)
        refz = oc.conv(cpu, x, w, b, (pd, pd), (st, st), grp, activ, z=z, coef=coef)
        gotz = conv_f16(gpu, x, w, b, (pd, pd), (st, st), grp, activ, _abi.NHWC, z=z)
        np.testing.assert_allclose(gotz.astype(np.float32), refz.astype(np.float32), rtol=4e-3, atol=4e-3, err_msg=what + " + z")
        np.testing.assert_array_equal(conv_f16(gpu, x, w, b, (pd, pd), (st, st), grp, activ, _abi.NHWC, z=z, inplace=True), gotz,
                                      err_msg=what + " in place")


def test_rowwise_ops_random_shapes(gpu, cpu):
    """Seeded sweeps of soft-max, LayerNorm, ReduceMean and the poolings over shapes around their kernels'
    boundaries (row lengths on both sides of 4-element groups, of the in-register limit and of a wavefront;
    reductions over an inner, a middle and an outer run), fp32 and fp16, against the oracle."""
    r = np.random.default_rng(77)
    for i in range(60):
        rows = int(r.choice([1, 2, 3, 7, 64, 130]))
        L = int(r.choice([1, 2, 3, 4, 5, 31, 32, 33, 63, 64, 65, 127, 128, 255, 256, 257, 768, 1000, 1024, 2047, 2048, 2049, 2052, 3000, 4100]))
        for dtype, tol in ((np.float32, 1e-4), (np.float16, 4e-3)):
            x = (r.standard_normal((rows, L)) * 2 + 0.5).astype(dtype)
            close(oc.softmax(gpu, x, 1), oc.softmax(cpu, x, 1), tol, tol * 1e-2 if dtype == np.float32 else tol)
            if L > 1:
                g, b = r.standard_normal(L).astype(dtype), r.standard_normal(L).astype(dtype)
                close(oc.layernorm(gpu, x, g, b, 1e-5), oc.layernorm(cpu, x, g, b, 1e-5), max(tol, 2e-4), max(tol, 2e-4) * 4)
    for i in range(40):
        outer, red, inner = (int(v) for v in (r.integers(1, 9), r.choice([1, 2, 5, 7, 49, 64, 100, 257]), r.choice([1, 2, 3, 4, 8, 16, 48, 130])))
        for dtype, tol in ((np.float32, 1e-5), (np.float16, 2e-3)):
            x = r.standard_normal((outer, red, inner)).astype(dtype)
            close(oc.reduce_mean(gpu, x, (outer, 1, inner)), oc.reduce_mean(cpu, x, (outer, 1, inner)), tol, tol)
    for i in range(40):
        N, C, H, W = (int(v) for v in (r.integers(1, 4), r.choice([1, 3, 8, 16, 24, 33]), r.integers(2, 24), r.integers(2, 24)))
        k = (int(r.integers(1, 4)), int(r.integers(1, 4)))
        st = (int(r.integers(1, 4)), int(r.integers(1, 4)))
        pd = (int(r.integers(0, (k[0] + 1) // 2 + (k[0] > 1) - (k[0] == 2))), int(r.integers(0, (k[1] + 1) // 2 + (k[1] > 1) - (k[1] == 2))))
        pd = (min(pd[0], k[0] // 2), min(pd[1], k[1] // 2))
        if H + 2 * pd[0] < k[0] or W + 2 * pd[1] < k[1]:
            continue
        for dtype in (np.float32, np.float16):
            x = r.standard_normal((N, C, H, W)).astype(dtype)
            if i % 5 == 0:
                x[0, 0, H // 2, W // 2] = np.nan
            got, ref = oc.pool(gpu, "max", x, k, pd, st), oc.pool(cpu, "max", x, k, pd, st)
            np.testing.assert_array_equal(got, ref, err_msg=f"max pool {x.shape} k {k} pads {pd} strides {st} {dtype.__name__}")
            if i % 5:
                tol = 1e-5 if dtype == np.float32 else 2e-3
                close(oc.pool(gpu, "avg", x, k, pd, st), oc.pool(cpu, "avg", x, k, pd, st), tol, tol)


def test_products_random_shapes(gpu, cpu):
    """Seeded sweeps of the 2-D product (every layout, alpha / beta, row and matrix C) and the batched product with
    bias, residual and GELU over ragged shapes, fp32 and fp16, against the oracle."""
    r = np.random.default_rng(78)
    dims = [1, 2, 3, 5, 8, 17, 31, 32, 33, 64, 65, 100, 128, 130, 257]
    for i in range(50):
        M, K, N = (int(r.choice(dims)) for _ in range(3))
        tA, tB = int(r.integers(0, 2)), int(r.integers(0, 2))
        for dtype, tol in ((np.float32, (1e-4, 1e-4)), (np.float16, (4e-3, 8e-3))):
            a = r.standard_normal((K, M) if tA else (M, K)).astype(dtype)
            b = (r.standard_normal((N, K) if tB else (K, N)) / np.sqrt(K)).astype(dtype)
            kw = [dict(), dict(alpha=0.5), dict(c=r.standard_normal((M, N)).astype(dtype), alpha=1.5, beta=0.5)][i % 3]
            got, ref = oc.matmul2d(gpu, a, b, transA=tA, transB=tB, **kw), oc.matmul2d(cpu, a, b, transA=tA, transB=tB, **kw)
            np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=tol[0], atol=tol[1],
                                       err_msg=f"[{M},{K}]x[{K},{N}] transA {tA} transB {tB} {kw.keys()} {dtype.__name__}")
    for i in range(40):
        M, K, N = (int(r.choice(dims)) for _ in range(3))
        batch = [(), (2,), (3, 2)][i % 3]
        shared_b = i % 2 == 0
        for dtype, tol in ((np.float32, (1e-4, 1e-4)), (np.float16, (1e-2, 1e-2))):
            a = r.standard_normal(batch + (M, K)).astype(dtype)
            b = (r.standard_normal((() if shared_b else batch) + (K, N)) / np.sqrt(K)).astype(dtype)
            bias = r.standard_normal(N).astype(dtype)
            z = r.standard_normal(batch + (M, N)).astype(dtype)
            kw = [dict(), dict(z=z), dict(gelu=True), dict(z=z, gelu=True)][i % 4]
            got, ref = oc.matmul_nd_bias(gpu, a, b, bias, **kw), oc.matmul_nd_bias(cpu, a, b, bias, **kw)
            np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=tol[0], atol=tol[1],
                                       err_msg=f"{a.shape} x {b.shape} {list(kw)} {dtype.__name__}")
            got, ref = oc.matmul_nd(gpu, a, b), oc.matmul_nd(cpu, a, b)
            np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=tol[0], atol=tol[1], err_msg=f"{a.shape} x {b.shape}")


def test_conv_closed_forms(gpu):
    x = rng(1).standard_normal((1, 3, 8, 8)).astype(np.float32)
    w = np.zeros((3, 3, 3, 3), np.float32)
    for c in range(3):
        w[c, c, 1, 1] = 1
    np.testing.assert_array_equal(oc.conv(gpu, x, w, None, (1, 1), (1, 1)), x)
    w = np.zeros((1, 1, 3, 3), np.float32)
    w[0, 0, 0, 2] = 1
    xi = np.arange(36, dtype=np.float32).reshape(1, 1, 6, 6)
    exp = np.zeros((6, 6), np.float32)
    exp[1:, :-1] = xi[0, 0, :-1, 1:]
    np.testing.assert_array_equal(oc.conv(gpu, xi, w, None, (1, 1), (1, 1))[0, 0], exp)


def test_conv_errors(gpu):
    x = np.zeros((1, 4, 4, 4), np.float32)
    with pytest.raises(RuntimeError):
        oc.conv(gpu, x, np.zeros((4, 3, 1, 1), np.float32))
    with pytest.raises(RuntimeError):
        oc.conv(gpu, x, np.zeros((4, 4, 7, 7), np.float32))


# ---- elementwise -----------------------------------------------------------------

@pytest.mark.parametrize("n", [1, 3, 255, 256, 1025, 200704])
def test_unary_exact(gpu, cpu, n):
    x = np.concatenate([rng(n).standard_normal(n) * 3]).astype(np.float32)
    x[0] = -0.0
    for name, kw in [("relu", {}), ("negative", {}), ("clip", {"lo": 0.0, "hi": 6.0})]:
        np.testing.assert_array_equal(oc.unary(gpu, name, x, **kw), oc.unary(cpu, name, x, **kw))
    nz = np.where(x == 0, np.float32(1), x)
    np.testing.assert_array_equal(oc.unary(gpu, "reciprocal", nz), oc.unary(cpu, "reciprocal", nz))
    np.testing.assert_array_equal(oc.unary(gpu, "sqrt", np.abs(x)), oc.unary(cpu, "sqrt", np.abs(x)))
    np.testing.assert_array_equal(oc.pow_(gpu, x, 2.0), oc.pow_(cpu, x, 2.0))
    for name in ("erf", "gelu", "sigmoid", "tanh"):
        close(oc.unary(gpu, name, x), oc.unary(cpu, name, x))
    close(oc.pow_(gpu, np.abs(x) + 0.5, 1.5), oc.pow_(cpu, np.abs(x) + 0.5, 1.5))


def test_unary_misc(gpu, cpu):
    assert np.isnan(oc.unary(gpu, "relu", np.array([np.nan, 1.0], np.float32))[0])
    i = rng(2).integers(-2 ** 40, 2 ** 40, 777)
    np.testing.assert_array_equal(oc.cast(gpu, i), oc.cast(cpu, i))
    # 4-D shape through dnnrtActive, and an unaligned view (pointer + 4 bytes)
    x = rng(3).standard_normal((2, 3, 5, 7)).astype(np.float32)
    np.testing.assert_array_equal(oc.unary(gpu, "relu", x), oc.unary(cpu, "relu", x))
    t = gpu.put(rng(4).standard_normal(1030).astype(np.float32))
    y = gpu.empty(1030)
    gpu.ops.negative(gpu.ptr(t) + 4, gpu.ptr(y) + 4, [1029])
    gpu.sync()
    np.testing.assert_array_equal(gpu.get(y)[1:], -gpu.get(t)[1:])
    # fp16 storage
    h = (rng(5).standard_normal(5000) * 4).astype(np.float16)
    for name, kw in [("relu", {}), ("negative", {}), ("clip", {"lo": 0.0, "hi": 6.0})]:
        np.testing.assert_array_equal(oc.unary(gpu, name, h, **kw), oc.unary(cpu, name, h, **kw))
    close(oc.unary(gpu, "gelu", h).astype(np.float32), oc.unary(cpu, "gelu", h).astype(np.float32), 2e-2, 1e-3)


def test_tensor_op(gpu, cpu):
    r = rng(7)
    shapes = [((2, 5, 3, 4), (2, 5, 3, 4)), ((2, 5, 3, 4), (1, 5, 1, 1)), ((2, 5, 3, 4), (1, 1, 1, 4)),
              ((2, 5, 3, 4), (2, 1, 3, 1)), ((2, 5, 3, 4), (1, 1, 1, 1)), ((2, 5, 3, 4), (1, 5, 3, 1)),
              ((1, 256, 56, 56), (1, 256, 56, 56)), ((1, 256, 56, 56), (1, 256, 1, 1)),
              ((1, 1000), (1, 1000)), ((1, 128, 768), (1, 1, 768)), ((1, 128, 768), (1, 128, 1)),
              ((3, 7), (1, 7)), ((5,), (5,)), ((5,), (1,))]
    for sa, sb in shapes:
        a = r.standard_normal(sa).astype(np.float32)
        b = r.standard_normal(sb).astype(np.float32)
        for op in (_abi.OP_ADD, _abi.OP_MUL):
            np.testing.assert_array_equal(oc.tensor_op(gpu, op, a, b), oc.tensor_op(cpu, op, a, b))
            np.testing.assert_array_equal(oc.tensor_op(gpu, op, a, b, coef=-2.5), oc.tensor_op(cpu, op, a, b, coef=-2.5))
        np.testing.assert_array_equal(oc.tensor_op(gpu, _abi.OP_ADD, a, b, inplace=True),
                                      oc.tensor_op(cpu, _abi.OP_ADD, a, b, inplace=True))
    with pytest.raises(RuntimeError):
        oc.tensor_op(gpu, _abi.OP_ADD, np.zeros((2, 4), np.float32), np.zeros((2, 3), np.float32))
    a = r.standard_normal((2, 3, 4, 8)).astype(np.float16)
    b = r.standard_normal((1, 3, 1, 1)).astype(np.float16)
    np.testing.assert_array_equal(oc.tensor_op(gpu, _abi.OP_ADD, a, b), oc.tensor_op(cpu, _abi.OP_ADD, a, b))
    # 16-byte broadcast path (innermost run a multiple of 16 bytes) next to the element-wise one, both dtypes
    for dtype in (np.float32, np.float16):
        for sa, sb in [((2, 6, 4, 8), (1, 6, 1, 1)), ((2, 6, 4, 8), (2, 1, 4, 8)), ((2, 6, 4, 8), (2, 6, 1, 1)),
                       ((2, 6, 4, 8), (1, 1, 1, 8)), ((2, 6, 4, 8), (1, 6, 1, 8)), ((2, 6, 4, 8), (1, 1, 4, 1)),
                       ((3, 5, 16), (3, 1, 16)), ((3, 5, 16), (1, 5, 1)), ((4, 24), (1, 1)), ((4, 24), (4, 1)),
                       ((2, 6, 3, 6), (1, 6, 1, 1)), ((1, 64, 96, 96), (1, 1, 1, 1)), ((2, 64, 28, 28), (1, 64, 1, 1))]:
            a = r.standard_normal(sa).astype(dtype)
            b = r.standard_normal(sb).astype(dtype)
            want = (a.astype(np.float32) + b.astype(np.float32)).astype(dtype)
            np.testing.assert_array_equal(oc.tensor_op(gpu, _abi.OP_ADD, a, b), want)
            np.testing.assert_array_equal(oc.tensor_op(gpu, _abi.OP_MUL, a, b), oc.tensor_op(cpu, _abi.OP_MUL, a, b))


# ---- reductions --------------------------------------------------------------------

def test_reduce_mean(gpu, cpu):
    r = rng(9)
    for shape, out in [((1, 2048, 7, 7), (1, 2048, 1, 1)), ((2, 6, 7, 7), (2, 1, 7, 7)), ((2, 6, 7, 7), (1, 6, 7, 7)),
                       ((1, 128, 768), (1, 128, 1)), ((3, 1000), (3, 1)), ((1, 1280, 7, 7), (1, 1280, 1, 1))]:
        x = r.standard_normal(shape).astype(np.float32)
        close(oc.reduce_mean(gpu, x, out), oc.reduce_mean(cpu, x, out))
    # a middle dim reduced over an inner run of whole 8-byte units (what a channels-last global average
    # pool is): 7 + 3, 49 and 5 reduction steps, both element types, against numpy's float64 mean
    for shape, out in [((3, 10, 16), (3, 1, 16)), ((4, 49, 256), (4, 1, 256)), ((2, 5, 3, 8), (2, 1, 3, 8)), ((1, 7, 6), (1, 1, 6))]:
        for dtype, tol in ((np.float32, 1e-5), (np.float16, 2e-3)):
            x = r.standard_normal(shape).astype(dtype)
            got = oc.reduce_mean(gpu, x, out)
            close(got, oc.reduce_mean(cpu, x, out), tol, tol)
            np.testing.assert_allclose(got.astype(np.float64), x.astype(np.float64).mean(1, keepdims=True), rtol=tol, atol=tol)
    with pytest.raises(RuntimeError):
        oc.reduce_mean(gpu, np.zeros((2, 3, 4, 5), np.float32), (1, 3, 1, 5))


def test_softmax(gpu, cpu):
    r = rng(10)
    x = (r.standard_normal((1, 12, 128, 128)) * 3).astype(np.float32)
    got = oc.softmax(gpu, x, 3)
    close(got, oc.softmax(cpu, x, 3), 1e-4, 1e-7)
    close(got.sum(3), 1.0, 1e-5)
    x = (r.standard_normal((2, 3, 5, 17)) * 4).astype(np.float32)
    for axis in (3, -1, 1, 0, 2):
        close(oc.softmax(gpu, x, axis), oc.softmax(cpu, x, axis), 1e-4, 1e-7)
    big = np.array([[1000.0, 1000.0, -1000.0]], np.float32)
    close(oc.softmax(gpu, big, 1), [[0.5, 0.5, 0.0]], 1e-6, 1e-7)


def test_layernorm(gpu, cpu):
    r = rng(12)
    # rows held in registers (L % 4 == 0, up to 2048: one to eight groups of four per lane, few and
    # many rows) and the general kernel (odd L, long rows)
    for shape in [(1, 128, 768), (2, 7, 48), (5, 1000), (3, 1), (3, 4), (2, 300), (1, 2048), (1300, 256), (2, 1540), (2, 4096), (4, 1026)]:
        L = shape[-1]
        x = (r.standard_normal(shape) * 3 + 1).astype(np.float32)
        g = r.standard_normal(L).astype(np.float32)
        b = r.standard_normal(L).astype(np.float32)
        close(oc.layernorm(gpu, x, g, b, 1e-12 if L > 1 else 1e-5), oc.layernorm(cpu, x, g, b, 1e-12 if L > 1 else 1e-5), 1e-4, 1e-4)
    for shape in [(16, 768), (3, 64), (2, 2052)]:
        L = shape[-1]
        x = (r.standard_normal(shape) * 3 + 1).astype(np.float16)
        g, b = r.standard_normal(L).astype(np.float16), r.standard_normal(L).astype(np.float16)
        np.testing.assert_allclose(oc.layernorm(gpu, x, g, b, 1e-5).astype(np.float32), oc.layernorm(cpu, x, g, b, 1e-5).astype(np.float32),
                                   rtol=2e-2, atol=2e-2)


# ---- pooling ---------------------------------------------------------------------------

def test_pooling(gpu, cpu):
    r = rng(13)
    x = r.standard_normal((1, 64, 112, 112)).astype(np.float32)
    np.testing.assert_array_equal(oc.pool(gpu, "max", x, (3, 3), (1, 1), (2, 2)), oc.pool(cpu, "max", x, (3, 3), (1, 1), (2, 2)))
    x = r.standard_normal((2, 3, 13, 12)).astype(np.float32)
    for k, p, s in [(3, 1, 2), (2, 0, 2), (3, 0, 1), (3, 1, 1)]:
        np.testing.assert_array_equal(oc.pool(gpu, "max", x, (k, k), (p, p), (s, s)), oc.pool(cpu, "max", x, (k, k), (p, p), (s, s)))
        close(oc.pool(gpu, "avg", x, (k, k), (p, p), (s, s)), oc.pool(cpu, "avg", x, (k, k), (p, p), (s, s)))
    xn = x.copy()
    xn[0, 0, 0, 0] = np.nan
    np.testing.assert_array_equal(np.isnan(oc.pool(gpu, "max", xn, (3, 3), (1, 1), (2, 2))),
                                  np.isnan(oc.pool(cpu, "max", xn, (3, 3), (1, 1), (2, 2))))


# ---- matrix products --------------------------------------------------------------------

def test_matmul2d(gpu, cpu):
    r = rng(14)
    # the few-row shapes take the dot-product kernel with 1, 4 or 16 wavefronts per output
    for M, K, N in [(1, 2048, 1000), (1, 1280, 1000), (5, 9, 7), (64, 64, 64), (130, 70, 33), (3, 2048, 10), (16, 250, 40),
                    (2, 50176, 496), (8, 8194, 33), (1, 9216, 4096), (7, 2049, 5)]:
        a = r.standard_normal((M, K)).astype(np.float32)
        b = (r.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
        c = r.standard_normal((M, N)).astype(np.float32)
        ref = oc.matmul2d(cpu, a, b)
        close(oc.matmul2d(gpu, a, b), ref)
        close(oc.matmul2d(gpu, a.T.copy(), b, transA=1), ref)
        close(oc.matmul2d(gpu, a, b.T.copy(), transB=1), ref)
        close(oc.matmul2d(gpu, a.T.copy(), b.T.copy(), transA=1, transB=1), ref)
        close(oc.matmul2d(gpu, a, b.T.copy(), c.copy(), alpha=0.5, beta=-2.0, transB=1),
              oc.matmul2d(cpu, a, b.T.copy(), c.copy(), alpha=0.5, beta=-2.0, transB=1))
        # C as one row (a Gemm's bias folded into the product): equal to product-then-add on the GPU, bit for bit
        row = c[0].copy()
        for tb, bb in ((0, b), (1, b.T.copy())):
            fused = oc.matmul2d_row(gpu, a, bb, row, transB=tb)
            close(fused, oc.matmul2d_row(cpu, a, bb, row, transB=tb))
            np.testing.assert_array_equal(fused, oc.tensor_op(gpu, _abi.OP_ADD, oc.matmul2d(gpu, a, bb, transB=tb), row.reshape(1, -1)))
    with pytest.raises(RuntimeError):
        oc.matmul2d(gpu, np.zeros((5, 9), np.float32), np.zeros((9, 7), np.float32), transB=1)


def test_matmul_nd(gpu, cpu):
    r = rng(15)
    cases = [((1, 128, 768), (768, 768)), ((1, 12, 128, 64), (1, 12, 64, 128)), ((1, 12, 128, 128), (1, 12, 128, 64)),
             ((1, 128, 768), (768, 3072)), ((1, 128, 3072), (3072, 768)),
             ((4, 6), (6, 3)), ((2, 4, 6), (6, 3)), ((2, 3, 4, 6), (2, 3, 6, 5)), ((2, 4, 6), (2, 6, 3)), ((4, 6), (3, 6, 2)),
             # the LDS-staged row-major kernel: ragged rows and columns, 1 to 11 reduction splits (odd counts too)
             # (it takes products of 1.5e8 multiply-adds and more)
             ((1, 100, 1056), (1056, 1540)), ((1, 33, 3072), (3072, 1604)), ((200, 2048), (2048, 388)), ((300, 1024), (1024, 512)),
             ((2, 77, 1024), (1024, 1028)), ((1024, 256), (256, 1024)), ((1, 128, 768), (768, 2304))]
    for sa, sb in cases:
        a = r.standard_normal(sa).astype(np.float32)
        b = (r.standard_normal(sb) / np.sqrt(sb[-2])).astype(np.float32)
        ref = oc.matmul_nd(cpu, a, b)
        close(oc.matmul_nd(gpu, a, b), ref)
        close(oc.matmul_nd(gpu, a, b), ref)   # again: the split-reduction counters must be back at zero
    # fp16 tensors (fp32 accumulation, one rounding): the transformer shapes, broadcast batches, ragged tiles
    for sa, sb in [((1, 128, 768), (768, 768)), ((1, 12, 128, 64), (1, 12, 64, 128)), ((1, 12, 128, 128), (1, 12, 128, 64)),
                   ((4, 6), (6, 3)), ((2, 4, 6), (6, 3)), ((2, 3, 4, 6), (2, 3, 6, 5)), ((2, 4, 6), (2, 6, 3)), ((4, 6), (3, 6, 2)),
                   ((2, 77, 130), (130, 70)),
                   # few tiles and long reductions: split over 2 to 16 workgroups (odd step counts too), twice each
                   # (the arrival counters must be back at zero)
                   ((1, 128, 768), (768, 3072)), ((1, 128, 3072), (3072, 768)), ((1, 33, 1100), (1100, 100)), ((3, 64, 4000), (4000, 64))]:
        a = r.standard_normal(sa).astype(np.float16)
        b = (r.standard_normal(sb) / np.sqrt(sb[-2])).astype(np.float16)
        ref = oc.matmul_nd(cpu, a, b).astype(np.float32)
        first = oc.matmul_nd(gpu, a, b)
        np.testing.assert_allclose(first.astype(np.float32), ref, rtol=2e-3, atol=2e-3)
        np.testing.assert_array_equal(oc.matmul_nd(gpu, a, b), first)


def test_split_reduction_hand_over_is_deterministic(gpu, cpu):
    """Reductions split over workgroups meet through partial tiles and arrival counters in the handle's scratch;
    partial tiles are added in split order, so the result does not depend on who arrives last.  The deepest
    split of ResNet-50 at batch 1 (3x3 over 512 channels at 7x7), a 1x1 layer over 2048 channels and the
    768 -> 3072 product, 200 times each on one handle: every repetition bit-identical to the first, which
    matches the oracle."""
    r = rng(91)
    def repeat(call, ref):
        first = call()
        close(gpu.get(first), ref)
        first = first.clone()
        for i in range(200):
            again = call()
            assert gpu.torch.equal(again, first), f"repetition {i} differs"
    for case in [(1, 512, 7, 7, 512, 3, 1, 1), (1, 2048, 7, 7, 512, 1, 1, 0), (1, 1024, 14, 14, 256, 1, 1, 0)]:
        N, C, H, W, K, R, st, pd = case
        x = r.standard_normal((N, C, H, W)).astype(np.float32)
        w = (r.standard_normal((K, C, R, R)) * np.sqrt(2.0 / (C * R * R))).astype(np.float32)
        b = r.uniform(-0.1, 0.1, K).astype(np.float32)
        ref = oc.conv(cpu, x, w, b, (pd, pd), (st, st), 1, _abi.ACT_RELU)
        P, Q = oc.conv_out_hw(H, W, R, R, (pd, pd), (st, st))
        X, Wt, B, Y = gpu.put(x), gpu.put(w), gpu.put(b), gpu.empty((N, K, P, Q))
        def conv_call():
            gpu.ops.conv_bias_activ(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), (pd, pd), (st, st), _abi.ACT_RELU,
                                    gpu.ptr(Y), 1, _abi.F32)
            gpu.sync()
            return Y
        repeat(conv_call, ref)
    a = r.standard_normal((1, 128, 768)).astype(np.float32)
    b = (r.standard_normal((768, 3072)) / np.sqrt(768)).astype(np.float32)
    ref = oc.matmul_nd(cpu, a, b)
    A, Bm, Y = gpu.put(a), gpu.put(b), gpu.empty((1, 128, 3072))
    def mm_call():
        gpu.ops.matmul_nd(gpu.ptr(A), a.shape, gpu.ptr(Bm), b.shape, gpu.ptr(Y), (1, 128, 3072), _abi.F32)
        gpu.sync()
        return Y
    repeat(mm_call, ref)
    # the fp16 product splits its reduction the same way (3072 -> 768: eleven workgroups per tile, 768 -> 3072: none)
    for K, N in ((3072, 768), (768, 768)):
        a16 = r.standard_normal((1, 128, K)).astype(np.float16)
        b16 = (r.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
        ref16 = oc.matmul_nd(cpu, a16, b16).astype(np.float32)
        A16, B16, Y16 = gpu.put(a16), gpu.put(b16), gpu.empty((1, 128, N), np.float16)
        def mm16_call():
            gpu.ops.matmul_nd(gpu.ptr(A16), a16.shape, gpu.ptr(B16), b16.shape, gpu.ptr(Y16), (1, 128, N), _abi.F16)
            gpu.sync()
            return Y16
        first = mm16_call()
        np.testing.assert_allclose(gpu.get(first).astype(np.float32), ref16, rtol=4e-3, atol=8e-3)
        first = first.clone()
        for i in range(200):
            assert gpu.torch.equal(mm16_call(), first), f"fp16 product {K} -> {N}: repetition {i} differs"


def test_matmul_nd_bias(gpu, cpu):
    r = rng(44)
    # transformer Linear layers (one tall product, the dot-product kernel for few rows) and batched products
    for sa, sb in [((1, 128, 768), (768, 768)), ((1, 128, 768), (768, 3072)), ((1, 128, 3072), (3072, 768)), ((5, 7), (7, 3)),
                   ((3, 6, 5), (3, 5, 4)), ((2, 12, 40, 64), (2, 12, 64, 40)), ((1, 3, 33), (33, 130))]:
        a = r.standard_normal(sa).astype(np.float32)
        b = (r.standard_normal(sb) / np.sqrt(sb[-2])).astype(np.float32)
        bias = r.standard_normal(sb[-1]).astype(np.float32)
        close(oc.matmul_nd_bias(gpu, a, b, bias), oc.matmul_nd_bias(cpu, a, b, bias))
        z = r.standard_normal(np.broadcast_shapes(sa[:-2], sb[:-2]) + (sa[-2], sb[-1])).astype(np.float32)
        close(oc.matmul_nd_bias(gpu, a, b, bias, z=z), oc.matmul_nd_bias(cpu, a, b, bias, z=z))
        close(oc.matmul_nd_bias(gpu, a, b, bias, gelu=True), oc.matmul_nd_bias(cpu, a, b, bias, gelu=True))
    # fp16 tensors: the generic fp16 product (fp32 accumulation, bias, residual and GELU before the one rounding;
    # the oracle rounds to fp16 after the product and after each of the three)
    for sa, sb in [((1, 128, 768), (768, 768)), ((5, 7), (7, 3)), ((3, 6, 5), (3, 5, 4)), ((2, 12, 40, 64), (2, 12, 64, 40)), ((1, 3, 33), (33, 130))]:
        a = r.standard_normal(sa).astype(np.float16)
        b = (r.standard_normal(sb) / np.sqrt(sb[-2])).astype(np.float16)
        bias = r.standard_normal(sb[-1]).astype(np.float16)
        z = r.standard_normal(np.broadcast_shapes(sa[:-2], sb[:-2]) + (sa[-2], sb[-1])).astype(np.float16)
        for kw in (dict(), dict(z=z), dict(gelu=True), dict(z=z, gelu=True)):
            np.testing.assert_allclose(oc.matmul_nd_bias(gpu, a, b, bias, **kw).astype(np.float32),
                                       oc.matmul_nd_bias(cpu, a, b, bias, **kw).astype(np.float32), rtol=1e-2, atol=1e-2)


def test_attention(gpu, cpu):
    r = rng(45)
    # BERT-base's shape; key counts around the 32-key wavefront slice and the 128-key block; every head size
    for B, Sq, Sk, H, D in [(1, 128, 128, 12, 64), (2, 50, 77, 3, 32), (1, 300, 300, 2, 128), (1, 1, 5, 1, 64), (1, 33, 129, 4, 64),
                            (3, 64, 31, 2, 64), (1, 40, 512, 2, 64)]:
        q, k, v = (r.standard_normal((B, S, H * D)).astype(np.float32) for S in (Sq, Sk, Sk))
        q *= 2.0                                              # sharper soft-max: the running maximum moves between blocks
        close(oc.attention(gpu, q, k, v, H, 1.0 / np.sqrt(D)), oc.attention(cpu, q, k, v, H, 1.0 / np.sqrt(D)), 1e-4, 1e-5)
    qkv = r.standard_normal((2, 130, 3 * 256)).astype(np.float32)          # Q | K | V per row
    close(oc.attention_packed(gpu, qkv, 4, 0.125), oc.attention_packed(cpu, qkv, 4, 0.125), 1e-4, 1e-5)
    with pytest.raises(RuntimeError):
        oc.attention(gpu, q[:, :, :96], k[:, :, :96], v[:, :, :96], 2, 1.0)   # head size 48
    # fp16 tensors: widened on the way in, fp32 in between, one rounding on the way out (the oracle does the same)
    for B, Sq, Sk, H, D in [(1, 128, 128, 12, 64), (2, 50, 77, 3, 32), (1, 33, 129, 4, 64), (1, 40, 300, 2, 128)]:
        q, k, v = (r.standard_normal((B, S, H * D)).astype(np.float16) for S in (Sq, Sk, Sk))
        np.testing.assert_allclose(oc.attention(gpu, q, k, v, H, 1.0 / np.sqrt(D)).astype(np.float32),
                                   oc.attention(cpu, q, k, v, H, 1.0 / np.sqrt(D)).astype(np.float32), rtol=2e-3, atol=2e-3)
    qkv = r.standard_normal((2, 130, 3 * 256)).astype(np.float16)
    np.testing.assert_allclose(oc.attention_packed(gpu, qkv, 4, 0.125).astype(np.float32),
                               oc.attention_packed(cpu, qkv, 4, 0.125).astype(np.float32), rtol=2e-3, atol=2e-3)


# ---- data movement -------------------------------------------------------------------------

def test_data_movement(gpu, cpu):
    r = rng(16)
    x = r.standard_normal((2, 3, 4, 5)).astype(np.float32)
    np.testing.assert_array_equal(oc.flatten(gpu, x, 1), x.reshape(2, 60))
    np.testing.assert_array_equal(oc.reshape(gpu, x, (6, 20)), x.reshape(6, 20))
    for perm in [(0, 2, 1, 3), (0, 2, 3, 1), (3, 2, 1, 0), (1, 0, 2, 3)]:
        np.testing.assert_array_equal(oc.transpose(gpu, x, perm), x.transpose(perm))
    h = r.standard_normal((1, 128, 12, 64)).astype(np.float32)
    np.testing.assert_array_equal(oc.transpose(gpu, h, (0, 2, 1, 3)), h.transpose(0, 2, 1, 3))
    np.testing.assert_array_equal(oc.transpose(gpu, h, (0, 2, 3, 1)), h.transpose(0, 2, 3, 1))
    np.testing.assert_array_equal(oc.transpose(gpu, x[0], (1, 0, 2)), x[0].transpose(1, 0, 2))
    xi = r.integers(-5, 5, (3, 4)).astype(np.int64)
    np.testing.assert_array_equal(oc.transpose(gpu, xi, (1, 0)), xi.T)
    x6 = r.standard_normal((2, 3, 2, 2, 3, 2)).astype(np.float32)
    np.testing.assert_array_equal(oc.transpose(gpu, x6, (0, 1, 4, 2, 5, 3)), x6.transpose(0, 1, 4, 2, 5, 3))
    table = r.standard_normal((30522, 768)).astype(np.float32)
    idx = r.integers(0, 30522, (1, 128))
    np.testing.assert_array_equal(oc.gather(gpu, table, idx, 0), np.take(table, idx, 0))
    np.testing.assert_array_equal(oc.gather(gpu, x, np.array([2, -1]), 2), np.take(x, [2, -1], 2))
    ti = r.integers(-1000, 1000, (70, 3, 20)).astype(np.int64)
    np.testing.assert_array_equal(oc.gather(gpu, ti, np.array([[6, 0], [3, -2]]), 0), np.take(ti, [[6, 0], [3, -2]], 0))
    np.testing.assert_array_equal(oc.gather(gpu, ti, np.array([19, 1]), 2), oc.gather(cpu, ti, np.array([19, 1]), 2))
    # every permutation of a rank-4 tensor whose dims allow 1-, 2-, 4- and 8-element units, each dtype,
    # plus shapes with size-1 dims and runs of dims that stay together
    import itertools
    for dtype in (np.float32, np.float16, np.int64):
        t = r.integers(-999, 999, (4, 6, 8, 16)).astype(dtype)
        for perm in itertools.permutations(range(4)):
            np.testing.assert_array_equal(oc.transpose(gpu, t, perm), t.transpose(perm))
        for shape, perm in [((2, 1, 8, 4), (2, 1, 0, 3)), ((1, 64, 2, 2, 12, 12), (0, 1, 4, 2, 5, 3)), ((3, 5, 7), (2, 0, 1)),
                            ((2, 3, 4, 5, 6), (0, 3, 4, 1, 2)), ((1, 1, 1), (2, 1, 0)), ((6, 8), (0, 1))]:
            t = r.integers(-999, 999, shape).astype(dtype)
            np.testing.assert_array_equal(oc.transpose(gpu, t, perm), t.transpose(perm))
            np.testing.assert_array_equal(oc.transpose(gpu, t, perm), oc.transpose(cpu, t, perm))
    with pytest.raises(RuntimeError):
        oc.transpose(gpu, x, (0, 1, 1, 3))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_conv_clipped_and_leaky_relu(gpu, cpu, dtype):
    r = rng(43)
    tol = dict(rtol=1e-4, atol=1e-5) if dtype == np.float32 else dict(rtol=2e-2, atol=2e-3)
    # dense 3x3 and 1x1 (the MFMA kernels), a depthwise 3x3, and a product large enough for the LDS-tiled kernel
    for (N, C, H, K, R, st, pd, grp) in [(1, 64, 14, 64, 3, 1, 1, 1), (2, 32, 9, 48, 1, 1, 0, 1), (1, 32, 12, 32, 3, 2, 1, 32),
                                          (4, 64, 28, 128, 3, 1, 1, 1)]:
        if dtype == np.float16 and grp != 1:
            continue
        x = r.standard_normal((N, C, H, H)).astype(dtype)
        w = (r.standard_normal((K, C // grp, R, R)) * (0.5 / np.sqrt(C // grp * R * R))).astype(dtype)
        b = r.standard_normal(K).astype(dtype)
        P = (H + 2 * pd - R) // st + 1
        z = r.standard_normal((N, K, P, P)).astype(dtype)
        for activ, coef in [(_abi.ACT_CLIPPED_RELU, 0.75), (_abi.ACT_LEAKY_RELU, 0.1)]:
            for zz in (None, z):
                got = oc.conv(gpu, x, w, b, (pd, pd), (st, st), grp, activ, z=zz, coef=coef)
                ref = oc.conv(cpu, x, w, b, (pd, pd), (st, st), grp, activ, z=zz, coef=coef)
                np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), **tol)
                if activ == _abi.ACT_CLIPPED_RELU:
                    assert got.max() <= 0.75 and got.min() >= 0
    x = r.standard_normal((3, 5, 7, 2)).astype(dtype)
    X, Y = gpu.put(x), gpu.empty(x.shape, x.dtype)
    gpu.ops.set_activation_coef(0.25)
    gpu.ops.active(gpu.ptr(X), x.shape, _abi.ACT_LEAKY_RELU, gpu.ptr(Y), oc.DT[np.dtype(dtype)])
    gpu.sync()
    np.testing.assert_array_equal(gpu.get(Y), oc.leaky_relu(cpu, x, 0.25))
    with pytest.raises(RuntimeError):
        oc.conv(gpu, x, np.zeros((4, 5, 1, 1), dtype), np.zeros(4, dtype), activ=4)


def test_leaky_relu_prelu(gpu, cpu):
    r = rng(41)
    for dtype in (np.float32, np.float16):
        for shape in [(2, 24, 13, 13), (1, 64, 56, 56), (5,), (3, 7)]:
            x = r.standard_normal(shape).astype(dtype)
            np.testing.assert_array_equal(oc.leaky_relu(gpu, x, 0.1), oc.leaky_relu(cpu, x, 0.1))
            np.testing.assert_array_equal(oc.prelu(gpu, x, np.array([0.25], dtype)), oc.prelu(cpu, x, np.array([0.25], dtype)))
        x = r.standard_normal((2, 24, 13, 13)).astype(dtype)
        for sshape in [(24, 1, 1), (1, 24, 1, 1), (13,), (2, 24, 13, 13), (1, 1, 13, 1)]:
            sl = r.uniform(-0.5, 0.5, sshape).astype(dtype)
            np.testing.assert_array_equal(oc.prelu(gpu, x, sl), oc.prelu(cpu, x, sl))
    with pytest.raises(RuntimeError):
        oc.prelu(gpu, x, np.ones((7, 1, 1), x.dtype))
    # channels-last: the tensor is a dense [N,H,W,C] array, the slope runs along C
    x = r.standard_normal((2, 24, 5, 7)).astype(np.float16)
    sl = r.uniform(-0.5, 0.5, (24, 1, 1)).astype(np.float16)
    gpu.ops.set_format(_abi.NHWC)
    try:
        X, S = gpu.put(np.ascontiguousarray(x.transpose(0, 2, 3, 1))), gpu.put(sl)
        Y = gpu.empty((2, 5, 7, 24), np.float16)
        gpu.ops.prelu(gpu.ptr(X), gpu.ptr(Y), x.shape, gpu.ptr(S), sl.shape, _abi.F16)
        gpu.sync()
    finally:
        gpu.ops.set_format(_abi.NCHW)
    np.testing.assert_array_equal(gpu.get(Y).transpose(0, 3, 1, 2), oc.prelu(cpu, x, sl))


def test_concat_squeeze_unsqueeze(gpu, cpu):
    r = rng(42)
    for dtype in (np.float32, np.float16, np.int64):
        mk = (lambda s: r.integers(-99, 99, s).astype(np.int64)) if dtype == np.int64 else (lambda s: r.standard_normal(s).astype(dtype))
        for axis in range(4):
            for sizes in [(1, 3, 7), (4, 4), (8, 16, 8)]:         # element-wise and 16-byte paths
                shapes = []
                for k in sizes:
                    sh = [2, 8, 4, 8]
                    sh[axis] = k
                    shapes.append(sh)
                xs = [mk(s) for s in shapes]
                got = oc.concat(gpu, xs, axis)
                np.testing.assert_array_equal(got, np.concatenate(xs, axis))
                np.testing.assert_array_equal(got, oc.concat(cpu, xs, axis))
    many = [r.standard_normal((3, k + 1, 5)).astype(np.float32) for k in range(16)]
    np.testing.assert_array_equal(oc.concat(gpu, many, 1), np.concatenate(many, 1))
    big = [r.standard_normal((2, c, 52, 52)).astype(np.float32) for c in (128, 256)]  # a detection neck's concat
    np.testing.assert_array_equal(oc.concat(gpu, big, 1), np.concatenate(big, 1))
    with pytest.raises(RuntimeError):
        oc.concat(gpu, many + [many[0]], 1)
    with pytest.raises(RuntimeError):
        oc.concat(gpu, [big[0], big[1][:, :, :50]], 1)
    # channels-last: concatenating channels interleaves per pixel
    xs = [r.standard_normal((2, c, 6, 5)).astype(np.float16) for c in (8, 24, 3)]
    gpu.ops.set_format(_abi.NHWC)
    try:
        Xs = [gpu.put(np.ascontiguousarray(x.transpose(0, 2, 3, 1))) for x in xs]
        Y = gpu.empty((2, 6, 5, 35), np.float16)
        gpu.ops.concat([gpu.ptr(X) for X in Xs], [x.shape for x in xs], gpu.ptr(Y), (2, 35, 6, 5), 1, _abi.F16)
        gpu.sync()
    finally:
        gpu.ops.set_format(_abi.NCHW)
    np.testing.assert_array_equal(gpu.get(Y).transpose(0, 3, 1, 2), np.concatenate(xs, 1))
    s = r.standard_normal((2, 1, 4, 1)).astype(np.float32)
    np.testing.assert_array_equal(oc.squeeze(gpu, s, (2, 4)), s.reshape(2, 4))
    np.testing.assert_array_equal(oc.squeeze(gpu, s.reshape(2, 4), (1, 2, 1, 4), un=True), s.reshape(1, 2, 1, 4))
    with pytest.raises(RuntimeError):
        oc.squeeze(gpu, s, (4, 2))


def test_expand_and_nonzero(gpu, cpu):
    r = rng(43)
    for shape, out in [((3, 1, 5), (3, 1, 5)), ((3, 1, 5), (2, 3, 4, 5)), ((1,), (1000,)), ((64, 1), (64, 300)),
                       ((1, 1, 1), (2, 3, 4)), ((2, 1, 3, 1, 2), (2, 4, 3, 5, 2)), ((1, 1, 128, 128), (2, 12, 128, 128))]:
        for dtype in (np.int64, np.float32, np.float16):
            x = r.integers(-99, 99, shape).astype(dtype)
            got = oc.expand(gpu, x, out)
            np.testing.assert_array_equal(got, np.broadcast_to(x, out))
            np.testing.assert_array_equal(got, oc.expand(cpu, x, out))
    with pytest.raises(RuntimeError):
        oc.expand(gpu, np.zeros((3, 1, 5), np.int64), (3, 4, 6))
    # sizes around the 1024-element chunk and the 64-lane wavefront, sparse and dense
    for n, density in [(1, 1.0), (63, 0.5), (64, 1.0), (65, 0.3), (1023, 0.9), (1024, 1.0), (1025, 0.01), (5000, 0.5),
                       (100_003, 0.1), (4096, 0.0)]:
        for dtype in (np.float32, np.int64, np.float16):
            x = (r.integers(1, 5, (n,)) * (r.random((n,)) < density)).astype(dtype)
            got = oc.nonzero(gpu, x, (n,), -3)
            want = np.flatnonzero(x)
            np.testing.assert_array_equal(got, oc.nonzero(cpu, x, (n,), -3))
            if dtype != np.float16:  # fp16 cannot hold indices above 2048 exactly: the oracle comparison covers it
                np.testing.assert_array_equal(got[: want.size], want.astype(dtype))
            np.testing.assert_array_equal(got[want.size:], np.full(n - want.size, -3, dtype))
    x = (r.random((7, 9, 11)) < 0.5).astype(np.float32)
    cut = oc.nonzero(gpu, x, (2, 10), -1.0)          # output rank differs from the input's; capacity 20
    np.testing.assert_array_equal(cut.reshape(-1), np.flatnonzero(x.reshape(-1))[:20].astype(np.float32))
    z = np.array([0.0, -0.0, np.nan, 1e-45, 0.0], np.float32)
    np.testing.assert_array_equal(oc.nonzero(gpu, z, (5,), -1.0), np.array([2, 3, -1, -1, -1], np.float32))


def test_empty_tensors_are_no_ops(gpu, cpu):
    # an empty batch (or an empty tensor of any kind) launches nothing, writes nothing, raises nothing,
    # and leaves no error behind; the oracle agrees entry point by entry point
    got = oc.empty_tensor_behaviour(gpu)
    assert got == oc.empty_tensor_behaviour(cpu)
    assert set(got.values()) == {"untouched"}, got


# ---- fp16, channels-last -----------------------------------------------------------------

def conv_f16(gpu, x, w, b, pads, strides, group, activ, fmt, z=None, inplace=False):
    """x, w (and the residual z) in logical NCHW / KCRS order; returns logical NCHW.  inplace: the result buffer
    holds z and is passed as both Z and Y."""
    N, C, H, W = x.shape
    K, Cg, R, S = w.shape
    P, Q = oc.conv_out_hw(H, W, R, S, pads, strides)
    xin = x if fmt != _abi.NHWC else np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    win = w if fmt == _abi.NCHW else np.ascontiguousarray(w.transpose(0, 2, 3, 1))  # K,R,S,C
    X, Wt, B = gpu.put(xin), gpu.put(win), gpu.put(b)
    Y = gpu.empty((N * K * P * Q,), np.float16)
    gpu.ops.set_format(fmt)
    try:
        if z is None:
            gpu.ops.conv_bias_activ(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), pads, strides, activ,
                                    gpu.ptr(Y), group, _abi.F16)
        else:  # laid out like Y
            Z = gpu.put(z if fmt == _abi.NCHW else np.ascontiguousarray(z.transpose(0, 2, 3, 1)))
            if inplace:
                Y = Z
            gpu.ops.conv_bias_add_activ(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), gpu.ptr(Z), pads, strides,
                                        activ, gpu.ptr(Y), group, _abi.F16)
        gpu.sync()
    finally:
        gpu.ops.set_format(_abi.NCHW)
    y = gpu.get(Y)
    return y.reshape(N, K, P, Q) if fmt == _abi.NCHW else y.reshape(N, P, Q, K).transpose(0, 3, 1, 2)


F16_CASES = [
    # N, C, H, W, K, R, stride, pad
    (2, 64, 56, 56, 64, 3, 1, 1),      # fast path, K_out = 64 tile
    (2, 64, 56, 56, 256, 1, 1, 0),
    (2, 256, 28, 28, 128, 3, 2, 1),    # strided 3x3
    (3, 512, 7, 7, 512, 3, 1, 1),      # ragged pixel tile (147 pixels)
    (2, 256, 14, 14, 1000, 1, 1, 0),   # K_out not a multiple of the tile
    (1, 1024, 14, 14, 2048, 1, 2, 0),
    (2, 32, 9, 11, 40, 3, 1, 1),       # smallest C the fast path takes
    (2, 64, 9, 11, 40, 3, 1, 1),       # 64 x 128 tile, ragged in both directions
    (2, 64, 9, 11, 40, 1, 1, 0),       # one-step reduction (single LDS stage), ragged in both directions
    (1, 64, 12, 12, 72, 1, 2, 0),      # the same with stride 2 and two k_out tiles
    (2, 128, 9, 11, 40, 1, 1, 0),      # two, three and four steps taking turns in the one LDS stage
    (1, 192, 10, 7, 72, 1, 1, 0),
    (2, 256, 7, 7, 136, 1, 1, 0),
    (64, 2048, 1, 1, 1000, 1, 1, 0),   # few pixels (a fully connected layer): 16 filters x 32 pixels per workgroup
    (1, 512, 1, 1, 1000, 1, 1, 0),     # the same with one pixel
    (3, 320, 3, 5, 72, 1, 1, 0),       # 45 pixels, five chunks over four wavefronts, half a block of filters
    (1, 1088, 7, 7, 24, 1, 1, 0),      # 49 pixels, 17 chunks
    (2, 3, 32, 32, 64, 7, 2, 3),       # 3 channels: first-layer kernel (NCHW in, NHWC out), generic otherwise
    (2, 3, 45, 37, 64, 7, 2, 3),       # first-layer kernel, ragged tiles (23 x 19 output pixels)
    (1, 3, 224, 224, 64, 7, 2, 3),     # the ResNet first layer at full size
    (1, 20, 9, 9, 24, 3, 1, 1),        # generic path: C % 32 != 0
    # channels-last 1x1 layers over a multiple of 8 channels that is not one of 64: one wavefront per 32 pixels
    (2, 16, 20, 20, 96, 1, 1, 0),      # one 16-channel step
    (3, 24, 9, 11, 144, 1, 1, 0),      # half of the second step is past the channels; 297 pixels: a ragged last wavefront
    (2, 144, 7, 9, 24, 1, 1, 0),       # nine steps, fewer filters than a block
    (1, 160, 7, 7, 960, 1, 1, 0),      # 49 pixels: the filter blocks are dealt over the grid
    (5, 8, 3, 3, 8, 1, 1, 0),          # the smallest
    (1, 248, 6, 5, 40, 1, 1, 0),       # sixteen steps, the last one half empty
    (1, 200, 9, 9, 72, 1, 1, 0),
    (8, 24, 56, 56, 144, 1, 1, 0),     # a MobileNetV2 expansion layer
    # first layers other than the 7x7 one (N,C,H,W in, channels-last out): a thread per output pixel
    (2, 3, 33, 30, 32, 3, 2, 1),       # MobileNetV2's, on a ragged image
    (1, 3, 224, 224, 32, 3, 2, 1),     # ... at full size
    (2, 3, 20, 17, 64, 3, 1, 1),       # a VGG's
    (3, 1, 12, 12, 16, 3, 1, 0),       # one channel, no padding
    (2, 4, 9, 9, 24, 1, 1, 0),         # four channels, 1x1
    (1, 2, 10, 11, 48, 2, 2, 1),       # 2x2 filter
]


@pytest.mark.parametrize("case", F16_CASES, ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("fmt", [_abi.NHWC, _abi.NCHW_TO_NHWC, _abi.NCHW])
def test_conv_f16(gpu, cpu, case, fmt):
    N, C, H, W, K, R, st, pd = case
    r = rng(sum(case) + fmt)
    x = r.standard_normal((N, C, H, W)).astype(np.float16)
    w = (r.standard_normal((K, C, R, R)) * np.sqrt(2.0 / (C * R * R))).astype(np.float16)
    b = r.uniform(-0.1, 0.1, K).astype(np.float16)
    ref = oc.conv(cpu, x, w, b, (pd, pd), (st, st), 1, _abi.ACT_RELU)          # fp16 storage, exact accumulate
    got = conv_f16(gpu, x, w, b, (pd, pd), (st, st), 1, _abi.ACT_RELU, fmt)
    # fp32 accumulation then one rounding to fp16: within 1 fp16 ulp of the oracle
    np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=2e-3, atol=2e-3)
    if fmt == _abi.NHWC:
        ident = conv_f16(gpu, x, w, b, (pd, pd), (st, st), 1, _abi.ACT_IDENTITY, fmt)
        refi = oc.conv(cpu, x, w, b, (pd, pd), (st, st), 1, _abi.ACT_IDENTITY)
        np.testing.assert_allclose(ident.astype(np.float32), refi.astype(np.float32), rtol=2e-3, atol=2e-3)
    z = r.standard_normal(ref.shape).astype(np.float16)
    refz = oc.conv(cpu, x, w, b, (pd, pd), (st, st), 1, _abi.ACT_RELU, z=z)
    gotz = conv_f16(gpu, x, w, b, (pd, pd), (st, st), 1, _abi.ACT_RELU, fmt, z=z)
    np.testing.assert_allclose(gotz.astype(np.float32), refz.astype(np.float32), rtol=4e-3, atol=4e-3)
    if fmt != _abi.NCHW_TO_NHWC:  # written over the residual operand: the same bits
        np.testing.assert_array_equal(conv_f16(gpu, x, w, b, (pd, pd), (st, st), 1, _abi.ACT_RELU, fmt, z=z, inplace=True), gotz)


@pytest.mark.parametrize("case", [(2, 32, 14, 14, 32, 3, 1, 1, 32), (1, 96, 28, 28, 96, 3, 2, 1, 96), (2, 6, 7, 7, 12, 3, 1, 1, 6),
                                  (1, 16, 10, 10, 32, 3, 1, 1, 4), (2, 128, 9, 9, 128, 1, 1, 0, 2), (3, 144, 13, 9, 144, 3, 2, 1, 144),
                                  (1, 960, 7, 7, 960, 3, 1, 1, 960), (2, 24, 9, 9, 24, 5, 1, 2, 24), (1, 12, 6, 6, 12, 3, 1, 1, 12)],
                         ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("fmt", [_abi.NHWC, _abi.NCHW])
def test_conv_f16_grouped_and_depthwise(gpu, cpu, case, fmt):
    """fp16 convolutions with groups (depthwise: the channels-last kernel of its own for channel counts that are
    multiples of eight, MobileNetV2's shapes among them, the generic kernel otherwise; depthwise with a channel
    multiplier; a few wide groups), with bias, ReLU and a residual operand, channels-last and N,C,H,W, against the
    oracle to the fp16 convolution tolerance."""
    N, C, H, W, K, R, st, pd, grp = case
    r = rng(sum(case) + fmt)
    x = r.standard_normal((N, C, H, W)).astype(np.float16)
    w = (r.standard_normal((K, C // grp, R, R)) * np.sqrt(2.0 / (C // grp * R * R))).astype(np.float16)
    b = r.uniform(-0.1, 0.1, K).astype(np.float16)
    ref = oc.conv(cpu, x, w, b, (pd, pd), (st, st), grp, _abi.ACT_RELU)
    got = conv_f16(gpu, x, w, b, (pd, pd), (st, st), grp, _abi.ACT_RELU, fmt)
    np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=2e-3, atol=2e-3)
    z = r.standard_normal(ref.shape).astype(np.float16)
    refz = oc.conv(cpu, x, w, b, (pd, pd), (st, st), grp, _abi.ACT_RELU, z=z)
    gotz = conv_f16(gpu, x, w, b, (pd, pd), (st, st), grp, _abi.ACT_RELU, fmt, z=z)
    np.testing.assert_allclose(gotz.astype(np.float32), refz.astype(np.float32), rtol=4e-3, atol=4e-3)
    np.testing.assert_array_equal(conv_f16(gpu, x, w, b, (pd, pd), (st, st), grp, _abi.ACT_RELU, fmt, z=z, inplace=True), gotz)


def stem_pool_f16(gpu, x, w, b, activ, fmt=_abi.NCHW_TO_NHWC, kernel=(3, 3), ppads=(1, 1, 1, 1), pstrides=(2, 2)):
    """The fused first layer through the C-ABI; x in N,C,H,W, w logical K,C,R,S; returns logical N,K,PP,QQ."""
    N, C, H, W = x.shape
    K = w.shape[0]
    P, Q = oc.conv_out_hw(H, W, 7, 7, (3, 3), (2, 2))
    PP, QQ = oc.conv_out_hw(P, Q, 3, 3, (1, 1), (2, 2))
    X, Wt, B = gpu.put(x), gpu.put(np.ascontiguousarray(w.transpose(0, 2, 3, 1))), gpu.put(b)
    Y = gpu.empty((N * K * PP * QQ,), np.float16)
    gpu.ops.set_format(fmt)
    try:
        gpu.ops.conv_bias_activ_max_pool(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), (3, 3), (2, 2), activ, kernel,
                                         ppads, pstrides, gpu.ptr(Y), (N, K, PP, QQ))
        gpu.sync()
    finally:
        gpu.ops.set_format(_abi.NCHW)
    return gpu.get(Y).reshape(N, PP, QQ, K).transpose(0, 3, 1, 2)


@pytest.mark.parametrize("case", [(2, 32, 32), (2, 45, 38), (3, 64, 80), (1, 224, 224), (5, 23, 62), (70, 16, 16), (1, 7, 2)],
                         ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("activ", [_abi.ACT_RELU, _abi.ACT_IDENTITY])
def test_first_layer_with_its_max_pool_in_one_call(gpu, cpu, case, activ):
    """dnnrtConvBiasActivMaxPool against the two calls it replaces: the oracle's chain to the convolution's
    tolerance (one rounding to fp16 of an fp32 sum; the maximum adds none), and this library's own two calls
    bit for bit (same products in the same order, then an exact maximum).  Identity activation leaves negative
    values, so a padding of zeros instead of -inf would show; odd heights and widths that are not multiples of 28
    leave ragged strips and a last pooled row and column whose windows hang over the edge."""
    N, H, W = case
    r = rng(N + H + W + activ)
    x = r.standard_normal((N, 3, H, W)).astype(np.float16)
    w = (r.standard_normal((64, 3, 7, 7)) * np.sqrt(2.0 / 147)).astype(np.float16)
    b = r.uniform(-0.5, 0.1, 64).astype(np.float16)
    if case == (5, 23, 62):
        x[1, 2, 11, 30] = np.nan  # reaches a 4 x 4 block of convolution outputs of image 1, every channel
        x[3, 0, 5, 40] = np.inf   # infinities of both signs in one window's reach: inf - inf is a NaN as well,
        x[3, 1, 6, 41] = -np.inf  # and around it results of +inf and -inf
    got = stem_pool_f16(gpu, x, w, b, activ)
    conv_ref = oc.conv(cpu, x, w, b, (3, 3), (2, 2), 1, activ)
    ref = oc.pool(cpu, "max", conv_ref, (3, 3), (1, 1), (2, 2))
    assert got.shape == ref.shape
    np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=2e-3, atol=2e-3)
    if case == (5, 23, 62):
        assert np.isnan(got[1]).any() and np.isnan(got[3]).any() and not np.isnan(got[[0, 2, 4]]).any()
        assert (np.isnan(got) == np.isnan(ref)).all()
    # the two calls on the GPU, channels-last in between
    conv_gpu = conv_f16(gpu, x, w, b, (3, 3), (2, 2), 1, activ, _abi.NCHW_TO_NHWC)       # logical NCHW
    mid = gpu.put(np.ascontiguousarray(conv_gpu.transpose(0, 2, 3, 1)))
    P, Q = conv_gpu.shape[2:]
    PP, QQ = ref.shape[2:]
    Y2 = gpu.empty((N * 64 * PP * QQ,), np.float16)
    gpu.ops.set_format(_abi.NHWC)
    try:
        gpu.ops.maxpool(gpu.ptr(mid), (N, 64, P, Q), gpu.ptr(Y2), (N, 64, PP, QQ), (3, 3), (1, 1, 1, 1), (2, 2), _abi.F16)
        gpu.sync()
    finally:
        gpu.ops.set_format(_abi.NCHW)
    two = gpu.get(Y2).reshape(N, PP, QQ, 64).transpose(0, 3, 1, 2)
    np.testing.assert_array_equal(got, two)


def test_first_layer_with_its_max_pool_refuses_other_shapes(gpu):
    r = rng(3)
    x = r.standard_normal((1, 3, 32, 32)).astype(np.float16)
    w = r.standard_normal((64, 3, 7, 7)).astype(np.float16)
    b = np.zeros(64, np.float16)
    for kw, word in ((dict(fmt=_abi.NHWC), "NCHW_TO_NHWC"), (dict(kernel=(2, 2)), "3x3"), (dict(pstrides=(1, 1)), "stride 2"),
                     (dict(ppads=(0, 0, 0, 0)), "pad 1")):
        with pytest.raises(RuntimeError, match=word):
            stem_pool_f16(gpu, x, w, b, _abi.ACT_RELU, **kw)
    with pytest.raises(RuntimeError, match="even width"):
        stem_pool_f16(gpu, r.standard_normal((1, 3, 32, 33)).astype(np.float16), w, b, _abi.ACT_RELU)
    with pytest.raises(RuntimeError, match="7x7"):
        w5 = r.standard_normal((64, 3, 5, 5)).astype(np.float16)
        X, Wt, B = gpu.put(x), gpu.put(np.ascontiguousarray(w5.transpose(0, 2, 3, 1))), gpu.put(b)
        Y = gpu.empty((64 * 8 * 8,), np.float16)
        gpu.ops.set_format(_abi.NCHW_TO_NHWC)
        try:
            gpu.ops.conv_bias_activ_max_pool(gpu.ptr(X), x.shape, gpu.ptr(Wt), w5.shape, gpu.ptr(B), (2, 2), (2, 2), _abi.ACT_RELU,
                                             (3, 3), (1, 1, 1, 1), (2, 2), gpu.ptr(Y), (1, 64, 8, 8))
        finally:
            gpu.ops.set_format(_abi.NCHW)


@pytest.mark.parametrize("case", [(1, 224, 224), (2, 64, 64), (3, 37, 51), (1, 9, 9), (2, 30, 61)], ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("crsk", [False, True])
@pytest.mark.parametrize("activ", [_abi.ACT_RELU, _abi.ACT_IDENTITY])
def test_first_layer_fp32_alone_and_with_its_max_pool(gpu, cpu, case, crsk, activ):
    """The fp32 N,C,H,W first layer (3 -> 64 channels, 7x7, stride 2, pad 3) through dnnrtConvBiasActiv and, with the
    3x3 stride-2 pooling behind it, through dnnrtConvBiasActivMaxPool, against the oracle's convolution and its chain:
    rtol 1e-4, atol 1e-5 as for every fp32 convolution (the maximum adds no rounding).  Both filter layouts; the
    benchmark's size, odd sizes with ragged tiles in both directions, an image smaller than one tile; identity
    activation leaves negative values, so a padding of zeros instead of -inf would show."""
    N, H, W = case
    r = rng(N + H + W + activ)
    x = r.standard_normal((N, 3, H, W)).astype(np.float32)
    w = (r.standard_normal((64, 3, 7, 7)) * np.sqrt(2.0 / 147)).astype(np.float32)
    b = r.uniform(-0.5, 0.1, 64).astype(np.float32)
    if case == (3, 37, 51):
        x[1, 2, 11, 30] = np.nan
        x[2, 0, 5, 40] = np.inf
        x[2, 1, 6, 41] = -np.inf
    conv_ref = oc.conv(cpu, x, w, b, (3, 3), (2, 2), 1, activ)
    ref = oc.pool(cpu, "max", conv_ref, (3, 3), (1, 1), (2, 2))
    lay = (lambda t: np.ascontiguousarray(t.transpose(1, 2, 3, 0))) if crsk else (lambda t: t)
    X, Wt, B = gpu.put(x), gpu.put(lay(w)), gpu.put(b)
    Yc, Yp = gpu.empty(conv_ref.shape, np.float32), gpu.empty(ref.shape, np.float32)
    gpu.ops.set_filter_layout(_abi.FILTER_CRSK if crsk else _abi.FILTER_KCRS)
    try:
        gpu.ops.conv_bias_activ(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), (3, 3), (2, 2), activ, gpu.ptr(Yc))
        gpu.ops.conv_bias_activ_max_pool(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), (3, 3), (2, 2), activ,
                                         (3, 3), (1, 1, 1, 1), (2, 2), gpu.ptr(Yp), ref.shape, dtype=_abi.F32)
        gpu.sync()
    finally:
        gpu.ops.set_filter_layout(_abi.FILTER_KCRS)
    got_c, got = gpu.get(Yc), gpu.get(Yp)
    finite = np.isfinite(conv_ref)
    assert (np.isnan(got_c) == np.isnan(conv_ref)).all() and (np.isnan(got) == np.isnan(ref)).all()
    np.testing.assert_allclose(got_c[finite], conv_ref[finite], rtol=1e-4, atol=1e-5)
    np.testing.assert_array_equal(got_c[~finite & ~np.isnan(conv_ref)], conv_ref[~finite & ~np.isnan(conv_ref)])
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-5)
    if case == (3, 37, 51):
        assert np.isnan(got[1]).any() and np.isnan(got[2]).any() and not np.isnan(got[0]).any()
    # the pooled result is the exact maximum of this library's own convolution
    Y2 = gpu.empty(ref.shape, np.float32)
    gpu.ops.maxpool(gpu.ptr(Yc), conv_ref.shape, gpu.ptr(Y2), ref.shape, (3, 3), (1, 1, 1, 1), (2, 2), _abi.F32)
    gpu.sync()
    np.testing.assert_array_equal(got, gpu.get(Y2))


def test_first_layer_fp32_with_its_max_pool_refuses_other_shapes(gpu):
    r = rng(4)
    x = r.standard_normal((1, 3, 32, 32)).astype(np.float32)
    b = np.zeros(64, np.float32)
    X, B = gpu.put(x), gpu.put(b)
    Y = gpu.empty((64 * 8 * 8,), np.float32)
    w5 = r.standard_normal((64, 3, 5, 5)).astype(np.float32)
    with pytest.raises(RuntimeError, match="7x7"):
        gpu.ops.conv_bias_activ_max_pool(gpu.ptr(X), x.shape, gpu.ptr(gpu.put(w5)), w5.shape, gpu.ptr(B), (2, 2), (2, 2), _abi.ACT_RELU,
                                         (3, 3), (1, 1, 1, 1), (2, 2), gpu.ptr(Y), (1, 64, 8, 8), dtype=_abi.F32)
    w7 = r.standard_normal((64, 3, 7, 7)).astype(np.float32)
    with pytest.raises(RuntimeError, match="ReLU or identity"):
        gpu.ops.conv_bias_activ_max_pool(gpu.ptr(X), x.shape, gpu.ptr(gpu.put(w7)), w7.shape, gpu.ptr(B), (3, 3), (2, 2), _abi.ACT_LEAKY_RELU,
                                         (3, 3), (1, 1, 1, 1), (2, 2), gpu.ptr(Y), (1, 64, 8, 8), dtype=_abi.F32)


def dual_conv_f16(gpu, x, w, b, x2, w2, b2, stride2, activ, algo=0):
    """dnnrtConvBiasAddConvBiasActiv through the C-ABI; tensors in logical NCHW / KCRS order; returns logical NCHW."""
    N, C, P, Q = x.shape
    K = w.shape[0]
    nhwc = lambda t: np.ascontiguousarray(t.transpose(0, 2, 3, 1))  # noqa: E731
    X, Wt, B, X2, Wt2, B2 = gpu.put(nhwc(x)), gpu.put(nhwc(w)), gpu.put(b), gpu.put(nhwc(x2)), gpu.put(nhwc(w2)), gpu.put(b2)
    Y = gpu.empty((N * K * P * Q,), np.float16)
    gpu.ops.set_format(_abi.NHWC)
    try:
        gpu.ops.conv_bias_add_conv_bias_activ(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), (0, 0), (1, 1), gpu.ptr(X2), x2.shape,
                                              gpu.ptr(Wt2), w2.shape, gpu.ptr(B2), (0, 0), (stride2, stride2), activ, gpu.ptr(Y),
                                              algo=algo)
        gpu.sync()
    finally:
        gpu.ops.set_format(_abi.NCHW)
    return gpu.get(Y).reshape(N, P, Q, K).transpose(0, 3, 1, 2)


@pytest.mark.parametrize("case", [(2, 9, 11, 64, 64, 72, 1), (3, 13, 13, 128, 256, 200, 2), (2, 14, 10, 192, 128, 256, 2), (8, 56, 56, 64, 64, 256, 1), (4, 56, 56, 128, 256, 512, 2), (3, 9, 13, 128, 256, 136, 2), (2, 10, 10, 128, 128, 72, 1), (2, 12, 12, 64, 256, 64, 2), (1, 9, 9, 192, 256, 40, 1),
                                  (1, 7, 7, 64, 128, 64, 1)], ids=lambda c: "x".join(map(str, c)))
def test_last_convolution_and_projection_shortcut_in_one_call(gpu, cpu, case):
    """dnnrtConvBiasAddConvBiasActiv against the two calls it replaces: the oracle's chain to the fp16 convolutions'
    tolerance.  N, H2, W2, C, C2, K, stride of the shortcut; ragged tiles in both directions.  64 + 64 and 128 + 256
    channels take the kernel that gives this library's own two calls bit for bit (each conv + bias rounded to fp16 on
    its own, the sum and ReLU in fp32); other multiples of 64 take one reduction over both convolutions' channels,
    rounded once, which is as close to the oracle as the two calls are but not their bits."""
    N, H2, W2, C, C2, K, st = case
    P, Q = (H2 - 1) // st + 1, (W2 - 1) // st + 1
    r = rng(sum(case))
    x = r.standard_normal((N, C, P, Q)).astype(np.float16)
    x2 = r.standard_normal((N, C2, H2, W2)).astype(np.float16)
    w = (r.standard_normal((K, C, 1, 1)) * np.sqrt(2.0 / C)).astype(np.float16)
    w2 = (r.standard_normal((K, C2, 1, 1)) * np.sqrt(2.0 / C2)).astype(np.float16)
    b, b2 = r.uniform(-0.2, 0.2, K).astype(np.float16), r.uniform(-0.2, 0.2, K).astype(np.float16)
    got = dual_conv_f16(gpu, x, w, b, x2, w2, b2, st, _abi.ACT_RELU)
    z_ref = oc.conv(cpu, x2, w2, b2, (0, 0), (st, st), 1, _abi.ACT_IDENTITY)
    ref = oc.conv(cpu, x, w, b, (0, 0), (1, 1), 1, _abi.ACT_RELU, z=z_ref)
    np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=4e-3, atol=4e-3)
    z_gpu = conv_f16(gpu, x2, w2, b2, (0, 0), (st, st), 1, _abi.ACT_IDENTITY, _abi.NHWC)
    two = conv_f16(gpu, x, w, b, (0, 0), (1, 1), 1, _abi.ACT_RELU, _abi.NHWC, z=z_gpu)
    if (C, C2) in ((64, 64), (128, 256)):
        np.testing.assert_array_equal(got, two)
    else:
        np.testing.assert_allclose(got.astype(np.float32), two.astype(np.float32), rtol=4e-3, atol=4e-3)
    if case[0] == 2 and C == 64:  # the oracle's own entry point is that chain
        X, Wt, B, X2, Wt2, B2 = cpu.put(x), cpu.put(w), cpu.put(b), cpu.put(x2), cpu.put(w2), cpu.put(b2)
        Y = cpu.empty(ref.shape, np.float16)
        cpu.ops.conv_bias_add_conv_bias_activ(cpu.ptr(X), x.shape, cpu.ptr(Wt), w.shape, cpu.ptr(B), (0, 0), (1, 1), cpu.ptr(X2), x2.shape,
                                              cpu.ptr(Wt2), w2.shape, cpu.ptr(B2), (0, 0), (st, st), _abi.ACT_RELU, cpu.ptr(Y))
        np.testing.assert_array_equal(cpu.get(Y), ref)


@pytest.mark.parametrize("case", [(64, 28, 28, 256, 512, 1024, 2), (64, 14, 14, 512, 1024, 2048, 2), (3, 13, 13, 128, 256, 200, 2),
                                  (2, 14, 10, 192, 128, 256, 2), (5, 9, 13, 64, 64, 136, 1)], ids=lambda c: "x".join(map(str, c)))
def test_shortcut_pair_as_one_reduction_every_variant(gpu, cpu, case):
    """The one-reduction form of dnnrtConvBiasAddConvBiasActiv on every tile variant it is compiled in, asked for
    through the call's `algo` operand (DNNRT_CONV_ALGO_BASE + id), ResNet-50's two long pairs at batch 64 among the
    cases and the short pairs too (which take this form only when asked): the oracle's chain to the fp16
    convolutions' tolerance."""
    N, H2, W2, C, C2, K, st = case
    P, Q = (H2 - 1) // st + 1, (W2 - 1) // st + 1
    r = rng(sum(case) + 1)
    x = r.standard_normal((N, C, P, Q)).astype(np.float16)
    x2 = r.standard_normal((N, C2, H2, W2)).astype(np.float16)
    w = (r.standard_normal((K, C, 1, 1)) * np.sqrt(2.0 / C)).astype(np.float16)
    w2 = (r.standard_normal((K, C2, 1, 1)) * np.sqrt(2.0 / C2)).astype(np.float16)
    b, b2 = r.uniform(-0.2, 0.2, K).astype(np.float16), r.uniform(-0.2, 0.2, K).astype(np.float16)
    z_ref = oc.conv(cpu, x2, w2, b2, (0, 0), (st, st), 1, _abi.ACT_IDENTITY)
    ref = oc.conv(cpu, x, w, b, (0, 0), (1, 1), 1, _abi.ACT_RELU, z=z_ref).astype(np.float32)
    for vid in (33, 37, 39, 61, 64, 66):
        got = dual_conv_f16(gpu, x, w, b, x2, w2, b2, st, _abi.ACT_RELU, algo=_abi.CONV_ALGO_BASE + vid)
        np.testing.assert_allclose(got.astype(np.float32), ref, rtol=4e-3, atol=4e-3, err_msg=f"variant {vid}")


@pytest.mark.parametrize("case", [(1, 56, 56, 64, 64, 256, 1), (1, 56, 56, 128, 256, 512, 2), (1, 28, 28, 256, 512, 1024, 2),
                                  (1, 14, 14, 512, 1024, 2048, 2), (2, 9, 11, 24, 40, 72, 1), (16, 28, 28, 128, 256, 512, 2)],
                         ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("crsk", [False, True])
def test_last_convolution_and_projection_shortcut_fp32(gpu, cpu, case, crsk):
    """The same call on fp32 N,C,H,W tensors with both filter layouts: ResNet-50's four shortcut pairs at batch 1 (one
    launch of the small 1x1 kernel, the second reduction appended to the first: one rounding of the whole sum where the
    chain has three), an odd-sized pair and a batch-16 pair (the two convolutions one after the other through Y: the
    chain's bits).  Against the oracle's chain: rtol 1e-4, atol 1e-5 as for every fp32 convolution."""
    N, H2, W2, C, C2, K, st = case
    P, Q = (H2 - 1) // st + 1, (W2 - 1) // st + 1
    r = rng(sum(case))
    x = r.standard_normal((N, C, P, Q)).astype(np.float32)
    x2 = r.standard_normal((N, C2, H2, W2)).astype(np.float32)
    w = (r.standard_normal((K, C, 1, 1)) * np.sqrt(2.0 / C)).astype(np.float32)
    w2 = (r.standard_normal((K, C2, 1, 1)) * np.sqrt(2.0 / C2)).astype(np.float32)
    b, b2 = r.uniform(-0.2, 0.2, K).astype(np.float32), r.uniform(-0.2, 0.2, K).astype(np.float32)
    z_ref = oc.conv(cpu, x2, w2, b2, (0, 0), (st, st), 1, _abi.ACT_IDENTITY)
    ref = oc.conv(cpu, x, w, b, (0, 0), (1, 1), 1, _abi.ACT_RELU, z=z_ref)
    lay = (lambda t: np.ascontiguousarray(t.transpose(1, 2, 3, 0))) if crsk else (lambda t: t)
    X, Wt, B, X2, Wt2, B2 = gpu.put(x), gpu.put(lay(w)), gpu.put(b), gpu.put(x2), gpu.put(lay(w2)), gpu.put(b2)
    Y = gpu.empty(ref.shape, np.float32)
    gpu.ops.set_filter_layout(_abi.FILTER_CRSK if crsk else _abi.FILTER_KCRS)
    try:
        for _ in range(2):  # twice: the split reduction's counters must be back at zero
            gpu.ops.conv_bias_add_conv_bias_activ(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), (0, 0), (1, 1), gpu.ptr(X2), x2.shape,
                                                  gpu.ptr(Wt2), w2.shape, gpu.ptr(B2), (0, 0), (st, st), _abi.ACT_RELU, gpu.ptr(Y), dtype=_abi.F32)
            gpu.sync()
            np.testing.assert_allclose(gpu.get(Y), ref, rtol=1e-4, atol=1e-5)
    finally:
        gpu.ops.set_filter_layout(_abi.FILTER_KCRS)


def test_last_convolution_and_projection_shortcut_with_other_convolutions(gpu, cpu):
    """Shapes the one-kernel forms do not take run as the two convolutions through Y and give the chain's bits: a 3x3
    closing convolution in fp16 channels-last."""
    r = rng(11)
    x = r.standard_normal((2, 64, 9, 9)).astype(np.float16)
    x2 = r.standard_normal((2, 128, 9, 9)).astype(np.float16)
    w = (r.standard_normal((72, 64, 3, 3)) * 0.06).astype(np.float16)
    w2 = (r.standard_normal((72, 128, 1, 1)) * 0.1).astype(np.float16)
    b, b2 = r.uniform(-0.2, 0.2, 72).astype(np.float16), r.uniform(-0.2, 0.2, 72).astype(np.float16)
    nhwc = lambda t: np.ascontiguousarray(t.transpose(0, 2, 3, 1))  # noqa: E731
    X, Wt, B, X2, Wt2, B2 = gpu.put(nhwc(x)), gpu.put(nhwc(w)), gpu.put(b), gpu.put(nhwc(x2)), gpu.put(nhwc(w2)), gpu.put(b2)
    Y = gpu.empty((2 * 72 * 9 * 9,), np.float16)
    gpu.ops.set_format(_abi.NHWC)
    try:
        gpu.ops.conv_bias_add_conv_bias_activ(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), (1, 1), (1, 1), gpu.ptr(X2), x2.shape,
                                              gpu.ptr(Wt2), w2.shape, gpu.ptr(B2), (0, 0), (1, 1), _abi.ACT_RELU, gpu.ptr(Y))
        gpu.sync()
    finally:
        gpu.ops.set_format(_abi.NCHW)
    got = gpu.get(Y).reshape(2, 9, 9, 72).transpose(0, 3, 1, 2)
    z_gpu = conv_f16(gpu, x2, w2, b2, (0, 0), (1, 1), 1, _abi.ACT_IDENTITY, _abi.NHWC)
    two = conv_f16(gpu, x, w, b, (1, 1), (1, 1), 1, _abi.ACT_RELU, _abi.NHWC, z=z_gpu)
    np.testing.assert_array_equal(got, two)
    z_ref = oc.conv(cpu, x2, w2, b2, (0, 0), (1, 1), 1, _abi.ACT_IDENTITY)
    ref = oc.conv(cpu, x, w, b, (1, 1), (1, 1), 1, _abi.ACT_RELU, z=z_ref)
    np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=4e-3, atol=4e-3)


def test_last_convolution_and_projection_shortcut_refuses_other_shapes(gpu):
    r = rng(4)
    x = r.standard_normal((1, 64, 8, 8)).astype(np.float16)
    w = r.standard_normal((64, 64, 1, 1)).astype(np.float16)
    b = np.zeros(64, np.float16)
    X, Wt, B = gpu.put(x), gpu.put(w), gpu.put(b)
    Y = gpu.empty((64 * 64,), np.float16)
    gpu.ops.set_format(_abi.NHWC)
    try:
        with pytest.raises(RuntimeError, match="give"):  # the two convolutions must land on the same tensor
            gpu.ops.conv_bias_add_conv_bias_activ(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), (0, 0), (1, 1), gpu.ptr(X), (1, 64, 4, 16),
                                                  gpu.ptr(Wt), w.shape, gpu.ptr(B), (0, 0), (1, 1), _abi.ACT_RELU, gpu.ptr(Y))
        with pytest.raises(RuntimeError, match="dtype"):
            gpu.ops.conv_bias_add_conv_bias_activ(gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), (0, 0), (1, 1), gpu.ptr(X), x.shape,
                                                  gpu.ptr(Wt), w.shape, gpu.ptr(B), (0, 0), (1, 1), _abi.ACT_RELU, gpu.ptr(Y), dtype=_abi.I64)
    finally:
        gpu.ops.set_format(_abi.NCHW)


# Problems of the size ResNet-50 has at batch 64: the dispatcher picks its large tiles (128 x 128 and up,
# four or eight wavefronts) only when a launch has hundreds of tiles, so these are the only cases that reach
# them.  N, C, H, W, K, R, stride, pad
F16_BATCH64_CASES = [
    (64, 128, 28, 28, 128, 3, 1, 1),   # 392 tiles of 128 x 128, padded taps
    (32, 128, 28, 28, 128, 3, 1, 1),   # 196 tiles: about one per CU
    (64, 512, 28, 28, 128, 1, 1, 0),   # 1x1, no taps to mask, eight steps
    (64, 256, 14, 14, 256, 3, 1, 1),   # 14 x 14: 196 tiles
    (64, 128, 56, 56, 128, 3, 2, 1),   # strided 3x3
    (64, 256, 56, 56, 512, 1, 2, 0),   # strided 1x1 (downsample branch)
    (64, 64, 56, 56, 64, 3, 1, 1),     # K_out = 64: 64-filter tiles
    (61, 128, 28, 28, 136, 3, 1, 1),   # ragged in pixels (47824 = 373.6 x 128) and in filters
    (64, 512, 7, 7, 512, 3, 1, 1),     # 7 x 7: few, deep tiles
    (64, 1024, 14, 14, 256, 1, 1, 0),  # sixteen steps
    (64, 2048, 7, 7, 512, 1, 1, 0),    # 7 x 7, 1x1: 64-row tiles on eight wavefronts
    (64, 512, 14, 14, 512, 3, 2, 1),   # the same, strided 3x3
]


def f16_problem(case, seed):
    N, C, H, W, K, R, st, pd = case
    r = rng(seed)
    x = r.standard_normal((N, C, H, W), dtype=np.float32).astype(np.float16)
    w = (r.standard_normal((K, C, R, R), dtype=np.float32) * np.sqrt(2.0 / (C * R * R))).astype(np.float16)
    b = r.uniform(-0.1, 0.1, K).astype(np.float16)
    return x, w, b, (pd, pd), (st, st)


@pytest.mark.parametrize("case", F16_BATCH64_CASES, ids=lambda c: "x".join(map(str, c)))
def test_conv_f16_at_batch_64_sizes(gpu, cpu, case):
    x, w, b, pads, strides = f16_problem(case, sum(case))
    ref = oc.conv(cpu, x, w, b, pads, strides, 1, _abi.ACT_RELU)
    got = conv_f16(gpu, x, w, b, pads, strides, 1, _abi.ACT_RELU, _abi.NHWC)
    np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=2e-3, atol=2e-3)
    z = rng(1 + sum(case)).standard_normal(ref.shape, dtype=np.float32).astype(np.float16)
    refz = oc.conv(cpu, x, w, b, pads, strides, 1, _abi.ACT_RELU, z=z)
    gotz = conv_f16(gpu, x, w, b, pads, strides, 1, _abi.ACT_RELU, _abi.NHWC, z=z)
    np.testing.assert_allclose(gotz.astype(np.float32), refz.astype(np.float32), rtol=4e-3, atol=4e-3)
    np.testing.assert_array_equal(conv_f16(gpu, x, w, b, pads, strides, 1, _abi.ACT_RELU, _abi.NHWC, z=z, inplace=True), gotz)


def test_every_compiled_f16_conv_variant(gpu, cpu):
    """Each variant dnnrtListConvTiles names, forced with dnnrtSetConvTile, on a padded 3x3 problem, a 1x1
    problem over 128 channels and one over 512, and two 3x3 problems on small images whose runs of pixels cross
    image boundaries (one to three per tile), all ragged in both directions: it either matches the
    oracle or refuses the problem loudly (the single-stage variants take reductions of up to four steps)."""
    tiles = gpu.ops.conv_tiles()
    assert tiles and 0 not in tiles
    cases = [(3, 128, 19, 23, 200, 3, 1, 1), (5, 128, 19, 23, 200, 1, 1, 0), (5, 512, 9, 13, 136, 1, 2, 0),
             (11, 192, 14, 14, 136, 3, 1, 1), (23, 128, 7, 7, 72, 3, 1, 1), (5, 64, 13, 20, 72, 3, 1, 1), (2, 64, 56, 56, 64, 3, 1, 1)]
    ran = {t: 0 for t in tiles}
    for case in cases:
        x, w, b, pads, strides = f16_problem(case, 5 + sum(case))
        z = rng(6).standard_normal((case[0], case[4]) + oc.conv_out_hw(case[2], case[3], case[5], case[5], pads, strides),
                                   dtype=np.float32).astype(np.float16)
        ref = oc.conv(cpu, x, w, b, pads, strides, 1, _abi.ACT_RELU)
        refz = oc.conv(cpu, x, w, b, pads, strides, 1, _abi.ACT_RELU, z=z)
        for t in tiles:
            gpu.ops.set_conv_tile(t)
            try:
                got = conv_f16(gpu, x, w, b, pads, strides, 1, _abi.ACT_RELU, _abi.NHWC)
                try:
                    gotz = conv_f16(gpu, x, w, b, pads, strides, 1, _abi.ACT_RELU, _abi.NHWC, z=z)
                    np.testing.assert_array_equal(conv_f16(gpu, x, w, b, pads, strides, 1, _abi.ACT_RELU, _abi.NHWC, z=z, inplace=True), gotz,
                                                  err_msg=f"variant {t} on {case} written over its residual operand")
                except RuntimeError as e:  # a variant without the residual operand says so
                    assert "residual" in str(e), str(e)
                    gotz = None
            except RuntimeError as e:
                assert "tile" in str(e) or "variant" in str(e), str(e)
                continue
            finally:
                gpu.ops.set_conv_tile(0)
            ran[t] += 1
            np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=2e-3, atol=2e-3,
                                       err_msg=f"variant {t} on {case}")
            if gotz is not None:
                np.testing.assert_allclose(gotz.astype(np.float32), refz.astype(np.float32), rtol=4e-3, atol=4e-3,
                                           err_msg=f"variant {t} on {case} with a residual")
    assert all(ran.values()), f"variants that ran no case: {[t for t, n in ran.items() if not n]}"
    with pytest.raises(RuntimeError):
        gpu.ops.set_conv_tile(9999)


def test_f16_channels_last_ops(gpu, cpu):
    r = rng(77)
    x = r.standard_normal((2, 64, 28, 28)).astype(np.float16)
    xl = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    gpu.ops.set_format(_abi.NHWC)
    try:
        X = gpu.put(xl)
        Y = gpu.empty((2 * 64 * 14 * 14,), np.float16)
        gpu.ops.maxpool(gpu.ptr(X), x.shape, gpu.ptr(Y), (2, 64, 14, 14), (3, 3), (1, 1, 1, 1), (2, 2), _abi.F16)
        G = gpu.empty((2 * 64,), np.float16)
        gpu.ops.reduce_mean(gpu.ptr(X), x.shape, gpu.ptr(G), (2, 64, 1, 1), _abi.F16)
        bias = r.standard_normal((1, 64, 1, 1)).astype(np.float16)
        Bv = gpu.put(bias.reshape(64))
        O = gpu.empty(xl.shape, np.float16)
        gpu.ops.tensor_op(_abi.OP_ADD, gpu.ptr(X), x.shape, gpu.ptr(Bv), (1, 64, 1, 1), gpu.ptr(O), 1.0, _abi.F16)
        gpu.sync()
    finally:
        gpu.ops.set_format(_abi.NCHW)
    np.testing.assert_array_equal(gpu.get(Y).reshape(2, 14, 14, 64).transpose(0, 3, 1, 2),
                                  oc.pool(cpu, "max", x, (3, 3), (1, 1), (2, 2)))
    np.testing.assert_allclose(gpu.get(G).reshape(2, 64, 1, 1).astype(np.float32),
                               oc.reduce_mean(cpu, x, (2, 64, 1, 1)).astype(np.float32), rtol=2e-3, atol=1e-3)
    np.testing.assert_array_equal(gpu.get(O).transpose(0, 3, 1, 2), oc.tensor_op(cpu, _abi.OP_ADD, x, bias))


@pytest.mark.parametrize("C", [64, 12])          # 16-byte vector kernel / scalar kernel
@pytest.mark.parametrize("kind", ["max", "avg"])
def test_pooling_f16_channels_last(gpu, cpu, C, kind):
    r = rng(79 + C)
    x = r.standard_normal((3, C, 15, 13)).astype(np.float16)
    x[1, 3, 4, 5] = np.nan                        # NaN must reach every window that sees it
    for kernel, pads, strides in [((3, 3), (1, 1), (2, 2)), ((2, 2), (0, 0), (2, 2)), ((3, 2), (1, 0), (1, 2))]:
        P, Q = oc.conv_out_hw(15, 13, kernel[0], kernel[1], pads, strides)
        gpu.ops.set_format(_abi.NHWC)
        try:
            X = gpu.put(np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
            Y = gpu.empty((3 * C * P * Q,), np.float16)
            fn = gpu.ops.maxpool if kind == "max" else gpu.ops.avgpool
            fn(gpu.ptr(X), x.shape, gpu.ptr(Y), (3, C, P, Q), kernel, [pads[0], pads[1], pads[0], pads[1]], strides, _abi.F16)
            gpu.sync()
        finally:
            gpu.ops.set_format(_abi.NCHW)
        got = gpu.get(Y).reshape(3, P, Q, C).transpose(0, 3, 1, 2)
        ref = oc.pool(cpu, kind, x, kernel, pads, strides)
        if kind == "max":
            np.testing.assert_array_equal(got, ref)
        else:
            np.testing.assert_allclose(got.astype(np.float32), ref.astype(np.float32), rtol=2e-3, atol=1e-3)


def test_matmul2d_f16(gpu, cpu):
    r = rng(78)
    for M, K, N in [(64, 2048, 1000), (2, 64, 8), (130, 96, 72)]:
        a = r.standard_normal((M, K)).astype(np.float16)
        b = (r.standard_normal((N, K)) / np.sqrt(K)).astype(np.float16)
        np.testing.assert_allclose(oc.matmul2d(gpu, a, b, transB=1).astype(np.float32),
                                   oc.matmul2d(cpu, a, b, transB=1).astype(np.float32), rtol=2e-3, atol=2e-3)
        # C as one row with beta 1 (a Gemm's bias): the convolution kernel's bias; the oracle runs product, then add
        row = r.standard_normal(N).astype(np.float16)
        np.testing.assert_allclose(oc.matmul2d_row(gpu, a, b, row, transB=1).astype(np.float32),
                                   oc.matmul2d_row(cpu, a, b, row, transB=1).astype(np.float32), rtol=2e-3, atol=4e-3)
    # every other form on the generic fp16 kernel: the four operand layouts, alpha and beta with a row or a matrix C
    # (the matrix updated in place), ragged tiles
    for M, K, N in [(130, 96, 72), (5, 7, 3), (64, 200, 65)]:
        for tA in (0, 1):
            for tB in (0, 1):
                a = r.standard_normal((K, M) if tA else (M, K)).astype(np.float16)
                b = (r.standard_normal((N, K) if tB else (K, N)) / np.sqrt(K)).astype(np.float16)
                c = r.standard_normal((M, N)).astype(np.float16)
                row = r.standard_normal(N).astype(np.float16)
                for kw in (dict(), dict(alpha=0.5), dict(c=c, alpha=1.5, beta=0.5), dict(c=c, beta=1.0)):
                    np.testing.assert_allclose(oc.matmul2d(gpu, a, b, transA=tA, transB=tB, **kw).astype(np.float32),
                                               oc.matmul2d(cpu, a, b, transA=tA, transB=tB, **kw).astype(np.float32), rtol=4e-3, atol=6e-3)
                if not tA:
                    np.testing.assert_allclose(oc.matmul2d_row(gpu, a, b, row, beta=0.5, transB=tB).astype(np.float32),
                                               oc.matmul2d_row(cpu, a, b, row, beta=0.5, transB=tB).astype(np.float32), rtol=4e-3, atol=6e-3)
