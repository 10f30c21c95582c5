"""One function per operator that runs it through a backend (tests/helpers.py)
on numpy inputs and returns a numpy output.  Used by the oracle tests (oracle
vs. closed forms / torch CPU) and by the GPU parity tests (HIP vs. oracle)."""
import numpy as np

from occamy_amd import _abi

DT = {np.dtype(np.float32): _abi.F32, np.dtype(np.float16): _abi.F16, np.dtype(np.int64): _abi.I64}


def conv_out_hw(H, W, R, S, pads, strides):
    return (H + 2 * pads[0] - R) // strides[0] + 1, (W + 2 * pads[1] - S) // strides[1] + 1


def conv(be, x, w, b=None, pads=(0, 0), strides=(1, 1), group=1, activ=None, crsk=False, z=None, coef=None, inplace=False):
    """crsk: hand the filter over stored C,R,S,K (the dims stay logical K,C,R,S).
    z: residual tensor shaped like the result (needs b): act((conv + b) + z); inplace: the result buffer holds z
    and is passed as both Z and Y.
    coef: the handle's activation coefficient (ceiling of ACT_CLIPPED_RELU, slope of ACT_LEAKY_RELU)."""
    N, C, H, W = x.shape
    K, Cg, R, S = w.shape
    P, Q = conv_out_hw(H, W, R, S, pads, strides)
    dt = DT[x.dtype]
    X = be.put(x)
    Wt = be.put(np.ascontiguousarray(w.transpose(1, 2, 3, 0)) if crsk else w)
    Y = be.empty((N, K, max(P, 1), max(Q, 1)), x.dtype)  # the call rejects empty outputs itself
    if crsk:
        be.ops.set_filter_layout(_abi.FILTER_CRSK)
    if coef is not None:
        be.ops.set_activation_coef(coef)
    try:
        if b is None:
            assert activ is None
            be.ops.conv(be.ptr(X), x.shape, be.ptr(Wt), w.shape, pads, strides, be.ptr(Y), group, dt)
        elif z is not None:
            B, Z = be.put(b), be.put(z)
            if inplace:
                Y = Z
            be.ops.conv_bias_add_activ(be.ptr(X), x.shape, be.ptr(Wt), w.shape, be.ptr(B), be.ptr(Z), pads, strides,
                                       activ if activ is not None else _abi.ACT_IDENTITY, be.ptr(Y), group, dt)
        else:
            B = be.put(b)
            be.ops.conv_bias_activ(be.ptr(X), x.shape, be.ptr(Wt), w.shape, be.ptr(B), pads, strides,
                                   activ if activ is not None else _abi.ACT_IDENTITY, be.ptr(Y), group, dt)
    finally:
        if crsk:
            be.ops.set_filter_layout(_abi.FILTER_KCRS)
    be.sync()
    return be.get(Y)


def unary(be, name, x, **kw):
    X = be.put(x)
    Y = be.empty(x.shape, x.dtype)
    dt = DT[x.dtype]
    if name == "relu":
        be.ops.active(be.ptr(X), x.shape, _abi.ACT_RELU, be.ptr(Y), dt)
    elif name == "sigmoid":
        be.ops.active(be.ptr(X), x.shape, _abi.ACT_SIGMOID, be.ptr(Y), dt)
    elif name == "tanh":
        be.ops.active(be.ptr(X), x.shape, _abi.ACT_TANH, be.ptr(Y), dt)
    elif name == "clip":
        be.ops.clip(be.ptr(X), be.ptr(Y), x.shape, kw["lo"], kw["hi"], dt)
    elif name == "sqrt":
        be.ops.tensor_op(_abi.OP_SQRT, be.ptr(X), x.shape, None, x.shape, be.ptr(Y), 1.0, dt)
    else:
        getattr(be.ops, name)(be.ptr(X), be.ptr(Y), x.shape, dt)
    be.sync()
    return be.get(Y)


def pow_(be, x, e):
    X, E = be.put(x), be.put(np.array([e], dtype=x.dtype))
    Y = be.empty(x.shape, x.dtype)
    be.ops.pow(be.ptr(X), be.ptr(E), be.ptr(Y), x.shape, DT[x.dtype])
    be.sync()
    return be.get(Y)


def cast(be, x, out_dtype=np.float32):
    X = be.put(x)
    Y = be.empty(x.shape, out_dtype)
    be.ops.cast_i64_to_float(be.ptr(X), be.ptr(Y), x.shape, DT[np.dtype(out_dtype)])
    be.sync()
    return be.get(Y)


def tensor_op(be, op, a, b, coef=1.0, inplace=False):
    A, B = be.put(a), be.put(b)
    O = A if inplace else be.empty(a.shape, a.dtype)
    be.ops.tensor_op(op, be.ptr(A), a.shape, be.ptr(B), b.shape, be.ptr(O), coef, DT[a.dtype])
    be.sync()
    return be.get(O)


def reduce_mean(be, x, out_shape):
    X = be.put(x)
    Y = be.empty(out_shape, x.dtype)
    be.ops.reduce_mean(be.ptr(X), x.shape, be.ptr(Y), out_shape, DT[x.dtype])
    be.sync()
    return be.get(Y)


def softmax(be, x, axis):
    X = be.put(x)
    Y = be.empty(x.shape, x.dtype)
    be.ops.softmax(be.ptr(X), x.shape, be.ptr(Y), axis, DT[x.dtype])
    be.sync()
    return be.get(Y)


def layernorm(be, x, g, b, eps):
    X, G, B = be.put(x), be.put(g), be.put(b)
    Y = be.empty(x.shape, x.dtype)
    be.ops.layernorm(be.ptr(X), x.shape, be.ptr(G), be.ptr(B), eps, be.ptr(Y), DT[x.dtype])
    be.sync()
    return be.get(Y)


def pool(be, kind, x, kernel, pads, strides):
    N, C, H, W = x.shape
    P, Q = conv_out_hw(H, W, kernel[0], kernel[1], pads, strides)
    X = be.put(x)
    Y = be.empty((N, C, P, Q), x.dtype)
    fn = be.ops.maxpool if kind == "max" else be.ops.avgpool
    fn(be.ptr(X), x.shape, be.ptr(Y), (N, C, P, Q), kernel, [pads[0], pads[1], pads[0], pads[1]],
       strides, DT[x.dtype])
    be.sync()
    return be.get(Y)


def matmul2d(be, a, b, c=None, alpha=1.0, beta=0.0, transA=0, transB=0):
    M = a.shape[1] if transA else a.shape[0]
    N = b.shape[0] if transB else b.shape[1]
    A, B = be.put(a), be.put(b)
    Out = be.put(c) if c is not None else be.empty((M, N), a.dtype)
    be.ops.matmul2d(be.ptr(A), a.shape, be.ptr(B), b.shape, be.ptr(Out), (M, N), alpha, beta, transA,
                    transB, be.ptr(Out) if c is not None else None, DT[a.dtype])
    be.sync()
    return be.get(Out)


def matmul2d_row(be, a, b, row, alpha=1.0, beta=1.0, transB=0):
    """Out = alpha a b + beta row, the row [N] added to every row of the product."""
    M, N = a.shape[0], (b.shape[0] if transB else b.shape[1])
    A, B, C_ = be.put(a), be.put(b), be.put(row.reshape(1, N))
    Out = be.empty((M, N), a.dtype)
    be.ops.matmul2d(be.ptr(A), a.shape, be.ptr(B), b.shape, be.ptr(Out), (M, N), alpha, beta, 0, transB,
                    be.ptr(C_), DT[a.dtype], dimC=(1, N))
    be.sync()
    return be.get(Out)


def matmul_nd(be, a, b):
    y_shape = np.matmul(np.zeros(a.shape, np.float32), np.zeros(b.shape, np.float32)).shape
    A, B = be.put(a), be.put(b)
    Y = be.empty(y_shape, a.dtype)
    be.ops.matmul_nd(be.ptr(A), a.shape, be.ptr(B), b.shape, be.ptr(Y), y_shape, DT[a.dtype])
    be.sync()
    return be.get(Y)


def flatten(be, x, axis):
    out = (int(np.prod(x.shape[:axis])), int(np.prod(x.shape[axis:])))
    X = be.put(x)
    Y = be.empty(out, x.dtype)
    be.ops.flatten(be.ptr(X), x.shape, be.ptr(Y), out, axis, DT[x.dtype])
    be.sync()
    return be.get(Y)


def reshape(be, x, out):
    X = be.put(x)
    Y = be.empty(out, x.dtype)
    be.ops.reshape(be.ptr(X), x.shape, be.ptr(Y), DT[x.dtype])
    be.sync()
    return be.get(Y)


def transpose(be, x, perm):
    X = be.put(x)
    Y = be.empty([x.shape[p] for p in perm], x.dtype)
    be.ops.transpose(be.ptr(X), x.shape, be.ptr(Y), perm, DT[x.dtype])
    be.sync()
    return be.get(Y)


def gather(be, x, idx, axis):
    out = x.shape[:axis] + idx.shape + x.shape[axis + 1:]
    X, I = be.put(x), be.put(idx.astype(np.int64))
    Y = be.empty(out, x.dtype)
    be.ops.gather(be.ptr(X), x.shape, be.ptr(Y), out, be.ptr(I), idx.shape, axis, DT[x.dtype])
    be.sync()
    return be.get(Y)


def leaky_relu(be, x, alpha):
    X = be.put(x)
    Y = be.empty(x.shape, x.dtype)
    be.ops.leaky_relu(be.ptr(X), be.ptr(Y), x.shape, alpha, DT[x.dtype])
    be.sync()
    return be.get(Y)


def prelu(be, x, slope):
    X, S = be.put(x), be.put(slope)
    Y = be.empty(x.shape, x.dtype)
    be.ops.prelu(be.ptr(X), be.ptr(Y), x.shape, be.ptr(S), slope.shape, DT[x.dtype])
    be.sync()
    return be.get(Y)


def concat(be, xs, axis):
    out = list(xs[0].shape)
    out[axis] = sum(x.shape[axis] for x in xs)
    Xs = [be.put(x) for x in xs]
    Y = be.empty(out, xs[0].dtype)
    be.ops.concat([be.ptr(X) for X in Xs], [x.shape for x in xs], be.ptr(Y), out, axis, DT[xs[0].dtype])
    be.sync()
    return be.get(Y)


def squeeze(be, x, out, un=False):
    X = be.put(x)
    Y = be.empty(out, x.dtype)
    (be.ops.unsqueeze if un else be.ops.squeeze)(be.ptr(X), x.shape, be.ptr(Y), out, DT[x.dtype])
    be.sync()
    return be.get(Y)


def expand(be, x, out):
    X = be.put(x)
    Y = be.empty(out, x.dtype)
    be.ops.expand(be.ptr(X), x.shape, be.ptr(Y), out, DT[x.dtype])
    be.sync()
    return be.get(Y)


def nonzero(be, x, out, fill):
    """Y starts as `fill` everywhere: the call writes only the front."""
    X = be.put(x)
    Y = be.put(np.full(out, fill, x.dtype))
    be.ops.nonzero(be.ptr(X), x.shape, be.ptr(Y), out, DT[x.dtype])
    be.sync()
    return be.get(Y)


def matmul_nd_bias(be, a, b, bias, z=None, gelu=False):
    y_shape = np.broadcast_shapes(a.shape[:-2], b.shape[:-2]) + (a.shape[-2], b.shape[-1])
    A, B, Bi = be.put(a), be.put(b), be.put(bias)
    Z = be.put(z) if z is not None else None
    Y = be.empty(y_shape, a.dtype)
    be.ops.matmul_nd_bias(be.ptr(A), a.shape, be.ptr(B), b.shape, be.ptr(Bi), be.ptr(Y), y_shape, DT[a.dtype],
                          Z=be.ptr(Z) if Z is not None else None, gelu=gelu)
    be.sync()
    return be.get(Y)


def attention(be, q, k, v, heads, scale):
    """q [B, Sq, heads*D], k and v [B, Sk, heads*D]."""
    B, Sq, hidden = q.shape
    Q, K, V = be.put(q), be.put(k), be.put(v)
    Y = be.empty(q.shape, q.dtype)
    be.ops.attention(be.ptr(Q), be.ptr(K), be.ptr(V), be.ptr(Y), B, Sq, k.shape[1], heads, hidden // heads, scale, DT[q.dtype])
    be.sync()
    return be.get(Y)


def attention_packed(be, qkv, heads, scale):
    """qkv [B, S, 3*hidden]: every row holds Q | K | V."""
    B, S, three = qkv.shape
    hidden = three // 3
    X = be.put(qkv)
    Y = be.empty((B, S, hidden), qkv.dtype)
    es = qkv.dtype.itemsize
    p = be.ptr(X)
    be.ops.attention(p, p + hidden * es, p + 2 * hidden * es, be.ptr(Y), B, S, S, heads, hidden // heads, scale,
                     DT[qkv.dtype], ld_in=three)
    be.sync()
    return be.get(Y)


def empty_tensor_behaviour(be):
    """Every entry point with a tensor that has a zero dim.  Buffers are real
    (64 sentinel floats) so that only the dims say "empty".  Returns
    {entry point: "refused" | "untouched" | "wrote"}: a clean error, or a
    successful call that left the output alone."""
    f32 = np.float32
    o = be.ops
    out = {}

    def probe(name, call, outputs):
        try:
            call()
            be.sync()
        except RuntimeError:
            out[name] = "refused"
            return
        out[name] = "untouched" if all(np.array_equal(be.get(y), np.full(64, 7.0, f32)) for y in outputs) else "wrote"

    def buf():
        return be.put(np.full(64, 7.0, f32))

    def idx():
        return be.put(np.zeros(8, np.int64))

    X, W, B, Z, Y = buf(), buf(), buf(), buf(), buf()
    p = be.ptr
    probe("conv", lambda: o.conv(p(X), (0, 4, 3, 3), p(W), (2, 4, 1, 1), (0, 0), (1, 1), p(Y)), [Y])
    probe("conv_bias_activ", lambda: o.conv_bias_activ(p(X), (0, 4, 3, 3), p(W), (2, 4, 1, 1), p(B), (0, 0), (1, 1), _abi.ACT_RELU, p(Y)), [Y])
    probe("conv_bias_add_activ", lambda: o.conv_bias_add_activ(p(X), (0, 4, 3, 3), p(W), (2, 4, 1, 1), p(B), p(Z), (0, 0), (1, 1), _abi.ACT_RELU, p(Y)), [Y])
    probe("active", lambda: o.active(p(X), (0, 4), _abi.ACT_RELU, p(Y)), [Y])
    probe("tensor_op", lambda: o.tensor_op(_abi.OP_ADD, p(X), (0, 4), p(B), (1, 4), p(Y)), [Y])
    probe("clip", lambda: o.clip(p(X), p(Y), (0, 4), 0.0, 1.0), [Y])
    probe("leaky_relu", lambda: o.leaky_relu(p(X), p(Y), (0, 4), 0.1), [Y])
    probe("prelu", lambda: o.prelu(p(X), p(Y), (0, 4), p(B), (1, 4)), [Y])
    probe("erf", lambda: o.erf(p(X), p(Y), (0, 4)), [Y])
    probe("gelu", lambda: o.gelu(p(X), p(Y), (0, 4)), [Y])
    probe("pow", lambda: o.pow(p(X), p(B), p(Y), (0, 4)), [Y])
    probe("cast", lambda: o.cast_i64_to_float(p(idx()), p(Y), (0, 4)), [Y])
    probe("reduce_mean", lambda: o.reduce_mean(p(X), (0, 4), p(Y), (0, 1)), [Y])
    probe("softmax", lambda: o.softmax(p(X), (0, 4), p(Y), 1), [Y])
    probe("layernorm", lambda: o.layernorm(p(X), (0, 4), p(W), p(B), 1e-5, p(Y)), [Y])
    probe("maxpool", lambda: o.maxpool(p(X), (0, 2, 4, 4), p(Y), (0, 2, 2, 2), (2, 2), (0, 0, 0, 0), (2, 2)), [Y])
    probe("avgpool", lambda: o.avgpool(p(X), (0, 2, 4, 4), p(Y), (0, 2, 2, 2), (2, 2), (0, 0, 0, 0), (2, 2)), [Y])
    probe("matmul2d", lambda: o.matmul2d(p(X), (0, 4), p(W), (4, 3), p(Y), (0, 3)), [Y])
    probe("matmul_nd", lambda: o.matmul_nd(p(X), (0, 2, 4), p(W), (4, 3), p(Y), (0, 2, 3)), [Y])
    probe("matmul_nd_bias", lambda: o.matmul_nd_bias(p(X), (0, 2, 4), p(W), (4, 3), p(B), p(Y), (0, 2, 3)), [Y])
    probe("attention", lambda: o.attention(p(X), p(W), p(Z), p(Y), 0, 4, 4, 1, 32, 1.0), [Y])
    probe("flatten", lambda: o.flatten(p(X), (0, 2, 2), p(Y), (0, 4), 1), [Y])
    probe("reshape", lambda: o.reshape(p(X), (0, 4), p(Y)), [Y])
    probe("squeeze", lambda: o.squeeze(p(X), (0, 1, 4), p(Y), (0, 4)), [Y])
    probe("unsqueeze", lambda: o.unsqueeze(p(X), (0, 4), p(Y), (0, 1, 4)), [Y])
    probe("expand", lambda: o.expand(p(X), (0, 1), p(Y), (0, 4), _abi.F32), [Y])
    probe("nonzero", lambda: o.nonzero(p(X), (0, 4), p(Y), (0,), _abi.F32), [Y])
    probe("concat", lambda: o.concat([p(X), p(W)], [(0, 2), (0, 3)], p(Y), (0, 5), 1), [Y])
    probe("transpose", lambda: o.transpose(p(X), (0, 4), p(Y), (1, 0)), [Y])
    probe("gather", lambda: o.gather(p(X), (4, 0), p(Y), (2, 0), p(idx()), (2,), 0), [Y])
    # the handle is still good: a real call after all of the above
    a = np.arange(6, dtype=f32).reshape(2, 3)
    assert np.array_equal(tensor_op(be, _abi.OP_ADD, a, a), a + a)
    return out
