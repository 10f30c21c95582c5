"""Python mirror of the runtime's operator interface.

One method per entry point of ``include/dnnrt.h`` with the reference
wrapper's argument meaning (src/Tools/dnn-wrapper/** in the reference tree):
tensors are raw device addresses (ints), shapes are Python sequences.  Every
method raises ``RuntimeError`` with the library's error text when a call
fails, instead of the reference's printf + exit(-1).
"""
import ctypes as C

from . import _abi
from ._abi import dims


class Ops:
    def __init__(self, cdll=None):
        # cdll is the already-bound runtime library; the default (and the only
        # one the package itself ever passes) is the gfx950 library.
        self.lib = cdll if cdll is not None else _abi.load_runtime()
        h = C.c_void_p()
        self._check(self.lib.dnnrtCreate(C.byref(h)), "dnnrtCreate")
        self.handle = h
        self.stream = None

    def close(self):
        if self.handle is not None:
            self.lib.dnnrtDestroy(self.handle)
            self.handle = None

    # -- helpers ---------------------------------------------------------
    def _err(self):
        return self.lib.dnnrtLastError().decode()

    def _check(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} failed ({rc}): {self._err()}")

    def _ret(self, p, what):
        if not p:
            raise RuntimeError(f"{what}: {self._err()}")
        return p

    # -- handle state ------------------------------------------------------
    def set_stream(self, stream):
        self._check(self.lib.dnnrtSetStream(self.handle, stream), "dnnrtSetStream")
        self.stream = stream

    def set_format(self, fmt):
        self._check(self.lib.dnnrtSetTensorFormat(self.handle, fmt), "dnnrtSetTensorFormat")

    def set_activation_coef(self, coef):
        """Ceiling of ACT_CLIPPED_RELU / slope of ACT_LEAKY_RELU for the calls that follow."""
        self._check(self.lib.dnnrtSetActivationCoef(self.handle, coef), "dnnrtSetActivationCoef")

    def set_filter_layout(self, layout):
        self._check(self.lib.dnnrtSetFilterLayout(self.handle, layout), "dnnrtSetFilterLayout")

    def conv_tiles(self):
        """Ids of the fp16 channels-last convolution variants in the library."""
        n = self.lib.dnnrtListConvTiles(None, 0)
        ids = (C.c_int32 * max(n, 1))()
        self.lib.dnnrtListConvTiles(ids, n)
        return list(ids[:n])

    def set_conv_tile(self, tile):
        """Force one fp16 convolution variant for the calls that follow (0: automatic)."""
        self._check(self.lib.dnnrtSetConvTile(self.handle, tile), "dnnrtSetConvTile")

    def sync(self):
        self._check(self.lib.dnnrtSync(self.handle), "dnnrtSync")

    # -- memory --------------------------------------------------------------
    def mempool_init(self, nbytes):
        p = C.c_void_p()
        self._check(self.lib.dnnrtMemPoolInit(C.byref(p), nbytes), "dnnrtMemPoolInit")
        return p.value

    def mem_offset(self, base, offset, nbytes):
        p = C.c_void_p()
        self._check(self.lib.dnnrtMemOffset(C.byref(p), base, offset, nbytes), "dnnrtMemOffset")
        return p.value

    def memcpy(self, dst, src, nbytes, kind, stream=None):
        self._check(self.lib.dnnrtMemcpy(dst, src, nbytes, kind, stream), "dnnrtMemcpy")

    def malloc(self, nbytes):
        p = C.c_void_p()
        self._check(self.lib.dnnrtMalloc(C.byref(p), nbytes), "dnnrtMalloc")
        return p.value

    def dealloc(self, p):
        self._check(self.lib.dnnrtDealloc(p), "dnnrtDealloc")

    # -- compute ---------------------------------------------------------------
    def conv(self, X, dimX, W, dimW, pads, strides, Y, group=1, dtype=_abi.F32, algo=0):
        return self._ret(self.lib.dnnrtConv(self.handle, X, dims(dimX), W, dims(dimW), None, 0, algo,
                                            group, dims(pads), dims(strides), Y, dtype), "dnnrtConv")

    def conv_bias_activ(self, X, dimX, W, dimW, B, pads, strides, activ, Y, group=1, dtype=_abi.F32, algo=1):
        dimB = [1, dimW[0], 1, 1]
        return self._ret(self.lib.dnnrtConvBiasActiv(self.handle, X, dims(dimX), W, dims(dimW), B,
                                                     dims(dimB), None, 0, algo, group, dims(pads),
                                                     dims(strides), activ, Y, dtype),
                         "dnnrtConvBiasActiv")

    def conv_bias_activ_no_alloc(self, stream, X, dimX, W, dimW, B, pads, strides, activ, Y, group=1, dtype=_abi.F32):
        """dnnrtConvBiasActivNoAlloc: takes a stream (may be None: the default stream), not this object's handle."""
        dimB = [1, dimW[0], 1, 1]
        return self._ret(self.lib.dnnrtConvBiasActivNoAlloc(stream, X, dims(dimX), W, dims(dimW), B, dims(dimB), group,
                                                            dims(pads), dims(strides), activ, Y, dtype),
                         "dnnrtConvBiasActivNoAlloc")

    def conv_bias_add_activ(self, X, dimX, W, dimW, B, Z, pads, strides, activ, Y, group=1, dtype=_abi.F32, algo=1):
        dimB = [1, dimW[0], 1, 1]
        return self._ret(self.lib.dnnrtConvBiasAddActiv(self.handle, X, dims(dimX), W, dims(dimW), B,
                                                        dims(dimB), Z, None, 0, algo, group, dims(pads),
                                                        dims(strides), activ, Y, dtype),
                         "dnnrtConvBiasAddActiv")

    def conv_bias_activ_max_pool(self, X, dimX, W, dimW, B, pads, strides, activ, kernel, pool_pads, pool_strides, Y, dimY,
                                 group=1, dtype=_abi.F16):
        dimB = [1, dimW[0], 1, 1]
        return self._ret(self.lib.dnnrtConvBiasActivMaxPool(self.handle, X, dims(dimX), W, dims(dimW), B, dims(dimB), group,
                                                            dims(pads), dims(strides), activ, dims(kernel), dims(pool_pads),
                                                            dims(pool_strides), Y, dims(dimY), dtype),
                         "dnnrtConvBiasActivMaxPool")

    def conv_bias_add_conv_bias_activ(self, X, dimX, W, dimW, B, pads, strides, X2, dimX2, W2, dimW2, B2, pads2, strides2, activ, Y,
                                      dtype=_abi.F16, algo=0, algo2=0):
        return self._ret(self.lib.dnnrtConvBiasAddConvBiasActiv(self.handle, X, dims(dimX), W, dims(dimW), B, dims(pads), dims(strides),
                                                                X2, dims(dimX2), W2, dims(dimW2), B2, dims(pads2), dims(strides2),
                                                                activ, algo, algo2, Y, dtype),
                         "dnnrtConvBiasAddConvBiasActiv")

    def active(self, X, dimX, mode, Y, dtype=_abi.F32):
        d = list(dimX) + [1] * (4 - len(dimX))
        return self._ret(self.lib.dnnrtActive(self.handle, X, dims(d), mode, Y, dtype), "dnnrtActive")

    def tensor_op(self, op, A, dimA, B, dimB, O, coef=1.0, dtype=_abi.F32):
        r = len(dimA)
        return self._ret(self.lib.dnnrtTensorOp(self.handle, op, A, dims(dimA), r, B, dims(dimB), r, O,
                                                dims(dimA), r, coef, dtype), "dnnrtTensorOp")

    def clip(self, X, Y, dimY, lo, hi, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtClip(self.handle, X, Y, dims(dimY), lo, hi, len(dimY), dtype),
                         "dnnrtClip")

    def leaky_relu(self, X, Y, dimY, alpha, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtLeakyRelu(self.handle, X, Y, dims(dimY), alpha, len(dimY), dtype),
                         "dnnrtLeakyRelu")

    def prelu(self, X, Y, dimY, slope, dimSlope, dtype=_abi.F32):
        """dimSlope is right-aligned to dimY here (ONNX's unidirectional broadcast)."""
        ds = [1] * (len(dimY) - len(dimSlope)) + list(dimSlope)
        return self._ret(self.lib.dnnrtPRelu(self.handle, X, Y, dims(dimY), slope, dims(ds), len(dimY), dtype),
                         "dnnrtPRelu")

    def _unary(self, name, X, Y, dim, dtype):
        fn = getattr(self.lib, name)
        return self._ret(fn(self.handle, X, Y, dims(dim), len(dim), dtype), name)

    def erf(self, X, Y, dim, dtype=_abi.F32):
        return self._unary("dnnrtErf", X, Y, dim, dtype)

    def negative(self, X, Y, dim, dtype=_abi.F32):
        return self._unary("dnnrtNegative", X, Y, dim, dtype)

    def reciprocal(self, X, Y, dim, dtype=_abi.F32):
        return self._unary("dnnrtReciprocal", X, Y, dim, dtype)

    def gelu(self, X, Y, dim, dtype=_abi.F32):
        return self._unary("dnnrtGelu", X, Y, dim, dtype)

    def pow(self, X, E, Y, dimY, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtPow(self.handle, X, E, Y, dims(dimY), len(dimY), dtype), "dnnrtPow")

    def cast_i64_to_float(self, X, Y, dimY, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtCastI64toFloat(self.handle, X, Y, dims(dimY), len(dimY), dtype),
                         "dnnrtCastI64toFloat")

    def reduce_mean(self, X, dimX, Y, dimY, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtReduce(self.handle, len(dimX), X, dims(dimX), Y, dims(dimY),
                                              _abi.REDUCE_AVG, dtype), "dnnrtReduce")

    def softmax(self, X, dimX, Y, axis, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtSoftmax(self.handle, X, dims(dimX), Y, dims(dimX), axis,
                                               len(dimX), dtype), "dnnrtSoftmax")

    def layernorm(self, X, dimX, gamma, beta, eps, Y, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtLayerNorm(self.handle, X, dims(dimX), len(dimX), gamma, beta,
                                                 eps, Y, dtype), "dnnrtLayerNorm")

    def maxpool(self, X, dimX, Y, dimY, kernel, pads, strides, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtMaxPool(self.handle, X, dims(dimX), Y, dims(dimY), dims(kernel),
                                               dims(pads), dims(strides), dtype), "dnnrtMaxPool")

    def avgpool(self, X, dimX, Y, dimY, kernel, pads, strides, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtAveragePool(self.handle, X, dims(dimX), Y, dims(dimY),
                                                   dims(kernel), dims(pads), dims(strides), dtype),
                         "dnnrtAveragePool")

    def matmul2d(self, A, dimA, B, dimB, Out, dimOut, alpha=1.0, beta=0.0, transA=0, transB=0, C_=None,
                 dtype=_abi.F32, dimC=None):
        """dimC: [M, N] (default) or [1, N] for one row added to every row of the product."""
        return self._ret(self.lib.dnnrtMatmul2d(self.handle, 2, A, dims(dimA), B, dims(dimB), C_,
                                                dims(dimC if dimC is not None else dimOut), Out, dims(dimOut), alpha,
                                                beta, transA, transB, dtype), "dnnrtMatmul2d")

    def matmul_nd(self, A, dimA, B, dimB, Y, dimY, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtMatmulNd(self.handle, A, dims(dimA), len(dimA), B, dims(dimB),
                                                len(dimB), Y, dims(dimY), len(dimY), dtype),
                         "dnnrtMatmulNd")

    def matmul_nd_bias(self, A, dimA, B, dimB, bias, Y, dimY, dtype=_abi.F32, Z=None, gelu=False):
        """Y = act((A B + bias) + Z); Z: optional residual shaped like Y; act: Gelu or identity."""
        return self._ret(self.lib.dnnrtMatmulNdBias(self.handle, A, dims(dimA), len(dimA), B, dims(dimB),
                                                    len(dimB), bias, Z, int(gelu), Y, dims(dimY), len(dimY), dtype),
                         "dnnrtMatmulNdBias")

    def attention(self, Q, K, V, Y, batch, seq_q, seq_k, heads, head_dim, scale, dtype=_abi.F32, ld_in=0):
        """Q [batch, seq_q, heads*head_dim], K and V [batch, seq_k, heads*head_dim], Y like Q;
        ld_in: row stride of Q, K, V in elements when they are slices of a wider tensor."""
        return self._ret(self.lib.dnnrtAttention(self.handle, Q, K, V, Y, batch, seq_q, seq_k, heads, head_dim,
                                                 ld_in, scale, dtype), "dnnrtAttention")

    def flatten(self, X, dimX, Y, dimY, axis, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtFlatten(self.handle, X, dims(dimX), Y, dims(dimY), axis,
                                               len(dimX), dtype), "dnnrtFlatten")

    def reshape(self, X, dimX, Y, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtReshape(self.handle, X, dims(dimX), len(dimX), Y, dtype),
                         "dnnrtReshape")

    def squeeze(self, X, dimX, Y, dimY, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtSqueeze(self.handle, X, dims(dimX), len(dimX), Y, dims(dimY), len(dimY),
                                               dtype), "dnnrtSqueeze")

    def unsqueeze(self, X, dimX, Y, dimY, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtUnsqueeze(self.handle, X, dims(dimX), len(dimX), Y, dims(dimY), len(dimY),
                                                 dtype), "dnnrtUnsqueeze")

    def expand(self, X, dimX, Y, dimY, dtype=_abi.I64):
        return self._ret(self.lib.dnnrtExpand(self.handle, X, dims(dimX), len(dimX), Y, dims(dimY), len(dimY),
                                              dtype), "dnnrtExpand")

    def nonzero(self, X, dimX, Y, dimY, dtype=_abi.F32):
        """Flat indices of the non-zero elements, in X's element type, at the front of Y."""
        return self._ret(self.lib.dnnrtNonZero(self.handle, X, dims(dimX), len(dimX), Y, dims(dimY), len(dimY),
                                               dtype), "dnnrtNonZero")

    def concat(self, Xs, dimXs, Y, dimY, axis, dtype=_abi.F32):
        """Xs: device pointers (ints), dimXs: one dim list per input."""
        n = len(Xs)
        ptrs = (C.c_void_p * n)(*Xs)
        dim_arrays = [dims(d) for d in dimXs]  # kept alive until the call returns
        dim_ptrs = (C.c_void_p * n)(*[C.cast(a, C.c_void_p) for a in dim_arrays])
        return self._ret(self.lib.dnnrtConcat(self.handle, ptrs, dim_ptrs, Y, dims(dimY), axis, n, len(dimY),
                                              dtype), "dnnrtConcat")

    def transpose(self, X, dimX, Y, perm, dtype=_abi.F32):
        dimY = [dimX[p] for p in perm]
        return self._ret(self.lib.dnnrtTranspose(self.handle, X, dims(dimX), Y, dims(dimY), dims(perm),
                                                 len(dimX), dtype), "dnnrtTranspose")

    def gather(self, X, dimX, Y, dimY, idx, dimIdx, axis, dtype=_abi.F32):
        return self._ret(self.lib.dnnrtGather(self.handle, X, dims(dimX), len(dimX), Y, dims(dimY),
                                              len(dimY), idx, dims(dimIdx), len(dimIdx), axis, dtype),
                         "dnnrtGather")
