"""ctypes binding of the runtime's C ABI (include/dnnrt.h).

``SIGNATURES`` restates every prototype of the header; ``bind`` applies it to
a loaded shared object and fails if a symbol is missing.  ``load_runtime``
loads the gfx950 library and nothing else.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
RUNTIME_PATH = os.path.join(_HERE, "lib", "libdnnrt.so")

P = C.c_void_p
I64P = C.POINTER(C.c_int64)
i64, i32, f32 = C.c_int64, C.c_int32, C.c_float

# name -> (restype, argtypes); order and types as in include/dnnrt.h
SIGNATURES = {
    "dnnrtCreate": (i32, [C.POINTER(P)]),
    "dnnrtDestroy": (i32, [P]),
    "dnnrtDeviceMemoryStats": (i32, [I64P, I64P, I64P, i32]),
    "dnnrtStreamCreate": (i32, [C.POINTER(P)]),
    "dnnrtStreamDestroy": (i32, [P]),
    "dnnrtSetStream": (i32, [P, P]),
    "dnnrtSetTensorFormat": (i32, [P, i32]),
    "dnnrtSetFilterLayout": (i32, [P, i32]),
    "dnnrtListConvTiles": (i32, [C.POINTER(i32), i32]),
    "dnnrtSetConvTile": (i32, [P, i32]),
    "dnnrtSetActivationCoef": (i32, [P, f32]),
    "dnnrtSync": (i32, [P]),
    "dnnrtGraphBegin": (i32, [P]),
    "dnnrtGraphEnd": (i32, [P, C.POINTER(P)]),
    "dnnrtGraphLaunch": (i32, [P, P]),
    "dnnrtGraphDestroy": (i32, [P]),
    "dnnrtEventCreate": (i32, [C.POINTER(P)]),
    "dnnrtEventRecord": (i32, [P, P]),
    "dnnrtEventElapsedMs": (i32, [P, P, C.POINTER(f32)]),
    "dnnrtEventDestroy": (i32, [P]),
    "dnnrtLastError": (C.c_char_p, []),
    "dnnrtIsHostBackend": (i32, []),
    "dnnrtMemPoolInit": (i32, [C.POINTER(P), i64]),
    "dnnrtMemOffset": (i32, [C.POINTER(P), P, i64, i64]),
    "dnnrtMemFill": (i32, [P, i32, i64, P]),
    "dnnrtMemcpy": (i32, [P, P, i64, i32, P]),
    "dnnrtMalloc": (i32, [C.POINTER(P), i64]),
    "dnnrtDealloc": (i32, [P]),
    "dnnrtHostAlloc": (i32, [C.POINTER(P), i64]),
    "dnnrtHostFree": (i32, [P]),
    "dnnrtConv": (P, [P, P, I64P, P, I64P, P, i64, i64, i64, I64P, I64P, P, i32]),
    "dnnrtConvBiasActiv": (P, [P, P, I64P, P, I64P, P, I64P, P, i64, i64, i64, I64P, I64P, i64, P, i32]),
    "dnnrtConvBiasAddActiv": (P, [P, P, I64P, P, I64P, P, I64P, P, P, i64, i64, i64, I64P, I64P, i64, P, i32]),
    "dnnrtConvBiasActivMaxPool": (P, [P, P, I64P, P, I64P, P, I64P, i64, I64P, I64P, i64, I64P, I64P, I64P, P, I64P, i32]),
    "dnnrtConvBiasAddConvBiasActiv": (P, [P, P, I64P, P, I64P, P, I64P, I64P, P, I64P, P, I64P, P, I64P, I64P, i64, i64, i64, P, i32]),
    "dnnrtConvBiasActivNoAlloc": (P, [P, P, I64P, P, I64P, P, I64P, i64, I64P, I64P, i64, P, i32]),
    "dnnrtActive": (P, [P, P, I64P, i32, P, i32]),
    "dnnrtTensorOp": (P, [P, i64, P, I64P, i32, P, I64P, i32, P, I64P, i32, f32, i32]),
    "dnnrtClip": (P, [P, P, P, I64P, f32, f32, i64, i32]),
    "dnnrtLeakyRelu": (P, [P, P, P, I64P, f32, i64, i32]),
    "dnnrtPRelu": (P, [P, P, P, I64P, P, I64P, i64, i32]),
    "dnnrtErf": (P, [P, P, P, I64P, i64, i32]),
    "dnnrtNegative": (P, [P, P, P, I64P, i64, i32]),
    "dnnrtReciprocal": (P, [P, P, P, I64P, i64, i32]),
    "dnnrtPow": (P, [P, P, P, P, I64P, i64, i32]),
    "dnnrtCastI64toFloat": (P, [P, P, P, I64P, i64, i32]),
    "dnnrtGelu": (P, [P, P, P, I64P, i64, i32]),
    "dnnrtReduce": (P, [P, i32, P, I64P, P, I64P, i32, i32]),
    "dnnrtSoftmax": (P, [P, P, I64P, P, I64P, i64, i64, i32]),
    "dnnrtLayerNorm": (P, [P, P, I64P, i64, P, P, f32, P, i32]),
    "dnnrtMaxPool": (P, [P, P, I64P, P, I64P, I64P, I64P, I64P, i32]),
    "dnnrtAveragePool": (P, [P, P, I64P, P, I64P, I64P, I64P, I64P, i32]),
    "dnnrtMatmul2d": (P, [P, i64, P, I64P, P, I64P, P, I64P, P, I64P, f32, f32, i64, i64, i32]),
    "dnnrtMatmulNd": (P, [P, P, I64P, i32, P, I64P, i32, P, I64P, i32, i32]),
    "dnnrtMatmulNdBias": (P, [P, P, I64P, i32, P, I64P, i32, P, P, i32, P, I64P, i32, i32]),
    "dnnrtAttention": (P, [P, P, P, P, P, i64, i64, i64, i64, i64, i64, f32, i32]),
    "dnnrtFlatten": (P, [P, P, I64P, P, I64P, i32, i64, i32]),
    "dnnrtReshape": (P, [P, P, I64P, i64, P, i32]),
    "dnnrtSqueeze": (P, [P, P, I64P, i64, P, I64P, i64, i32]),
    "dnnrtUnsqueeze": (P, [P, P, I64P, i64, P, I64P, i64, i32]),
    "dnnrtConcat": (P, [P, P, P, P, I64P, i64, i64, i32, i32]),
    "dnnrtExpand": (P, [P, P, I64P, i64, P, I64P, i64, i32]),
    "dnnrtNonZero": (P, [P, P, I64P, i64, P, I64P, i64, i32]),
    "dnnrtTranspose": (P, [P, P, I64P, P, I64P, I64P, i64, i32]),
    "dnnrtGather": (P, [P, P, I64P, i64, P, I64P, i64, P, I64P, i64, i64, i32]),
}

F32, F16, I64 = 0, 1, 2
NCHW, NHWC, NCHW_TO_NHWC = 0, 1, 2
FILTER_KCRS, FILTER_CRSK = 0, 1
ACT_SIGMOID, ACT_RELU, ACT_TANH, ACT_CLIPPED_RELU, ACT_IDENTITY, ACT_LEAKY_RELU = 0, 1, 2, 3, 5, 6
OP_ADD, OP_MUL, OP_SQRT = 0, 1, 4
REDUCE_AVG = 5
H2D, D2H, D2D = 1, 2, 3
CONV_ALGO_BASE = 1000


def bind(cdll):
    """Set restype/argtypes of every ABI symbol on ``cdll``; raise if one is missing."""
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(cdll, name)
        except AttributeError as e:
            raise RuntimeError(f"{cdll._name}: ABI symbol {name} is missing") from e
        fn.restype, fn.argtypes = res, args
    return cdll


_runtime = None


def load_runtime():
    """The gfx950 runtime library.  There is no fallback: a missing build is an error."""
    global _runtime
    if _runtime is None:
        if not os.path.exists(RUNTIME_PATH):
            raise RuntimeError(
                f"{RUNTIME_PATH} is not built; run `make -C occamy_amd/csrc` "
                "(or __graft_entry__.build()) first")
        _runtime = bind(C.CDLL(RUNTIME_PATH))
    return _runtime


def dims(seq):
    """A host int64 array as the ABI wants its dims/pads/strides arguments."""
    seq = [int(v) for v in seq]
    return (C.c_int64 * max(len(seq), 1))(*seq)
