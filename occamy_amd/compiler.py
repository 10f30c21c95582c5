"""Python front end of the DNN program compiler/executor (include/dnnc.h).

``Graph`` collects an ONNX-level graph (inputs, constants, nodes in ONNX
operator vocabulary), ``Graph.compile`` runs the reference's pass pipeline on
it (src/Compiler/CoreDNNPasses.cpp:24-28 and CoreDNNUtils.cpp:773-780: ONNX to
DNN, function arguments to device, dummy-constant removal, optional fusion,
dealloc placement, pool planning) and ``Program.session`` binds the result to
the gfx950 runtime.  The compile flags carry the reference's names and the
values its own tests use (test/models/simpleconv/run.py:50-54).
"""
import ctypes as C
import os

import numpy as np

from . import _abi

_HERE = os.path.dirname(os.path.abspath(__file__))
# DNNC_PATH in the environment names another build of the same library (the sanitizer build, `make asan`)
DNNC_PATH = os.environ.get("DNNC_PATH") or os.path.join(_HERE, "lib", "libdnnc.so")

F32, F16, I64 = 0, 1, 2
_NP = {F32: np.float32, F16: np.float16, I64: np.int64}
_DT = {np.dtype(np.float32): F32, np.dtype(np.float16): F16, np.dtype(np.int64): I64}
MODE_OCCAMY, MODE_RESIDENT = 0, 1


class _Options(C.Structure):
    _fields_ = [("const_at_use", C.c_int32), ("fusion", C.c_int32), ("dealloc_opt", C.c_int32),
                ("pool_opt", C.c_int32), ("channels_last", C.c_int32), ("fuse_residual", C.c_int32),
                ("fuse_activations", C.c_int32), ("recompose", C.c_int32), ("fuse_matmul_bias", C.c_int32),
                ("fuse_attention", C.c_int32), ("fuse_first_layer_maxpool", C.c_int32),
                ("fuse_projection_shortcut", C.c_int32), ("alias_copies", C.c_int32), ("inplace_residual", C.c_int32), ("compact_pool", C.c_int32)]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(DNNC_PATH):
        raise RuntimeError(f"{DNNC_PATH} is not built; run `make -C occamy_amd/csrc` first")
    L = C.CDLL(DNNC_PATH)
    P, I64P, I32P = C.c_void_p, C.POINTER(C.c_int64), C.POINTER(C.c_int32)
    sig = {
        "dnncLastError": (C.c_char_p, []),
        "dnncGraphCreate": (P, []),
        "dnncGraphDestroy": (None, [P]),
        "dnncGraphAddInput": (C.c_int32, [P, C.c_char_p, C.c_int32, C.c_int32, I64P]),
        "dnncGraphAddConstant": (C.c_int32, [P, C.c_char_p, C.c_int32, C.c_int32, I64P, P]),
        "dnncGraphAddNode": (C.c_int32, [P, C.c_char_p, C.c_int32, C.POINTER(C.c_char_p), C.c_char_p, C.c_char_p]),
        "dnncGraphAddOutput": (C.c_int32, [P, C.c_char_p]),
        "dnncGraphFromOnnx": (P, [C.c_char_p, C.c_int64]),
        "dnncGraphNumInputs": (C.c_int32, [P]),
        "dnncGraphNumOutputs": (C.c_int32, [P]),
        "dnncGraphInputName": (C.c_char_p, [P, C.c_int32]),
        "dnncGraphOutputName": (C.c_char_p, [P, C.c_int32]),
        "dnncGraphInputInfo": (C.c_int32, [P, C.c_int32, I32P, I32P, I64P, C.c_int32]),
        "dnncCompile": (P, [P, C.POINTER(_Options)]),
        "dnncProgramDestroy": (None, [P]),
        "dnncProgramText": (C.c_char_p, [P]),
        "dnncProgramPoolBytes": (C.c_int64, [P]),
        "dnncProgramPoolExtent": (C.c_int64, [P]),
        "dnncProgramEvents": (C.c_int64, [P, I32P, I64P, I64P, I64P, C.c_int64]),
        "dnncProgramNumInputs": (C.c_int32, [P]),
        "dnncProgramNumOutputs": (C.c_int32, [P]),
        "dnncProgramOutputInfo": (C.c_int32, [P, C.c_int32, I32P, I32P, I64P]),
        "dnncProgramNumOps": (C.c_int64, [P, C.c_int32]),
        "dnncProgramComputeOp": (C.c_int32, [P, C.c_int64, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p),
                                 C.POINTER(C.c_double), C.POINTER(C.c_double)]),
        "dnncSessionProfile": (C.c_int64, [P, C.POINTER(P), C.c_int32, C.POINTER(C.c_float), C.c_int64]),
        "dnncPlanPool": (C.c_int64, [C.c_int64, I32P, I64P, I64P, I64P]),
        "dnncPlanFreeList": (C.c_int64, [C.c_int64, I32P, I64P, I64P, C.c_int64, I64P, C.c_int64]),
        "dnncSessionCreate": (P, [P, C.c_char_p, C.c_int32]),
        "dnncSessionDestroy": (None, [P]),
        "dnncSessionRun": (C.c_int32, [P, C.POINTER(P), C.POINTER(P)]),
        "dnncSessionRunResident": (C.c_int32, [P, C.POINTER(P), C.POINTER(P), C.c_int32, C.c_int32]),
        "dnncSessionSync": (C.c_int32, [P]),
        "dnncSessionSetConvTile": (C.c_int32, [P, C.c_int32]),
        "dnncSessionTune": (C.c_int64, [P, C.POINTER(P), C.c_int32, C.c_int32]),
        "dnncSessionGetAlgos": (C.c_int64, [P, I64P, C.c_int64]),
        "dnncSessionSetAlgos": (C.c_int32, [P, I64P, C.c_int64]),
        "dnncSessionSetDebugFill": (C.c_int32, [P, C.c_int32]),
        "dnncSessionWeightsBytes": (C.c_int64, [P]),
        "dnncSessionLastPoolBytes": (C.c_int64, [P]),
        "dnncSessionDeviceBytes": (C.c_int32, [P, I64P, I64P, I64P, C.c_int32]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


def _err():
    return lib().dnncLastError().decode()


def plan_pool(events):
    """The planner alone.  events: (kind, id, bytes) with kind 0 = malloc, 1 = dealloc.
    Returns (offsets per event, pool bytes)."""
    n = len(events)
    kind = (C.c_int32 * max(n, 1))(*[e[0] for e in events])
    ids = (C.c_int64 * max(n, 1))(*[e[1] for e in events])
    byt = (C.c_int64 * max(n, 1))(*[e[2] for e in events])
    off = (C.c_int64 * max(n, 1))()
    peak = lib().dnncPlanPool(n, kind, ids, byt, off)
    if peak < 0:
        raise RuntimeError("planner: dealloc of a tensor that is not live")
    return list(off[:n]), peak


def plan_free_list(events, upto):
    n = len(events)
    kind = (C.c_int32 * max(n, 1))(*[e[0] for e in events])
    ids = (C.c_int64 * max(n, 1))(*[e[1] for e in events])
    byt = (C.c_int64 * max(n, 1))(*[e[2] for e in events])
    out = (C.c_int64 * 2048)()
    m = lib().dnncPlanFreeList(n, kind, ids, byt, upto, out, 1024)
    return [(out[2 * i], out[2 * i + 1]) for i in range(m)]


def load_onnx(source):
    """An ONNX model file (a path, or the file's bytes) as a Graph: what the
    reference is given on its command line (``core-dnn --EmitLib model.onnx``).
    The Python-side mirror holds the inputs and outputs only."""
    data = source if isinstance(source, (bytes, bytearray)) else open(source, "rb").read()
    h = lib().dnncGraphFromOnnx(bytes(data), len(data))
    if not h:
        raise RuntimeError(_err())
    g = Graph(_handle=h)
    for i in range(lib().dnncGraphNumInputs(h)):
        dt, rank, d = C.c_int32(), C.c_int32(), (C.c_int64 * 8)()
        if lib().dnncGraphInputInfo(h, i, C.byref(dt), C.byref(rank), d, 8):
            raise RuntimeError(_err())
        g.input_shapes[lib().dnncGraphInputName(h, i).decode()] = (tuple(d[:rank.value]), np.dtype(_NP[dt.value]))
    g.outputs = [lib().dnncGraphOutputName(h, i).decode() for i in range(lib().dnncGraphNumOutputs(h))]
    return g


class Graph:
    """An ONNX-level graph: named tensors, constants, nodes with ONNX operator names."""

    def __init__(self, _handle=None):
        self._g = _handle if _handle is not None else lib().dnncGraphCreate()
        self._n = 0
        # Python-side mirror of what was added, for inspection and for
        # evaluating the same graph with another engine
        self.input_shapes = {}
        self.constants = {}
        self.nodes = []
        self.outputs = []

    def __del__(self):
        if getattr(self, "_g", None) and lib is not None:  # module globals are gone at interpreter exit
            lib().dnncGraphDestroy(self._g)
            self._g = None

    def _name(self, prefix):
        self._n += 1
        return f"{prefix}_{self._n}"

    def input(self, name, shape, dtype=np.float32):
        d = _abi.dims(shape)
        if lib().dnncGraphAddInput(self._g, name.encode(), _DT[np.dtype(dtype)], len(shape), d):
            raise RuntimeError(_err())
        self.input_shapes[name] = (tuple(shape), np.dtype(dtype))
        return name

    def constant(self, array, name=None):
        a = np.ascontiguousarray(array)
        name = name or self._name("const")
        d = _abi.dims(a.shape)
        if lib().dnncGraphAddConstant(self._g, name.encode(), _DT[a.dtype], a.ndim, d, a.ctypes.data):
            raise RuntimeError(_err())
        self.constants[name] = a
        return name

    def node(self, op_type, inputs, name=None, **attrs):
        out = name or self._name(op_type.lower())
        arr = (C.c_char_p * max(len(inputs), 1))(*[(i or "").encode() for i in inputs])
        parts = []
        for k, v in attrs.items():
            if isinstance(v, float):
                parts.append(f"{k}={v!r}")  # repr of a float always has '.', 'e', 'inf' or 'nan'
            elif isinstance(v, (list, tuple)):
                parts.append(f"{k}=" + ",".join(str(int(x)) for x in v))
            else:
                parts.append(f"{k}={int(v)}")
        if lib().dnncGraphAddNode(self._g, op_type.encode(), len(inputs), arr, out.encode(), ";".join(parts).encode()):
            raise RuntimeError(_err())
        self.nodes.append((op_type, list(inputs), out, dict(attrs)))
        return out

    def output(self, name):
        if lib().dnncGraphAddOutput(self._g, name.encode()):
            raise RuntimeError(_err())
        self.outputs.append(name)

    def compile(self, fusion=False, dealloc_opt=True, pool_opt=True, const_at_use=True, channels_last=False,
                fuse_residual=False, fuse_activations=False, recompose=False, fuse_matmul_bias=False,
                fuse_attention=False, fuse_first_layer_maxpool=False, alias_copies=False, fuse_projection_shortcut=False,
                inplace_residual=False, compact_pool=False):
        opt = _Options(int(const_at_use), int(fusion), int(dealloc_opt), int(pool_opt), int(channels_last),
                       int(fuse_residual), int(fuse_activations), int(recompose), int(fuse_matmul_bias),
                       int(fuse_attention), int(fuse_first_layer_maxpool), int(fuse_projection_shortcut), int(alias_copies),
                       int(inplace_residual), int(compact_pool))
        p = lib().dnncCompile(self._g, C.byref(opt))
        if not p:
            raise RuntimeError("compile: " + _err())
        return Program(p, self)


class Program:
    def __init__(self, handle, graph):
        self._p = handle
        self._graph = graph  # owns the constants the program points at

    def __del__(self):
        if getattr(self, "_p", None) and lib is not None:
            lib().dnncProgramDestroy(self._p)
            self._p = None

    @property
    def text(self):
        return lib().dnncProgramText(self._p).decode()

    @property
    def pool_bytes(self):
        return lib().dnncProgramPoolBytes(self._p)

    @property
    def pool_extent(self):
        return lib().dnncProgramPoolExtent(self._p)

    def num_ops(self, compute_only=False):
        return lib().dnncProgramNumOps(self._p, int(compute_only))

    def compute_ops(self):
        """[(mnemonic, work class, algorithmic FLOPs, algorithmic bytes)] per compute op, program order."""
        out = []
        for i in range(self.num_ops(compute_only=True)):
            name, cls, fl, by = C.c_char_p(), C.c_char_p(), C.c_double(), C.c_double()
            if lib().dnncProgramComputeOp(self._p, i, C.byref(name), C.byref(cls), C.byref(fl), C.byref(by)):
                raise RuntimeError(_err())
            out.append((name.value.decode(), cls.value.decode(), fl.value, by.value))
        return out

    def events(self):
        """[(kind, id, bytes, offset)] in execution order."""
        n = lib().dnncProgramEvents(self._p, None, None, None, None, 0)
        kind = (C.c_int32 * max(n, 1))()
        ids, byt, off = (C.c_int64 * max(n, 1))(), (C.c_int64 * max(n, 1))(), (C.c_int64 * max(n, 1))()
        lib().dnncProgramEvents(self._p, kind, ids, byt, off, n)
        return [(kind[i], ids[i], byt[i], off[i]) for i in range(n)]

    def output_info(self):
        out = []
        for i in range(lib().dnncProgramNumOutputs(self._p)):
            dt, rank, d = C.c_int32(), C.c_int32(), (C.c_int64 * 8)()
            if lib().dnncProgramOutputInfo(self._p, i, C.byref(dt), C.byref(rank), d):
                raise RuntimeError(_err())
            out.append((tuple(d[:rank.value]), _NP[dt.value]))
        return out

    def session(self, mode=MODE_OCCAMY, runtime_library=None):
        """Bind to a runtime.  The default, and the only one this package ever
        chooses, is the gfx950 library; a missing build is an error."""
        if runtime_library is None:
            _abi.load_runtime()  # fail loudly when the HIP library is absent
            runtime_library = _abi.RUNTIME_PATH
        return Session(self, runtime_library, mode)


class Session:
    def __init__(self, program, runtime_library, mode):
        self.program = program
        self.mode = mode
        self._s = lib().dnncSessionCreate(program._p, runtime_library.encode(), mode)
        if not self._s:
            raise RuntimeError("session: " + _err())
        self._out_info = program.output_info()

    def close(self):
        if getattr(self, "_s", None) and lib is not None:
            lib().dnncSessionDestroy(self._s)
            self._s = None

    def __del__(self):
        self.close()

    def run(self, *inputs):
        """Host arrays in, host arrays out (the reference's ``sess.run``)."""
        ins = [np.ascontiguousarray(a) for a in inputs]
        outs = [np.empty(s, d) for s, d in self._out_info]
        ip = (C.c_void_p * max(len(ins), 1))(*[a.ctypes.data for a in ins])
        op = (C.c_void_p * max(len(outs), 1))(*[a.ctypes.data for a in outs])
        if lib().dnncSessionRun(self._s, ip, op):
            raise RuntimeError("run: " + _err())
        return outs

    def run_device(self, in_ptrs, out_ptrs, use_graph=True, in_place=False):
        """Resident mode: device addresses in and out; returns without waiting.  in_place: the kernels read the
        input buffers where they are (no copy into the pool) and the operations that produce the results write them
        into the result buffers (no copy out of the pool): the inputs must stay unchanged and the result buffers
        untouched until the run is over, and neither may overlap the other."""
        ip = (C.c_void_p * max(len(in_ptrs), 1))(*in_ptrs)
        op = (C.c_void_p * max(len(out_ptrs), 1))(*out_ptrs)
        if lib().dnncSessionRunResident(self._s, ip, op, 2 if in_place else 1, int(use_graph)):
            raise RuntimeError("run_device: " + _err())

    def profile(self, in_ptrs_or_arrays, on_device=False, by_class=False):
        """Resident mode: milliseconds per compute op (device timestamps), program order."""
        if on_device:
            ip = (C.c_void_p * max(len(in_ptrs_or_arrays), 1))(*in_ptrs_or_arrays)
        else:
            keep = [np.ascontiguousarray(a) for a in in_ptrs_or_arrays]
            ip = (C.c_void_p * max(len(keep), 1))(*[a.ctypes.data for a in keep])
        n = self.program.num_ops(compute_only=True)
        ms = (C.c_float * max(n, 1))()
        if lib().dnncSessionProfile(self._s, ip, int(on_device) | (2 if by_class else 0), ms, n) < 0:
            raise RuntimeError("profile: " + _err())
        return list(ms[:n])

    def set_debug_fill(self, byte):
        """Per-inference mode: fill the pool and every tensor's slot with `byte` before use (-1: off)."""
        if lib().dnncSessionSetDebugFill(self._s, byte):
            raise RuntimeError("set_debug_fill: " + _err())

    def set_conv_tile(self, tile):
        """Force one fp16 convolution variant (dnnrtListConvTiles) for every following run; 0 = automatic."""
        if lib().dnncSessionSetConvTile(self._s, tile):
            raise RuntimeError("set_conv_tile: " + _err())

    def tune(self, in_ptrs_or_arrays, on_device=False, reps=7):
        """Resident mode: time every convolution variant on every fp16 channels-last convolution of the program, in
        place, and keep the winners as the calls' `algo` operands; returns how many operations got a variant."""
        if on_device:
            ip = (C.c_void_p * max(len(in_ptrs_or_arrays), 1))(*in_ptrs_or_arrays)
        else:
            keep = [np.ascontiguousarray(a) for a in in_ptrs_or_arrays]
            ip = (C.c_void_p * max(len(keep), 1))(*[a.ctypes.data for a in keep])
        n = lib().dnncSessionTune(self._s, ip, int(on_device), reps)
        if n < 0:
            raise RuntimeError("tune: " + _err())
        return n

    def algos(self):
        """[(variant of the convolution, variant of a fused pair's second convolution)] per operation that launches;
        0 = the runtime's own choice."""
        n = lib().dnncSessionGetAlgos(self._s, None, 0)
        buf = (C.c_int64 * max(n, 1))()
        lib().dnncSessionGetAlgos(self._s, buf, n)
        return [(buf[i], buf[i + 1]) for i in range(0, n, 2)]

    def set_algos(self, pairs):
        flat = [int(v) for p in pairs for v in p]
        buf = (C.c_int64 * max(len(flat), 1))(*flat)
        if lib().dnncSessionSetAlgos(self._s, buf, len(flat)):
            raise RuntimeError("set_algos: " + _err())

    def sync(self):
        if lib().dnncSessionSync(self._s):
            raise RuntimeError("sync: " + _err())

    @property
    def weights_bytes(self):
        return lib().dnncSessionWeightsBytes(self._s)

    @property
    def last_pool_bytes(self):
        return lib().dnncSessionLastPoolBytes(self._s)

    def device_bytes(self, reset_peak=False):
        """(bytes the runtime library holds from the device allocator now, the peak of that sum, the size of the
        library's static device arrays); counted per process over every session bound to the same library."""
        now, peak, static = C.c_int64(), C.c_int64(), C.c_int64()
        if lib().dnncSessionDeviceBytes(self._s, C.byref(now), C.byref(peak), C.byref(static), int(reset_peak)):
            raise RuntimeError("device_bytes: " + _err())
        return now.value, peak.value, static.value
