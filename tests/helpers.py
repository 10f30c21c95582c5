"""Test-side plumbing: run the same operator call against the CPU oracle
(numpy buffers) and against the gfx950 library (torch CUDA buffers)."""
import ctypes as C
import os

import numpy as np

from occamy_amd import _abi
from occamy_amd.ops import Ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_PATH = os.path.join(ROOT, "oracle", "libdnnrt_oracle.so")
PLANNER_ORACLE_PATH = os.path.join(ROOT, "oracle", "libpool_planner_oracle.so")

_oracle = None


def oracle_lib():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_PATH):
            raise RuntimeError("oracle not built: run `make -C oracle`")
        _oracle = _abi.bind(C.CDLL(ORACLE_PATH))
    return _oracle


NP_DT = {_abi.F32: np.float32, _abi.F16: np.float16, _abi.I64: np.int64}


class OracleBackend:
    """Buffers are numpy arrays; pointers are their host addresses."""
    name = "oracle"

    def __init__(self):
        self.ops = Ops(oracle_lib())
        self._keep = []

    def put(self, a):
        a = np.array(a, copy=True, order="C")  # calls may write in place
        self._keep.append(a)
        return a

    def empty(self, shape, dtype=np.float32):
        a = np.full(shape, np.nan if np.issubdtype(dtype, np.floating) else -1, dtype=dtype)
        self._keep.append(a)
        return a

    def ptr(self, a):
        return a.ctypes.data

    def get(self, a):
        return np.array(a)

    def sync(self):
        pass


class GpuBackend:
    """Buffers are torch CUDA tensors; pointers are device addresses."""
    name = "gpu"

    def __init__(self):
        import torch
        self.torch = torch
        self.ops = Ops()
        self._keep = []

    def put(self, a):
        t = self.torch.from_numpy(np.ascontiguousarray(a)).cuda()
        self._keep.append(t)
        return t

    def empty(self, shape, dtype=np.float32):
        t = self.torch.from_numpy(
            np.full(shape, np.nan if np.issubdtype(dtype, np.floating) else -1, dtype=dtype)).cuda()
        self._keep.append(t)
        return t

    def ptr(self, t):
        return t.data_ptr()

    def get(self, t):
        self.torch.cuda.synchronize()
        return t.cpu().numpy()

    def sync(self):
        self.ops.sync()
        self.torch.cuda.synchronize()


def rng(seed):
    return np.random.default_rng(seed)
