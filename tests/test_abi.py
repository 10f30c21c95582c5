"""The C-ABI boundary: every function include/dnnrt.h declares is exported by
the gfx950 library and by the oracle build, and the Python binding restates
exactly that set.  No compute call is made here (no GPU needed)."""
import ctypes as C
import os
import re

from helpers import ORACLE_PATH, ROOT
from occamy_amd import _abi, compiler


def declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(dnn(?:rt|c)[A-Z]\w*)\s*\(", text))


def test_header_matches_binding():
    assert declared("dnnrt.h") == set(_abi.SIGNATURES)


def test_gpu_library_exports_every_symbol():
    lib = C.CDLL(_abi.RUNTIME_PATH)  # loads without a GPU: nothing is initialised until dnnrtCreate
    for name in declared("dnnrt.h"):
        assert hasattr(lib, name), name
    _abi.bind(lib)
    assert lib.dnnrtIsHostBackend() == 0


def test_oracle_exports_every_symbol():
    lib = _abi.bind(C.CDLL(ORACLE_PATH))
    assert lib.dnnrtIsHostBackend() == 1


def test_compiler_library_exports_every_symbol():
    lib = C.CDLL(compiler.DNNC_PATH)
    for name in declared("dnnc.h"):
        assert hasattr(lib, name), name


def test_missing_library_is_loud(monkeypatch):
    monkeypatch.setattr(_abi, "_runtime", None)
    monkeypatch.setattr(_abi, "RUNTIME_PATH", "/nonexistent/libdnnrt.so")
    try:
        _abi.load_runtime()
    except RuntimeError as e:
        assert "not built" in str(e)
    else:
        raise AssertionError("a missing HIP library must raise")
