"""The drop-in boundary against the reference's own table.

Where the reference is mounted (this container; never the GPU box), parse
``src/Conversion/DNNToLLVM/DNNAPISpecs.inc`` and apply the row transformations a
maintainer is told to make (rename; handle first; dtype last; ``group`` on the
fused convolution; the handful of rows whose operand list changes): the result
must be exactly the prototype ``include/dnnrt.h`` / ``_abi.SIGNATURES`` declare.
A row added to the reference's table, or an operand reordered here, fails."""
import ctypes as C
import os
import re

import pytest

from occamy_amd import _abi

SPECS = "/root/reference/src/Conversion/DNNToLLVM/DNNAPISpecs.inc"
pytestmark = pytest.mark.skipif(not os.path.exists(SPECS), reason="the reference is not mounted here")

H, D = "handle", "dtype"


def kind(ty):
    """An LLVM type of the table, or a ctypes type of the binding, as one of p / i64 / i32 / f32."""
    if isinstance(ty, str):
        return {"int64Ty": "i64", "int32Ty": "i32", "floatTy": "f32"}.get(ty, "p" if "Ptr" in ty else None)
    if ty in (C.c_int64,):
        return "i64"
    if ty in (C.c_int32,):
        return "i32"
    if ty in (C.c_float,):
        return "f32"
    return "p"


def reference_rows():
    text = open(SPECS).read()
    rows = {}
    for _, name, ret, ops in re.findall(r'DNNRuntimeAPI\(API::(\w+),\s*"(\w+)",\s*(\w+),\s*\{([^}]*)\}\)', text, flags=re.S):
        kinds = [kind(o.strip()) for o in ops.replace("\n", " ").split(",") if o.strip()]
        assert None not in kinds, (name, ops)
        rows[name] = (kind(ret), kinds)
    return rows


# reference symbol -> (symbol here, transformation of the operand kinds)
def same(k):
    return k


def handle_first_dtype_last(k):  # the CUDA / cuBLAS rows: they take no handle in the reference
    return ["p"] + k + ["i32"]


def dtype_last(k):  # the cuDNN-backed rows: the handle is already first
    return k + ["i32"]


def fused_conv(k):  # + group after algo (the reference drops it), + dtype
    return k[:10] + ["i64"] + k[10:] + ["i32"]


def prelu(k):  # (X, Y, dimX, slope, rank): + the slope's dims after the slope
    return ["p"] + k[:4] + ["p"] + k[4:] + ["i32"]


def shape_triplets(k):  # squeeze / unsqueeze / expand / nonzero: (X, dimX, rankX, Y, dimY, rankY)
    return ["p", "p", "p", "i64", "p", "p", "i64", "i32"]


MAP = {
    "cudnnCreate": ("dnnrtCreate", same), "cudnnDestroy": ("dnnrtDestroy", same),
    "cudaStreamCreate": ("dnnrtStreamCreate", same), "cudaStreamDestroy": ("dnnrtStreamDestroy", same),
    "wrapDNNDealloc": ("dnnrtDealloc", same), "wrapDNNMalloc": ("dnnrtMalloc", same), "wrapDNNMemcpy": ("dnnrtMemcpy", same),
    "wrapDNNMemOffset": ("dnnrtMemOffset", same), "wrapDNNMemPoolInit": ("dnnrtMemPoolInit", same),
    "DNNConvFunc": ("dnnrtConv", dtype_last), "DNNConvBiasActivFunc": ("dnnrtConvBiasActiv", fused_conv),
    "DNNActiveFunc": ("dnnrtActive", dtype_last), "DNNTensorOpFunc": ("dnnrtTensorOp", dtype_last),
    "DNNReduceFunc": ("dnnrtReduce", dtype_last), "DNNMaxPoolFunc": ("dnnrtMaxPool", dtype_last),
    "DNNAveragePoolFunc": ("dnnrtAveragePool", dtype_last),
    "CUBLASMatmul2dFunc": ("dnnrtMatmul2d", handle_first_dtype_last), "CUDAMatmulNdFunc": ("dnnrtMatmulNd", handle_first_dtype_last),
    "CUDASoftmaxFunc": ("dnnrtSoftmax", handle_first_dtype_last), "CUDAClipFunc": ("dnnrtClip", handle_first_dtype_last),
    "CUDAErfFunc": ("dnnrtErf", handle_first_dtype_last), "CUDANegativeFunc": ("dnnrtNegative", handle_first_dtype_last),
    "CUDAReciprocalFunc": ("dnnrtReciprocal", handle_first_dtype_last), "CUDAPowFunc": ("dnnrtPow", handle_first_dtype_last),
    "CUDACastI64toFloatFunc": ("dnnrtCastI64toFloat", handle_first_dtype_last),
    "CUDAFlattenFunc": ("dnnrtFlatten", handle_first_dtype_last), "CUDAReshapeFunc": ("dnnrtReshape", handle_first_dtype_last),
    "CUDAGatherFloatFunc": ("dnnrtGather", handle_first_dtype_last), "CUDAGatherInt64Func": ("dnnrtGather", handle_first_dtype_last),
    "CUDALeakyReluFunc": ("dnnrtLeakyRelu", handle_first_dtype_last), "CUDAPReluFunc": ("dnnrtPRelu", prelu),
    "CUDAConcatFloatFunc": ("dnnrtConcat", handle_first_dtype_last), "CUDAConcatInt64Func": ("dnnrtConcat", handle_first_dtype_last),
    "CUDASqueezeFloatFunc": ("dnnrtSqueeze", shape_triplets), "CUDASqueezeInt64Func": ("dnnrtSqueeze", shape_triplets),
    "CUDAUnsqueezeFloatFunc": ("dnnrtUnsqueeze", shape_triplets), "CUDAUnsqueezeInt64Func": ("dnnrtUnsqueeze", shape_triplets),
    "CUDAExpandInt64Func": ("dnnrtExpand", shape_triplets),
    "CUDANonZeroFloatFunc": ("dnnrtNonZero", shape_triplets), "CUDANonZeroInt64Func": ("dnnrtNonZero", shape_triplets),
}
for rank in (2, 3, 4, 6):
    for ty in ("Float", "Int64"):
        MAP[f"CUDATranspose{rank}D{ty}Func"] = ("dnnrtTranspose", handle_first_dtype_last)

# entry points with no row in the reference's table (include/dnnrt.h says "New" on each)
NEW = {"dnnrtLastError", "dnnrtIsHostBackend", "dnnrtDeviceMemoryStats", "dnnrtSetStream", "dnnrtSetTensorFormat", "dnnrtSetFilterLayout",
       "dnnrtSetActivationCoef", "dnnrtListConvTiles", "dnnrtSetConvTile", "dnnrtSync", "dnnrtGraphBegin", "dnnrtGraphEnd",
       "dnnrtGraphLaunch", "dnnrtGraphDestroy", "dnnrtEventCreate", "dnnrtEventRecord", "dnnrtEventElapsedMs",
       "dnnrtEventDestroy", "dnnrtHostAlloc", "dnnrtHostFree", "dnnrtMemFill", "dnnrtConvBiasAddActiv", "dnnrtConvBiasActivNoAlloc", "dnnrtConvBiasActivMaxPool", "dnnrtConvBiasAddConvBiasActiv",
       "dnnrtGelu", "dnnrtLayerNorm", "dnnrtMatmulNdBias", "dnnrtAttention", "dnnrtSqrt", "dnnrtSigmoid", "dnnrtTanh"}


def test_every_reference_row_has_its_counterpart_with_the_documented_operands():
    rows = reference_rows()
    assert len(rows) >= 48
    missing = sorted(set(rows) - set(MAP))
    assert not missing, f"rows of the reference's table with no counterpart here: {missing}"
    for ref_name, (ret, kinds) in rows.items():
        ours, change = MAP[ref_name]
        assert ours in _abi.SIGNATURES, ours
        res, args = _abi.SIGNATURES[ours]
        assert [kind(a) for a in args] == change(list(kinds)), f"{ref_name} -> {ours}"
        assert kind(res) == ret, f"{ref_name} -> {ours}: result"


def test_everything_else_is_declared_new():
    from_table = {ours for ours, _ in MAP.values()}
    extra = set(_abi.SIGNATURES) - from_table
    undeclared = sorted(n for n in extra if n not in NEW and not n.startswith("dnnrtOracle"))
    assert not undeclared, f"entry points that neither replace a row of the reference nor are listed as new: {undeclared}"


def test_retargeted_table_declares_the_prototypes_of_the_header():
    """occamy_amd/integration/retarget.py rewrites the reference's table from the checkout's own text; what it
    writes must name, row by row, an entry point of include/dnnrt.h with exactly its operand kinds, and the
    other three edits must apply to the mounted sources."""
    from occamy_amd.integration import retarget
    new_table = retarget.retarget_table(open(SPECS).read())
    rows = re.findall(r'DNNRuntimeAPI\(API::(\w+),\s*"(\w+)",\s*(\w+),\s*\{([^}]*)\}\)', new_table, flags=re.S)
    assert len(rows) == len(reference_rows()) + 2  # + dnnrtSetStream, dnnrtSync
    for _, name, ret, ops in rows:
        assert name in _abi.SIGNATURES, name
        res, args = _abi.SIGNATURES[name]
        kinds = [kind(o.strip()) for o in ops.replace("\n", " ").split(",") if o.strip()]
        assert kinds == [kind(a) for a in args], name
        assert kind(ret) == kind(res), name
    root = SPECS[:SPECS.index("/src/")]
    edits = {rel: (old, new) for rel, old, new in retarget.all_edits(root)}
    for rel in (retarget.DIALECT, retarget.FUSION, retarget.FUSED_LOWERING):
        old, new = edits[rel]
        assert new != old and "group" in new.lower(), rel


def test_every_retargeted_call_site_passes_what_its_row_declares():
    """The script rewrites every callApi site under src/Conversion/DNNToLLVM (Ops/** and the handle / stream set-up
    of DNNToLLVMCommon.cpp) from the checkout's own text.  On the mounted sources: every site names an API
    enumerator with a row in the rewritten table and passes exactly as many operands as that row declares; the
    handle is the first operand and the element type the last one wherever the header has them; dnnrtSetStream is
    called after the two creates and dnnrtSync in front of dnnrtDestroy."""
    from occamy_amd.integration import retarget
    root = SPECS[:SPECS.index("/src/")]
    edits = {rel: new for rel, _, new in retarget.all_edits(root)}
    table = edits[retarget.SPECS]
    rows = {api: (name, [o.strip() for o in ops.replace("\n", " ").split(",") if o.strip()])
            for api, name, _, ops in re.findall(r'DNNRuntimeAPI\(API::(\w+),\s*"(\w+)",\s*(\w+),\s*\{([^}]*)\}\)', table, flags=re.S)}
    enum = edits[retarget.API_HPP]
    assert "SET_STREAM," in enum and "SYNC," in enum
    sites = 0
    for rel in retarget.ops_files(root):
        text = edits.get(rel) or open(os.path.join(root, rel)).read()
        for api, _, _, ops in retarget.call_sites(text):
            name, declared = rows[api]
            assert len(ops) == len(declared), (rel, api, ops, declared)
            assert name in _abi.SIGNATURES
            if declared[0] == "handlePtrTy" and name not in ("dnnrtCreate", "dnnrtDestroy"):
                assert ops[0] in ("handleLoad", retarget.HANDLE_X), (rel, ops[0])
            if _abi.SIGNATURES[name][0] is C.c_void_p and name not in ("dnnrtMalloc",):   # a compute entry point: dtype last
                assert ops[-1] in (retarget.DTYPE_X, "dtypeConst"), (rel, api, ops[-1])
            sites += 1
    assert sites >= 46
    common = edits[retarget.COMMON_CPP]
    gen = common[common.index("void generateDNNHandle("):]
    assert gen.index("API::SYNC") < gen.index("API::CUDNN_DESTROY")
    assert gen.index("handleSync.getDefiningOp()->moveBefore") < gen.index("handleDestroy.getDefiningOp()->moveBefore")
    assert "dnnrtHandleSlot = handleAlloca;" in gen
    stream = common[common.index("void generateCUDAStream("):]
    assert stream.index("API::STREAM_CREATE") < stream.index("API::SET_STREAM") < stream.index("API::STREAM_DESTROY")
    for fn in ("dnnrtHandle", "dnnrtElementType", "dnnrtRank", "dnnrtDims"):
        assert f"mlir::Value {fn}(" in common and f"mlir::Value {fn}(" in edits[retarget.COMMON_HPP]
    # the set-up's own calls also match their rows
    for api, want in (("SET_STREAM", 2), ("SYNC", 1)):
        m = re.search(r"API::" + api + r",\s*\{([^}]*)\}", common)
        assert m and len(retarget.split_operands(m.group(1))) == want == len(rows[api][1])
