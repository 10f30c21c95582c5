"""dnnrtConvBiasActivNoAlloc, the entry point for callers that cannot allocate device memory: through the C ABI,
against dnnrtConvBiasActiv on a fresh handle (same kernels, same split: bit-identical) and against the CPU oracle
(rtol 1e-4 / atol 1e-5), on two calls in a row, the second on a smaller input.  Every GPU shares one static
scratch array between all calls, so the second call finds what the first left there."""
import numpy as np
import pytest

import opcases as oc
from helpers import GpuBackend, OracleBackend, rng
from occamy_amd import _abi

pytestmark = pytest.mark.gpu

# N, C, H, W, K, R, stride, pad: batch-1 layers whose reduction is split over workgroups (partial tiles and arrival
# counters in the scratch), larger first
CALLS = [
    (1, 512, 14, 14, 512, 3, 2, 1),
    (1, 2048, 7, 7, 512, 1, 1, 0),
    (1, 256, 7, 7, 64, 3, 1, 1),
]


def problem(case, seed):
    N, C, H, W, K, R, st, pd = case
    r = rng(seed)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = (r.standard_normal((K, C, R, R)) * np.sqrt(2.0 / (C * R * R))).astype(np.float32)
    b = r.uniform(-0.1, 0.1, K).astype(np.float32)
    return x, w, b, (pd, pd), (st, st)


def no_alloc_conv(gpu, x, w, b, pads, strides, activ):
    P, Q = oc.conv_out_hw(x.shape[2], x.shape[3], w.shape[2], w.shape[3], pads, strides)
    X, Wt, B = gpu.put(x), gpu.put(w), gpu.put(b)
    Y = gpu.empty((x.shape[0], w.shape[0], P, Q), np.float32)
    gpu.torch.cuda.synchronize()
    free_before = gpu.torch.cuda.mem_get_info()[0]
    gpu.ops.conv_bias_activ_no_alloc(None, gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), pads, strides, activ,
                                     gpu.ptr(Y), 1, _abi.F32)
    gpu.torch.cuda.synchronize()
    free_after = gpu.torch.cuda.mem_get_info()[0]
    return gpu.get(Y), free_before - free_after


def test_no_alloc_conv_twice_second_smaller():
    gpu, cpu = GpuBackend(), OracleBackend()
    for i, case in enumerate(CALLS):
        x, w, b, pads, strides = problem(case, 40 + i)
        got, taken = no_alloc_conv(gpu, x, w, b, pads, strides, _abi.ACT_RELU)
        same = oc.conv(gpu, x, w, b, pads, strides, 1, _abi.ACT_RELU)
        ref = oc.conv(cpu, x, w, b, pads, strides, 1, _abi.ACT_RELU)
        assert np.array_equal(got, same), f"call {i} {case}: differs from dnnrtConvBiasActiv"
        np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-5, err_msg=f"call {i} {case}")
        if i > 0:  # the first call may load the library's code object
            assert taken == 0, f"call {i} took {taken} bytes of device memory"


def test_no_alloc_conv_other_paths_and_errors():
    gpu, cpu = GpuBackend(), OracleBackend()
    # a layer that fills the chip without a split, identity activation; then what the call refuses
    x, w, b, pads, strides = problem((2, 64, 56, 56, 64, 3, 1, 1), 50)
    got, _ = no_alloc_conv(gpu, x, w, b, pads, strides, _abi.ACT_IDENTITY)
    np.testing.assert_allclose(got, oc.conv(cpu, x, w, b, pads, strides, 1, _abi.ACT_IDENTITY), rtol=1e-4, atol=1e-5)
    with pytest.raises(RuntimeError, match="activMode"):
        no_alloc_conv(gpu, x, w, b, pads, strides, 2)
    with pytest.raises(RuntimeError, match="group"):
        P, Q = oc.conv_out_hw(56, 56, 3, 3, pads, strides)
        X, Wt, B, Y = gpu.put(x), gpu.put(w), gpu.put(b), gpu.empty((2, 64, P, Q))
        gpu.ops.conv_bias_activ_no_alloc(None, gpu.ptr(X), x.shape, gpu.ptr(Wt), w.shape, gpu.ptr(B), pads, strides,
                                         _abi.ACT_RELU, gpu.ptr(Y), 3, _abi.F32)
