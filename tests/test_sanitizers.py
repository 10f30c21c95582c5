"""The host side (ONNX reader, pass pipeline, planner, executor) under AddressSanitizer and
UndefinedBehaviorSanitizer: `make asan` in occamy_amd/csrc builds those sources with a small driver into one
executable, which reads ONNX files and seeded mutations of them (truncations, changed, dropped and doubled bytes),
compiles what the reader accepts with the reference's flags and with every fusion, and runs small accepted
programs through the sanitizer build of the CPU oracle.  A refusal is fine; a sanitizer finding aborts the
process."""
import os
import shutil
import subprocess

import numpy as np
import pytest

import onnx_writer as ow
from occamy_amd import compiler, models

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "occamy_amd", "lib", "dnnc_sanitize")
ORACLE_ASAN = os.path.join(ROOT, "oracle", "libdnnrt_oracle_asan.so")


def _residual_block():
    r = np.random.default_rng(21)
    g = compiler.Graph()
    g.input("x", (1, 8, 10, 10))
    conv = lambda src, cin, cout, k: g.node("Conv", [src, g.constant((r.standard_normal((cout, cin, k, k)) * 0.2).astype(np.float32)),  # noqa: E731
                                                      g.constant(r.uniform(-0.1, 0.1, cout).astype(np.float32))],
                                            kernel_shape=[k, k], pads=[k // 2] * 4, strides=[1, 1], group=1)
    o = conv(g.node("Relu", [conv("x", 8, 4, 1)]), 4, 16, 3)
    y = g.node("Relu", [g.node("Add", [o, conv("x", 8, 16, 1)])])
    y = g.node("Flatten", [g.node("GlobalAveragePool", [y])], axis=1)
    w = g.constant((r.standard_normal((5, 16)) * 0.2).astype(np.float32))
    g.output(g.node("Gemm", [y, w, g.constant(np.zeros(5, np.float32))], alpha=1.0, beta=1.0, transB=1))
    return g


@pytest.fixture(scope="module")
def driver():
    if not shutil.which("g++") or not shutil.which("make"):
        pytest.skip("no host compiler")
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "occamy_amd", "csrc"), os.path.join("..", "lib", "dnnc_sanitize")],
                          stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "libdnnrt_oracle_asan.so"], stdout=subprocess.DEVNULL)
    return DRIVER


def test_reader_compiler_and_executor_on_mutated_onnx_files(driver, tmp_path):
    files = []
    builders = {"single_conv": lambda: models.single_conv()[0], "residual_block": _residual_block,
                "bert": lambda: models.bert_encoder(layers=1, hidden=32, heads=2, ffn=64, seq=8, vocab=50)[0]}
    for name, b in builders.items():
        g = b()
        for i, layout in enumerate((dict(), dict(typed_fields=True, packed=False), dict(constants_as_nodes=True))):
            if name == "single_conv" and i:
                continue
            path = tmp_path / f"{name}_{i}.onnx"
            path.write_bytes(ow.model_bytes(g, **layout))
            files.append(str(path))
            g = b()
    assert len(files) >= 4
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([driver, *files, "--mutations", "400", "--seed", "7", "--run", ORACLE_ASAN], capture_output=True, text=True,
                       env=env, timeout=600)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-6000:])
    assert "AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-6000:]
    assert int(r.stdout.split(",")[0].split()[-1]) == len(files) * 401, r.stdout
    # some mutations are still well-formed models and compile; most are refused
    accepted = int(r.stdout.split("accepted by the reader")[1].split(",")[0])
    ran = int(r.stdout.strip().split("ran")[-1])
    assert accepted >= len(files) and ran >= 2 * len(files), r.stdout
