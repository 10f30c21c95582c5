#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

A "step" is one inference of the workload with its input and all weights
already resident in HBM: input copy into its pool slot (device to device),
every kernel of the compiled DNN program (replayed from a captured graph),
output copy to the caller's device buffer.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

workloads: resnet50_fp32_bs1 (default), resnet50_fp16_bs64, mobilenet_v2_fp32_bs1,
bert_base_fp32_seq128, single_conv_fp32
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"mfma_f32": 157.3e12, "mfma_f16": 2.5e15, "hbm": 8.0e12}


def build_workload(name):
    from occamy_amd import models
    if name == "resnet50_fp32_bs1":
        return models.resnet50(1, np.float32), dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True), 1, "img/s", "f32"
    if name == "resnet50_fp16_bs64":
        return models.resnet50(64, np.float16, seed=5), dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, channels_last=True), 64, "img/s", "f16"
    if name == "mobilenet_v2_fp32_bs1":
        return models.mobilenet_v2(1, np.float32), dict(fusion=True, fuse_residual=True, fuse_activations=True, fuse_matmul_bias=True), 1, "img/s", "f32"
    if name == "bert_base_fp32_seq128":
        return models.bert_encoder(), dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True), 1, "seq/s", "f32"
    if name == "single_conv_fp32":
        return models.single_conv(), dict(fusion=True), 1, "img/s", "f32"
    if name == "alexnet_fp32_bs1":
        return models.alexnet(1, np.float32), dict(fusion=True, fuse_matmul_bias=True), 1, "img/s", "f32"
    if name == "yolo_v1_fp32_bs2":
        return models.yolo_v1(2, np.float32), dict(fusion=True, fuse_activations=True, fuse_matmul_bias=True), 2, "img/s", "f32"
    if name == "srgan_fp32_96x96":
        return models.srgan_generator(1, np.float32, height=96, width=96), dict(fusion=True, fuse_residual=True, fuse_activations=True), 1, "img/s", "f32"
    raise SystemExit(f"unknown workload {name}")


def recorded_traffic(workload, cls):
    """HBM bytes per launch of kernel class `cls`, from the counter runs whose
    summary is kept under profiles/ (FETCH_SIZE and WRITE_SIZE scaled by the
    copy-kernel calibration); None if no such summary exists for the workload."""
    path = os.path.join(ROOT, "profiles", f"{workload}_traffic.txt")
    try:
        for line in open(path):
            if line.startswith(f"traffic_bytes_per_launch[{cls}]:"):
                return float(line.split(":", 1)[1])
    except OSError:
        pass
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="resnet50_fp32_bs1")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the CPU-baseline leg")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--extra", action="store_true", help="also time the other workloads (reported under 'extra')")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only launch the library's plain copy kernel on 256 MiB a few times: the run that the "
                         "FETCH_SIZE / WRITE_SIZE counters of the other runs are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this path has no exchange step between devices, "
                         "N GPUs are N independent copies of this run (run with --gpus 1)")

    import torch
    from occamy_amd import compiler

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")

    if args.calibrate_copy:
        from occamy_amd import _abi
        from occamy_amd.ops import Ops
        n = 64 << 20  # floats: 256 MiB read + 256 MiB written per launch
        src = torch.ones(n, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        ops = Ops()
        for _ in range(5):
            ops.reshape(src.data_ptr(), (n,), dst.data_ptr(), _abi.F32)
        ops.sync()
        print(json.dumps({"calibration": "copy16_kernel", "launches": 5, "bytes_read_per_launch": 4 * n,
                          "bytes_written_per_launch": 4 * n}))
        return

    def measure(name, steps, warmup, want_profile):
        (graph, inputs), flags, batch, unit, dtype = build_workload(name)
        prog = graph.compile(**flags)
        sess = prog.session(compiler.MODE_RESIDENT)
        dev_in = [torch.from_numpy(a).cuda() for a in inputs]
        dev_out = [torch.empty(s, dtype=torch.from_numpy(np.empty(0, d)).dtype, device="cuda") for s, d in prog.output_info()]
        ip, op = [t.data_ptr() for t in dev_in], [t.data_ptr() for t in dev_out]
        torch.cuda.synchronize()
        for _ in range(max(warmup, 1)):
            sess.run_device(ip, op, use_graph=True)
        sess.sync()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            sess.run_device(ip, op, use_graph=True)
        sess.sync()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        res = dict(name=name, batch=batch, unit=unit, dtype=dtype, ms_per_step=1e3 * dt / steps,
                   value=batch * steps / dt, pool_bytes=prog.pool_bytes, weights_bytes=sess.weights_bytes,
                   kernels_per_step=prog.num_ops(compute_only=True), flags=flags)
        if want_profile:
            # device timestamps on the session's own stream, eager launches: one pair per operation
            # class around that class's launches issued back to back (a timestamp between two kernels
            # of a few microseconds costs about as much as the kernels themselves)
            ops = prog.compute_ops()
            acc = np.zeros(len(ops))
            reps = 20
            sess.profile(ip, on_device=True, by_class=True)
            for _ in range(reps):
                acc += np.array(sess.profile(ip, on_device=True, by_class=True))
            acc /= reps
            by_class = {}
            for (mn, cls, fl, by), ms in zip(ops, acc):
                c = by_class.setdefault(cls, dict(launches=0, flops=0.0, bytes=0.0, ms=0.0))
                c["launches"] += 1
                c["flops"] += fl
                c["bytes"] += by
                c["ms"] += float(ms)
            res["by_class"] = by_class
        # the reference's per-inference semantics: pool alloc, all weights H2D, kernels, D2H, sync, pool free
        # (compiled with the reference's own flags: no residual fusion)
        (ref_graph, _), _, _, _, _ = build_workload(name)  # a graph compiles once; the builders are seeded
        ref_prog = ref_graph.compile(**{k: v for k, v in flags.items() if k not in ("fuse_residual", "fuse_activations", "recompose", "fuse_matmul_bias", "fuse_attention")})
        res["pool_bytes_reference_flags"] = ref_prog.pool_bytes
        so = ref_prog.session(compiler.MODE_OCCAMY)
        so.run(*inputs)
        n = max(3, min(20, steps // 10))
        t0 = time.perf_counter()
        for _ in range(n):
            so.run(*inputs)
        res["occamy_semantics_value"] = batch * n / (time.perf_counter() - t0)
        so.close()
        sess.close()
        return res, (graph, inputs, prog)

    main_res, (graph, inputs, prog) = measure(args.workload, args.steps, args.warmup, True)

    # dominant kernel class by measured time
    cls, c = max(main_res["by_class"].items(), key=lambda kv: kv[1]["ms"])
    mfma_bound = cls in ("conv_dense", "gemm", "matmul")
    if mfma_bound:
        peak = PEAK["mfma_f16" if main_res["dtype"] == "f16" else "mfma_f32"]
        achieved = c["flops"] / (c["ms"] * 1e-3)
        roof = dict(bound="mfma", achieved=achieved / 1e12, peak=peak / 1e12, unit="TFLOP/s", frac=achieved / peak)
    else:
        achieved = c["bytes"] / (c["ms"] * 1e-3)
        roof = dict(bound="hbm", achieved=achieved / 1e9, peak=PEAK["hbm"] / 1e9, unit="GB/s", frac=achieved / PEAK["hbm"])
    roof.update(kernel=cls, launches_per_step=c["launches"], avg_launch_us=1e3 * c["ms"] / c["launches"],
                traffic=recorded_traffic(args.workload, cls))

    cpu = None
    if not args.no_cpu:
        # CPU baseline: the oracle build of the same ABI runs the same program on the host cores.
        import ctypes
        oracle_path = os.path.join(ROOT, "oracle", "libdnnrt_oracle.so")
        olib = ctypes.CDLL(oracle_path)
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
        olib.dnnrtOracleSetThreads(cores)
        cpu_prog = prog
        _, wl_flags, _, _, _ = build_workload(args.workload)
        if wl_flags.get("channels_last"):
            # the oracle keeps the reference's N,C,H,W layout: same graph, same flags otherwise
            (cpu_graph, _), _, _, _, _ = build_workload(args.workload)
            cpu_prog = cpu_graph.compile(**{k: v for k, v in wl_flags.items() if k != "channels_last"})
        so = cpu_prog.session(compiler.MODE_RESIDENT, runtime_library=oracle_path)
        t0 = time.perf_counter()
        so.run(*inputs)
        first = time.perf_counter() - t0
        n = int(max(1, min(50, args.cpu_seconds / max(first, 1e-3))))
        t0 = time.perf_counter()
        for _ in range(n):
            so.run(*inputs)
        dt = (time.perf_counter() - t0) / n
        so.close()
        cpu = dict(value=main_res["batch"] / dt, unit=main_res["unit"], cores=cores, kind="port",
                   sample=f"{n} inference(s) of {args.workload} (batch {main_res['batch']}) through the in-repo CPU oracle, "
                          f"OpenMP {cores} threads; the reference's onnx-mlir CPU lowering is not available")

    line = {
        "metric": "ResNet-50 img/s at bs1/bs64 on 1 GPU" if args.workload.startswith("resnet50") else f"{args.workload} throughput",
        "value": main_res["value"], "unit": main_res["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_res["dtype"], "data": "synthetic",
        "config": {"workload": args.workload, "batch": main_res["batch"],
                   "fusion": ", ".join(k for k, v in main_res["flags"].items() if v and (k.startswith("fus") or k == "recompose")),
                   "mode": "weights and input resident in HBM, kernels replayed from a captured graph",
                   "kernels_per_step": main_res["kernels_per_step"]},
        "roofline": roof,
        "cpu_baseline": cpu,
        "pool_bytes": main_res["pool_bytes"], "pool_bytes_reference_flags": main_res["pool_bytes_reference_flags"],
        "weights_bytes": main_res["weights_bytes"],
        "occamy_semantics": {"value": main_res["occamy_semantics_value"], "unit": main_res["unit"],
                             "what": "reference flags (no residual fusion); per inference: pool hipMalloc, every weight H2D into its pool slot, kernels, D2H, sync, pool free"},
        "by_class": {k: {"launches": v["launches"], "ms": round(v["ms"], 4),
                         "TFLOP/s": round(v["flops"] / max(v["ms"], 1e-9) / 1e9, 3),
                         "GB/s": round(v["bytes"] / max(v["ms"], 1e-9) / 1e6, 1)} for k, v in main_res["by_class"].items()},
    }
    if args.extra:
        extra = {}
        for name in ["resnet50_fp16_bs64", "mobilenet_v2_fp32_bs1", "bert_base_fp32_seq128", "single_conv_fp32",
                     "alexnet_fp32_bs1", "yolo_v1_fp32_bs2", "srgan_fp32_96x96"]:
            if name == args.workload:
                continue
            try:
                r, _ = measure(name, max(20, args.steps // 4), max(5, args.warmup // 2), True)
                extra[name] = {k: r[k] for k in ("value", "unit", "ms_per_step", "pool_bytes", "weights_bytes", "occamy_semantics_value")}
                extra[name]["by_class"] = {k: {"launches": v["launches"], "ms": round(v["ms"], 4)} for k, v in r["by_class"].items()}
            except Exception as e:  # a workload that cannot run yet is reported, not hidden
                extra[name] = {"error": str(e)}
        line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
