#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

A "step" is one inference of the workload with its input and all weights
already resident in HBM: every kernel of the compiled DNN program (replayed
from a captured graph), the first reading the caller's input buffer and the
last writing the caller's result buffer.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--layers FILE] [--profile-only]

The default workload, "resnet50", is the metric's two halves in one line: the
headline record (value, roofline, cpu_baseline ...) is ResNet-50 fp16 batch 64
and the key "fp32_bs1" holds the same record for ResNet-50 fp32 batch 1; the
key "configs" holds a compact record (value, ms_per_step, roofline, the
figures the configuration is asked for) of the three other configurations:
single_conv_fp32, mobilenet_v2_fp32_bs1, bert_base_fp32_seq128.
Other workloads: resnet50_fp32_bs1, resnet50_fp16_bs64, mobilenet_v2_fp32_bs1,
bert_base_fp32_seq128, single_conv_fp32, alexnet_fp32_bs1, yolo_v1_fp32_bs2,
srgan_fp32_96x96, ssd_resnet50_fp32_bs3, mobilenet_v2_fp16_bs64, bert_base_fp16_seq128.  --layers writes a per-operation table (algorithmic FLOP and
bytes, the roofline bound, measured time) of the headline workload to FILE.
--profile-only runs nothing but the timed program of --workload (one eager
pass, which a graph recording needs, then W + K replays; no CPU leg, no
reference-flag leg, no per-class or per-operation timing passes, no tuning
sweep): the run to put under rocprofv3, whose kernel counts are then whole
multiples of the program's.
"""
import argparse
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"mfma_f32": 157.3e12, "mfma_f16": 2.5e15, "hbm": 8.0e12}
RESIDENT_ONLY_FLAGS = ("fuse_residual", "fuse_activations", "recompose", "fuse_matmul_bias", "fuse_attention", "fuse_first_layer_maxpool", "fuse_projection_shortcut", "alias_copies", "inplace_residual", "compact_pool")


def build_workload(name, batch=None):
    """((graph, inputs), compile flags, batch, unit, dtype); `batch` overrides the workload's own batch size."""
    from occamy_amd import models
    if name == "resnet50_fp32_bs1":
        b = batch or 1
        return models.resnet50(b, np.float32), dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, fuse_first_layer_maxpool=True, fuse_projection_shortcut=True, alias_copies=True), b, "img/s", "f32"
    if name == "resnet50_fp16_bs64":
        b = batch or 64
        return (models.resnet50(b, np.float16, seed=5),
                dict(fusion=True, fuse_residual=True, fuse_matmul_bias=True, channels_last=True, fuse_first_layer_maxpool=True, fuse_projection_shortcut=True,
                     alias_copies=True, inplace_residual=True, compact_pool=True),
                b, "img/s", "f16")
    if batch is not None:
        raise SystemExit(f"{name}: no batch override")
    if name == "mobilenet_v2_fp32_bs1":
        return models.mobilenet_v2(1, np.float32), dict(fusion=True, fuse_residual=True, fuse_activations=True, fuse_matmul_bias=True, alias_copies=True), 1, "img/s", "f32"
    if name == "bert_base_fp32_seq128":
        return models.bert_encoder(), dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True, alias_copies=True), 1, "seq/s", "f32"
    if name == "bert_base_fp32_seq128_unfused_attention":
        return models.bert_encoder(), dict(recompose=True, fusion=True, fuse_matmul_bias=True, alias_copies=True), 1, "seq/s", "f32"
    if name == "mobilenet_v2_fp16_bs64":
        return (models.mobilenet_v2(64, np.float16),
                dict(fusion=True, fuse_residual=True, fuse_activations=True, fuse_matmul_bias=True, channels_last=True, alias_copies=True,
                     inplace_residual=True, compact_pool=True), 64, "img/s", "f16")
    if name == "bert_base_fp16_seq128":
        return (models.bert_encoder(dtype=np.float16),
                dict(recompose=True, fusion=True, fuse_matmul_bias=True, fuse_attention=True, alias_copies=True, compact_pool=True), 1, "seq/s", "f16")
    if name == "single_conv_fp32":
        return models.single_conv(), dict(fusion=True), 1, "img/s", "f32"
    if name == "alexnet_fp32_bs1":
        return models.alexnet(1, np.float32), dict(fusion=True, fuse_matmul_bias=True), 1, "img/s", "f32"
    if name == "yolo_v1_fp32_bs2":
        return models.yolo_v1(2, np.float32), dict(fusion=True, fuse_activations=True, fuse_matmul_bias=True), 2, "img/s", "f32"
    if name == "ssd_resnet50_fp32_bs3":  # the reference's test runs three images
        return (models.ssd_resnet50(3, np.float32),
                dict(fusion=True, fuse_residual=True, fuse_first_layer_maxpool=True, fuse_projection_shortcut=True, inplace_residual=True, compact_pool=True), 3, "img/s", "f32")
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


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


MFMA_CLASSES = ("conv_dense", "gemm", "matmul", "attention")


def timed_steps(sess, ip, op, steps, warmup):
    """W untimed graph-replayed steps, then exactly K timed ones between two host-side waits; seconds."""
    import torch
    for _ in range(max(warmup, 1)):
        sess.run_device(ip, op, use_graph=True, in_place=True)
    sess.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        sess.run_device(ip, op, use_graph=True, in_place=True)
    sess.sync()
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def measure(name, steps, warmup, profile_only=False, tune=True, reference_leg=True, per_op=True):
    """One workload on the GPU: K graph-replayed steps timed as a whole (value), individually timed steps (median,
    P90), per-class and per-operation device times, and the reference's per-inference semantics."""
    import torch
    from occamy_amd import compiler
    (graph, inputs), flags, batch, unit, dtype = build_workload(name)
    prog = graph.compile(**flags)
    sess = prog.session(compiler.MODE_RESIDENT)
    dev_in = [torch.from_numpy(a).cuda() for a in inputs]
    dev_out = [torch.empty(s, dtype=torch.from_numpy(np.empty(0, d)).dtype, device="cuda") for s, d in prog.output_info()]
    ip, op = [t.data_ptr() for t in dev_in], [t.data_ptr() for t in dev_out]
    torch.cuda.synchronize()
    dt = timed_steps(sess, ip, op, steps, warmup)
    res = dict(name=name, batch=batch, unit=unit, dtype=dtype, pool_bytes=prog.pool_bytes, weights_bytes=sess.weights_bytes,
               kernels_per_step=prog.num_ops(compute_only=True), flags=flags)
    now, _, static = sess.device_bytes()
    res["device_bytes"] = dict(allocated=now, static=static, total=now + static,
                               what="everything the runtime library holds on the device during the timed steps: the pool and the "
                                    "constants' arena from the allocator (counted by the library: dnnrtDeviceMemoryStats), and "
                                    "its static arrays (split-reduction scratch)")
    if profile_only:
        res.update(ms_per_step=1e3 * dt / steps, value=batch * steps / dt)
        sess.close()
        return res
    # The measured choice of variant per convolution (the reference times cuDNN's algorithms at compile time and
    # passes the winner as `algo`): the same K steps again with the tuned program, and the faster of the two
    # programs is the one reported, the other one's time beside it.
    res["tuning"] = None
    if tune and dtype == "f16":
        t0 = time.perf_counter()
        try:
            changed = sess.tune(ip, on_device=True, reps=5)
        except RuntimeError as e:  # the runtime's own choices stay in force; say what happened
            changed = 0
            res["tuning_error"] = str(e)
        tune_s = time.perf_counter() - t0
        res["tuning"] = dict(operations_with_a_measured_variant=changed, seconds=round(tune_s, 2),
                             ms_per_step_runtime_choice=1e3 * dt / steps)
        if changed:
            tuned_algos = sess.algos()
            dt2 = timed_steps(sess, ip, op, steps, warmup)
            res["tuning"]["ms_per_step_measured_choice"] = 1e3 * dt2 / steps
            if dt2 < dt:
                dt = dt2
                res["tuning"]["used"] = "measured choice"
            else:
                sess.set_algos([(0, 0)] * len(tuned_algos))
                timed_steps(sess, ip, op, 1, 1)  # record the graph of the runtime's own choices again
                res["tuning"]["used"] = "runtime choice"
        else:
            res["tuning"]["used"] = "runtime choice"
    res.update(ms_per_step=1e3 * dt / steps, value=batch * steps / dt)
    # the distribution: the same step, each one waited for (what a caller that needs every answer sees)
    lat = []
    for _ in range(max(20, min(steps, 100))):
        t1 = time.perf_counter()
        sess.run_device(ip, op, use_graph=True, in_place=True)
        sess.sync()
        lat.append(1e3 * (time.perf_counter() - t1))
    res["latency_ms"] = {"median": float(np.median(lat)), "p90": float(np.percentile(lat, 90)), "samples": len(lat),
                         "what": "one step at a time, each waited for on the host"}
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
    res["ops"] = ops
    res["text"] = prog.text
    if per_op:
        # ... and one pair per operation, in program order (each kernel finds the caches as the network leaves them)
        per = np.zeros(len(ops))
        sess.profile(ip, on_device=True)
        for _ in range(reps):
            per += np.array(sess.profile(ip, on_device=True))
        res["per_op_ms"] = list(per / reps)
    if reference_leg:
        # the reference's per-inference semantics: pool alloc, all weights H2D, kernels, D2H, sync, pool free
        # (compiled with the reference's own flags: no residual fusion)
        (ref_graph, _), _, _, _, _ = build_workload(name)  # a graph compiles once; the builders are seeded
        ref_prog = ref_graph.compile(**{k: v for k, v in flags.items() if k not in RESIDENT_ONLY_FLAGS})
        res["pool_bytes_reference_flags"] = ref_prog.pool_bytes
        sess.close()  # so that the per-inference session is the only one alive: its handle then has the static scratch
        so = ref_prog.session(compiler.MODE_OCCAMY)
        base, _, _ = so.device_bytes(reset_peak=True)
        so.run(*inputs)
        _, peak, _ = so.device_bytes()
        res["device_bytes_reference_flags"] = peak - base
        n = max(3, min(20, steps // 10))
        t0 = time.perf_counter()
        for _ in range(n):
            so.run(*inputs)
        res["occamy_semantics_value"] = batch * n / (time.perf_counter() - t0)
        so.close()
    sess.close()
    return res


def class_figures(res):
    """Per operation class: launches, device time, and the achieved rate as a fraction of the peak that bounds the
    class (MFMA for products, HBM for everything else)."""
    peak_mfma = PEAK["mfma_f16" if res["dtype"] == "f16" else "mfma_f32"]
    out = {}
    for k, v in res["by_class"].items():
        ms = max(v["ms"], 1e-9)
        tf, gb = v["flops"] / ms / 1e9, v["bytes"] / ms / 1e6
        out[k] = {"launches": v["launches"], "ms": round(v["ms"], 4), "TFLOP/s": round(tf, 3), "GB/s": round(gb, 1),
                  "bound": "mfma" if k in MFMA_CLASSES else "hbm",
                  "frac": round(tf * 1e12 / peak_mfma if k in MFMA_CLASSES else gb * 1e9 / PEAK["hbm"], 4)}
    return out


def roofline_of(res):
    """The roofline record of the workload's dominant kernel class (by measured time)."""
    cls, c = max(res["by_class"].items(), key=lambda kv: kv[1]["ms"])
    if cls in MFMA_CLASSES:
        peak = PEAK["mfma_f16" if res["dtype"] == "f16" else "mfma_f32"]
        achieved = c["flops"] / (c["ms"] * 1e-3)
        roof = dict(bound="mfma", achieved=achieved / 1e12, peak=peak / 1e12, unit="TFLOP/s", frac=achieved / peak)
    else:
        achieved = c["bytes"] / (c["ms"] * 1e-3)
        roof = dict(bound="hbm", achieved=achieved / 1e9, peak=PEAK["hbm"] / 1e9, unit="GB/s", frac=achieved / PEAK["hbm"])
    roof.update(kernel=cls, launches_per_step=c["launches"], avg_launch_us=1e3 * c["ms"] / c["launches"],
                traffic=recorded_traffic(res["name"], cls))
    return roof


def cpu_leg(name, threads, seconds, batch=None):
    """The same DNN program through the oracle build of the same ABI on `threads` host threads; images (sequences)
    per second over a bounded number of inferences."""
    import ctypes
    from occamy_amd import compiler
    oracle_path = os.path.join(ROOT, "oracle", "libdnnrt_oracle.so")
    ctypes.CDLL(oracle_path).dnnrtOracleSetThreads(threads)
    (graph, inputs), flags, b, unit, _ = build_workload(name, batch)
    # the oracle keeps the reference's N,C,H,W layout: same graph, same flags otherwise
    prog = graph.compile(**{k: v for k, v in flags.items() if k != "channels_last"})
    so = prog.session(compiler.MODE_RESIDENT, runtime_library=oracle_path)
    t0 = time.perf_counter()
    so.run(*inputs)
    first = time.perf_counter() - t0
    n = int(max(1, min(50, (seconds - first) / max(first, 1e-3))))
    times = [first] if first > seconds / 3 else []  # a long first inference is itself a sample
    for _ in range(n):
        t0 = time.perf_counter()
        so.run(*inputs)
        times.append(time.perf_counter() - t0)
    so.close()
    return b / float(np.median(times)), len(times), b


def cpu_baseline(res, seconds):
    name, batch = res["name"], res["batch"]
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    threads = max(1, min(threads, os.cpu_count() or 1))
    cpu_batch = None if batch <= 16 else 16  # the same per-image work in more, shorter samples
    value, n, bt = cpu_leg(name, threads, seconds, cpu_batch)
    small = None if batch <= 2 else 2  # one thread gets a batch it finishes in seconds (same per-image work)
    v1, n1, b1 = cpu_leg(name, 1, seconds / 2, small)
    return dict(value=value, unit=res["unit"], cores=threads, kind="port", cpu=cpu_model(), host_cpus=os.cpu_count(),
                sample=f"median of {n} inference(s) of {name} at batch {bt} through the in-repo CPU oracle (plain C, "
                       f"double accumulation) on {threads} OpenMP threads = this job's share of the host "
                       f"(OMP_NUM_THREADS); the reference's onnx-mlir CPU lowering is not available",
                one_thread=dict(value=v1, unit=res["unit"], cores=1,
                                sample=f"median of {n1} inference(s) of the same network at batch {b1} on one thread"))


def record(res, steps, warmup, cpu_seconds):
    """The JSON record of one measured workload (the keys of the headline line)."""
    return {
        "value": res["value"], "unit": res["unit"], "steps": steps, "warmup": warmup, "ms_per_step": res["ms_per_step"],
        "latency_ms": res["latency_ms"], "dtype": res["dtype"], "data": "synthetic",
        "config": {"workload": res["name"], "batch": res["batch"],
                   "fusion": ", ".join(k for k, v in res["flags"].items() if v and (k.startswith("fus") or k in ("recompose", "alias_copies", "channels_last", "inplace_residual", "compact_pool"))),
                   "mode": "weights and input resident in HBM (the first layer reads the input buffer in place, the last one writes the result buffer), "
                           + ("kernels replayed from a captured graph" if res["kernels_per_step"] > 3 else "kernels launched one by one (up to three: a graph launch costs the host more)"),
                   "kernels_per_step": res["kernels_per_step"]},
        "roofline": roofline_of(res),
        "cpu_baseline": cpu_baseline(res, cpu_seconds) if cpu_seconds > 0 else None,
        "pool_bytes": res["pool_bytes"], "pool_bytes_reference_flags": res["pool_bytes_reference_flags"],
        "weights_bytes": res["weights_bytes"], "device_bytes": res["device_bytes"],
        "occamy_semantics": {"value": res["occamy_semantics_value"], "unit": res["unit"],
                             "device_bytes_peak": res["device_bytes_reference_flags"],
                             "what": "reference flags (no residual fusion); per inference: pool hipMalloc, every weight H2D into its pool slot, kernels, D2H, sync, pool free; "
                                     "device_bytes_peak = what the runtime library took from the allocator at the peak of one inference (= pool_bytes_reference_flags)"},
        "tuning": res["tuning"],
        "by_class": class_figures(res),
    }


def compact_record(res, steps, warmup):
    """One of the other configurations in the default line: throughput, the dominant class's roofline, every
    class's rate against its bound, memory."""
    return {"value": res["value"], "unit": res["unit"], "steps": steps, "warmup": warmup, "ms_per_step": res["ms_per_step"],
            "latency_ms": res["latency_ms"], "dtype": res["dtype"],
            "config": {"workload": res["name"], "batch": res["batch"], "kernels_per_step": res["kernels_per_step"]},
            "roofline": roofline_of(res), "by_class": class_figures(res), "tuning": res.get("tuning"),
            "pool_bytes": res["pool_bytes"], "pool_bytes_reference_flags": res["pool_bytes_reference_flags"],
            "weights_bytes": res["weights_bytes"], "device_bytes_total": res["device_bytes"]["total"],
            "occamy_semantics_value": res["occamy_semantics_value"]}


def layer_table(res):
    """Per operation, in program order: algorithmic FLOP and bytes, the time the roofline allows
    (max of FLOP / MFMA peak and bytes / HBM peak), the measured time, and their ratio."""
    peak = PEAK["mfma_f16" if res["dtype"] == "f16" else "mfma_f32"]
    names = {o[0] for o in res["ops"]}
    lines = [l for l in res["text"].splitlines() if any(f"= {n} " in l for n in names)]
    out = [f"{res['name']}: per operation, program order.  t_mfma = FLOP / {peak / 1e12:.1f} TFLOP/s, t_hbm = bytes / 8 TB/s,",
           "bound = the larger; measured = device timestamps around each launch inside the network (a pair of",
           f"timestamps adds to a kernel of a few microseconds; the graph-replayed step takes {res['ms_per_step'] * 1e3:.0f} us,",
           f"the measured column sums to {sum(res['per_op_ms']) * 1e3:.0f} us); frac = bound / measured.", "",
           f"{'#':>3s} {'operation':28s} {'result':22s} {'red.':>5s} {'attrs':28s} {'MFLOP':>9s} {'KB':>9s} {'t_mfma':>7s} {'t_hbm':>7s} "
           f"{'by':>4s} {'meas_us':>8s} {'frac':>5s} {'TF/s':>7s} {'GB/s':>7s}"]
    for i, ((mn, cls, fl, by), ms) in enumerate(zip(res["ops"], res["per_op_ms"])):
        line = lines[i] if len(lines) == len(res["ops"]) else ""
        shape = re.search(r": \w+(\[[^\]]*\])\s*$", line)
        attrs = re.search(r"\{([^}]*)\}", line)
        a = attrs.group(1) if attrs else ""
        a = re.sub(r"group=1, |activMode=\d+|, $", "", a).strip(", ")
        n_out = np.prod([int(v) for v in shape.group(1)[1:-1].split(",")]) if shape else 0
        red = f"{int(round(fl / (2 * n_out)))}" if cls == "conv_dense" and n_out else ""
        t_m, t_h = fl / peak * 1e6, by / PEAK["hbm"] * 1e6
        bound = max(t_m, t_h)
        us = ms * 1e3
        out.append(f"{i:3d} {mn[4:]:28s} {shape.group(1) if shape else '':22s} {red:>5s} {a[:28]:28s} {fl / 1e6:9.1f} {by / 1e3:9.1f} "
                   f"{t_m:7.2f} {t_h:7.2f} {'mfma' if t_m >= t_h else 'hbm':>4s} {us:8.2f} {bound / max(us, 1e-9):5.2f} "
                   f"{fl / max(us, 1e-9) / 1e6:7.1f} {by / max(us, 1e-9) / 1e3:7.1f}")
    tot_b = sum(max(fl / peak, by / PEAK["hbm"]) for _, _, fl, by in res["ops"]) * 1e6
    out.append("")
    out.append(f"sum of bounds {tot_b:.0f} us; sum of measured {sum(res['per_op_ms']) * 1e3:.0f} us")
    return "\n".join(out) + "\n"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="resnet50")
    ap.add_argument("--cpu-seconds", type=float, default=24.0, help="budget of the CPU-baseline leg of the headline workload")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--layers", metavar="FILE", help="write the per-operation table of the headline workload to FILE")
    ap.add_argument("--extra", action="store_true", help="also time the workloads outside the five configurations (reported under 'extra')")
    ap.add_argument("--profile-only", action="store_true",
                    help="run only the timed program of --workload (no CPU leg, no reference-flag leg, no timing passes, no tuning): the run to profile")
    ap.add_argument("--no-tune", action="store_true", help="fp16 workloads: skip the measured choice of convolution variants")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only launch the library's plain copy kernel on 256 MiB a few times: the run that the "
                         "FETCH_SIZE / WRITE_SIZE counters of the other runs are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this path has no exchange step between devices, "
                         "N GPUs are N independent copies of this run (run with --gpus 1)")

    import torch

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

    both = args.workload == "resnet50"
    head_name = "resnet50_fp16_bs64" if both else args.workload
    if args.profile_only:
        r = measure(head_name, args.steps, args.warmup, profile_only=True)
        print(json.dumps({"profile_only": head_name, "value": r["value"], "unit": r["unit"], "steps": args.steps, "warmup": max(args.warmup, 1),
                          "ms_per_step": r["ms_per_step"], "kernels_per_step": r["kernels_per_step"],
                          "passes_over_the_program": 1 + max(args.warmup, 1) + args.steps if r["kernels_per_step"] > 3 else max(args.warmup, 1) + args.steps,
                          "device_bytes": r["device_bytes"]}))
        return
    cpu_seconds = 0.0 if args.no_cpu else args.cpu_seconds
    head = measure(head_name, args.steps, args.warmup, tune=not args.no_tune)
    rec = record(head, args.steps, args.warmup, cpu_seconds)
    if args.layers:
        with open(args.layers, "w") as f:
            f.write(layer_table(head))
    line = {"metric": "ResNet-50 img/s at bs1/bs64 on 1 GPU" if head_name.startswith("resnet50") else f"{head_name} throughput",
            "value": rec.pop("value"), "unit": rec.pop("unit"), "n_gpus": 1, "steps": rec.pop("steps"), "warmup": rec.pop("warmup"),
            "ms_per_step": rec.pop("ms_per_step"), "higher_is_better": True, "scaling": "weak", "vs_baseline": None}
    line.update(rec)
    if both:
        line["headline"] = ("resnet50_fp16_bs64 (the half of the metric with a stated target); the fp32 batch-1 half is under fp32_bs1 with the "
                            "same keys, the three other configurations under configs")
        # batch 1: more steps for the same wall time (a step is under half a millisecond)
        small = measure("resnet50_fp32_bs1", args.steps, args.warmup)
        line["fp32_bs1"] = record(small, args.steps, args.warmup, cpu_seconds / 2)
        configs = {}
        for name in ("single_conv_fp32", "mobilenet_v2_fp32_bs1", "bert_base_fp32_seq128"):
            r = measure(name, args.steps, args.warmup, per_op=False)
            configs[name] = compact_record(r, args.steps, args.warmup)
        # config 4 is asked for its softmax rate too, and the timed program has no softmax launch of its own (it is
        # inside the fused attention call): the same encoder without that fusion, for its softmax and matmul classes
        r = measure("bert_base_fp32_seq128_unfused_attention", max(5, args.steps // 2), max(2, args.warmup // 2), per_op=False, reference_leg=False)
        cf = class_figures(r)
        configs["bert_base_fp32_seq128"]["without_attention_fusion"] = {
            "ms_per_step": r["ms_per_step"], "kernels_per_step": r["kernels_per_step"],
            "by_class": {k: cf[k] for k in ("softmax", "matmul", "layernorm") if k in cf}}
        line["configs"] = configs
    if args.extra:
        extra = {}
        for name in ["alexnet_fp32_bs1", "yolo_v1_fp32_bs2", "srgan_fp32_96x96", "ssd_resnet50_fp32_bs3", "mobilenet_v2_fp16_bs64", "bert_base_fp16_seq128"]:
            if name == head_name:
                continue
            try:
                r = measure(name, max(20, args.steps // 4), max(5, args.warmup // 2), per_op=False)
                extra[name] = compact_record(r, max(20, args.steps // 4), max(5, args.warmup // 2))
            except Exception as e:  # a workload that cannot run yet is reported, not hidden
                extra[name] = {"error": str(e)}
        line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
