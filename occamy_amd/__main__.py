"""``python -m occamy_amd model.onnx``: compile an ONNX file with the reference's
flags and time it, the way the reference's test scripts do
(test/models/*/run.py: export, ``core-dnn --EmitLib --dnn-dealloc-opt=true
--dnn-malloc-pool-opt=true model.onnx``, run N times discarding the first,
report mean / P90 / P95 / P99 in milliseconds)."""
import argparse
import json
import time

import numpy as np

from . import compiler


def main():
    ap = argparse.ArgumentParser(prog="python -m occamy_amd")
    ap.add_argument("model", help="ONNX model file (static shapes)")
    ap.add_argument("--dnn-kernel-fusion", dest="fusion", action="store_true")
    ap.add_argument("--fuse-residual", action="store_true", help="with fusion: conv+bias -> add -> relu as one call")
    ap.add_argument("--recompose", action="store_true", help="LayerNormalization / Gelu written in primitive operators become one call each")
    ap.add_argument("--fuse-attention", action="store_true", help="head split, QK^T, Softmax, PV, head merge as one call")
    ap.add_argument("--fuse-matmul-bias", action="store_true", help="with fusion: MatMul -> Add(bias row) as one call")
    ap.add_argument("--fuse-activations", action="store_true",
                    help="with fusion: conv+bias -> Clip(0, c) / LeakyRelu / one-slope PRelu as one call")
    ap.add_argument("--no-dnn-dealloc-opt", dest="dealloc_opt", action="store_false")
    ap.add_argument("--no-onnx-const-at-use", dest="const_at_use", action="store_false")
    ap.add_argument("--channels-last", action="store_true", help="fp16 graphs: NHWC on the device")
    ap.add_argument("--fuse-projection-shortcut", action="store_true",
                    help="with --dnn-kernel-fusion, --fuse-residual and --channels-last: a residual block's projection shortcut and last convolution in one call")
    ap.add_argument("--alias-copies", action="store_true", help="Flatten / Reshape / Squeeze / Unsqueeze reuse their input's buffer")
    ap.add_argument("--compact-pool", action="store_true", help="plan the pool with every lifetime known (largest first) instead of the reference's first fit")
    ap.add_argument("--inplace-residual", action="store_true", help="a fused conv + add + activation writes over its residual operand when nothing reads it afterwards")
    ap.add_argument("--fuse-first-layer-maxpool", action="store_true",
                    help="with --dnn-kernel-fusion and --channels-last: a ResNet's first convolution and its max-pool in one call")
    ap.add_argument("--resident", action="store_true", help="keep pool and weights on the device between runs")
    ap.add_argument("--tune", metavar="FILE", help="with --resident: time the runtime's convolution variants on this model's layers, in place, "
                    "keep the winners as the calls' algo operands (the reference picks cuDNN's algorithm the same way when it compiles a model) and write them to FILE")
    ap.add_argument("--algos", metavar="FILE", help="with --resident: apply the choices an earlier --tune wrote to FILE")
    ap.add_argument("--runtime", default=None, help="shared object exporting include/dnnrt.h (default: the gfx950 library)")
    ap.add_argument("--iterations", type=int, default=100)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--emit", action="store_true", help="print the DNN program and stop")
    args = ap.parse_args()

    graph = compiler.load_onnx(args.model)
    prog = graph.compile(fusion=args.fusion, fuse_residual=args.fuse_residual, fuse_activations=args.fuse_activations, recompose=args.recompose, fuse_matmul_bias=args.fuse_matmul_bias, fuse_attention=args.fuse_attention, dealloc_opt=args.dealloc_opt,
                         const_at_use=args.const_at_use, channels_last=args.channels_last,
                         fuse_first_layer_maxpool=args.fuse_first_layer_maxpool, alias_copies=args.alias_copies, fuse_projection_shortcut=args.fuse_projection_shortcut,
                         inplace_residual=args.inplace_residual, compact_pool=args.compact_pool)
    print(f"inputs: {graph.input_shapes}")
    print(f"pool: {prog.pool_bytes} bytes (maxAllocByte); {prog.num_ops(compute_only=True)} runtime calls per inference")
    if args.emit:
        print(prog.text)
        return
    rng = np.random.default_rng(args.seed)
    inputs = []
    for name, (shape, dt) in graph.input_shapes.items():
        inputs.append(rng.integers(0, 100, shape).astype(dt) if dt == np.int64 else rng.standard_normal(shape).astype(dt))
    sess = prog.session(compiler.MODE_RESIDENT if args.resident else compiler.MODE_OCCAMY, runtime_library=args.runtime)
    if (args.tune or args.algos) and not args.resident:
        raise SystemExit("--tune and --algos need --resident")
    if args.algos:
        with open(args.algos) as f:
            saved = json.load(f)
        if saved.get("program_ops") != prog.num_ops(compute_only=True):
            raise SystemExit(f"{args.algos} was written for another program")
        sess.set_algos([tuple(a) for a in saved["algos"]])
    if args.tune:
        sess.run(*inputs)
        changed = sess.tune(inputs)
        with open(args.tune, "w") as f:
            json.dump({"program_ops": prog.num_ops(compute_only=True), "algos": sess.algos()}, f)
        print(f"tuned: {changed} operation(s) got a measured variant; written to {args.tune}")
    times = []
    for i in range(args.iterations + 1):
        t0 = time.perf_counter()
        out = sess.run(*inputs)
        dt = (time.perf_counter() - t0) * 1e3
        if i:
            times.append(dt)
        else:
            print(f"first run: {dt:.3f} ms")
    sess.close()
    t = np.array(times)
    print(f"outputs: {[o.shape for o in out]}")
    print(f"mean {t.mean():.3f} ms  P90 {np.percentile(t, 90):.3f}  P95 {np.percentile(t, 95):.3f}  P99 {np.percentile(t, 99):.3f}")


if __name__ == "__main__":
    main()
