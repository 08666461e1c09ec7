#!/usr/bin/env python3
"""Benchmark: ResNet-50 training step (fwd + bwd + SGD-momentum), fp32, batch 64, 3x224x224,
1000 classes, synthetic data, on one MI355X through the lantern_hip C ABI.

Prints ONE JSON line: training samples/s, the MFMA roofline fraction of the convolution kernels
(measured live with HIP events on the library's stream over the timed steps), and the CPU oracle
timed on the host cores on a bounded sample of the same workload.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 64] [--hw 224] [--no-cpu]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

PEAK_FP32_MFMA_TFLOPS = 157.3
CATS = ["conv_fwd", "conv_bwd_data", "conv_bwd_filter", "gemm", "bn_fwd", "bn_bwd", "elementwise", "pool", "reduce", "optim", "fill", "rnn"]


def conv_flops(model, batch, hw):
    """Algorithmic conv work of one step: 2*N*K*C*R*S*P*Q per direction; every conv has a filter
    gradient, every conv but the stem an input gradient."""
    from lantern_amd.nn import Conv2D
    fwd = 0
    first = True
    total = 0
    shapes = []

    def visit(m, h):
        return h
    # walk the network the way __call__ does, tracking spatial size
    h = hw
    convs = []
    c1 = model.conv1
    def out_hw(h, conv):
        k = conv.kernel.x.shape
        return (h + 2 * conv.pad[0] - k[2]) // conv.stride[0] + 1
    def f(conv, h):
        k = conv.kernel.x.shape
        p = out_hw(h, conv)
        return 2.0 * batch * k[0] * k[1] * k[2] * k[3] * p * p, p
    fl, h = f(c1, h); convs.append((fl, False))
    if model.imagenet_stem:
        h = (h + 2 - 3) // 2 + 1
    for blk in model.blocks:
        fl1, h1 = f(blk.conv1, h); convs.append((fl1, True))
        fl2, h2 = f(blk.conv2, h1); convs.append((fl2, True))
        fl3, h3 = f(blk.conv3, h2); convs.append((fl3, True))
        if blk.down is not None:
            fld, _ = f(blk.down[0], h); convs.append((fld, True))
        h = h3
    fwd = sum(c[0] for c in convs)
    bwd_filter = fwd
    bwd_data = sum(c[0] for c in convs if c[1])
    return fwd, bwd_data, bwd_filter


def run_gpu(args):
    import lantern_amd as la
    from lantern_amd.apps.resnet50 import ResNet50, Trainer
    be = la.BackendHIP(heap_bytes=int(args.heap_gb * (1 << 30)))
    be.setup()
    la.set_backend(be)
    model = ResNet50(num_classes=args.classes, imagenet_stem=args.hw > 64)
    tr = Trainer(model, args.batch, args.hw, args.classes, lr=0.1, momentum=0.9)
    lib = be.lib
    losses = []
    for _ in range(args.warmup):
        l = tr.step(); tr.end_step()
    be.sync()
    conv_mask = 0b111
    lib.lh_prof_enable(conv_mask)
    ms = (C.c_double * len(CATS))(); calls = (C.c_int64 * len(CATS))()
    lib.lh_prof_collect(ms, calls, len(CATS))       # reset
    be.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        l = tr.step()
        losses.append(l)
        tr.end_step()
    be.sync()
    t1 = time.perf_counter()
    lib.lh_prof_collect(ms, calls, len(CATS))
    conv_ms = [ms[i] / args.steps for i in range(3)]
    conv_calls = [int(calls[i]) // args.steps for i in range(3)]
    # a separate, untimed pass with every category instrumented (breakdown for the log)
    lib.lh_prof_enable((1 << len(CATS)) - 1)
    tr.step(); tr.end_step()
    lib.lh_prof_collect(ms, calls, len(CATS))
    breakdown = {CATS[i]: {"ms": round(ms[i], 3), "calls": int(calls[i])} for i in range(len(CATS))}
    lib.lh_prof_enable(0)
    loss_val = float(tr.step().toCPU()[0]); tr.end_step()
    peak_gb = lib.lh_heap_peak() / 2 ** 30
    fl = conv_flops(model, args.batch, args.hw)
    be.cleanup()
    return {"sec": t1 - t0, "conv_ms": conv_ms, "conv_calls": conv_calls, "conv_flops": fl, "breakdown": breakdown,
            "loss": loss_val, "arena_peak_gib": peak_gb}


def run_cpu(args):
    """The oracle (a C restatement of Lantern's BackendCPU: per-sample im2col + own SGEMM) on the
    host cores, same network and input shape, on a bounded sample: `cpu_batch` images per step."""
    import lantern_amd as la
    from oracle.backend_cpu import BackendCPU
    from lantern_amd.apps.resnet50 import ResNet50, Trainer
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
    be = BackendCPU(threads=threads)
    be.setup()
    la.set_backend(be)
    model = ResNet50(num_classes=args.classes, imagenet_stem=args.hw > 64)
    tr = Trainer(model, args.cpu_batch, args.hw, args.classes, lr=0.1, momentum=0.9)
    tr.step(); tr.end_step()                     # warm-up
    t0 = time.perf_counter()
    n = 0
    while n < args.cpu_steps:
        tr.step(); tr.end_step(); n += 1
        if time.perf_counter() - t0 > 30.0:
            break
    dt = time.perf_counter() - t0
    return {"value": args.cpu_batch * n / dt, "cores": threads, "steps": n}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--hw", type=int, default=224)
    ap.add_argument("--classes", type=int, default=1000)
    ap.add_argument("--heap-gb", type=float, default=48.0)
    ap.add_argument("--cpu-batch", type=int, default=4)
    ap.add_argument("--cpu-steps", type=int, default=2)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--verbose", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the reference is single-device; nothing here shards); use --gpus 1")

    g = run_gpu(args)
    ms_per_step = 1000.0 * g["sec"] / args.steps
    value = args.batch * args.steps / g["sec"]
    conv_time_s = sum(g["conv_ms"]) / 1000.0
    conv_fl = sum(g["conv_flops"])
    achieved = conv_fl / conv_time_s / 1e12 if conv_time_s > 0 else 0.0
    out = {
        "metric": "train samples/s (fwd+bwd+SGD), ResNet-50 b64 fp32; % of MFMA/HBM roofline",
        "value": round(value, 2), "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "ResNet-50 training step (configs[3]): batch %d, 3x%dx%d, %d classes, SGD lr 0.1 momentum 0.9, Kaiming-normal init"
                               % (args.batch, args.hw, args.hw, args.classes),
                   "global_batch": args.batch, "loss_after_run": round(g["loss"], 5), "arena_peak_gib": round(g["arena_peak_gib"], 2)},
        "roofline": {"bound": "mfma", "kernel": "k_igemm (conv fwd + bwd-data + bwd-filter, %d launches/step)" % sum(g["conv_calls"]),
                     "achieved": round(achieved, 2), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": None,
                     "flop_per_step": conv_fl, "ms_per_step": {"fwd": round(g["conv_ms"][0], 3), "bwd_data": round(g["conv_ms"][1], 3),
                                                               "bwd_filter": round(g["conv_ms"][2], 3)},
                     "tflops_by_pass": {k: round(f / (m / 1000.0) / 1e12, 2) if m > 0 else None
                                        for k, f, m in zip(("fwd", "bwd_data", "bwd_filter"), g["conv_flops"], g["conv_ms"])}},
    }
    if args.verbose:
        print(json.dumps(g["breakdown"], indent=1), file=sys.stderr)
    if not args.no_cpu:
        c = run_cpu(args)
        out["cpu_baseline"] = {"value": round(c["value"], 3), "unit": "samples/s", "cores": c["cores"], "kind": "port",
                               "sample": "same network and 3x%dx%d input, %d step(s) of batch %d (bounded sample; own SGEMM, not OpenBLAS)"
                                         % (args.hw, args.hw, c["steps"], args.cpu_batch)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
