#!/usr/bin/env python3
"""Benchmark: one training step (fwd + bwd + optimizer), fp32, synthetic data, on one MI355X through
the lantern_hip C ABI.  Default workload: ResNet-50, batch 64, 3x224x224, 1000 classes (the headline
configuration); `--workload` selects one of the other four application programs.

Prints ONE JSON line: training samples/s over the timed steps, the roofline fraction of the dominant
kernel family (measured live with HIP events on the library's stream around every launch, over a
second run of the same number of steps), and the CPU oracle timed on the host cores on a bounded
sample of the same workload.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload resnet50|squeezenet|lenet|treelstm|deepspeech2]
                  [--batch B] [--hw 224] [--no-cpu] [--verbose]
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

import numpy as np  # noqa: E402,F401

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
# conv kernels of the headline step under rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/resnet50_b64_hbm_traffic_and_mfma_counters.md)
# 16.85 GB read + 7.98 GB written per step over 158 launches.  The measured launch plans decide how many launches a step has
# (a strided input gradient runs as one grouped launch or one per residue class), the bytes of the step hardly depend on it.
PROFILED_TRAFFIC = {"bytes_per_step": 24.83e9, "launches_per_step": 158}
CATS = ["conv_fwd", "conv_bwd_data", "conv_bwd_filter", "gemm", "bn_fwd", "bn_bwd", "elementwise", "pool", "reduce", "optim", "fill", "rnn", "cmdlist"]

TREE_C_PROGRAM = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "host_c", "_build", "treelstm_step")
DEFAULT_BATCH = {"resnet50": 64, "squeezenet": 64, "lenet": 100, "treelstm": 1, "deepspeech2": 32}


def make_trainer(args, batch, cpu=False):
    """(trainer, samples per step, description).  `cpu`: the bounded sample for the oracle."""
    w = args.workload
    if w == "resnet50":
        from lantern_amd.apps.resnet50 import ResNet50, Trainer
        model = ResNet50(num_classes=args.classes, imagenet_stem=args.hw > 64)
        return Trainer(model, batch, args.hw, args.classes, lr=0.1, momentum=0.9, streamed=not cpu and not args.resident and not args.graph), batch, \
            "ResNet-50 training step (configs[3]): batch %d, 3x%dx%d, %d classes, SGD lr 0.1 momentum 0.9, Kaiming-normal init" % (batch, args.hw, args.hw, args.classes)
    if w == "squeezenet":
        from lantern_amd.apps.squeezenet import Trainer
        return Trainer(batch=batch, hw=32, num_classes=10, lr=0.005, momentum=0.9), batch, \
            "SqueezeNet training step (configs[2]): batch %d, 3x32x32, 10 classes, SGD lr 0.005 momentum 0.9" % batch
    if w == "lenet":
        from lantern_amd.apps.lenet import Trainer
        return Trainer(batch=batch, lr=0.0005), batch, "LeNet-style CNN training step (configs[0]): batch %d, 1x28x28, SGD lr 0.0005, dropout 0.5" % batch
    if w == "treelstm":
        from lantern_amd.apps.treelstm import Trainer
        if args.tree_file:
            from lantern_amd.apps.treelstm import read_trees
            return Trainer(vocab=20000, trees=read_trees(args.tree_file)), 1, \
                "TreeLSTM sentiment step (configs[1]): one tree of %s per step, hidden 150, embedding 300, Adagrad lr 0.05" % os.path.basename(args.tree_file)
        return Trainer(n_trees=64, vocab=20000), 1, \
            "TreeLSTM sentiment step (configs[1]): one tree of 5-50 leaves per step, hidden 150, embedding 300, Adagrad lr 0.05"
    if w == "deepspeech2":
        from lantern_amd.apps.deepspeech2 import Trainer
        # learning rate 1e-5: the reference program's 3e-4 (DeepSpeech.scala:127) diverges within ten steps on random spectrograms
        return Trainer(batch=batch, freq=161, frames=args.frames, hidden=args.hidden, layers=3, label_len=50, lr=1e-5), batch, \
            "DeepSpeech2-style step (configs[4]): batch %d, 1x161x%d, 3 bidirectional tanh RNN layers hidden %d with sequence-wise batch norm in front of layers 2 and 3 " \
            "(the reference program builds them with useBatchNorm = false), CTC over 29 symbols, Nesterov SGD lr 1e-5" % (batch, args.frames, args.hidden)
    raise SystemExit("unknown workload %r" % w)


def run_gpu(args):
    import lantern_amd as la
    be = la.BackendHIP(heap_bytes=int(args.heap_gb * (1 << 30)))
    be.setup()
    la.set_backend(be)
    tr, per_step, desc = make_trainer(args, args.batch)
    lib = be.lib
    if args.no_side_stream:
        lib.lh_set_side_stream(0)
    if args.deterministic:
        be.setDeterministic(True)
    if args.no_fusion:
        lib.lh_set_fusion(0)
    streamed = bool(getattr(tr, "streamed", False))
    loss_first = None
    for i in range(args.warmup):
        l = tr.step()
        if i == 0:
            loss_first = float(l.toCPU()[0])      # before any update: ln(classes) for a freshly initialised classifier
        tr.end_step()
    be.sync()
    if streamed:
        # The host link's clock ramps up under sustained traffic (the first ~0.5 s of per-step uploads run 2-4 % slower than the
        # steady state an epoch of thousands of steps sees): about a second of untimed uploads into a scratch buffer first.
        scratch = be.mallocArray(tr.hx[0].size, zero=False)
        t_w = time.perf_counter()
        while time.perf_counter() - t_w < 1.0:
            for _ in range(32):
                be.uploadAsync(scratch, tr.hx[1])
            be.sync()
        tr.end_step()
    t_issued = None
    resident_sec = None
    if args.graph:
        # the step recorded once (after the warm-up measured the launch plans) and replayed: one host call per step
        g = la.StepGraph(tr, eager_steps=0)
        g.launch(); be.sync()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            g.launch()
        be.sync()
        t1 = time.perf_counter()
        g.close()
    else:
        # the timed region: exactly `steps` steps, nothing else on the stream.  Streamed (the headline program): every step
        # uploads its batch from pinned host memory and reads its loss back, as the reference's loop does.
        t0 = time.perf_counter()
        for _ in range(args.steps):
            tr.step()
            tr.end_step()
        t_issued = time.perf_counter()      # the host has enqueued everything; the device may still be working
        be.sync()
        t1 = time.perf_counter()
        if streamed:
            assert np.isfinite(tr.losses()[-min(args.steps, tr.LOSS_RING):]).all(), "a streamed step's loss did not arrive"
            # the same steps on a resident batch, no upload and no read-back (second figure; not the metric)
            tr.streamed = False
            tr.step(); tr.end_step(); be.sync()
            r0 = time.perf_counter()
            for _ in range(args.steps):
                tr.step()
                tr.end_step()
            be.sync()
            resident_sec = time.perf_counter() - r0
    # the same `steps` steps again with a HIP event pair around every matrix-kernel launch (conv x3, gemm, rnn).
    # Kept out of the timed region: an event between two launches drains the pipeline and costs about 1 ms per step.
    # (a program that runs from the command list times only the interpreter launches: an event elsewhere would cut the list short)
    lib.lh_prof_enable((1 << CATS.index("cmdlist")) if getattr(tr, "batching", False) else (0b1111 | (1 << CATS.index("rnn"))))
    ms = (C.c_double * len(CATS))(); calls = (C.c_int64 * len(CATS))()
    lib.lh_prof_collect(ms, calls, len(CATS))       # reset
    be.work = {}; be.count_work = True
    for _ in range(args.steps):
        tr.step()
        tr.end_step()
    be.sync()
    lib.lh_prof_collect(ms, calls, len(CATS))
    timed = {CATS[i]: (ms[i] / args.steps, int(calls[i]) // args.steps) for i in range(len(CATS))}
    work = {k: v / args.steps for k, v in be.work.items()}
    be.count_work = False
    # the same again around the HBM-bound families (batch norm forward / backward, element-wise, pooling, optimizer)
    hbm_cats = ("bn_fwd", "bn_bwd", "elementwise", "pool", "optim")
    timed_hbm = {}
    if not getattr(tr, "batching", False):
        lib.lh_prof_enable(sum(1 << CATS.index(c) for c in hbm_cats))
        lib.lh_prof_collect(ms, calls, len(CATS))
        wb = (C.c_double * len(CATS))()
        lib.lh_work_collect(wb, len(CATS))          # reset: the library counts the algorithmic bytes of the kernels it chooses to run
        for _ in range(args.steps):
            tr.step()
            tr.end_step()
        be.sync()
        lib.lh_prof_collect(ms, calls, len(CATS))
        lib.lh_work_collect(wb, len(CATS))
        timed_hbm = {c: (ms[CATS.index(c)] / args.steps, int(calls[CATS.index(c)]) // args.steps) for c in hbm_cats}
        for c, key in (("bn_fwd", "bn_fwd_bytes"), ("bn_bwd", "bn_bwd_bytes"), ("elementwise", "elementwise_bytes")):
            work[key] = wb[CATS.index(c)] / args.steps
    # a separate, untimed pass with every category instrumented (breakdown for the log)
    lib.lh_prof_enable((1 << CATS.index("cmdlist")) if getattr(tr, "batching", False) else (1 << len(CATS)) - 1)
    tr.step(); tr.end_step()
    lib.lh_prof_collect(ms, calls, len(CATS))
    breakdown = {CATS[i]: {"ms": round(ms[i], 3), "calls": int(calls[i])} for i in range(len(CATS))}
    lib.lh_prof_enable(0)
    loss_val = float(tr.step().toCPU()[0]); tr.end_step()
    peak_gb = lib.lh_heap_peak() / 2 ** 30
    fstats = (C.c_int64 * 8)()
    lib.lh_fusion_stats(fstats, 8)
    unfused_sec = None
    if args.workload == "resnet50" and not args.no_fusion and not args.graph:
        # the same steps with the library running every call as issued (no chains fused, every lh_malloc cleared, every
        # gradient accumulated, one optimizer launch per parameter): what the call sequence costs without the deferred work
        lib.lh_set_fusion(0)
        tr.step(); tr.end_step(); be.sync()
        u0 = time.perf_counter()
        for _ in range(args.steps):
            tr.step()
            tr.end_step()
        be.sync()
        unfused_sec = time.perf_counter() - u0
        lib.lh_set_fusion(1)
    c_host = None
    c_dir = None
    if args.workload == "treelstm" and os.path.exists(TREE_C_PROGRAM):
        # the same loop as a plain-C host program over the C-ABI (what the reference's generated code is): fresh parameters of the
        # same distribution, the same trees; it runs after this process has released the device
        import tempfile
        from lantern_amd.apps.treelstm import write_c_program_inputs
        c_dir = args.keep_c_inputs or tempfile.mkdtemp(prefix="lantern_treelstm_")
        os.makedirs(c_dir, exist_ok=True)
        tr.close(); tr.end_step()
        tr2, _, _ = make_trainer(args, args.batch)
        write_c_program_inputs(c_dir, tr2)
        tr2.close()
    emitted = None
    if args.c_host and args.workload != "treelstm":
        # the step written out as straight-line C (what the reference's LMS back end emits), compiled, and timed after this process
        # has released the device: the library without the Python mirror between two calls
        import tempfile
        from lantern_amd import emit_c
        e_dir = tempfile.mkdtemp(prefix="lantern_emitted_")
        text, data, tr3, _ = emit_c.record(lambda: make_trainer(args, args.batch)[0], be, desc, be.heap_bytes,
                                           frame=(["lh_set_deterministic(1);"] if args.deterministic else []) + (["lh_set_side_stream(0);"] if args.no_side_stream else []))
        open(os.path.join(e_dir, "step.c"), "w").write(text)
        open(os.path.join(e_dir, "data.bin"), "wb").write(data)
        emitted = (e_dir, text.count("\n"))
    be.cleanup()
    if emitted is not None:
        import subprocess, shutil
        e_dir, lines = emitted
        exe = os.path.join(e_dir, "step")
        cc = subprocess.run(emit_c.compile_line(os.path.dirname(os.path.abspath(__file__)), os.path.join(e_dir, "step.c"), exe), capture_output=True, text=True)
        if cc.returncode != 0:
            sys.exit("bench.py: the emitted C program does not compile: " + cc.stderr[-2000:])
        r = subprocess.run([exe, os.path.join(e_dir, "data.bin"), str(args.steps), str(args.warmup)], capture_output=True, text=True, timeout=900)
        if r.returncode != 0 or not r.stdout.startswith("ms_per_step"):
            sys.exit("bench.py: the emitted C program failed: " + r.stdout + r.stderr)
        f = r.stdout.split()
        emitted = {"ms_per_step": float(f[1]), "value": round(per_step / (float(f[1]) / 1000.0), 2), "first_loss": float(f[5]), "last_loss": float(f[7]), "lines_of_c": lines,
                   "note": "the same step written out by lantern_amd/emit_c.py as a plain-C host program (one library call per operator, the loss read back with a wait every step), "
                           "compiled with gcc and run on its own after this process released the device"}
        shutil.rmtree(e_dir, ignore_errors=True)
    if c_dir is not None:
        import subprocess
        r = subprocess.run([TREE_C_PROGRAM, os.path.join(c_dir, "params.bin"), os.path.join(c_dir, "trees.txt"), os.path.join(c_dir, "out.bin"),
                            str(args.steps), str(args.warmup), "1"], capture_output=True, text=True, timeout=600)
        if r.returncode != 0 or not r.stdout.startswith("trees_per_s"):
            sys.exit("bench.py: the C host program failed: " + r.stdout + r.stderr)
        f = r.stdout.split()
        c_host = {"trees_per_s": float(f[1]), "ms_per_tree": float(f[3]), "host_issue_ms_per_tree": float(f[7])}
        losses = np.fromfile(os.path.join(c_dir, "out.bin"), np.float32, count=args.steps)
        assert np.isfinite(losses).all() and (losses > 0).all(), "the C host program's losses"
        if not args.keep_c_inputs:
            import shutil
            shutil.rmtree(c_dir, ignore_errors=True)
    return {"fusion_stats": [int(v) for v in fstats], "unfused_sec": unfused_sec, "emitted": emitted, "c_host": c_host, "streamed": streamed, "resident_sec": resident_sec, "timed_hbm": timed_hbm, "sec": t1 - t0, "issue_sec": (t_issued - t0) if t_issued is not None else None, "timed": timed, "work": work, "breakdown": breakdown, "loss": loss_val, "loss_first": loss_first, "arena_peak_gib": peak_gb,
            "per_step": per_step, "desc": desc}


def run_cpu(args):
    """The oracle (a C restatement of Lantern's BackendCPU: per-sample im2col + own SGEMM) on the
    host cores, same program and input shape, on a bounded sample (a smaller batch, a few steps)."""
    import lantern_amd as la
    from oracle.backend_cpu import BackendCPU
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
    be = BackendCPU(threads=threads)
    be.setup()
    la.set_backend(be)
    batch = {"resnet50": args.cpu_batch, "squeezenet": 64, "lenet": 100, "treelstm": 1, "deepspeech2": 4}[args.workload]
    tr, per_step, _ = make_trainer(args, batch, cpu=True)
    if args.workload == "treelstm":              # the very trees the device run times: W warm-up trees, then the next K, three times over
        for _ in range(args.warmup):
            tr.step(); tr.end_step()
        t0 = time.perf_counter()
        n = 0
        for _ in range(3):
            tr.next = args.warmup
            for _ in range(args.steps):
                tr.step(); tr.end_step(); n += 1
        dt = time.perf_counter() - t0
        return {"value": per_step * n / dt, "cores": threads, "steps": n, "batch": batch}
    tr.step(); tr.end_step()                     # warm-up
    max_steps = {"resnet50": args.cpu_steps, "squeezenet": 30, "lenet": 200, "deepspeech2": 4}[args.workload]
    t0 = time.perf_counter()
    n = 0
    while n < max_steps:
        tr.step(); tr.end_step(); n += 1
        if time.perf_counter() - t0 > 25.0:
            break
    dt = time.perf_counter() - t0
    return {"value": per_step * n / dt, "cores": threads, "steps": n, "batch": batch}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="resnet50", choices=sorted(DEFAULT_BATCH))
    ap.add_argument("--batch", type=int, default=0)
    ap.add_argument("--hw", type=int, default=224)
    ap.add_argument("--classes", type=int, default=1000)
    ap.add_argument("--frames", type=int, default=400)
    ap.add_argument("--hidden", type=int, default=800)
    ap.add_argument("--heap-gb", type=float, default=48.0)
    ap.add_argument("--cpu-batch", type=int, default=8)
    ap.add_argument("--cpu-steps", type=int, default=4)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--c-host", action="store_true", help="also write the step out as a plain-C host program (lantern_amd/emit_c.py), compile and time it: "
                    "the library without the Python mirror between two calls (fixed-shape workloads; needs gcc)")
    ap.add_argument("--keep-c-inputs", default=None, help="treelstm: write the C host program's input files (params.bin, trees.txt) into this directory and leave them there")
    ap.add_argument("--tree-file", default=None, help="treelstm: trees in the reference's array_tree.txt format instead of random ones (tests/golden/array_tree_first24.txt)")
    ap.add_argument("--no-side-stream", action="store_true", help="filter gradients in line on the main stream (kernel profiles: no two kernels overlap)")
    ap.add_argument("--resident", action="store_true", help="resnet50: keep one batch resident on the device (no per-step upload, no loss read-back)")
    ap.add_argument("--deterministic", action="store_true", help="fixed-order reductions and rule-chosen launch plans (lh_set_deterministic): what run-to-run bit equality costs")
    ap.add_argument("--no-fusion", action="store_true", help="lh_set_fusion(0): every library call runs as issued (no chains fused, every block cleared when handed out)")
    ap.add_argument("--graph", action="store_true", help="time replays of the step recorded into a HIP graph (fixed-shape workloads)")
    ap.add_argument("--verbose", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the reference is single-device; nothing here shards); use --gpus 1")
    if args.batch <= 0:
        args.batch = DEFAULT_BATCH[args.workload]

    g = run_gpu(args)
    ms_per_step = 1000.0 * g["sec"] / args.steps
    value = g["per_step"] * args.steps / g["sec"]
    python_host = None
    if g.get("c_host"):
        # TreeLSTM issues ~7000 operator calls per tree: from Python the host is the bound, so the figure of the library is the
        # one measured from the C host program; the Python mirror's is kept beside it
        python_host = {"value": round(value, 2), "ms_per_step": round(ms_per_step, 3), "host_issue_ms_per_step": round(1000.0 * g["issue_sec"] / args.steps, 3)}
        value, ms_per_step = g["c_host"]["trees_per_s"], g["c_host"]["ms_per_tree"]
        g["issue_sec"] = g["c_host"]["host_issue_ms_per_tree"] * args.steps / 1000.0
    timed, work = g["timed"], g["work"]
    conv_ms = [timed[k][0] for k in ("conv_fwd", "conv_bwd_data", "conv_bwd_filter")]
    conv_calls = sum(timed[k][1] for k in ("conv_fwd", "conv_bwd_data", "conv_bwd_filter"))
    if args.workload == "treelstm":
        # matrix-vector path: the weight matrices are streamed once per product; the whole tree runs from the command
        # list (one workgroup interpreting ~90 small operations per node), so the step is latency-bound, not HBM-bound
        t = timed["cmdlist"][0] / 1000.0
        achieved = work.get("gemv_bytes", 0.0) / t / 1e9 if t > 0 else 0.0
        roof = {"bound": "hbm", "kernel": "k_cmdlist (%d interpreter launches/step running the gemv / rank-1 update / element-wise commands level by level "
                                          "over the library's workgroups; bound by memory round trips and the barrier per level at these sizes; timed under the Python mirror)" % timed["cmdlist"][1],
                "achieved": round(achieved, 2), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBS, 5), "traffic": None,
                "bytes_per_step": work.get("gemv_bytes", 0.0), "ms_per_step": round(timed["cmdlist"][0], 3)}
    else:
        conv_fl = work.get("conv_flop", 0.0)
        conv_t = sum(conv_ms) / 1000.0
        achieved = conv_fl / conv_t / 1e12 if conv_t > 0 else 0.0
        roof = {"bound": "mfma", "kernel": "k_igemm (conv fwd + bwd-data + bwd-filter, %d launches/step)" % conv_calls,
                "achieved": round(achieved, 2), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
                # HBM bytes per launch come from separate rocprofv3 FETCH_SIZE / WRITE_SIZE runs (profiles/), which this process cannot
                # make: the profiled bytes of a step over THIS run's launches per step, and only when that count is within
                # 5 % of the profiled run's (the same step, at most a few launches cut differently); otherwise null
                "traffic": round(PROFILED_TRAFFIC["bytes_per_step"] / conv_calls) if (args.workload == "resnet50" and args.batch == 64 and args.hw == 224 and not args.deterministic
                                                                    and conv_calls > 0 and abs(conv_calls - PROFILED_TRAFFIC["launches_per_step"]) <= 0.05 * PROFILED_TRAFFIC["launches_per_step"]) else None,
                "flop_per_step": conv_fl,
                "ms_per_step": {"fwd": round(conv_ms[0], 3), "bwd_data": round(conv_ms[1], 3), "bwd_filter": round(conv_ms[2], 3)}}
        # the HBM-bound families against the 8 TB/s peak: algorithmic bytes of what was issued / event-timed kernel time
        th = g["timed_hbm"]
        hbm = {}
        for fam, key in (("bn_fwd", "bn_fwd_bytes"), ("bn_bwd", "bn_bwd_bytes"), ("elementwise", "elementwise_bytes")):
            if fam in th and th[fam][0] > 0 and work.get(key, 0.0) > 0:
                gbs = work[key] / (th[fam][0] / 1000.0) / 1e9
                hbm[fam] = {"bytes_per_step": work[key], "ms_per_step": round(th[fam][0], 3), "launches": th[fam][1], "achieved": round(gbs, 1),
                            "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4)}
        for fam in ("pool", "optim"):
            if fam in th and th[fam][0] > 0:
                hbm[fam] = {"ms_per_step": round(th[fam][0], 3), "launches": th[fam][1]}
        if hbm:
            roof["hbm"] = hbm
        if work.get("gemm_flop", 0.0) > 0 and timed["gemm"][0] > 0:
            roof["gemm"] = {"flop_per_step": work["gemm_flop"], "ms_per_step": round(timed["gemm"][0], 3),
                            "tflops": round(work["gemm_flop"] / (timed["gemm"][0] / 1000.0) / 1e12, 2)}
        if timed["rnn"][0] > 0:
            roof["rnn_recurrence"] = {"flop_per_step": work.get("rnn_flop", 0.0), "ms_per_step": round(timed["rnn"][0], 3), "launches": timed["rnn"][1]}
    unit = "trees/s" if args.workload == "treelstm" else "samples/s"
    out = {
        "metric": "train samples/s (fwd+bwd+SGD), ResNet-50 b64 fp32; % of MFMA/HBM roofline" if args.workload == "resnet50"
                  else "train %s (fwd+bwd+optimizer), %s fp32; %% of MFMA/HBM roofline" % (unit, args.workload),
        "value": round(value, 2), "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": g["desc"], "global_batch": args.batch, "loss_first_step": round(g["loss_first"], 5) if g["loss_first"] is not None else None, "loss_after_run": round(g["loss"], 5), "arena_peak_gib": round(g["arena_peak_gib"], 2),
                   "launch": "hip graph replay" if args.graph else "one launch per kernel",
                   "calls": "one library call per Backend trait method (conv2D_batch, batchNormTraining, relu in place, +, one momentum_update per parameter; "
                            "every buffer from lh_malloc, every gradient accumulated): what scala/TensorDslHIP.scala emits; the library fuses the chains" +
                            (" (fusion switched OFF for this run)" if args.no_fusion else ""),
                   "host_issue_ms_per_step": round(1000.0 * g["issue_sec"] / args.steps, 3) if g["issue_sec"] is not None else None,
                   "h2d": ("included: the batch (%.1f MB) is uploaded from pinned host memory for every step on a copy stream, beside the previous step; "
                           "the loss is read back every step without a wait" % (args.batch * 3 * args.hw * args.hw * 4 / 1e6)) if g["streamed"] else "not included: inputs resident on the device",
                   "filter_gradients": "in line" if (args.no_side_stream or args.deterministic) else "side stream",
                   "reductions": "deterministic (two-pass, rule-chosen plans)" if args.deterministic else "atomic combine, measured plans"},
        "roofline": roof,
    }
    if python_host is not None:
        out["config"]["host"] = "plain-C host program over the C-ABI (tests/host_c/treelstm_step.c): the reference's generated-code shape, command list on"
        out["python_mirror_host"] = python_host
    if g.get("emitted"):
        out["emitted_c_program"] = g["emitted"]
    if g.get("unfused_sec"):
        out["calls_run_as_issued"] = {"value": round(g["per_step"] * args.steps / g["unfused_sec"], 2), "ms_per_step": round(1000.0 * g["unfused_sec"] / args.steps, 3),
                                      "note": "the same call sequence with lh_set_fusion(0): nothing fused, every lh_malloc cleared at once, gradients accumulated, 161 optimizer launches"}
    fs = g.get("fusion_stats")
    if fs:
        out["config"]["library_fusion_totals"] = {"forward_chains": fs[0], "backward_chains": fs[1], "optimizer_calls_gathered": fs[2], "zero_fills_avoided": fs[3],
                                                  "zero_fills_done": fs[4], "results_produced_on_demand": fs[5], "chains_ended_without_relu": fs[6], "filter_copies_reused": fs[7]}
    if g["resident_sec"] is not None:
        out["resident_input"] = {"value": round(g["per_step"] * args.steps / g["resident_sec"], 2), "ms_per_step": round(1000.0 * g["resident_sec"] / args.steps, 3),
                                 "note": "the same steps with the batch resident on the device: no upload, no loss read-back"}
    if args.verbose:
        print(json.dumps(g["breakdown"], indent=1), file=sys.stderr)
    if not args.no_cpu:
        c = run_cpu(args)
        out["cpu_baseline"] = {"value": round(c["value"], 3), "unit": unit, "cores": c["cores"], "kind": "port",
                               "sample": "same program and input shape, %d step(s) of batch %d (bounded sample; own SGEMM, not OpenBLAS)" % (c["steps"], c["batch"])}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
