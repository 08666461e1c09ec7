"""A training program of the host mirror written out as a plain-C host program over the C-ABI.

Lantern's LMS back end does not interpret a model: it emits straight-line C++ (`void Snippet(char*)`, DslGenC in
TensorDifferentiation.scala:1540-1700 and the `unchecked(...)` library calls of TensorDslCublas.scala:171-560) in which every operator
of one training step is one library call with its shapes as literals, and the step sits in a loop.  This module produces the same
shape of program for any fixed-shape application of `lantern_amd.apps`: the application runs one step through a recorder that stands
in for the ctypes library (every call is forwarded to the real library and noted with its arguments), and the noted calls are written
as C: arena blocks become variables (`void* p17 = lh_malloc(1048576);`), device pointers become a variable plus an offset, shapes and
scalars become literals (floats as C99 hexadecimal literals, so nothing is rounded), small host arrays (dims, permutations, pointer
tables) become initialised local arrays, and everything the application uploads (initial parameters, the synthetic batch) goes into one
data file the program reads at start.  The result links against liblantern_hip.so and nothing else: no Python, no interpreter between
two library calls, which is what the reference's generated programs are and what the library's host-side cost should be measured with.

Programs whose call sequence depends on the data (the TreeLSTM's recursion over a tree) are not straight-line code; that one is written
by hand (tests/host_c/treelstm_step.c).

    python -m lantern_amd.emit_c squeezenet out_dir [--batch 64]      # writes out_dir/step.c and out_dir/data.bin, prints the cc line
"""
import ctypes as C
import os
import struct

import numpy as np

from . import _lib

P, I, F, L, Z, U64 = _lib.P, _lib.I, _lib.F, _lib.L, _lib.Z, _lib.U64

# Host arrays behind pointer arguments: name -> [(argument index, element kind, how many elements given the argument list)].
# Kinds: "int" (int32), "i64", "float", "dev" (a table of device pointers).
_rank = lambda pos: (lambda a: a[pos])
HOST_ARRAYS = {
    "lh_mask4d": [(1, "int", lambda a: a[2])],
    "lh_bcast_op": [(2, "int", _rank(7)), (4, "int", _rank(7)), (6, "int", _rank(7))],
    "lh_bcast_op_grad": [(3, "int", _rank(11)), (7, "int", _rank(11)), (10, "int", _rank(11))],
    "lh_bcast_update": [(2, "int", _rank(5)), (4, "int", _rank(5))],
    "lh_permute": [(2, "int", _rank(4)), (3, "int", _rank(4))],
    "lh_permute_grad": [(2, "int", _rank(4)), (3, "int", _rank(4))],
    "lh_concat": [(1, "dev", _rank(0)), (2, "int", _rank(0))],
    "lh_concat_grad": [(1, "dev", _rank(0)), (2, "int", _rank(0))],
    "lh_concat_grad_beta": [(1, "dev", _rank(0)), (2, "float", _rank(0)), (3, "int", _rank(0))],
    "lh_multi_momentum": [(1, "dev", _rank(0)), (2, "dev", _rank(0)), (3, "dev", _rank(0)), (4, "i64", _rank(0))],
    "lh_multi_momentum_static": [(1, "dev", _rank(0)), (2, "dev", _rank(0)), (3, "dev", _rank(0)), (4, "i64", _rank(0))],
    "lh_multi_sgd": [(1, "dev", _rank(0)), (2, "dev", _rank(0)), (3, "i64", _rank(0))],
    "lh_ctc_loss": [(2, "int", None), (3, "int", _rank(7)), (4, "int", _rank(7))],       # labels: as many as the label lengths add up to
}
UPLOADS = {"lh_h2d": (0, 1, 2), "lh_h2d_async": (0, 1, 2)}          # (device argument, host argument, byte count argument)
DOWNLOADS = {"lh_d2h": (0, 1, 2), "lh_d2h_async": (0, 1, 2)}        # (host argument, device argument, byte count argument)
ALLOCATORS = ("lh_malloc", "lh_malloc_uninit")
# calls that only report (or that the program's own frame makes): forwarded, not written out
SILENT = {"lh_last_error", "lh_clear_error", "lh_set_error_mode", "lh_heap_used", "lh_heap_peak", "lh_prof_enable", "lh_prof_collect",
          "lh_tune_counters", "lh_event_create", "lh_event_record", "lh_event_elapsed_ms", "lh_event_destroy", "lh_side_forks",
          "lh_get_deterministic", "lh_cmdlist_stats", "lh_rnn_gated_reserve_floats", "lh_setup", "lh_cleanup"}
_CTYPE = {"int": ("int", C.c_int32, "%d"), "i64": ("int64_t", C.c_int64, "%dLL"), "float": ("float", C.c_float, None)}


def _address(v):
    if v is None:
        return 0
    if isinstance(v, int):
        return v
    if isinstance(v, np.ndarray):
        return v.ctypes.data
    got = C.cast(v, C.c_void_p).value
    return got or 0


def _float_literal(v):
    v = float(np.float32(v))
    if v != v:
        return "NAN"
    if v in (float("inf"), float("-inf")):
        return "INFINITY" if v > 0 else "-INFINITY"
    return float.hex(v) + "f"


class Recorder:
    """Stands in for the ctypes library: forwards every call, notes what a C program must do to repeat it."""

    def __init__(self, lib):
        self._lib = lib
        self.blocks = []            # live arena blocks: (address, bytes, variable name, arena bytes in use once it was handed out)
        self.pinned = []            # (address, bytes, variable name, [digest of what was last copied into it])
        self.marks = {}             # mark value -> variable name
        self.phase = "init"
        self.code = {"init": [], "step": []}
        self.globals = []           # variables made in init and used by the step
        self.data = bytearray()
        self.nvar = 0
        self.last_download = None
        self.max_download = 0

    # ---- naming -----------------------------------------------------------------------------------------------------------------
    def _new(self, prefix):
        self.nvar += 1
        return "%s%d" % (prefix, self.nvar)

    def _declare(self, ctype, name):
        if self.phase == "init":
            self.globals.append("static %s %s;" % (ctype, name))
            return name
        return "%s %s" % (ctype, name)

    def _device(self, addr):
        if addr == 0:
            return "NULL"
        for base, size, name, _ in reversed(self.blocks):
            if base <= addr < base + size:
                return "(void*)((char*)%s + %d)" % (name, addr - base) if addr != base else name
        raise ValueError("address %#x is in no live arena block (a device pointer the recorder did not see allocated)" % addr)

    def _pinned(self, addr):
        for base, size, name, _ in self.pinned:
            if base <= addr < base + size:
                return base, name, addr - base
        return None

    def _stash(self, raw):
        off = len(self.data)
        self.data += raw
        self.data += b"\0" * (-len(self.data) % 64)
        return off

    def emit(self, line):
        self.code[self.phase].append(line)

    # ---- the calls ----------------------------------------------------------------------------------------------------------------
    def __getattr__(self, name):
        fn = getattr(self._lib, name)
        if not name.startswith("lh_") or name not in _lib.SIGNATURES:
            return fn
        res, argtypes = _lib.SIGNATURES[name]

        def call(*args):
            pre = self._before(name, argtypes, args) if name not in SILENT else None
            out = fn(*args)
            if name not in SILENT:
                self._after(name, args, out, pre)
            return out
        return call

    def _before(self, name, argtypes, args):
        """The argument texts (host memory is read now: the call may change it, the caller may reuse it)."""
        texts, setup = [], []
        plain = [a.value if hasattr(a, "value") and not isinstance(a, (C.Array, C._Pointer)) else a for a in args]
        host = {i: (kind, count) for i, kind, count in HOST_ARRAYS.get(name, [])}
        up, down = UPLOADS.get(name), DOWNLOADS.get(name)
        for i, (t, a) in enumerate(zip(argtypes, plain)):
            if t is F:
                texts.append(_float_literal(a))
            elif t in (I, L, Z, U64, C.c_uint):
                v = int(a)
                if name == "lh_rewind" and v in self.marks:
                    texts.append(self.marks[v])
                else:
                    texts.append("%d%s" % (v, "ULL" if t is U64 else ("LL" if t is L else "")))
            elif t is P or (isinstance(t, type) and issubclass(t, C._Pointer)):
                addr = _address(a)
                if i in host and addr:
                    kind, count = host[i]
                    n = int(count(plain)) if count is not None else int(sum(np.ctypeslib.as_array(C.cast(_address(plain[3]), C.POINTER(C.c_int32)), (int(plain[7]),))))
                    var = self._new("t")
                    if kind == "dev":
                        vals = np.ctypeslib.as_array(C.cast(addr, C.POINTER(C.c_uint64)), (n,)) if n else []
                        setup.append("void* %s[%d] = {%s};" % (var, max(n, 1), ", ".join(self._device(int(v)) for v in vals)))
                    else:
                        cname, ct, fmt = _CTYPE[kind]
                        vals = np.ctypeslib.as_array(C.cast(addr, C.POINTER(ct)), (n,)) if n else []
                        body = ", ".join(_float_literal(v) if kind == "float" else fmt % int(v) for v in vals)
                        setup.append("%s %s[%d] = {%s};" % (cname, var, max(n, 1), body))
                    texts.append("(void*)%s" % var if kind == "dev" else var)
                elif up and i == up[1]:
                    nbytes = int(plain[up[2]])
                    pin = self._pinned(addr)
                    raw = C.string_at(addr, nbytes)
                    if pin:                      # a pinned buffer the program fills itself: the bytes are copied in when they change
                        base, var, off = pin
                        slot = [p for p in self.pinned if p[0] == base][0][3]
                        digest = hash(raw)
                        if slot.get(off) != digest:
                            slot[off] = digest
                            setup.append("memcpy((char*)%s + %d, DATA + %d, %d);" % (var, off, self._stash(raw), nbytes))
                        texts.append("(void*)((char*)%s + %d)" % (var, off))
                    else:
                        texts.append("(void*)(DATA + %d)" % self._stash(raw))
                elif down and i == down[0]:
                    nbytes = int(plain[down[2]])
                    pin = self._pinned(addr)
                    self.max_download = max(self.max_download, nbytes)
                    texts.append("(void*)((char*)%s + %d)" % (pin[1], pin[2]) if pin else "(void*)DOWNLOAD")
                    self.last_download = texts[-1]
                else:
                    texts.append(self._device(addr))
            else:
                raise TypeError("%s: argument %d has a type the emitter does not know (%r)" % (name, i, t))
        return texts, setup

    def _after(self, name, args, out, pre):
        texts, setup = pre
        call = "%s(%s)" % (name, ", ".join(texts))
        if name in ALLOCATORS:
            var = self._new("p")
            size = int(args[0].value if hasattr(args[0], "value") else args[0])
            self.blocks.append((int(out or 0), size, var, int(self._lib.lh_heap_used())))
            self.emit("%s = %s;" % (self._declare("void*", var), call))
        elif name == "lh_host_alloc":
            var = self._new("h")
            size = int(args[0].value if hasattr(args[0], "value") else args[0])
            self.pinned.append((int(out or 0), size, var, {}))
            self.emit("%s = %s;" % (self._declare("void*", var), call))
        elif name == "lh_host_free":
            addr = _address(args[0])
            hit = [p for p in self.pinned if p[0] == addr]
            if hit:
                self.pinned.remove(hit[0])
                self.emit("lh_host_free(%s);" % hit[0][2])
        elif name == "lh_mark":
            var = self._new("m")
            self.marks[int(out)] = var
            self.emit("%s = lh_mark();" % self._declare("size_t", var))
        else:
            for line in setup:
                self.emit(line)
            self.emit(call + ";")
            if name in ("lh_rewind", "lh_free_top"):        # the blocks handed out above what is still in use are gone: their addresses come again
                used = int(self._lib.lh_heap_used())
                while self.blocks and self.blocks[-1][3] > used:
                    self.blocks.pop()


PROGRAM = r'''/* Written by lantern_amd/emit_c.py from one recorded training step of `%(what)s`: one library call per operator, shapes as
 * literals, the step in a loop, as the reference's LMS back end emits its programs.
 *   cc -O2 -std=c99 -I<repo>/include step.c -L<repo>/lantern_amd/csrc -llantern_hip -Wl,-rpath,<repo>/lantern_amd/csrc -o step
 *   ./step data.bin <steps> <warm-up steps> [losses.bin] */
#define _POSIX_C_SOURCE 199309L
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#include "lantern_hip.h"

static char* DATA;
static char DOWNLOAD[%(download)d];
%(globals)s

static void init(void) {
%(init)s
}

static float step(void) {
%(step)s
  float loss; memcpy(&loss, %(loss_from)s, sizeof loss);
  return loss;
}

static double now_s(void) { struct timespec ts; clock_gettime(CLOCK_MONOTONIC, &ts); return ts.tv_sec + 1e-9 * ts.tv_nsec; }

int main(int argc, char** argv) {
  if (argc < 4) { fprintf(stderr, "usage: %%s data.bin steps warmup [losses.bin]\n", argv[0]); return 2; }
  FILE* f = fopen(argv[1], "rb");
  if (!f) { perror(argv[1]); return 2; }
  DATA = (char*)malloc(%(data_bytes)dUL);
  if (!DATA || fread(DATA, 1, %(data_bytes)dUL, f) != %(data_bytes)dUL) { fprintf(stderr, "%%s: short file\n", argv[1]); return 2; }
  fclose(f);
  const int steps = atoi(argv[2]), warmup = atoi(argv[3]);
  lh_setup(%(heap)dUL);
%(frame)s
  init();
  float* losses = (float*)calloc((size_t)(steps + warmup) + 1, sizeof(float));
  for (int i = 0; i < warmup; i++) losses[i] = step();
  lh_sync();
  const double t0 = now_s();
  for (int i = 0; i < steps; i++) losses[warmup + i] = step();
  lh_sync();
  const double t1 = now_s();
  const char* err = lh_last_error();
  if (err && err[0]) { fprintf(stderr, "library error: %%s\n", err); return 1; }
  printf("ms_per_step %%.4f steps %%d first_loss %%.9g last_loss %%.9g\n", (t1 - t0) / (steps > 0 ? steps : 1) * 1e3, steps, losses[0], losses[steps + warmup - 1]);
  if (argc > 4) { FILE* o = fopen(argv[4], "wb"); if (!o) { perror(argv[4]); return 2; } fwrite(losses, sizeof(float), (size_t)(steps + warmup), o); fclose(o); }
  lh_cleanup();
  return 0;
}
'''


def record(make_trainer, be, what, heap_bytes, frame=()):
    """Runs `make_trainer()` and two steps of it on backend `be` (set up, current) through a recorder; returns (C text, data bytes, the
    trainer, the losses of those two steps).  `frame`: C statements for main() between lh_setup and init (modes the caller turned on)."""
    real = _lib._lib
    rec = Recorder(real)
    _lib._lib = rec
    be.lib = rec
    try:
        trainer = make_trainer()
        first = float(trainer.step().toCPU()[0]); trainer.end_step()          # the first step may allocate what later steps reuse: it stays in init
        rec.phase = "step"
        second = float(trainer.step().toCPU()[0]); trainer.end_step()
    finally:
        _lib._lib = real
        be.lib = real
    if rec.last_download is None:
        raise RuntimeError("the step read nothing back: there is no loss to report")
    indent = lambda lines: "\n".join("  " + l for l in lines)
    text = PROGRAM % {"what": what, "download": max(rec.max_download, 4), "globals": "\n".join(rec.globals), "init": indent(rec.code["init"]),
                      "step": indent(rec.code["step"]), "loss_from": rec.last_download, "data_bytes": len(rec.data), "heap": heap_bytes,
                      "frame": indent(frame)}
    return text, bytes(rec.data), trainer, (first, second)


def compile_line(repo, src, exe):
    csrc = os.path.join(repo, "lantern_amd", "csrc")
    return ["gcc", "-O1", "-std=c99", "-I" + os.path.join(repo, "include"), src, "-L" + csrc, "-llantern_hip", "-lm", "-Wl,-rpath," + csrc, "-o", exe]


def main():
    import argparse
    import lantern_amd as la
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("workload", choices=["resnet50", "squeezenet", "lenet", "deepspeech2"])
    ap.add_argument("out_dir")
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--heap-gb", type=float, default=None)
    args = ap.parse_args()
    batch = args.batch or {"resnet50": 64, "squeezenet": 64, "lenet": 100, "deepspeech2": 32}[args.workload]
    heap = int((args.heap_gb or {"resnet50": 40, "squeezenet": 4, "lenet": 1, "deepspeech2": 16}[args.workload]) * (1 << 30))
    be = la.BackendHIP(heap_bytes=heap)
    be.setup(); la.set_backend(be)

    def make():
        if args.workload == "resnet50":
            from .apps.resnet50 import ResNet50, Trainer
            return Trainer(ResNet50(num_classes=1000, imagenet_stem=True), batch, 224, 1000, lr=0.1, momentum=0.9, streamed=True)
        if args.workload == "squeezenet":
            from .apps.squeezenet import Trainer
            return Trainer(batch=batch, hw=32, num_classes=10, lr=0.005, momentum=0.9)
        if args.workload == "lenet":
            from .apps.lenet import Trainer
            return Trainer(batch=batch, lr=0.0005)
        from .apps.deepspeech2 import Trainer
        return Trainer(batch=batch, freq=161, frames=400, hidden=800, layers=3, label_len=50, lr=1e-5)
    text, data, trainer, losses = record(make, be, "%s, batch %d" % (args.workload, batch), heap)
    os.makedirs(args.out_dir, exist_ok=True)
    src = os.path.join(args.out_dir, "step.c")
    open(src, "w").write(text)
    open(os.path.join(args.out_dir, "data.bin"), "wb").write(data)
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    print("wrote %s (%d lines) and data.bin (%.1f MB); losses of the recorded steps %.6f %.6f" % (src, text.count("\n"), len(data) / 1e6, *losses))
    print(" ".join(compile_line(repo, src, os.path.join(args.out_dir, "step"))))


if __name__ == "__main__":
    main()
