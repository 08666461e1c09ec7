"""The C-ABI library loads and exports every symbol include/lantern_hip.h declares; the Python
binding covers them all; the product never reaches into the oracle.  No GPU call is made."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lantern_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lh_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_families():
    names = _declared()
    for must in ("lh_setup", "lh_malloc", "lh_rewind", "lh_conv2d_fwd", "lh_conv2d_bwd_data", "lh_conv2d_bwd_filter", "lh_sgemm",
                 "lh_bn_train_fwd", "lh_bn_bwd", "lh_softmax", "lh_nll", "lh_maxpool_fwd", "lh_dropout_fwd", "lh_momentum", "lh_adagrad"):
        assert must in names
    assert len(names) >= 70


def test_library_exports_every_declared_symbol():
    from lantern_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first (python -c 'import __graft_entry__ as g; g.build()')"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in _declared() if not hasattr(lib, n)]
    assert not missing, "declared in the header but not exported: %s" % missing


def test_python_binding_covers_the_header():
    from lantern_amd import _lib
    decl = set(_declared())
    bound = set(_lib.SIGNATURES)
    assert decl - bound == set(), "declared but not bound: %s" % sorted(decl - bound)
    assert bound - decl == set(), "bound but not declared: %s" % sorted(bound - decl)
    _lib.load()     # resolves all of them


def test_no_extra_lh_symbols_exported():
    from lantern_amd import _lib
    out = subprocess.check_output(["nm", "-D", "--defined-only", _lib.LIB_PATH], text=True)
    exported = {l.split()[-1] for l in out.splitlines() if " T " in l and l.split()[-1].startswith("lh_")}
    assert exported == set(_declared())


def test_product_does_not_touch_the_oracle_or_torch():
    bad = []
    for dirpath, _, files in os.walk(os.path.join(ROOT, "lantern_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                if re.search(r"^\s*(from|import)\s+oracle\b|oracle/|liblantern_cpu", text, flags=re.M):
                    bad.append(f + ": oracle")
                if re.search(r"^\s*(from|import)\s+torch\b", text, flags=re.M):
                    bad.append(f + ": torch")
                if re.search(r"hipblas|rocblas|miopen|hipify|__HIP_PLATFORM", text, flags=re.I):
                    bad.append(f + ": vendor library / compat layer")
    assert not bad, bad


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from lantern_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError):
        _lib.load()


HOST_C = os.path.join(ROOT, "tests", "host_c")
HOST_BIN = os.path.join(HOST_C, "_build", "lenet_step")


def test_header_is_plain_c99(tmp_path):
    """The boundary is a C header: a C99 translation unit that only includes it compiles without warnings."""
    src = tmp_path / "only_header.c"
    src.write_text('#include "lantern_hip.h"\nint main(void) { return 0; }\n')
    subprocess.check_call(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", "-I",
                           os.path.join(ROOT, "include"), str(src)])


def _build_host_program():
    subprocess.check_call(["make", "-C", HOST_C], stdout=subprocess.DEVNULL)
    return HOST_BIN


def test_c_host_program_links_without_python_or_torch():
    """A plain-C program written against the header links to the library and loads it (no device call is made)."""
    exe = _build_host_program()
    out = subprocess.run([exe], env=dict(os.environ, LENET_STEP_LINK_ONLY="1"), capture_output=True, text=True, timeout=60)
    assert out.returncode == 0 and out.stdout.strip() == "linked", out.stdout + out.stderr
    deps = subprocess.run(["ldd", exe], capture_output=True, text=True).stdout
    assert "liblantern_hip.so" in deps and "torch" not in deps and "python" not in deps, deps


@pytest.mark.gpu
def test_c_host_program_trains_lenet_like_the_oracle():
    """Five SGD steps of the MNIST CNN issued from C through the C-ABI, against the oracle in the same process:
    losses within 1e-4 relative, parameters within 1e-3 of the largest one (the program's own exit code)."""
    exe = HOST_BIN if os.path.exists(HOST_BIN) else _build_host_program()
    env = {k: v for k, v in os.environ.items() if k != "LENET_STEP_LINK_ONLY"}
    out = subprocess.run([exe], env=env, capture_output=True, text=True, timeout=110)
    print(out.stdout, out.stderr)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout + out.stderr


# ---- the TreeLSTM loop from C ---------------------------------------------------------------------------------------------
TREE_BIN = os.path.join(HOST_C, "_build", "treelstm_step")


def write_treelstm_inputs(tmp_path, trainer, trees):
    from lantern_amd.apps.treelstm import write_c_program_inputs
    assert trees is trainer.trees
    return write_c_program_inputs(tmp_path, trainer)


def test_c_treelstm_program_links():
    exe = _build_host_program() and TREE_BIN
    out = subprocess.run([exe], env=dict(os.environ, TREELSTM_STEP_LINK_ONLY="1"), capture_output=True, text=True, timeout=60)
    assert out.returncode == 0 and out.stdout.strip() == "linked", out.stdout + out.stderr
    deps = subprocess.run(["ldd", exe], capture_output=True, text=True).stdout
    assert "liblantern_hip.so" in deps and "torch" not in deps and "python" not in deps and "lantern_cpu" not in deps, deps


@pytest.mark.gpu
@pytest.mark.parametrize("cmdlist", [0, 1], ids=["one_launch_per_op", "command_list"])
def test_c_treelstm_program_tracks_the_oracle(tmp_path, cpu_backend, cmdlist):
    """The recursion over the tree arrays written in C against the C-ABI (tests/host_c/treelstm_step.c), one Adagrad step per tree
    over the first eight trees of the reference's own evaluation set (tests/golden/array_tree_first24.txt: 8 to 34 leaves), against
    the same trees run through the host mirror on the CPU oracle from the same initial parameters: every loss within 1e-4
    relative, every parameter tensor within 1e-3 (relative L2)."""
    import numpy as np
    import lantern_amd as la
    from lantern_amd.apps.treelstm import Trainer, read_trees
    exe = TREE_BIN if os.path.exists(TREE_BIN) else (_build_host_program() and TREE_BIN)
    la.set_backend(cpu_backend)
    mark = cpu_backend.getMallocAddr()
    trees = read_trees(os.path.join(ROOT, "tests", "golden", "array_tree_first24.txt"))[:8]
    tr = Trainer(vocab=500, trees=trees)
    params = write_treelstm_inputs(tmp_path, tr, tr.trees)
    want_losses = []
    for _ in range(len(trees)):
        want_losses.append(float(tr.step().toCPU()[0])); tr.end_step()
    want = [p.x.toCPU().copy() for p in params]
    tr.close(); cpu_backend.resetMallocAddr(mark)
    out = subprocess.run([exe, str(tmp_path / "params.bin"), str(tmp_path / "trees.txt"), str(tmp_path / "out.bin"), str(len(trees)), "0", str(cmdlist)],
                         capture_output=True, text=True, timeout=110)
    print(out.stdout, out.stderr)
    assert out.returncode == 0 and out.stdout.startswith("trees_per_s"), out.stdout + out.stderr
    got = np.fromfile(tmp_path / "out.bin", np.float32)
    assert got.size == len(trees) + sum(w.size for w in want)
    np.testing.assert_allclose(got[:len(trees)], want_losses, rtol=1e-4)
    assert want_losses[0] != want_losses[-1]
    pos = len(trees)
    for w in want:
        g = got[pos:pos + w.size].reshape(w.shape); pos += w.size
        err = np.linalg.norm(g.astype(np.float64) - w) / max(np.linalg.norm(w.astype(np.float64)), 1e-30)
        assert err <= 1e-3 or np.abs(g - w).max() <= 1e-5, err


@pytest.mark.gpu
def test_c_treelstm_command_list_gives_the_same_bits_on_any_number_of_workgroups(tmp_path, cpu_backend):
    """No command of the list combines partial results with atomic adds and every sum has a fixed order, so eight training steps
    of the C program end in the same bits whether 1, 5 or 32 workgroups share the commands (LH_CMDLIST_GROUPS), twice over, and
    also when element-wise chains run command by command instead of as programs over LDS (LH_CMDLIST_SLOTS=0) or when nothing is
    chained at all and every dependent command opens a level (LH_CMDLIST_CHAINS=0): how the commands are scheduled is not
    allowed to show in the result."""
    import numpy as np
    import lantern_amd as la
    from lantern_amd.apps.treelstm import Trainer, read_trees
    exe = TREE_BIN if os.path.exists(TREE_BIN) else (_build_host_program() and TREE_BIN)
    la.set_backend(cpu_backend)
    mark = cpu_backend.getMallocAddr()
    trees = read_trees(os.path.join(ROOT, "tests", "golden", "array_tree_first24.txt"))[:8]
    tr = Trainer(vocab=500, trees=trees)
    write_treelstm_inputs(tmp_path, tr, tr.trees)
    tr.close(); cpu_backend.resetMallocAddr(mark)
    results = []
    for extra in ({"LH_CMDLIST_GROUPS": "1"}, {"LH_CMDLIST_GROUPS": "5"}, {}, {}, {"LH_CMDLIST_SLOTS": "0"}, {"LH_CMDLIST_CHAINS": "0"}):
        out_file = tmp_path / ("out_%d.bin" % len(results))
        out = subprocess.run([exe, str(tmp_path / "params.bin"), str(tmp_path / "trees.txt"), str(out_file), str(len(trees)), "0", "1"],
                             capture_output=True, text=True, timeout=110, env=dict(os.environ, **extra))
        assert out.returncode == 0 and out.stdout.startswith("trees_per_s"), out.stdout + out.stderr
        results.append(np.fromfile(out_file, np.uint32))
    assert results[0].size > len(trees) and np.isfinite(results[0].view(np.float32)).all()
    for r in results[1:]:
        assert np.array_equal(results[0], r)


@pytest.mark.gpu
def test_emitted_c_program_repeats_the_mirrors_training_steps(tmp_path, on_hip):
    """lantern_amd/emit_c.py writes a program of the mirror out as straight-line C over the C-ABI (what the reference's LMS back end
    emits: one library call per operator, shapes as literals, the step in a loop).  A small ResNet (bottleneck blocks, batch norm,
    pooling, the classifier, momentum SGD: 32x32 images, batch 8) is recorded, compiled with gcc and run for five steps in a process
    of its own; in deterministic mode its losses are, bit for bit, the losses of the mirror's own next five steps."""
    import shutil
    import numpy as np
    from lantern_amd import emit_c
    from lantern_amd.apps.resnet50 import ResNet50, Trainer
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    be = on_hip
    be.setDeterministic(True)
    try:
        make = lambda: Trainer(ResNet50(num_classes=10, layers=(1, 1, 1, 1), imagenet_stem=False), 8, 32, 10, lr=0.01, momentum=0.9)
        text, data, trainer, (first, second) = emit_c.record(make, be, "a small ResNet, batch 8", 1 << 30, frame=["lh_set_deterministic(1);"])
        want = [second]
        for _ in range(4):
            want.append(float(trainer.step().toCPU()[0])); trainer.end_step()
    finally:
        be.setDeterministic(False)
    assert text.count("lh_conv2d_fwd") >= 10 and "lh_multi_momentum" in text or "lh_momentum" in text
    (tmp_path / "step.c").write_text(text)
    (tmp_path / "data.bin").write_bytes(data)
    exe = str(tmp_path / "step")
    cc = subprocess.run(emit_c.compile_line(ROOT, str(tmp_path / "step.c"), exe), capture_output=True, text=True)
    assert cc.returncode == 0 and "warning" not in cc.stderr, cc.stderr[-3000:]
    deps = subprocess.run(["ldd", exe], capture_output=True, text=True).stdout
    assert "liblantern_hip.so" in deps and "python" not in deps and "torch" not in deps, deps
    out = subprocess.run([exe, str(tmp_path / "data.bin"), "5", "0", str(tmp_path / "losses.bin")], capture_output=True, text=True, timeout=110)
    assert out.returncode == 0 and out.stdout.startswith("ms_per_step"), out.stdout + out.stderr
    got = np.fromfile(tmp_path / "losses.bin", np.float32)
    assert got.size == 5 and first != second
    assert np.array_equal(got, np.array(want, np.float32)), (got, want)
