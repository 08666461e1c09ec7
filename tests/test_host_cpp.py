"""The library's host-side logic built on its own with -fsanitize=address,undefined (tests/host_cpp/) and checked by brute force:
the command list's record-time dependence analysis against a comparison of every pair of commands, and the deferred-work
bookkeeping (parked launches, zero fills on demand, results produced on demand) against the same random programs run with every
call executed as issued.  No GPU: the device is simulated by loops over host memory."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host_cpp")


@pytest.fixture(scope="module")
def built():
    if shutil.which("g++") is None or shutil.which("make") is None:
        pytest.skip("no host C++ compiler")
    r = subprocess.run(["make", "-C", HERE, "-j2"], capture_output=True, text=True)
    if r.returncode != 0 and "sanitize" in r.stderr and "cannot find" in r.stderr:
        pytest.skip("the sanitizer runtimes are not installed: " + r.stderr[-300:])
    assert r.returncode == 0, r.stderr[-3000:]
    return os.path.join(HERE, "_build")


def _run(exe, *args):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    env.pop("LD_PRELOAD", None)          # the sanitizer runtime has to come first in the library list
    r = subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, timeout=600, env=env)
    assert r.returncode == 0, (r.stdout + r.stderr)[-3000:]
    return r.stdout


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_command_list_levels_against_every_pair_of_commands(built, seed):
    out = _run(os.path.join(built, "levels_check"), 150, 700, seed)
    assert "no violation" in out


@pytest.mark.parametrize("seed", [1, 2])
def test_deferred_work_gives_what_the_calls_as_issued_give(built, seed):
    out = _run(os.path.join(built, "defer_check"), 1500, seed)
    assert "identical" in out and " 0 chains fused" not in out
