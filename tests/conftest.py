import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def _gpu_present():
    return os.path.exists("/dev/kfd")


@pytest.fixture(scope="session")
def hip_backend():
    """One BackendHIP for the whole session (the library owns one arena); fails loudly if the .so is missing."""
    import lantern_amd as la
    be = la.BackendHIP(heap_bytes=int(os.environ.get("LANTERN_TEST_HEAP", 16 << 30)))      # the headline step at full size needs 12.4 GiB
    be.setup()
    yield be
    be.cleanup()


@pytest.fixture(scope="session")
def cpu_backend():
    from oracle.backend_cpu import BackendCPU
    be = BackendCPU(threads=1)
    be.setup()
    return be


@pytest.fixture
def on_cpu(cpu_backend):
    import lantern_amd as la
    la.set_backend(cpu_backend)
    return cpu_backend


@pytest.fixture
def on_hip(hip_backend):
    import lantern_amd as la
    la.set_backend(hip_backend)
    mark = hip_backend.getMallocAddr()
    yield hip_backend
    hip_backend.batchSmallOps(False)
    hip_backend.sync()
    hip_backend.resetMallocAddr(mark)


BACKENDS = [pytest.param("cpu", id="oracle"), pytest.param("hip", id="hip", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def be(request):
    """The reference's unit tests run the same snippet per backend; so do these."""
    import lantern_amd as la
    if request.param == "cpu":
        b = request.getfixturevalue("cpu_backend")
        la.set_backend(b)
        yield b
    else:
        b = request.getfixturevalue("hip_backend")
        la.set_backend(b)
        mark = b.getMallocAddr()
        yield b
        b.sync()
        b.resetMallocAddr(mark)
