import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# The library reads these once, when it is loaded (reference: amem_nccl.cpp:711-718).
os.environ.setdefault("AMEM_ENABLE", "1")
os.environ.setdefault("GMM_LOG", "1")
os.environ.setdefault("GMM_IPC_DIR", os.environ.get("TMPDIR", "/tmp"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


_MEASURED = []


@pytest.fixture()
def measured():
    """Tests hand timings here (one line each); they are printed in the run's summary, where `-q` and
    output capture do not hide them."""
    return _MEASURED.append


def _fd_kinds():
    kinds = {}
    for f in os.listdir("/proc/self/fd"):
        try:
            t = os.readlink("/proc/self/fd/" + f)
        except OSError:
            continue
        k = t.split(":")[0] if not t.startswith("/") else ("/dmabuf" if t.startswith("/dmabuf") else t)
        kinds[k] = kinds.get(k, 0) + 1
    return kinds


@pytest.fixture(autouse=True)
def _descriptor_growth(request):
    """Notes every test after which this process holds noticeably more open descriptors than before it."""
    before = len(os.listdir("/proc/self/fd"))
    yield
    after = len(os.listdir("/proc/self/fd"))
    if after - before > 16:
        top = sorted(_fd_kinds().items(), key=lambda kv: -kv[1])[:4]
        _MEASURED.append("descriptors: %s left %d more open (%d -> %d); most common now: %s" %
                         (request.node.name, after - before, before, after, top))


def pytest_terminal_summary(terminalreporter):
    if _MEASURED:
        terminalreporter.section("measured")
        for line in _MEASURED:
            terminalreporter.write_line(line)


def _built():
    from asystem_amem_amd import binding, footprint
    import oracle
    return all(os.path.exists(p) for p in (binding.LIB_PATH, footprint.LIB_PATH, oracle.LIB_PATH))


@pytest.fixture(scope="session", autouse=True)
def _libraries():
    """Tests load what is built; they build only when nothing is."""
    if not _built():
        import __graft_entry__
        __graft_entry__.build()


@pytest.fixture(scope="session")
def lib():
    """The shipped library. Only the child pytest of tests/test_engine_on_host_standin.py sets
    AMEM_TEST_LIB, to run engine-logic tests against the test-only build on the host stand-in."""
    from asystem_amem_amd import binding
    return binding.load(os.environ.get("AMEM_TEST_LIB") or None)


@pytest.fixture(scope="session")
def orc():
    import oracle
    return oracle.load()


@pytest.fixture()
def fresh(lib):
    """Engine context reset to the state before the first tracked allocation."""
    assert lib.amem_shutdown() == 0
    lib.amem_set_enabled(1)
    yield lib
    assert lib.amem_shutdown() == 0


@pytest.fixture()
def fresh_orc(orc):
    orc.oracle_reset()
    yield orc
    orc.oracle_reset()
    orc.oracle_vmm_reset()      # regions a test left in the oracle's host-memory stand-in (one memfd each)


@pytest.fixture(scope="session")
def gpu(lib):
    if lib.amem_device_count() < 1:
        pytest.skip("no GPU visible")
    return lib
