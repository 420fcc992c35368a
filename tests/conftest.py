"""pytest configuration: the ``gpu`` marker and the package loader."""
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def et():
    """The ctypes binding of the native library (fails loudly if it is not built)."""
    import __graft_entry__ as entry

    pkg = entry.load_package()
    pkg.lib()
    return pkg


@pytest.fixture(autouse=True)
def _release_device_buffers(request):
    """Frees the buffers tests/harness.up() kept alive, after the device has drained; GPU tests then
    leave canary blocks in the heap they freed (tests/heap_canary.py)."""
    yield
    from tests import harness

    if harness.KEEP:
        import __graft_entry__ as entry

        entry.load_package().sync()
        harness.KEEP.clear()
    if request.node.get_closest_marker("gpu") is not None:
        import gc

        from tests import heap_canary

        gc.collect()  # handles the test dropped are destroyed now, not in the middle of the next test
        heap_canary.take(request.node.nodeid)
        heap_canary.release_older_than(2, f"after '{request.node.nodeid}'")


def pytest_terminal_summary(terminalreporter):
    from tests import heap_canary

    heap_canary.release_older_than(0, "at the end of the session")
    hits = heap_canary.report()
    if hits:
        terminalreporter.section("heap canaries: memory of the test process changed behind its owner's back")
        for h in hits:
            terminalreporter.write_line(h)
