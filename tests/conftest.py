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
def _release_device_buffers():
    """Frees the buffers tests/harness.up() kept alive, after the device has drained."""
    yield
    from tests import harness

    if harness.KEEP:
        import __graft_entry__ as entry

        entry.load_package().sync()
        harness.KEEP.clear()
