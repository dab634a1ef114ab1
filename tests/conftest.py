import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests"), str(ROOT / "tests" / "golden")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    import __graft_entry__ as entry
    return entry.load_package()


@pytest.fixture(scope="session")
def gpu(pkg):
    """The package, after checking that a GPU is there.  GPU tests never fall
    back to anything: without a device they are skipped, not emulated."""
    if pkg.device_count() < 1:
        pytest.skip("no HIP device in this container")
    return pkg
