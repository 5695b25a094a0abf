import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure)."""
    from oracle import oracle
    oracle.load()
    return oracle


@pytest.fixture(scope="session")
def lib():
    """The native library; built only when no built copy is present."""
    from rustorch_amd import _lib
    if not _lib.LIB_PATH.exists():
        from rustorch_amd import build
        build.build_all(verbose=False)
    return _lib.load()


@pytest.fixture(scope="session")
def ex(lib):
    """One executor on hip:0 for the whole GPU session; a missing device is a failure, not a skip."""
    from rustorch_amd.executor import HipKernelExecutor
    e = HipKernelExecutor(0)
    yield e
    e.close()
