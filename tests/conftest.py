import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = Path(__file__).resolve().parent / "golden"

# lets the tests switch kernel variants inside the process (oq_debug_override refuses without it);
# the library reads it at its first call, so it has to be there before any test loads the library
os.environ.setdefault("ORBITQUANT_DEBUG", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN


@pytest.fixture
def library_switch():
    """`library_switch(name, value)` sets one of the library's OQ_* experiment switches until the test
    ends.  The library reads the environment once per process, so changing os.environ afterwards does
    nothing; oq_debug_override changes what it read."""
    from orbitquant_amd import _lib

    lib = _lib.load()
    touched = []

    def switch(name: str, value) -> None:
        rc = lib.oq_debug_override(name.encode(), None if value is None else str(value).encode())
        assert rc == 0, lib.oq_last_error()
        touched.append(name)

    yield switch
    for name in touched:   # back to what the process started with
        start = os.environ.get(name)
        lib.oq_debug_override(name.encode(), None if start is None else start.encode())
