import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = Path(__file__).resolve().parent / "golden"


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
