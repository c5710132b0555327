import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (C restatement of the reference arithmetic), built on demand."""
    from oracle import oracle as o
    o.build()
    o.lib()
    return o


@pytest.fixture(autouse=True)
def _library_options_reset():
    """A test may override run-time options of the HIP library (tests/_util.py: set_option); none survives it."""
    yield
    from bittorch_amd import _lib
    if _lib._lib is not None:
        _lib.set_option(None)


def announce(*parts):
    """Name the case before a GPU step so a lost box still says what ran."""
    print("[case]", *parts, flush=True)
