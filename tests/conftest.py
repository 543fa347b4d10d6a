import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import ref
    ref.lib()
    return ref


@pytest.fixture(autouse=True)
def shipped_library_by_default():
    """Every test starts and ends on the shipped library: a test that pins a kernel instance
    loads the tuning build (`_lib.load_tuning()`), and its overrides are reset afterwards."""
    yield
    from kiln_amd import _lib
    _lib.use_shipped()


@pytest.fixture
def matrix_core_kernel_from_33_rows():
    """Projections of up to 32 M weights take M = 33...64 through the small-M kernel in slabs;
    tests that mean to exercise the matrix-core kernel on few rows pin the switch-over at 33
    rows for their duration (through the tuning build of the library)."""
    from kiln_amd import _lib
    lib = _lib.load_tuning()
    lib.kiln_w4a16_debug_prefill_min_m(33)
    yield
    lib.kiln_w4a16_debug_prefill_min_m(0)
