import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def has_gpu():
    import ctypes as C
    from puppygrad_amd import _lib
    info = _lib.pg_device_info()
    return _lib.load().pg_device_query(0, C.byref(info)) == 0
