import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    return GOLDEN


def _stale_library():
    """Names a kernel source that is newer than the built library (a GPU run would then test old code)."""
    lib = os.path.join(ROOT, "turbospark_amd", "libtsverify.so")
    if not os.path.exists(lib):
        return None
    built = os.path.getmtime(lib)
    for base in (os.path.join(ROOT, "turbospark_amd", "csrc"), os.path.join(ROOT, "include")):
        for f in sorted(os.listdir(base)):
            if os.path.getmtime(os.path.join(base, f)) > built + 1.0:
                return f
    return None


def pytest_report_header(config):
    stale = _stale_library()
    if stale:
        return f"WARNING: libtsverify.so is older than {stale}: the GPU tests would run old code; rebuild first"
    return None
