import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; runs the HIP path through the C ABI")


@pytest.fixture(scope="session", autouse=True)
def _native_libraries():
    """Tests load what is built; they build only if nothing is there."""
    lib = os.path.join(ROOT, "dvm_amd", "lib")
    if not (os.path.exists(os.path.join(lib, "libdvm.so")) and os.path.exists(os.path.join(lib, "libdvm_hip.so"))):
        from dvm_amd import build as _b
        _b.build()
    from oracle import oracle as _o
    _o.build()
