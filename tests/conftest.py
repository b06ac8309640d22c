import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def lib():
    from metalhlo_amd import _lib
    return _lib.load()


@pytest.fixture(scope="session")
def oracle_c():
    """ctypes handle of oracle/liboracle.so (the C restatement); built on demand
    on the CPU only — the GPU box receives the prebuilt file."""
    import ctypes
    path = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(path):
        import subprocess
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "liboracle.so"])
    return ctypes.CDLL(path)


@pytest.fixture(scope="module", autouse=True)
def shipped_tuning_table(request):
    """Every GPU test module starts in the product's configuration: the tuning table holds the
    entries that ship for this device and nothing else (a test of the heuristics clears it)."""
    if not any(item.get_closest_marker("gpu") for item in request.session.items if item.module is request.module):
        yield
        return
    import os
    from metalhlo_amd import kernels
    kernels.tuning_clear()
    path = kernels.shipped_tuning_table()
    if os.path.exists(path):
        kernels.tuning_load(path)
    yield
