import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _has_gpu():
    try:
        import cumo_amd
        return cumo_amd.device_count() > 0
    except Exception:
        return False


HAS_GPU = _has_gpu()


def pytest_collection_modifyitems(config, items):
    if HAS_GPU:
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session", autouse=True)
def no_kernel_gave_up_a_wait():
    """After the last GPU test of the process: no kernel's bounded wait has given up
    (a give-up means a result that is not valid; see tests/test_gpu_wait_give_up.py)."""
    yield
    if not HAS_GPU:
        return
    import ctypes as C
    from cumo_amd import _lib
    counts = (C.c_uint32 * 4)()
    f = _lib.fn("cumo_hip_wait_give_ups", C.c_int, [C.POINTER(C.c_uint32 * 4)])
    assert f(C.byref(counts)) == 0
    assert list(counts) == [0, 0, 0, 0], "kernels gave up bounded waits during this run: %s" % list(counts)
