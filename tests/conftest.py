import ctypes as C
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _device_count():
    try:
        from seq2seqsharp_amd._lib import lib
        n = C.c_int(0)
        lib().TSHip_GetDeviceCount.argtypes = [C.POINTER(C.c_int)]
        if lib().TSHip_GetDeviceCount(C.byref(n)) != 1:
            return 0
        return n.value
    except Exception:
        return 0


def pytest_collection_modifyitems(config, items):
    have = None
    for item in items:
        if "gpu" in item.keywords:
            if have is None:
                have = _device_count() > 0
            if not have:
                item.add_marker(pytest.mark.skip(reason="no HIP device visible"))


@pytest.fixture(scope="session")
def oracle():
    from oracle import ts_oracle as O
    O.build()
    O.set_threads(min(8, os.cpu_count() or 1))
    return O
