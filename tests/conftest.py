import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_c():
    """The plain-C quantiser restatement (oracle/quant_ref.c) through ctypes."""
    import ctypes
    path = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    lib = ctypes.CDLL(path)
    lib.oracle_quantize_ref128.restype = ctypes.c_int
    lib.oracle_quantize_ref128.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p,
                                           ctypes.c_void_p]
    return lib


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture
def tuning():
    """Sets launch-shape overrides through eet_set_tuning for one test and clears them afterwards."""
    from eet_amd._lib import check, lib
    used = []

    def set_(name, value):
        used.append(name)
        check(lib().eet_set_tuning(name.encode(), str(value).encode()), "eet_set_tuning")
    yield set_
    for name in used:
        lib().eet_set_tuning(name.encode(), None)
