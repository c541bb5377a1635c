import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from polarquant_amd import _ffi
    _ffi.lib()  # fail loudly if the HIP library has not been built
    return torch.device("cuda:0")


@pytest.fixture(scope="session")
def hooks_lib():
    """The test build of the library (-DPQ_TEST_HOOKS), the only one that honours PQ_TEST_SILENT_SCORER.  The package
    never loads it; same ABI as the shipping library."""
    import ctypes
    from polarquant_amd import _ffi
    path = os.path.join(os.path.dirname(_ffi.LIB_PATH), "libpolarquant_hip_testhooks.so")
    if not os.path.exists(path):
        pytest.fail("%s is missing; build it with `python -m polarquant_amd.build`" % path)
    handle = ctypes.CDLL(path)
    for name, (res, args) in _ffi.SIGNATURES.items():
        fn = getattr(handle, name)
        fn.restype = res
        fn.argtypes = args
    return handle
