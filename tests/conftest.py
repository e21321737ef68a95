import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    if os.environ.get("HCCL_AMD_TEST_EMU") == "1":
        # The run tests/test_emulated_kernels.py starts: the Python mirror calls the CPU emulation build instead of
        # libhccl_amd.so.  Only this test process does; the package itself knows nothing of the emulation.
        import ctypes

        import hccl_amd
        hccl_amd._lib = hccl_amd._bind(ctypes.CDLL(os.environ["HCCL_AMD_TEST_EMU_LIB"]))


@pytest.fixture(scope="session")
def orc():
    import oracle
    oracle.lib()
    return oracle
