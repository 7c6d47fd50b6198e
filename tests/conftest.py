import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def emu():
    """Planner + API linked against the host emulation of the runtime layer."""
    import subprocess

    import rocfft_amd.binding as B

    path = os.path.join(ROOT, "tests", "emu", "librocfft_amd_emu.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "tests", "emu")])
    lib = B.Library(path)
    lib.setup()
    return lib


@pytest.fixture(scope="session")
def gpu_lib():
    """The product library on a real GPU; fails loudly if it is not built."""
    import torch

    import rocfft_amd as rf

    assert torch.cuda.is_available()
    return rf.library()
