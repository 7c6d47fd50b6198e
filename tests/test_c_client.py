"""A client written in plain C99 (tests/cclient/client.c) builds against include/rocfft/rocfft.h
with -Wall -Wextra -Werror -pedantic and runs the call sequence of the reference's samples
(clients/samples/rocfft/rocfft_example_complexcomplex.cpp, rocfft_example_realcomplex.cpp):
on the CPU against the emulated runtime, on the GPU against the library itself with buffers
from the HIP runtime's C API.  The client checks its results against closed forms (a complex
exponential transforms to one spike; round trip = n x) and against the direct sum."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLIENT_DIR = os.path.join(ROOT, "tests", "cclient")


def _client(name):
    path = os.path.join(CLIENT_DIR, name)
    if not os.path.exists(path):
        subprocess.check_call(["make", "-s", "-C", CLIENT_DIR, name])
    return path


def test_c_client_on_the_emulated_runtime(emu):
    out = subprocess.run([_client("client_emu")], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert out.stdout.startswith("ok ")


@pytest.mark.gpu
def test_c_client_on_the_gpu():
    path = os.path.join(CLIENT_DIR, "client_gpu")
    assert os.path.exists(path), "tests/cclient/client_gpu is not built (run __graft_entry__.build())"
    out = subprocess.run([path], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr + out.stdout
    assert out.stdout.startswith("ok ")
