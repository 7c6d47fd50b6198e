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


def _env_with_this_library_first():
    env = dict(os.environ)
    env["LD_LIBRARY_PATH"] = os.path.join(ROOT, "rocfft_amd", "lib") + ":" + env.get("LD_LIBRARY_PATH", "")
    return env


def test_client_linked_with_lrocfft_resolves_to_this_library():
    """built with -lrocfft: the dynamic section asks for librocfft.so.0, the name the reference
    installs; with this library's directory first in LD_LIBRARY_PATH the loader takes its copy
    (without it, the system ROCm's)"""
    path = _client("client_refname")
    needed = subprocess.check_output(["readelf", "-d", path]).decode()
    assert "librocfft.so.0" in needed
    resolved = subprocess.check_output(["ldd", path], env=_env_with_this_library_first()).decode()
    line = [ln for ln in resolved.splitlines() if "librocfft.so.0" in ln]
    assert line and os.path.realpath(line[0].split("=>")[1].split()[0]).startswith(
        os.path.join(ROOT, "rocfft_amd", "lib")), resolved


@pytest.mark.gpu
def test_c_client_under_the_reference_library_name():
    path = os.path.join(CLIENT_DIR, "client_refname")
    assert os.path.exists(path), "tests/cclient/client_refname is not built (run __graft_entry__.build())"
    out = subprocess.run([path], capture_output=True, text=True, timeout=300, env=_env_with_this_library_first())
    assert out.returncode == 0, out.stderr + out.stdout
    assert out.stdout.startswith("ok ")
    # the client prints the version string of the library it reached: this library's, not the system's
    assert "amd-gfx950" in out.stdout, out.stdout
