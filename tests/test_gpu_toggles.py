"""The switches that turn single optimisations off (kernel variants compiled for plain passes,
half-precision arrays inside the kernels, folded tile axes, nontemporal accesses) must not change
a single bit of any result: every switch selects between two routes through the same arithmetic."""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def run_child(extra_env):
    env = dict(os.environ)
    # (nontemporal accesses from 1 MB a pass on, so that the short transforms of the list take them)
    env["ROCFFT_AMD_NT_MB"] = "1"
    env.update(extra_env)
    out = subprocess.run([sys.executable, os.path.join(HERE, "toggle_child.py")], env=env, capture_output=True,
                         text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    sums = [l for l in out.stdout.splitlines() if len(l) == 64]
    assert len(sums) == 12, out.stdout
    return sums


@pytest.mark.gpu
def test_switches_select_routes_through_the_same_arithmetic(gpu_lib):
    base = run_child({})
    assert base == run_child({}), "two runs of the same build differ"
    for switch in ("ROCFFT_AMD_NO_VARIANTS", "ROCFFT_AMD_NO_HALF_FUSE", "ROCFFT_AMD_NO_FOLD", "ROCFFT_AMD_NO_NT"):
        other = run_child({switch: "1"})
        diff = [i for i, (a, b) in enumerate(zip(base, other)) if a != b]
        assert not diff, (switch, diff)
