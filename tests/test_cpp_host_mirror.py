"""The C++ host-side mirror of the reference's table / operator classes
(include/tensornet_amd.hpp) compiles against the C ABI and behaves: host-only
checks here, a device round trip under -m gpu."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "host_mirror_test")


def _binary():
    if not os.path.exists(BIN):
        from tensornet_amd import build

        build.build_host_test(verbose=False)
    return BIN


def test_host_mirror_without_a_gpu():
    out = subprocess.run([_binary()], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "host mirror ok" in out.stdout


@pytest.mark.gpu
def test_host_mirror_on_the_gpu():
    assert os.path.exists(BIN), "build the host test on the CPU box first (python -m tensornet_amd.build)"
    out = subprocess.run([BIN, "--gpu"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "host mirror ok" in out.stdout
