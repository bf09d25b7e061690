"""Runs the C++ host-layer test driver (tests/host/host_api_test.cpp) on the GPU.

The driver exercises flame_amd/host/flame_host.hpp -- the C++ mirror of the reference's Rust operator
interface for this path -- against the CPU oracle (oracle/_build/liboracle.so, linked into the driver as its
checker), to the tolerances of tests/gpu_util.py, and exits 0 when every check passed.  It is built ahead of time
by `python -m tests.host.build` (after `python -m flame_amd.build` and `make -C oracle`)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "host", "host_api_test")


def test_host_layer_driver():
    assert os.path.exists(EXE), "build it first: python -m tests.host.build"
    print("[host api] running", EXE, flush=True)
    res = subprocess.run([EXE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    print(res.stdout, flush=True)
    assert res.returncode == 0, res.stdout[-2000:]
    assert "all checks passed" in res.stdout
