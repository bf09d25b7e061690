"""Compiles the C++ host-layer test driver (host_api_test.cpp) against the attention library and the CPU oracle.

`python -m tests.host.build` from the repository root, after `python -m flame_amd.build` and `make -C oracle`.  The
driver is test infrastructure: the oracle (oracle/_build/liboracle.so) is its checker and is linked into nothing else."""
from __future__ import annotations

import os
import subprocess

from flame_amd.build import HIPCC, LIB_DIR

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
EXE = os.path.join(HERE, "host_api_test")


def build_host_test(verbose: bool = False) -> str:
    src = os.path.join(HERE, "host_api_test.cpp")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-x", "hip",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", src, "-o", EXE,
           "-L" + LIB_DIR, "-lflame_attn_hip", "-Wl,-rpath,$ORIGIN/../../flame_amd/lib",
           "-L" + os.path.join(ROOT, "oracle", "_build"), "-loracle", "-Wl,-rpath,$ORIGIN/../../oracle/_build"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l))
    return EXE


if __name__ == "__main__":
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True)
    print(build_host_test(verbose=True))
