"""Compiles the HIP sources of the attention library for gfx950 into ``flame_amd/lib``.

``python -m flame_amd.build`` (or ``build_lib()``) cross-compiles with hipcc; no GPU is needed.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libflame_attn_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",   # keep packed fp32 VALU ops off
    "-Wall", "-Wno-unused-function", "-Wno-inline-asm",   # m0 is clobbered on purpose by the LDS-DMA helpers
]


def hipcc_version() -> str:
    """The compiler's own version line ("HIP version: ..." plus the clang version), one token string."""
    out = subprocess.run([HIPCC, "--version"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True).stdout
    hip = next((l.split(":", 1)[1].strip() for l in out.splitlines() if l.startswith("HIP version")), "?")
    clang = next((l.strip() for l in out.splitlines() if "clang version" in l), "?")
    clang = clang.split("clang version", 1)[1].split()[0] if "clang version" in clang else "?"
    return f"{hip} clang-{clang}"


STATIC_LIB_PATH = os.path.join(LIB_DIR, "libflame_attn_hip.a")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"{os.path.basename(cmd[0])} failed:\n" + out)
    if verbose and out.strip():
        print(out)


def build_lib(verbose: bool = False, extra=()) -> str:
    """One compilation of flame_attn.hip to an object, from which both the shared library (what the tests, the
    benchmark and the ctypes binding load) and the static archive (what a Rust build script links, as the reference's
    build.rs links its own kernels) are made."""
    os.makedirs(LIB_DIR, exist_ok=True)
    src = os.path.join(CSRC, "flame_attn.hip")
    obj = os.path.join(LIB_DIR, "flame_attn.o")
    compile_flags = [f for f in FLAGS if f != "-shared"]
    _run([HIPCC, *compile_flags, f'-DFLAME_ATTN_HIPCC_VERSION="{hipcc_version()}"', *extra, "-c", src, "-o", obj], verbose)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", obj, "-o", LIB_PATH], verbose)
    if os.path.exists(STATIC_LIB_PATH):
        os.remove(STATIC_LIB_PATH)
    _run(["ar", "rcs", STATIC_LIB_PATH, obj], verbose)
    os.remove(obj)
    return LIB_PATH




PROBE_LIB_PATH = os.path.join(LIB_DIR, "libflame_mfma_probe.so")


def build_probe(verbose: bool = False) -> str:
    """The MFMA-only loop that bench.py --mfma-ceiling times (a measurement aid in a library of its own: nothing of
    it is in the attention library's ABI)."""
    os.makedirs(LIB_DIR, exist_ok=True)
    _run([HIPCC, *FLAGS, os.path.join(CSRC, "mfma_probe.hip"), "-o", PROBE_LIB_PATH], verbose)
    return PROBE_LIB_PATH


if __name__ == "__main__":
    print(build_lib(verbose=True, extra=sys.argv[1:]))
    print(build_probe(verbose=True))
