#!/usr/bin/env python3
"""Writes tests/golden/sdpa_small.npz: seeded inputs of a small attention problem and the CPU oracle's
outputs for it (non-causal and causal).  The reference cannot be run in this environment (Rust + CUDA
+ cuDNN), and it ships no fixture data for this path, so the vectors come from the pinned oracle; the
file freezes them so that a later change to the oracle or to the generators is caught.

    python tests/golden/make_small_fixture.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from flame_amd import workloads as W  # noqa: E402
from oracle import oracle as O  # noqa: E402


def main():
    B, H, Sq, Sk, D = 1, 2, 96, 136, 64
    seed = 0x601D
    q, k, v, do = (W.f32_to_bf16_bits(W.normal_f32(seed, s, B * H * n * D).reshape(B, H, n, D))
                   for s, n in enumerate((Sq, Sk, Sk, Sq)))
    scale = np.float32(0.125)
    out = dict(q=q, k=k, v=v, do=do, scale=scale)
    for tag, causal in (("", False), ("_causal", True)):
        o, lse = O.sdpa_fwd(q, k, v, float(scale), causal=causal)
        dq, dk, dv = O.sdpa_bwd(q, k, v, o, do, float(scale), causal=causal)
        out.update({"o" + tag: o, "lse" + tag: lse, "dq" + tag: dq, "dk" + tag: dk, "dv" + tag: dv})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sdpa_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
