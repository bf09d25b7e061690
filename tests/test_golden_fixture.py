"""The committed small fixture (tests/golden/sdpa_small.npz) against the oracle (CPU) and, on a GPU,
against the HIP kernels through the C ABI."""
import os

import numpy as np
import pytest

from flame_amd import workloads as W

FIX = os.path.join(os.path.dirname(__file__), "golden", "sdpa_small.npz")


def test_oracle_reproduces_the_fixture(oracle):
    f = np.load(FIX)
    B, H, Sq, D = f["q"].shape
    # the generator is a pure function of (seed, stream, index): the inputs regenerate bit for bit
    q = W.f32_to_bf16_bits(W.normal_f32(0x601D, 0, B * H * Sq * D).reshape(B, H, Sq, D))
    assert np.array_equal(q, f["q"])
    for tag, causal in (("", False), ("_causal", True)):
        o, lse = oracle.sdpa_fwd(f["q"], f["k"], f["v"], float(f["scale"]), causal=causal)
        dq, dk, dv = oracle.sdpa_bwd(f["q"], f["k"], f["v"], o, f["do"], float(f["scale"]), causal=causal)
        # bit-identical O is expected on the same build; allow one bf16 ulp for a different libm / FMA choice
        for name, got in (("o", o), ("dq", dq), ("dk", dk), ("dv", dv)):
            a, b = oracle.bf16_to_f32(got), oracle.bf16_to_f32(f[name + tag])
            assert np.max(np.abs(a - b)) <= 2.0 ** -7 * max(1.0, np.max(np.abs(b))), name + tag
        assert np.max(np.abs(lse - f["lse" + tag])) <= 1e-5


@pytest.mark.gpu
def test_kernels_match_the_fixture(oracle):
    import torch
    from flame_amd import capi
    from tests.gpu_util import to_dev, to_f32
    f = np.load(FIX)
    q, k, v, do = (to_dev(f[n]) for n in ("q", "k", "v", "do"))
    for tag, causal in (("", False), ("_causal", True)):
        o, lse = capi.attn_fwd(q, k, v, float(f["scale"]), causal=causal)
        dq, dk, dv = capi.attn_bwd(q, k, v, o, do, lse, float(f["scale"]), causal=causal)
        torch.cuda.synchronize()
        for name, got in (("o", o), ("dq", dq), ("dk", dk), ("dv", dv)):
            ref = oracle.bf16_to_f32(f[name + tag])
            g = to_f32(got)
            assert oracle.max_abs(g, ref) <= 2e-2 and oracle.rel_l2(g, ref) <= 1e-2, name + tag
        assert oracle.max_abs(lse.cpu().numpy().reshape(f["lse" + tag].shape), f["lse" + tag]) <= 1e-3
