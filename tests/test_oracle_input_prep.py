"""Pins the oracle's restatement of the joint-attention input preparation (RMS-norm over the head
dim -> bf16 -> interleaved RoPE -> bf16, [B,N,H,D] -> [B,H,N,D]) without re-typing its formula:
the reference's RoPE known-answer case, closed forms of the normalisation, and invariants."""
import json
import math
import os

import numpy as np

from flame_amd import workloads as W

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _bits(x):
    return W.f32_to_bf16_bits(np.asarray(x, np.float32))


def _f32(b):
    return W.bf16_bits_to_f32(b)


def test_rope_only_matches_reference_known_answer(oracle):
    kat = json.load(open(os.path.join(GOLD, "kat_rope_1x2x3x4.json")))
    B, H, S, D = kat["B"], kat["H"], kat["S"], kat["D"]
    x = (np.arange(B * H * S * D, dtype=np.float32) * np.float32(0.01)).reshape(B, H, S, D)
    xr = _f32(_bits(x))           # the bf16 values the kernel sees
    want = np.zeros_like(x)
    for h in range(H):            # scalar loop from the reference test: pair p, freq = theta^(-2p/D), angle = s*freq
        for s in range(S):
            for p in range(D // 2):
                ang = s * (1.0 / kat["theta"] ** (2.0 * p / D))
                x0, x1 = float(xr[0, h, s, 2 * p]), float(xr[0, h, s, 2 * p + 1])
                want[0, h, s, 2 * p] = x0 * math.cos(ang) - x1 * math.sin(ang)
                want[0, h, s, 2 * p + 1] = x0 * math.sin(ang) + x1 * math.cos(ang)
    pos = np.arange(S, dtype=np.float64)[:, None]
    freq = kat["theta"] ** (-2.0 * np.arange(D // 2) / D)[None, :]
    x_bnhd = np.ascontiguousarray(np.transpose(_bits(x), (0, 2, 1, 3)))
    got = _f32(oracle.prep_rmsnorm_rope(x_bnhd, None, np.cos(pos * freq).astype(np.float32),
                                        np.sin(pos * freq).astype(np.float32), apply_norm=False))
    assert got.shape == (B, H, S, D)
    assert np.max(np.abs(got - want)) < kat["tol"]


def test_norm_closed_forms(oracle):
    D = 64
    x = np.zeros((1, 3, 1, D), np.float32)
    x[0, 0, 0, :] = 3.0                        # constant row: x / |x| = 1 everywhere
    x[0, 1, 0, 0], x[0, 1, 0, 1] = 3.0, 4.0    # (3,4,0,...): mean square 25/64 -> rsqrt = 8/5
    x[0, 2, 0, :] = 0.0                        # zero row stays zero (eps keeps rsqrt finite)
    got = _f32(oracle.prep_rmsnorm_rope(_bits(x), None, None, None, eps=0.0))
    assert got.shape == (1, 1, 3, D)
    assert np.all(got[0, 0, 0] == 1.0)
    assert got[0, 0, 1, 0] == _f32(_bits(np.float32(4.8))) and got[0, 0, 1, 1] == _f32(_bits(np.float32(6.4)))
    assert np.all(got[0, 0, 1, 2:] == 0.0)
    got0 = _f32(oracle.prep_rmsnorm_rope(_bits(x), None, None, None, eps=1e-6))
    assert np.all(got0[0, 0, 2] == 0.0) and np.all(np.isfinite(got0))
    # learned scale multiplies after the normalisation
    w = np.linspace(0.5, 2.0, D).astype(np.float32)
    gw = _f32(oracle.prep_rmsnorm_rope(_bits(x), _bits(w), None, None, eps=0.0))
    assert np.allclose(gw[0, 0, 0], _f32(_bits(w)), rtol=2 ** -8, atol=0)


def test_rotation_preserves_pair_norms_and_layout(oracle):
    B, N, H, D = 2, 24, 3, 128
    x = W.normal_f32(11, 0, B * N * H * D).reshape(B, N, H, D)
    cos, sin = W.axial_rope_tables(8, 4, 4, D)
    assert cos.shape == (N, D // 2)
    xb = _bits(x)
    normed = _f32(oracle.prep_rmsnorm_rope(xb, None, None, None))
    both = _f32(oracle.prep_rmsnorm_rope(xb, None, cos, sin))
    assert normed.shape == both.shape == (B, H, N, D)
    # unit RMS after the normalisation, rotation keeps the length of every pair
    rms = np.sqrt((normed.astype(np.float64) ** 2).mean(-1))
    assert np.max(np.abs(rms - 1.0)) < 4e-3
    pn = normed[..., 0::2].astype(np.float64) ** 2 + normed[..., 1::2].astype(np.float64) ** 2
    pb = both[..., 0::2].astype(np.float64) ** 2 + both[..., 1::2].astype(np.float64) ** 2
    assert np.max(np.abs(np.sqrt(pn) - np.sqrt(pb))) < 2e-2
    # position 0 of the text block has angle 0: rotation is the identity there
    assert np.array_equal(normed[:, :, 0], both[:, :, 0])
    # the layout change: output row (b,h,n) comes from input row (b,n,h)
    assert np.array_equal(normed[1, 2, 5], _f32(oracle.prep_rmsnorm_rope(xb[1:2, 5:6, 2:3], None, None, None))[0, 0, 0])
    # agrees with the generator used for the benchmark inputs, which normalises and rotates without
    # the intermediate rounding: differences stay within one bf16 step of values of size <= 4
    alt = W.apply_rope_interleaved(np.transpose(W.rms_normalise(_f32(xb)), (0, 2, 1, 3)), cos, sin)
    assert np.max(np.abs(alt - both)) < 3.2e-2
