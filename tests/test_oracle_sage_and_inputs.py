"""Pins the int8 quantiser of the oracle and the synthetic-input generators."""
import json
import math
import os
from fractions import Fraction

import numpy as np

from flame_amd import workloads as W

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _bits(x):
    return W.f32_to_bf16_bits(np.asarray(x, np.float32))


def _round_half_even(fr: Fraction) -> int:
    fl = math.floor(fr)
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        return fl + 1
    return fl


def test_quantiser_closed_form_brute_force(oracle):
    """scale = absmax/127 (fp32 division), q = clamp(round_half_even(x/scale)) with the quotient
    rounded to fp32 first -- evaluated here with exact rationals, not with the C code's calls."""
    B, H, S, D = 1, 2, 200, 8     # 200 rows: second Q block (128) and fourth K block (64) are short
    q = _bits(W.normal_f32(7, 0, B * H * S * D).reshape(B, H, S, D))
    k = _bits(W.normal_f32(7, 1, B * H * S * D).reshape(B, H, S, D))
    out = oracle.sage_quant(q, k, qblk=128, kblk=64, smooth_k=False)
    assert np.all(out["kmean"] == 0) and np.array_equal(out["ks"], k)
    for name, x, blk, qi, sc in (("q", q, 128, out["qi8"], out["sq"]), ("k", k, 64, out["ki8"], out["sk"])):
        xf = W.bf16_bits_to_f32(x)
        for h in range(H):
            for b0 in range(0, S, blk):
                blkv = xf[0, h, b0:b0 + blk]
                amax = np.float32(np.max(np.abs(blkv)))
                s = np.float32(amax) / np.float32(127.0)
                assert sc[0, h, b0 // blk] == s, name
                for val, got in zip(blkv.ravel()[:257], qi[0, h, b0:b0 + blk].ravel()[:257]):
                    quo = np.float32(val) / s                      # IEEE fp32 division
                    want = max(-128, min(127, _round_half_even(Fraction(float(quo)))))
                    assert int(got) == want, (name, val, s, got, want)
        # the absmax element of every block maps to +-127
        assert np.all(np.max(np.abs(qi.astype(np.int32).reshape(B, H, -1)), axis=-1) == 127)


def test_quantiser_ties_zero_block_and_extremes(oracle):
    D = 8
    # block 0 (rows 0..127): absmax 127 -> scale exactly 1; x = k + 0.5 are exact ties in bf16
    q = np.zeros((1, 1, 256, D), np.float32)
    q[0, 0, 0, :] = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5]
    q[0, 0, 1, :4] = [-127.0, 126.5, -126.5, 0.25]
    # block 1 (rows 128..255) stays all zero -> scale 0, codes 0
    out = oracle.sage_quant(_bits(q), _bits(q[:, :, :64]), qblk=128, kblk=64, smooth_k=False)
    assert out["sq"][0, 0, 0] == 1.0 and out["sq"][0, 0, 1] == 0.0
    assert out["qi8"][0, 0, 0].tolist() == [127, 0, 2, 2, 0, -2, -2, 4]
    assert out["qi8"][0, 0, 1, :4].tolist() == [-127, 126, -126, 0]
    assert np.all(out["qi8"][0, 0, 128:] == 0)


def test_k_smoothing_mean_and_shift_invariance(oracle):
    B, H, S, D = 1, 2, 192, 16
    q = _bits(W.normal_f32(9, 0, B * H * S * D).reshape(B, H, S, D))
    kf = W.normal_f32(9, 1, B * H * S * D).reshape(B, H, S, D)
    kf[..., 3] = kf[..., 3] * 3 + 2.0
    k = _bits(kf)
    v = _bits(W.normal_f32(9, 2, B * H * S * D).reshape(B, H, S, D))
    out = oracle.sage_quant(q, k, smooth_k=True)
    mu = W.bf16_bits_to_f32(k).astype(np.float64).mean(axis=2)
    assert np.array_equal(out["kmean"], mu.astype(np.float32))
    ks = W.f32_to_bf16_bits(W.bf16_bits_to_f32(k) - out["kmean"][:, :, None, :])
    assert np.array_equal(out["ks"], ks)
    # subtracting a per-channel constant from K shifts every logit of a row equally: softmax unchanged
    scale = 0.25
    o_sage, _ = oracle.sage_fwd(out["qi8"], out["ki8"], out["sq"], out["sk"], v, scale)
    o_ref, _ = oracle.sdpa_fwd(q, k, v, scale)
    assert oracle.cosine(oracle.bf16_to_f32(o_sage), oracle.bf16_to_f32(o_ref)) > 0.999


def test_generator_is_a_pure_function_and_gaussian():
    a = W.normal_f32(123, 4, 200000)
    b = W.normal_f32(123, 4, 200000, chunk=777)
    assert np.array_equal(a, b)
    assert not np.array_equal(a[:1000], W.normal_f32(123, 5, 1000))
    assert abs(a.mean()) < 0.01 and abs(a.std() - 1.0) < 0.01
    assert abs(np.mean(a ** 4) - 3.0) < 0.1


def test_rope_known_answer_from_reference_test():
    kat = json.load(open(os.path.join(GOLD, "kat_rope_1x2x3x4.json")))
    B, H, S, D = kat["B"], kat["H"], kat["S"], kat["D"]
    x = (np.arange(B * H * S * D, dtype=np.float32) * np.float32(0.01)).reshape(B, H, S, D)
    # scalar loop written from the formula of the reference test (pair p: freq = theta^(-2p/D), angle = s*freq)
    want = np.zeros_like(x)
    for h in range(H):
        for s in range(S):
            for p in range(D // 2):
                ang = s * (1.0 / kat["theta"] ** (2.0 * p / D))
                x0, x1 = x[0, h, s, 2 * p], x[0, h, s, 2 * p + 1]
                want[0, h, s, 2 * p] = x0 * math.cos(ang) - x1 * math.sin(ang)
                want[0, h, s, 2 * p + 1] = x0 * math.sin(ang) + x1 * math.cos(ang)
    pos = np.arange(S, dtype=np.float32)[:, None]
    freq = (kat["theta"] ** (-2.0 * np.arange(D // 2) / D)).astype(np.float32)[None, :]
    got = W.apply_rope_interleaved(x, np.cos(pos * freq), np.sin(pos * freq))
    assert np.max(np.abs(got - want)) < kat["tol"]


def test_config2_inputs_unit_rms_and_rotation_preserves_norm():
    w = W.config2(H=2, n_text=16, grid=8, D=128)
    assert w.shape == (1, 2, 80, 80, 128)
    for t in (w.q, w.k):
        x = W.bf16_bits_to_f32(t).astype(np.float64)
        rms = np.sqrt((x * x).mean(-1))
        assert np.max(np.abs(rms - 1.0)) < 1e-2          # rotation keeps the unit RMS of each row
    cos, sin = W.axial_rope_tables(16, 8, 8, 128)
    assert cos.shape == (80, 64)
    # image token (r=2,c=5): first half of the pairs uses y=2, second half x=5, frequency index p mod 32
    n = 16 + 8 * 2 + 5
    assert abs(cos[n, 0] - math.cos(2.0)) < 1e-6 and abs(cos[n, 32] - math.cos(5.0)) < 1e-6
    assert abs(sin[n, 33] - math.sin(5.0 * 10000.0 ** (-1 / 32))) < 1e-6
    assert abs(cos[7, 1] - math.cos(7.0 * 10000.0 ** (-1 / 32))) < 1e-6   # text token: y = x = t


def test_config_shapes_and_flops():
    w3 = W.config3(H=1, Sq=8)
    assert w3.k.shape == (4, 1, 2049, 64) and w3.kv_len.tolist() == [77, 333, 1024, 2049]
    assert W.bf16_bits_to_f32(w3.k)[0, 0, 77, 0] == W.bf16_bits_to_f32(W.f32_to_bf16_bits(np.float32([1e4])))[0]
    assert w3.valid_pairs() == 8 * (77 + 333 + 1024 + 2049)
    w1 = W.config1()
    assert w1.flops() == 14 * 4 * 256 * 256 * 64
    w4 = W.config4(H=1, S=64, D=8)
    assert w4.causal and w4.valid_pairs() == 64 * 65 // 2
    s = W.config2(H=1, n_text=0, grid=2).saved_activation_bytes()
    assert s["O_bf16"] == 4 * 128 * 2 and s["LSE_f32"] == 16 and s["materialised_P_f32"] == 64
