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


def test_sage_forward_literal_known_answer(oracle):
    """2 queries x 2 keys x head dim 1 with one block per row, worked by hand:
    S = qi8 * ki8 * sq[i] * sk[j] = [[2*1*0.5*1, 2*(-1)*0.5*2], [3*1*1*1, 3*(-1)*1*2]] = [[1, -2], [3, -6]];
    V = [1, 0], so O_i is the weight of key 0: 1/(1+e^-3), 1/(1+e^-9); LSE = 1 + ln(1+e^-3), 3 + ln(1+e^-9).
    Swapping sq and sk, or indexing either by the other's block, gives different logits."""
    qi8 = np.array([2, 3], np.int8).reshape(1, 1, 2, 1)
    ki8 = np.array([1, -1], np.int8).reshape(1, 1, 2, 1)
    sq = np.array([0.5, 1.0], np.float32).reshape(1, 1, 2)
    sk = np.array([1.0, 2.0], np.float32).reshape(1, 1, 2)
    v = _bits(np.array([1.0, 0.0], np.float32).reshape(1, 1, 2, 1))
    _, lse, o = oracle.sage_fwd(qi8, ki8, sq, sk, v, 1.0, qblk=1, kblk=1, want_f32=True)
    assert np.allclose(o.ravel(), [0.9525741268224334, 0.9998766054240137], rtol=0, atol=2e-7)
    assert np.allclose(lse.ravel(), [1.048587351573742, 3.000123402189723], rtol=0, atol=5e-7)
    # causal: key 1 is excluded for query 0 (j > i), not for query 1
    _, lse, o = oracle.sage_fwd(qi8, ki8, sq, sk, v, 1.0, qblk=1, kblk=1, causal=True, want_f32=True)
    assert np.allclose(o.ravel(), [1.0, 0.9998766054240137], rtol=0, atol=2e-7)
    assert np.allclose(lse.ravel(), [1.0, 3.000123402189723], rtol=0, atol=5e-7)
    # key length 1: key 1 is excluded for both; key length 0: nothing is attended
    _, lse, o = oracle.sage_fwd(qi8, ki8, sq, sk, v, 1.0, qblk=1, kblk=1, kv_len=[1], want_f32=True)
    assert np.allclose(o.ravel(), [1.0, 1.0], rtol=0, atol=2e-7) and np.allclose(lse.ravel(), [1.0, 3.0], atol=5e-7)
    ob, lse = oracle.sage_fwd(qi8, ki8, sq, sk, v, 1.0, qblk=1, kblk=1, kv_len=[0])
    assert np.all(ob == 0) and np.all(lse == -np.inf)


def _sage_case(oracle, B, H, Sq, Sk, D, seed):
    """Quantised operands whose blocks have deliberately different magnitudes, short last blocks."""
    qf = W.normal_f32(seed, 0, B * H * Sq * D).reshape(B, H, Sq, D)
    kf = W.normal_f32(seed, 1, B * H * Sk * D).reshape(B, H, Sk, D)
    for ib, mul in enumerate((1.0, 6.0, 0.5)):
        qf[:, :, 128 * ib:128 * (ib + 1)] *= np.float32(mul)
    for jb, mul in enumerate((1.0, 4.0, 0.25, 2.0, 8.0)):
        kf[:, :, 64 * jb:64 * (jb + 1)] *= np.float32(mul)
    v = _bits(W.normal_f32(seed, 2, B * H * Sk * D).reshape(B, H, Sk, D))
    z = oracle.sage_quant(_bits(qf), _bits(kf), qblk=128, kblk=64, smooth_k=False)
    # per-block scales differ by the factors above, so a wrong block index cannot go unnoticed
    assert z["sq"].max() / z["sq"].min() > 4 and z["sk"].max() / z["sk"].min() > 8
    return z, v


def _dequantised(z, Sq, Sk):
    qd = z["qi8"].astype(np.float64) * np.repeat(z["sq"].astype(np.float64), 128, axis=-1)[..., :Sq, None]
    kd = z["ki8"].astype(np.float64) * np.repeat(z["sk"].astype(np.float64), 64, axis=-1)[..., :Sk, None]
    return qd, kd


def test_sage_forward_against_fp64_brute_force_on_dequantised_operands(oracle):
    """oracle_sage_fwd must equal textbook attention on Q~ = qi8 * sq[block], K~ = ki8 * sk[block]:
    O (before rounding) and LSE within 2e-5, with and without the causal flag and key lengths,
    Sq != Sk, short last blocks (200 = 128 + 72 queries, 150 = 64 + 64 + 22 keys)."""
    B, H, Sq, Sk, D = 2, 2, 200, 150, 16
    z, v = _sage_case(oracle, B, H, Sq, Sk, D, seed=31)
    qd, kd = _dequantised(z, Sq, Sk)
    vf = W.bf16_bits_to_f32(v).astype(np.float64)
    scale = 0.03            # logits of a few units: fp32 rounding of the logits stays far below 2e-5
    i = np.arange(Sq)[:, None]
    j = np.arange(Sk)[None, :]
    kv_len = np.array([150, 97], np.int32)
    cases = {
        "plain": (False, None, None),
        "causal": (True, None, np.broadcast_to(j <= i, (B, H, Sq, Sk))),
        "kv_len": (False, kv_len, np.broadcast_to((j < kv_len[:, None, None, None]), (B, H, Sq, Sk))),
        "causal+kv_len": (True, kv_len, np.broadcast_to((j <= i) & (j < kv_len[:, None, None, None]), (B, H, Sq, Sk))),
    }
    for name, (causal, kvl, keep) in cases.items():
        want_o, want_lse, _ = oracle.brute_sdpa_f64(qd, kd, vf, scale, keep=keep)
        assert np.abs(want_lse).max() < 30 and np.abs(want_lse).max() > 1, name
        _, lse, o32 = oracle.sage_fwd(z["qi8"], z["ki8"], z["sq"], z["sk"], v, scale, causal=causal, kv_len=kvl,
                                      want_f32=True)
        assert oracle.max_abs(o32, want_o) <= 2e-5, (name, oracle.max_abs(o32, want_o))
        assert oracle.max_abs(lse, want_lse) <= 2e-5, (name, oracle.max_abs(lse, want_lse))
    # additive bias (the reference's attention_mask), per head and broadcast over heads, with excluded positions
    rng = np.random.default_rng(5)
    for shape in ((B, H, Sq, Sk), (B, 1, Sq, Sk), (1, 1, Sq, Sk)):
        bias = rng.normal(size=shape).astype(np.float32) * 2
        bias[..., 3::7] = -np.inf
        bias[0, 0, 5, :] = -np.inf                       # a row that loses every key
        want_o, want_lse, _ = oracle.brute_sdpa_f64(qd, kd, vf, scale, bias=np.broadcast_to(bias, (B, H, Sq, Sk)))
        _, lse, o32 = oracle.sage_fwd(z["qi8"], z["ki8"], z["sq"], z["sk"], v, scale, bias=bias, want_f32=True)
        fin = np.isfinite(want_lse)
        assert not fin[0, 0, 5] and np.array_equal(np.isfinite(lse), fin)
        assert oracle.max_abs(o32, want_o) <= 2e-5 and oracle.max_abs(lse[fin], want_lse[fin]) <= 2e-5, shape
    # the check has teeth: block scales indexed by the other operand's block size change the result
    bad_sq = np.repeat(z["sq"], 2, axis=-1)[..., :z["sq"].shape[-1]]     # as if Q blocks were 64 rows
    _, _, o_bad = oracle.sage_fwd(z["qi8"], z["ki8"], bad_sq, z["sk"], v, scale, want_f32=True)
    want_o, _, _ = oracle.brute_sdpa_f64(qd, kd, vf, scale)
    assert oracle.max_abs(o_bad, want_o) > 1e-2


def test_sage_forward_row_and_head_ranges(oracle):
    B, H, Sq, Sk, D = 1, 3, 200, 150, 16
    z, v = _sage_case(oracle, B, H, Sq, Sk, D, seed=32)
    full_o, full_lse = oracle.sage_fwd(z["qi8"], z["ki8"], z["sq"], z["sk"], v, 0.03, causal=True)
    o, lse = oracle.sage_fwd(z["qi8"], z["ki8"], z["sq"], z["sk"], v, 0.03, causal=True, heads=(1, 2), rows=(120, 140))
    assert np.array_equal(o[0, 1, 120:140], full_o[0, 1, 120:140]) and np.array_equal(lse[0, 1, 120:140], full_lse[0, 1, 120:140])
    o[0, 1, 120:140] = 0
    assert not o.any()


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
