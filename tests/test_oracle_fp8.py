"""Pins the CPU oracle of the BF16 <-> FP8 E4M3 pair of the activation offload pool (oracle/fp8_oracle.c restates
src/cuda/fp8_quant.cu:19-72 and src/cuda/fp8_dequant.cu:10-39 with frexpf and float mantissas, as the reference
does).  The reference holds no test vectors for the pair, so the oracle is checked against what the format fixes:
the E4M3 value table in exact rationals, a nearest-value search over it (ties to the larger magnitude, the
reference's early saturation and subnormal cap as stated rules), literal anchors, monotonicity and round trips.
A wrong bias, tie direction, carry into the exponent or subnormal step fails one of them."""
from fractions import Fraction

import numpy as np
import pytest
import torch

# value of code c (sign stripped) as the reference's decoder reads it: no NaN / inf codes
TABLE = [Fraction(c & 7, 8) * Fraction(1, 64) if c >> 3 == 0 else (1 + Fraction(c & 7, 8)) * Fraction(2) ** ((c >> 3) - 7)
         for c in range(128)]


def _bf16_bits_of_f32(x):
    """bf16 rounding by torch (round to nearest even), as an independent statement of __float2bfloat16."""
    t = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16)
    return t.view(torch.int16).numpy().view(np.uint16)


def _ftz32(x):
    x = np.asarray(x, dtype=np.float32).copy()
    u = x.view(np.uint32)
    u[(u & 0x7F800000) == 0] &= 0x80000000
    return x


def _round_to_f32(s: Fraction) -> Fraction:
    """Nearest fp32 (ties to even) of a positive rational inside the normal range."""
    e = 0
    while Fraction(2) ** (e + 1) <= s:
        e += 1
    while Fraction(2) ** e > s:
        e -= 1
    q = s / Fraction(2) ** (e - 23)
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return n * Fraction(2) ** (e - 23)


def _model_encode(v: Fraction) -> int:
    """Code of an exact fp32 product v (already flushed), stated from the format: see the module docstring."""
    sign = 0x80 if v < 0 else 0
    v = abs(v)
    if v == 0:
        return 0 if sign == 0 else 0x80        # only +0 reaches here in practice (-0 < 0 is false): see the callers
    v = min(v, Fraction(448))
    if v >= 256:
        return sign | 0x7F                      # saturates one binade early
    if v < Fraction(1, 64):
        k = int(_round_to_f32(v * 512 + Fraction(1, 2)))     # floor of the fp32 sum
        return sign | min(k, 7)                 # rounding up to the smallest normal is capped
    best = min(range(8, 0x79), key=lambda c: (abs(TABLE[c] - v) if c < 0x78 else abs(Fraction(256) - v), -c))
    return sign | (0x7F if best == 0x78 else best)


def test_decoder_reads_every_code_as_the_table_says(oracle):
    codes = np.arange(256, dtype=np.uint8)
    assert TABLE[0x38] == 1 and TABLE[0x08] == Fraction(1, 64) and TABLE[0x01] == Fraction(1, 512)
    assert TABLE[0x77] == 240 and TABLE[0x7E] == 448 and TABLE[0x7F] == 480
    for scale in (1.0, float(np.float32(8.0 / 448.0)), 0.37, 3.0e38, 2.0 ** -120):
        got = oracle.fp8_to_bf16(codes, scale)
        vals = np.array([float(TABLE[c & 0x7F]) * (-1.0 if c & 0x80 else 1.0) for c in range(256)], dtype=np.float32)
        with np.errstate(over="ignore"):
            prod = _ftz32(vals * np.float32(scale))
        want = _bf16_bits_of_f32(prod)
        # a flushed product keeps the sign of the code (sign-preserving zero); -0 * scale too
        want[128:][prod[128:] == 0] = 0x8000
        assert np.array_equal(got, want), scale
    # scale 1: the bf16 value is the table value itself (3 mantissa bits fit)
    got = oracle.fp8_to_bf16(codes[:128], 1.0)
    assert [Fraction(float(x)) for x in oracle.bf16_to_f32(got)] == TABLE


def test_encoder_literal_anchors(oracle):
    enc = oracle.f32_to_fp8_e4m3
    assert enc(0.0) == 0x00 and enc(-0.0) == 0x00          # `-0.0 < 0` is false
    assert enc(1.0) == 0x38 and enc(-1.0) == 0xB8
    assert enc(1.0625) == 0x39                             # tie between 1 and 1.125 goes up (half up, not to even)
    assert enc(1.1875) == 0x3A                             # tie between 1.125 and 1.25 goes up as well
    assert enc(1.96875) == 0x40                            # rounds up into the next binade: 2.0
    assert enc(240.0) == 0x77 and enc(247.9) == 0x77
    assert enc(248.0) == 0x7F                              # would be 256: saturates
    assert enc(256.0) == 0x7F and enc(448.0) == 0x7F and enc(1e30) == 0x7F and enc(float("inf")) == 0x7F
    assert enc(-300.0) == 0xFF
    assert enc(2.0 ** -6) == 0x08 and enc(2.0 ** -9) == 0x01
    assert enc(7.49 / 512) == 0x07 and enc(7.5 / 512) == 0x07 and enc(7.99 / 512) == 0x07   # capped, not 0x08
    assert enc(0.49 / 512) == 0x00 and enc(0.5 / 512) == 0x01
    # the sum product * 512 + 0.5 is rounded to fp32 before truncation: 0.5 - 2^-25 + 0.5 rounds to 1
    assert enc(float(np.float32((0.5 - 2.0 ** -25) / 512))) == 0x01
    assert enc(float(np.float32((0.5 - 2.0 ** -24) / 512))) == 0x00


def test_encoder_against_the_exact_model_at_every_rounding_boundary(oracle):
    pts = []
    for c in range(1, 0x79):                               # midpoints between neighbouring table values, and the values
        lo, hi = TABLE[c - 1], (TABLE[c] if c < 0x78 else Fraction(256))
        for x in (lo, hi, (lo + hi) / 2):
            f = np.float32(float(x))
            pts += [f, np.nextafter(f, np.float32(0)), np.nextafter(f, np.float32(1e9))]
    for k in range(0, 9):                                  # subnormal steps: (k + 0.5) / 512 and neighbours
        for d in (-2.0 ** -25, -2.0 ** -24, 0.0, 2.0 ** -24):
            pts.append(np.float32((k + 0.5 + d) / 512))
    pts += [np.float32(x) for x in (448.0, 449.0, 255.99998, 2.0 ** -126, 1.5 * 2.0 ** -126, 3e-20, 1e-10)]
    n = 0
    for f in pts:
        for s in (1.0, -1.0):
            v = float(f) * s
            if v == 0.0:
                continue
            assert oracle.f32_to_fp8_e4m3(v) == _model_encode(Fraction(v)), (v, hex(oracle.f32_to_fp8_e4m3(v)))
            n += 1
    assert n > 1500


def _vector_model(prod32):
    """Codes of flushed fp32 products, vectorised: table midpoints in float64 (exact for these values)."""
    v = np.abs(prod32.astype(np.float64))
    tab = np.array([float(TABLE[c]) for c in range(8, 0x78)] + [256.0])
    mids = (tab[:-1] + tab[1:]) / 2
    code = 8 + np.searchsorted(mids, v, side="right")      # a tie goes to the larger value
    code = np.where(code >= 0x78, 0x7F, code)
    code = np.where(v >= 248.0, 0x7F, code)
    with np.errstate(over="ignore", invalid="ignore"):
        k = (np.abs(prod32) * np.float32(512) + np.float32(0.5)).astype(np.float32)
    sub = np.minimum(np.floor(np.where(np.isfinite(k), k, 0)), 7).astype(np.int64)
    code = np.where(v < 2.0 ** -6, sub, code)
    code = np.where(prod32 < 0, code | 0x80, code)
    return np.where(v == 0, 0, code).astype(np.uint8)


@pytest.mark.parametrize("inv_scale", [1.0, 56.0, float(np.float32(1.0 / 0.37)), float(np.float32(448.0 / 3.0)), 2.0 ** -100, 2.0 ** 90])
def test_encoder_on_every_bf16_input(oracle, inv_scale):
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = _ftz32((bits.astype(np.uint32) << 16).view(np.float32))           # denormal inputs count as zero
    with np.errstate(over="ignore", invalid="ignore"):
        prod = _ftz32(x * np.float32(inv_scale))                            # ... and so do denormal products
    ok = ~np.isnan(prod)
    got = oracle.bf16_to_fp8(bits, inv_scale)
    want = _vector_model(prod)
    assert np.array_equal(got[ok], want[ok])
    # NaN inputs: sign | 0x7F by this build's choice (the reference leaves it open)
    assert np.all((got[~ok] & 0x7F) == 0x7F)


def test_encoder_is_monotone_and_round_trips(oracle):
    bits = np.arange(0x0080, 0x7F80, dtype=np.uint16)                       # positive normal bf16, ascending
    for inv_scale in (1.0, 56.0, 0.013):
        codes = oracle.bf16_to_fp8(bits, inv_scale).astype(np.int64)
        assert np.all(np.diff(codes) >= 0)
        neg = oracle.bf16_to_fp8(bits | 0x8000, inv_scale).astype(np.int64)
        with np.errstate(over="ignore"):
            prod = (bits.astype(np.uint32) << 16).view(np.float32) * np.float32(inv_scale)
        flushed = np.abs(prod) < np.float32(2.0 ** -126)
        # the sign is kept also where the magnitude rounds to 0 (the product is not zero), but not where the
        # product itself is flushed to zero
        assert np.array_equal(neg, np.where(flushed, 0, codes | 0x80))
    producible = np.array(list(range(0, 0x78)) + [0x7F], dtype=np.uint8)
    back = oracle.bf16_to_fp8(oracle.fp8_to_bf16(producible, 1.0), 1.0)
    assert np.array_equal(back, producible)
    # the codes the encoder never writes decode to values it maps to 0x7F
    dead = np.arange(0x78, 0x7F, dtype=np.uint8)
    assert np.all(oracle.bf16_to_fp8(oracle.fp8_to_bf16(dead, 1.0), 1.0) == 0x7F)


def test_round_trip_error_with_the_pool_scale(oracle):
    """|x| < 32/7 with the pool's scale 8/448: relative error at most 1/16 (3 mantissa bits, half-up) above the
    subnormal range, absolute error at most one subnormal step below it (half a step from rounding, a whole one
    where the cap keeps a product just under 2^-6 at the largest subnormal)."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal(200000).astype(np.float32)
    x = x[np.abs(x) < 4.5]
    xb = _bf16_bits_of_f32(x)
    scale = np.float32(8.0 / 448.0)
    back = oracle.bf16_to_f32(oracle.fp8_to_bf16(oracle.bf16_to_fp8(xb, float(np.float32(1.0) / scale)), float(scale)))
    ref = oracle.bf16_to_f32(xb)
    err = np.abs(back - ref)
    big = np.abs(ref) >= 2.0 ** -6 * scale
    assert np.all(err[big] <= np.abs(ref[big]) / 16 * 1.01 + 1e-9)
    assert np.all(err[~big] <= 2.0 ** -9 * scale * 1.01 + np.abs(ref[~big]) * 2.0 ** -8)
    assert np.sqrt(np.mean(err ** 2)) / np.sqrt(np.mean(ref ** 2)) < 0.03
