/* CPU restatement of the reference's BF16 <-> FP8 E4M3 pair of the activation offload pool
 * (reference: src/cuda/fp8_quant.cu:19-72, src/cuda/fp8_dequant.cu:10-39), written the way the reference writes it
 * (frexpf, a float mantissa, +0.5 and truncation), not the way the GPU code does it (bit patterns).
 * TEST INFRASTRUCTURE ONLY: loaded by tests/ and by nothing that ships.
 *
 * The reference is compiled with flush-to-zero (build.rs:261, :295: --use_fast_math), which this host does not
 * do by itself: denormal operands and results of the two multiplications are flushed by hand below.
 *
 * Pinning (tests/test_oracle_fp8.py):
 *   decoder   all 256 codes against the E4M3 value table written as (1 + m/8) 2^(e-7) / m 2^-9 in exact rationals,
 *             with the literal anchors 0x38 = 1, 0x08 = 2^-6, 0x01 = 2^-9, 0x77 = 240, 0x7F = 480 (no NaN code)
 *   encoder   against a nearest-value search over that table in exact rationals (ties to the larger magnitude;
 *             256 and above -> 0x7F; below 2^-6 the subnormal rule with its cap), for every bf16 input at several
 *             scales and for fp32 products chosen at the rounding boundaries; literal anchors; monotone in |x|;
 *             encode(decode(c)) = c for every code the encoder can produce
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <stddef.h>

static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float ftz(float f) { return (f2u(f) & 0x7f800000u) == 0 ? u2f(f2u(f) & 0x80000000u) : f; }

static uint16_t f32_to_bf16_rne(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* fp8_quant.cu:19-57, on a product that has already been flushed */
uint8_t oracle_f32_to_fp8_e4m3(float val) {
    uint8_t sign = 0;
    if (val != val) return (uint8_t)(((f2u(val) >> 24) & 0x80u) | 0x7fu);   /* not specified by the reference */
    if (val < 0.0f) { sign = 0x80; val = -val; }
    if (val > 448.0f) val = 448.0f;
    if (val == 0.0f) return sign;
    int exp;
    float frac = frexpf(val, &exp);          /* val = frac 2^exp, frac in [0.5, 1) */
    exp -= 1;
    int biased = exp + 7;
    if (biased <= 0) {
        float subnorm = val * ldexpf(1.0f, 6);
        int mant = (int)(subnorm * 8.0f + 0.5f);
        if (mant > 7) mant = 7;
        if (mant < 0) mant = 0;
        return (uint8_t)(sign | mant);
    }
    if (biased >= 15) return (uint8_t)(sign | 0x7f);
    float mant_f = (2.0f * frac - 1.0f) * 8.0f;
    int mant = (int)(mant_f + 0.5f);
    if (mant > 7) { mant = 0; biased += 1; }
    if (biased >= 15) return (uint8_t)(sign | 0x7f);
    return (uint8_t)(sign | (biased << 3) | mant);
}

/* fp8_quant.cu:59-72 */
void oracle_bf16_to_fp8(const uint16_t* in, uint8_t* out, float inv_scale, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        float x = ftz(u2f((uint32_t)in[i] << 16));
        out[i] = oracle_f32_to_fp8_e4m3(ftz(x * ftz(inv_scale)));
    }
}

/* fp8_dequant.cu:10-39 */
void oracle_fp8_to_bf16(const uint8_t* in, uint16_t* out, float scale, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        uint8_t bits = in[i];
        int sign = (bits >> 7) & 1, exp = (bits >> 3) & 0xf, mant = bits & 7;
        float val;
        if (exp == 0 && mant == 0) val = 0.0f;
        else if (exp == 0) val = ldexpf((float)mant / 8.0f, -6);
        else val = ldexpf(1.0f + (float)mant / 8.0f, exp - 7);
        if (sign) val = -val;
        val = ftz(val * ftz(scale));
        out[i] = f32_to_bf16_rne(val);
    }
}
