/* CPU restatement of the reference's element-wise primitives on score tiles
 * (reference: src/kernels/sdpa_kernels.cu).  TEST INFRASTRUCTURE ONLY: loaded by tests/, by the smoke check and
 * by nothing that ships.
 *
 * Pinning (tests/test_oracle_tile_ops.py):
 *   masks           exact: literal known answers written out by hand and an independent numpy statement of the
 *                   predicate on random tiles; the summation order of the additive tile mask by a case where
 *                   fp32 addition is not associative (1e30 + (-1e30) + 1)
 *   softmax / lse   against fp64 log-sum-exp and exp; rows of one element (lse = the element), rows shifted by
 *                   a constant (lse shifts by it), merge of two halves = lse of the whole row
 *   dropout         the uniform generator against literal values computed by hand from the xorshift recurrence
 *                   in Python integers; kept fraction against p; kept values exactly bf16(x / (1 - p))
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <float.h>

static float bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t f32_to_bf16_rne(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);   /* NaN stays NaN */
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* sdpa_kernels.cu:35-61 */
void oracle_tile_causal_mask(float* scores, int B, int H, int Q, int K, int q_offset, int k_offset) {
    for (int64_t bh = 0; bh < (int64_t)B * H; ++bh)
        for (int q = 0; q < Q; ++q)
            for (int k = 0; k < K; ++k)
                if (k_offset + k > q_offset + q) scores[(bh * Q + q) * K + k] = -1.0e9f;
}

/* sdpa_kernels.cu:63-79 */
void oracle_tile_attn_mask(float* scores, const uint8_t* mask, int64_t total) {
    for (int64_t i = 0; i < total; ++i)
        if (mask[i] == 0) scores[i] = -1.0e9f;
}

/* sdpa_kernels.cu:81-138: delta starts at 0 and takes the additive operand, the boolean exclusion and the causal
 * exclusion in that order; the logit then takes delta. */
void oracle_tile_add_mask(float* logits, const uint8_t* user_bool, const float* user_add, int BH, int q_t, int k_t,
                          int q_abs_start, int k_abs_start, int bool_rank, int add_rank, int k_total,
                          int zero_is_mask, int causal) {
    for (int bh = 0; bh < BH; ++bh)
        for (int qi = 0; qi < q_t; ++qi)
            for (int kj = 0; kj < k_t; ++kj) {
                const int64_t index = ((int64_t)bh * q_t + qi) * k_t + kj;
                const int k_abs = k_abs_start + kj;
                volatile float delta = 0.0f;            /* volatile: every partial sum is rounded to fp32 */
                if (user_add) {
                    if (add_rank == 3) delta += user_add[index];
                    else if (add_rank == 2) delta += user_add[(int64_t)bh * k_total + k_abs];
                }
                if (user_bool) {
                    uint8_t mv = 1;
                    if (bool_rank == 3) mv = user_bool[index];
                    else if (bool_rank == 2) mv = user_bool[(int64_t)bh * k_total + k_abs];
                    if (zero_is_mask ? mv == 0 : mv != 0) delta += -1.0e30f;
                }
                if (causal && k_abs > q_abs_start + qi) delta += -1.0e30f;
                logits[index] += delta;
            }
}

/* sdpa_kernels.cu:140-157 */
void oracle_tile_softmax_from_lse(const float* logits, const float* lse_row, uint16_t* probs, float* probs_f32, int BH,
                                  int q_t, int k_t) {
    for (int64_t row = 0; row < (int64_t)BH * q_t; ++row)
        for (int kj = 0; kj < k_t; ++kj) {
            const float p = expf(logits[row * k_t + kj] - lse_row[row]);
            probs[row * k_t + kj] = f32_to_bf16_rne(p);
            if (probs_f32) probs_f32[row * k_t + kj] = p;
        }
}

/* sdpa_kernels.cu:159-199: maximum from -FLT_MAX, then log(sum exp(x - max)) + max */
void oracle_tile_lse_from_logits(const float* logits, float* out, int BH, int q_t, int k_t) {
    for (int64_t row = 0; row < (int64_t)BH * q_t; ++row) {
        float mx = -FLT_MAX;
        for (int kj = 0; kj < k_t; ++kj) mx = fmaxf(mx, logits[row * k_t + kj]);
        double sum = 0.0;
        for (int kj = 0; kj < k_t; ++kj) sum += exp((double)logits[row * k_t + kj] - (double)mx);
        out[row] = (float)(log(sum) + (double)mx);
    }
}

/* sdpa_kernels.cu:201-214; two -inf give -inf (the reference's expression is NaN there) */
void oracle_tile_lse_merge(float* lse_row, const float* tile_lse_row, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        const float a = lse_row[i], b = tile_lse_row[i];
        const float m = fmaxf(a, b);
        if (m == -INFINITY) { lse_row[i] = -INFINITY; continue; }
        lse_row[i] = (float)((double)m + log(exp((double)a - m) + exp((double)b - m)));
    }
}

static uint32_t xorshift32(uint32_t x) {
    x ^= x << 13;
    x ^= x >> 17;
    x ^= x << 5;
    return x;
}

/* sdpa_kernels.cu:18-33 */
float oracle_tile_uniform01(uint64_t seed, int b, int qi, int kj) {
    const uint32_t s = (uint32_t)seed ^
                       (1103515245u * (((uint32_t)b * 73856093u) ^ ((uint32_t)qi * 19349663u) ^ ((uint32_t)kj * 83492791u)));
    return (float)(xorshift32(s) & 0x00FFFFFFu) / 16777216.0f;
}

/* sdpa_kernels.cu:216-243 */
void oracle_tile_dropout(uint16_t* probs, float p, uint64_t seed, int BH, int q_t, int k_t) {
    const float keep = 1.0f - p;
    const float scale = keep > 0.0f ? 1.0f / keep : 0.0f;
    for (int bh = 0; bh < BH; ++bh)
        for (int qi = 0; qi < q_t; ++qi)
            for (int kj = 0; kj < k_t; ++kj) {
                const int64_t index = ((int64_t)bh * q_t + qi) * k_t + kj;
                float val = bf16_to_f32(probs[index]);
                if (oracle_tile_uniform01(seed, bh, qi, kj) < p) val = 0.0f;
                else val *= scale;
                probs[index] = f32_to_bf16_rne(val);
            }
}
