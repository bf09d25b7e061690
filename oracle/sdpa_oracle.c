/*
 * CPU oracle for the activation-memory-saving attention path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library may link, load or
 * call this file; it exists so that the HIP kernels can be checked against a
 * plain restatement of the reference's naive, materialised, fp32-accumulated
 * scaled-dot-product attention, and so that the benchmark can time that naive
 * algorithm on the host cores as a reported baseline.
 *
 * Reference algorithm followed (paths relative to the reference tree):
 *   forward   tests/fa2_parity_naive.rs:90-140      (upcast, QK^T, scale, max/exp/sum/div, PV, bf16)
 *   backward  tests/cudnn_sdpa_bwd_parity.rs:31-98  (dV=P^T dO, dP=dO V^T, D=rowsum(dO*O),
 *                                                    dS=P*(dP-D), dQ=dS K scale, dK=dS^T Q scale)
 *   bias      src/sdpa.rs:232-328                   (additive fp32 bias on the scaled logits, forward only)
 *   keep-mask src/sdpa.rs:458-470, src/tests/attention_tests.rs:61-108 (mask < 0.5 => excluded)
 *   causal    kernels/sdpa_kernels.cu:129-135       (absolute k > q is excluded)
 *   LSE       third_party/cudnn_frontend/include/cudnn_frontend/node/softmax.h:139-213
 *             (Stats = max + ln(sum exp(s - max)), natural log of the scaled logits)
 *   int8 quantisation closed form  src/sage_attention.rs:524-541
 *             (scale = absmax/127, q = clamp(round_half_even(x/scale), -128, 127))
 *
 * Deviations that are deliberate and stated:
 *   - excluded positions are treated as exactly -inf (weight 0), where the
 *     reference adds a large negative constant (-1e9 / -1e30): the results
 *     agree unless a whole row is excluded; such a row here gives O = 0,
 *     LSE = -inf and zero gradients.
 *   - the backward forms D from the bf16-rounded O (what a kernel that reads
 *     the saved O sees), the reference test uses its un-rounded fp32 O.
 *
 * Pinning status (see tests/test_oracle_*.py):
 *   forward O        pinned: reference 2x2 known-answer test, fp64 brute force, torch CPU SDPA, invariants
 *   additive bias    pinned: torch CPU SDPA with a float attn_mask, shift invariance (bias constant
 *                    per row leaves O unchanged), bias = -inf-like values reproduce the keep-mask result
 *   LSE              pinned by the closed form and sum_j exp(s_ij - LSE_i) = 1 only;
 *                    no reference test asserts Stats values ("parity unpinned" by the reference itself)
 *   dQ, dK, dV       pinned: fp64 central finite differences, torch CPU autograd
 *   int8 quantiser   pinned: brute force in Python integers/fp64, tie and absmax unit vectors
 *   K-mean smoothing pinned: fp64 column means, softmax shift invariance
 *   int8-QK forward  (per-block 128/64 scales, causal flag, key lengths; new behaviour with no counterpart
 *                    in the reference) pinned: a hand-worked 2x2 known answer with distinct scales per
 *                    block; fp64 textbook attention on the dequantised operands qi8*sq[block],
 *                    ki8*sk[block] with block magnitudes 4-8x apart and short last blocks (O and LSE
 *                    within 2e-5), with a control that a wrong block index fails
 *   row bands        pinned: bit-identical to the rows of the full computation
 *   dropout          (src/autograd_v4/ops/sdpa.rs:229-231, :444, :600-649; generator src/rng/mod.rs:14-24) pinned:
 *                    the kept set of the unchunked and of the chunked draw against the xorshift recurrence, the
 *                    tile seeds and the tiles' own flat indices in Python integers; forward against fp64 attention
 *                    with that set; backward against fp64 central differences and closed-form fp64 gradients
 *
 * Layout: every tensor is contiguous [B,H,S,D]; bf16 is carried as uint16_t.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even, NaN kept quiet */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

void oracle_bf16_to_f32(const uint16_t* src, float* dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = bf16_to_f32(src[i]);
}
void oracle_f32_to_bf16(const float* src, uint16_t* dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = f32_to_bf16(src[i]);
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
void oracle_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

typedef struct {
    int causal;
    const int32_t* kv_len;   /* [B] or NULL: keys >= kv_len[b] are excluded          */
    const uint8_t* mask;     /* keep-mask (non-zero = attend) or NULL                 */
    int64_t msb, msh, msq, msk; /* element strides of mask over (b,h,q,k); 0 = broadcast */
    const float* bias;       /* additive fp32 bias on the scaled logits or NULL (src/sdpa.rs:288-305) */
    int64_t bsb, bsh, bsq, bsk; /* its element strides over (b,h,q,k); 0 = broadcast     */
    float drop_p;            /* dropout probability, 0 = none                          */
    uint64_t drop_seed;
    int drop_cq, drop_ck;    /* tiles of the draw along queries and keys; 0 = one draw over the whole tensor */
} mask_spec;

/* Dropout of the attention probabilities as the reference's autograd_v4 operator draws it when it is not
 * chunked (src/autograd_v4/ops/sdpa.rs:229-231, :600-649 with q_offset = k_offset = 0): one uniform per element of
 * the [B*H, Sq, Sk] probability tensor, u = (xorshift32(seed32 ^ index32) >> 8) / 2^24 with index the flat element
 * index and seed32 / index32 their low 32 bits (src/rng/mod.rs:14-24); an element is kept when u >= p, and kept
 * elements are multiplied by 1 / (1 - p), both in fp32.  The probabilities themselves, and the log-sum-exp, are
 * those of the undropped softmax. */
static inline uint32_t drop_xorshift32(uint32_t x) {
    x ^= x << 13;
    x ^= x >> 17;
    x ^= x << 5;
    return x;
}
int oracle_dropout_keep(uint64_t seed, uint64_t flat_index, float p) {
    const uint32_t s = drop_xorshift32((uint32_t)seed ^ (uint32_t)flat_index);
    const float u = (float)(s >> 8) * (1.0f / 16777216.0f);
    return u >= p;
}
/* The same operator when it is chunked (save = SaveLSE and a query or key chunk shorter than the sequence,
 * :180-199): it draws per tile of chunk_q x chunk_kv (the last ones shorter), over the tile's own [B*H, q_t, k_t]
 * tensor, with the seed derive_tile_seed gives (:600-602): (seed + ((q_offset << 32) ^ k_offset)) truncated to 32
 * bits, which is seed32 + k_offset: the query offset does not reach the low word.  Element (bh, i, j) therefore has
 * index (bh * q_t + i - q_offset) * k_t + j - k_offset under seed32 + k_offset. */
int oracle_dropout_keep_tiled(uint64_t seed, int bh, int i, int j, int Sq, int Sk, int cq, int ck, float p) {
    if (cq <= 0 || cq > Sq) cq = Sq;
    if (ck <= 0 || ck > Sk) ck = Sk;
    const int q_off = (i / cq) * cq, k_off = (j / ck) * ck;
    const int q_t = Sq - q_off < cq ? Sq - q_off : cq, k_t = Sk - k_off < ck ? Sk - k_off : ck;
    const uint64_t tile_seed = seed + ((((uint64_t)q_off) << 32) ^ (uint64_t)k_off);      /* wrapping, as the reference */
    const uint64_t idx = ((uint64_t)bh * (uint64_t)q_t + (uint64_t)(i - q_off)) * (uint64_t)k_t + (uint64_t)(j - k_off);
    return oracle_dropout_keep(tile_seed, idx, p);
}
/* Operand rounding (off by default).  A kernel that forms P V, P^T dO, dS K and dS^T Q on a bf16 matrix unit has to
 * round the left operands (the dropped and rescaled probabilities, and dS) to bf16 first; the plain oracle keeps them
 * in fp32, as the reference's fp32 operator does.  With this switch on, the oracle rounds exactly those operands
 * (round to nearest even) and nothing else, which separates what the rounding of the operands costs from any other
 * difference.  Used by the dropout GPU tests, whose probabilities P / (1 - p) reach into [1, 2). */
static int g_round_operands = 0;
void oracle_set_operand_rounding(int on) { g_round_operands = on != 0; }
static inline float operand(float x) { return g_round_operands ? bf16_to_f32(f32_to_bf16(x)) : x; }

/* factor applied to P[bh, i, j]: 0 or 1 / (1 - p); 1 without dropout */
static inline float drop_factor(const mask_spec* ms, int bh, int i, int j, int Sq, int Sk) {
    if (!(ms->drop_p > 0.f)) return 1.0f;
    const float keep = 1.0f - ms->drop_p;
    return oracle_dropout_keep_tiled(ms->drop_seed, bh, i, j, Sq, Sk, ms->drop_cq, ms->drop_ck, ms->drop_p) ? 1.0f / keep : 0.f;
}

static inline int excluded(const mask_spec* ms, int b, int h, int i, int j) {
    if (ms->causal && j > i) return 1;
    if (ms->kv_len && j >= ms->kv_len[b]) return 1;
    if (ms->mask && ms->mask[b * ms->msb + h * ms->msh + i * ms->msq + j * ms->msk] == 0) return 1;
    return 0;
}

/* P (fp32, R x Sk) for the query rows [row0, row0 + R) of one head; also their LSE.
 * q = those R rows in fp32, kt = K^T in fp32 [D][Sk]. */
static void head_probs(const float* q, const float* kt, int row0, int R, int Sk, int D, float scale,
                       const mask_spec* ms, int b, int h, float* P, float* lse) {
    for (int i = 0; i < R; ++i) {
        float* row = P + (size_t)i * Sk;
        for (int j = 0; j < Sk; ++j) row[j] = 0.f;
        for (int d = 0; d < D; ++d) {
            const float qv = q[(size_t)i * D + d];
            const float* kr = kt + (size_t)d * Sk;
            for (int j = 0; j < Sk; ++j) row[j] += qv * kr[j];
        }
        float m = -INFINITY;
        for (int j = 0; j < Sk; ++j) {
            float s = excluded(ms, b, h, row0 + i, j) ? -INFINITY : row[j] * scale;
            if (ms->bias && s != -INFINITY) s += ms->bias[b * ms->bsb + h * ms->bsh + (row0 + i) * ms->bsq + j * ms->bsk];
            row[j] = s;
            if (s > m) m = s;
        }
        if (m == -INFINITY) { /* whole row excluded */
            for (int j = 0; j < Sk; ++j) row[j] = 0.f;
            lse[i] = -INFINITY;
            continue;
        }
        float l = 0.f;
        for (int j = 0; j < Sk; ++j) {
            float e = expf(row[j] - m);
            row[j] = e;
            l += e;
        }
        const float inv = 1.0f / l;
        for (int j = 0; j < Sk; ++j) row[j] *= inv;
        lse[i] = m + logf(l);
    }
}

static int check_dims(int B, int H, int Sq, int Sk, int D) {
    return (B > 0 && H > 0 && Sq > 0 && Sk > 0 && D > 0) ? 0 : -1;
}

/*
 * Forward.  O: bf16 [B,H,Sq,D]; LSE: fp32 [B,H,Sq]; O32 (optional): un-rounded fp32 O.
 * heads_begin/heads_end restrict the work to flat (b*H+h) indices in [begin,end) so that
 * long configurations can be checked on a head subset; pass 0 and B*H for everything.
 */
static int sdpa_fwd_impl(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                         int B, int H, int Sq, int Sk, int D, float scale, mask_spec ms,
                         int heads_begin, int heads_end, int row_begin, int row_end,
                         uint16_t* O, float* LSE, float* O32);

int oracle_sdpa_fwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                    int B, int H, int Sq, int Sk, int D, float scale, int causal,
                    const int32_t* kv_len, const uint8_t* mask,
                    int64_t msb, int64_t msh, int64_t msq, int64_t msk,
                    int heads_begin, int heads_end,
                    uint16_t* O, float* LSE, float* O32) {
    mask_spec ms = {causal, kv_len, mask, msb, msh, msq, msk, NULL, 0, 0, 0, 0, 0.f, 0, 0, 0};
    return sdpa_fwd_impl(Q, K, V, B, H, Sq, Sk, D, scale, ms, heads_begin, heads_end, 0, Sq, O, LSE, O32);
}

/* The same forward restricted to the query rows [row_begin, row_end) of the chosen heads: a band of a
 * long sequence then costs rows x Sk instead of Sq x Sk.  Outputs keep the full [B,H,Sq,...] layout;
 * only the rows of the band are written. */
int oracle_sdpa_fwd_rows(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                         int B, int H, int Sq, int Sk, int D, float scale, int causal,
                         const int32_t* kv_len, const uint8_t* mask,
                         int64_t msb, int64_t msh, int64_t msq, int64_t msk,
                         int heads_begin, int heads_end, int row_begin, int row_end,
                         uint16_t* O, float* LSE, float* O32) {
    mask_spec ms = {causal, kv_len, mask, msb, msh, msq, msk, NULL, 0, 0, 0, 0, 0.f, 0, 0, 0};
    if (row_begin < 0 || row_end > Sq || row_begin > row_end) return -1;
    return sdpa_fwd_impl(Q, K, V, B, H, Sq, Sk, D, scale, ms, heads_begin, heads_end, row_begin, row_end, O, LSE, O32);
}

/* Forward with an additive fp32 bias on the scaled logits (T5-style relative position bias),
 * following src/sdpa.rs:232-328: scores * scale, + bias, fp32 softmax, P V. */
int oracle_sdpa_fwd_bias(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                         int B, int H, int Sq, int Sk, int D, float scale,
                         const float* bias, int64_t bsb, int64_t bsh, int64_t bsq, int64_t bsk,
                         uint16_t* O, float* LSE, float* O32) {
    mask_spec ms = {0, NULL, NULL, 0, 0, 0, 0, bias, bsb, bsh, bsq, bsk, 0.f, 0, 0, 0};
    return sdpa_fwd_impl(Q, K, V, B, H, Sq, Sk, D, scale, ms, 0, B * H, 0, Sq, O, LSE, O32);
}

static int sdpa_fwd_impl(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                         int B, int H, int Sq, int Sk, int D, float scale, mask_spec ms,
                         int heads_begin, int heads_end, int row_begin, int row_end,
                         uint16_t* O, float* LSE, float* O32) {
    if (check_dims(B, H, Sq, Sk, D)) return -1;
    const int R = row_end - row_begin;
    if (R <= 0) return 0;
    int fail = 0;
#pragma omp parallel for schedule(dynamic, 1)
    for (int bh = heads_begin; bh < heads_end; ++bh) {
        const int b = bh / H, h = bh % H;
        float* q = (float*)malloc(sizeof(float) * (size_t)R * D);
        float* kt = (float*)malloc(sizeof(float) * (size_t)Sk * D);
        float* v = (float*)malloc(sizeof(float) * (size_t)Sk * D);
        float* P = (float*)malloc(sizeof(float) * (size_t)R * Sk);
        float* o = (float*)malloc(sizeof(float) * (size_t)D);
        if (!q || !kt || !v || !P || !o) {
            fail = 1;
        } else {
            const uint16_t* Qh = Q + ((size_t)bh * Sq + row_begin) * D;
            const uint16_t* Kh = K + (size_t)bh * Sk * D;
            const uint16_t* Vh = V + (size_t)bh * Sk * D;
            for (size_t t = 0; t < (size_t)R * D; ++t) q[t] = bf16_to_f32(Qh[t]);
            for (int j = 0; j < Sk; ++j)
                for (int d = 0; d < D; ++d) {
                    kt[(size_t)d * Sk + j] = bf16_to_f32(Kh[(size_t)j * D + d]);
                    v[(size_t)j * D + d] = bf16_to_f32(Vh[(size_t)j * D + d]);
                }
            head_probs(q, kt, row_begin, R, Sk, D, scale, &ms, b, h, P, LSE + (size_t)bh * Sq + row_begin);
            for (int i = 0; i < R; ++i) {
                for (int d = 0; d < D; ++d) o[d] = 0.f;
                const float* row = P + (size_t)i * Sk;
                for (int j = 0; j < Sk; ++j) {
                    const float p = operand(row[j] * drop_factor(&ms, bh, row_begin + i, j, Sq, Sk));
                    if (p == 0.f) continue;
                    const float* vr = v + (size_t)j * D;
                    for (int d = 0; d < D; ++d) o[d] += p * vr[d];
                }
                for (int d = 0; d < D; ++d) {
                    const size_t idx = ((size_t)bh * Sq + row_begin + i) * D + d;
                    O[idx] = f32_to_bf16(o[d]);
                    if (O32) O32[idx] = o[d];
                }
            }
        }
        free(q); free(kt); free(v); free(P); free(o);
    }
    return fail ? -2 : 0;
}

/*
 * Backward.  Recomputes P from Q,K (it does not consume a saved LSE, so it is independent of the
 * forward under test).  O is the bf16-rounded forward output.  Outputs bf16 dQ [B,H,Sq,D],
 * dK,dV [B,H,Sk,D]; optional fp32 copies dQ32,dK32,dV32 (NULL to skip).
 *
 * Only the query rows [row_begin, row_end) of the chosen heads take part: dQ is written for those
 * rows, and dK / dV hold the sums over those rows only (the whole gradient when the band is
 * [0, Sq), and also for every key that no query outside the band attends to, e.g. the last keys
 * of a causal problem when the band is the last rows).
 */
static int sdpa_bwd_impl(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                         const uint16_t* O, const uint16_t* dO,
                         int B, int H, int Sq, int Sk, int D, float scale, mask_spec ms,
                         int heads_begin, int heads_end, int row_begin, int row_end,
                         uint16_t* dQ, uint16_t* dK, uint16_t* dV,
                         float* dQ32, float* dK32, float* dV32) {
    if (check_dims(B, H, Sq, Sk, D)) return -1;
    if (row_begin < 0 || row_end > Sq || row_begin > row_end) return -1;
    const int R = row_end - row_begin;
    int fail = 0;
#pragma omp parallel for schedule(dynamic, 1)
    for (int bh = heads_begin; bh < heads_end; ++bh) {
        const int b = bh / H, h = bh % H;
        const size_t nq = (size_t)Sq * D, nk = (size_t)Sk * D, nr = (size_t)R * D;
        float* q = (float*)malloc(sizeof(float) * (nr + 1));
        float* g = (float*)malloc(sizeof(float) * (nr + 1));   /* dO */
        float* k = (float*)malloc(sizeof(float) * nk);
        float* kt = (float*)malloc(sizeof(float) * nk);
        float* vt = (float*)malloc(sizeof(float) * nk);
        float* P = (float*)malloc(sizeof(float) * ((size_t)R * Sk + 1));
        float* dp = (float*)malloc(sizeof(float) * (size_t)Sk);
        float* lse = (float*)malloc(sizeof(float) * (size_t)(R + 1));
        float* dq = (float*)calloc(nr + 1, sizeof(float));
        float* dk = (float*)calloc(nk, sizeof(float));
        float* dv = (float*)calloc(nk, sizeof(float));
        if (!q || !g || !k || !kt || !vt || !P || !dp || !lse || !dq || !dk || !dv) {
            fail = 1;
        } else {
            const uint16_t* Qh = Q + (size_t)bh * nq + (size_t)row_begin * D;
            const uint16_t* Gh = dO + (size_t)bh * nq + (size_t)row_begin * D;
            const uint16_t* Oh = O + (size_t)bh * nq + (size_t)row_begin * D;
            const uint16_t* Kh = K + (size_t)bh * nk;
            const uint16_t* Vh = V + (size_t)bh * nk;
            for (size_t t = 0; t < nr; ++t) { q[t] = bf16_to_f32(Qh[t]); g[t] = bf16_to_f32(Gh[t]); }
            for (int j = 0; j < Sk; ++j)
                for (int d = 0; d < D; ++d) {
                    const float kv = bf16_to_f32(Kh[(size_t)j * D + d]);
                    k[(size_t)j * D + d] = kv;
                    kt[(size_t)d * Sk + j] = kv;
                    vt[(size_t)d * Sk + j] = bf16_to_f32(Vh[(size_t)j * D + d]);
                }
            head_probs(q, kt, row_begin, R, Sk, D, scale, &ms, b, h, P, lse);
            for (int i = 0; i < R; ++i) {
                const float* gi = g + (size_t)i * D;
                const float* qi = q + (size_t)i * D;
                float* row = P + (size_t)i * Sk;
                float delta = 0.f;
                for (int d = 0; d < D; ++d) delta += gi[d] * bf16_to_f32(Oh[(size_t)i * D + d]);
                for (int j = 0; j < Sk; ++j) dp[j] = 0.f;
                for (int d = 0; d < D; ++d) {
                    const float gv = gi[d];
                    const float* vr = vt + (size_t)d * Sk;
                    for (int j = 0; j < Sk; ++j) dp[j] += gv * vr[j];
                }
                float* dqi = dq + (size_t)i * D;
                for (int j = 0; j < Sk; ++j) {
                    const float p = row[j];
                    if (p == 0.f) continue;
                    /* with dropout O = (P * f) V, f = 0 or 1 / (1 - p): dV takes P * f, dP = f * (dO V^T), and
                     * rowsum(dP * P) = rowsum(dO * O) = delta as without it */
                    const float f = drop_factor(&ms, bh, row_begin + i, j, Sq, Sk);
                    const float ds = operand(p * (f * dp[j] - delta));
                    const float pd = operand(p * f);
                    float* dvj = dv + (size_t)j * D;
                    float* dkj = dk + (size_t)j * D;
                    const float* kj = k + (size_t)j * D;
                    for (int d = 0; d < D; ++d) {
                        dvj[d] += pd * gi[d];
                        dqi[d] += ds * kj[d];
                        dkj[d] += ds * qi[d];
                    }
                }
            }
            for (size_t t = 0; t < nr; ++t) {
                const float x = dq[t] * scale;
                const size_t idx = (size_t)bh * nq + (size_t)row_begin * D + t;
                dQ[idx] = f32_to_bf16(x);
                if (dQ32) dQ32[idx] = x;
            }
            for (size_t t = 0; t < nk; ++t) {
                const float x = dk[t] * scale;
                dK[(size_t)bh * nk + t] = f32_to_bf16(x);
                dV[(size_t)bh * nk + t] = f32_to_bf16(dv[t]);
                if (dK32) dK32[(size_t)bh * nk + t] = x;
                if (dV32) dV32[(size_t)bh * nk + t] = dv[t];
            }
        }
        free(q); free(g); free(k); free(kt); free(vt); free(P); free(dp); free(lse);
        free(dq); free(dk); free(dv);
    }
    return fail ? -2 : 0;
}

int oracle_sdpa_bwd_rows(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                         const uint16_t* O, const uint16_t* dO,
                         int B, int H, int Sq, int Sk, int D, float scale, int causal,
                         const int32_t* kv_len, const uint8_t* mask,
                         int64_t msb, int64_t msh, int64_t msq, int64_t msk,
                         int heads_begin, int heads_end, int row_begin, int row_end,
                         uint16_t* dQ, uint16_t* dK, uint16_t* dV,
                         float* dQ32, float* dK32, float* dV32) {
    mask_spec ms = {causal, kv_len, mask, msb, msh, msq, msk, NULL, 0, 0, 0, 0, 0.f, 0, 0, 0};
    return sdpa_bwd_impl(Q, K, V, O, dO, B, H, Sq, Sk, D, scale, ms, heads_begin, heads_end, row_begin, row_end,
                         dQ, dK, dV, dQ32, dK32, dV32);
}

/* Forward and backward with dropout of the probabilities (see drop_factor). */
int oracle_sdpa_fwd_dropout(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                            int B, int H, int Sq, int Sk, int D, float scale, int causal, const int32_t* kv_len,
                            const uint8_t* mask, int64_t msb, int64_t msh, int64_t msq, int64_t msk,
                            float drop_p, uint64_t drop_seed, int drop_cq, int drop_ck, uint16_t* O, float* LSE, float* O32) {
    mask_spec ms = {causal, kv_len, mask, msb, msh, msq, msk, NULL, 0, 0, 0, 0, drop_p, drop_seed, drop_cq, drop_ck};
    return sdpa_fwd_impl(Q, K, V, B, H, Sq, Sk, D, scale, ms, 0, B * H, 0, Sq, O, LSE, O32);
}

int oracle_sdpa_bwd_dropout(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                            const uint16_t* O, const uint16_t* dO,
                            int B, int H, int Sq, int Sk, int D, float scale, int causal, const int32_t* kv_len,
                            const uint8_t* mask, int64_t msb, int64_t msh, int64_t msq, int64_t msk,
                            float drop_p, uint64_t drop_seed, int drop_cq, int drop_ck,
                            uint16_t* dQ, uint16_t* dK, uint16_t* dV, float* dQ32, float* dK32, float* dV32) {
    mask_spec ms = {causal, kv_len, mask, msb, msh, msq, msk, NULL, 0, 0, 0, 0, drop_p, drop_seed, drop_cq, drop_ck};
    return sdpa_bwd_impl(Q, K, V, O, dO, B, H, Sq, Sk, D, scale, ms, 0, B * H, 0, Sq, dQ, dK, dV, dQ32, dK32, dV32);
}

int oracle_sdpa_bwd(const uint16_t* Q, const uint16_t* K, const uint16_t* V,
                    const uint16_t* O, const uint16_t* dO,
                    int B, int H, int Sq, int Sk, int D, float scale, int causal,
                    const int32_t* kv_len, const uint8_t* mask,
                    int64_t msb, int64_t msh, int64_t msq, int64_t msk,
                    int heads_begin, int heads_end,
                    uint16_t* dQ, uint16_t* dK, uint16_t* dV,
                    float* dQ32, float* dK32, float* dV32) {
    return oracle_sdpa_bwd_rows(Q, K, V, O, dO, B, H, Sq, Sk, D, scale, causal, kv_len, mask, msb, msh, msq, msk,
                                heads_begin, heads_end, 0, Sq, dQ, dK, dV, dQ32, dK32, dV32);
}

/* ------------------------------------------------------------------------------------------
 * SageAttention int8-QK inference variant.
 *
 * Spec (all fp32 unless stated):
 *   kmean[b,h,c] = (float)( (double) sum_t K[b,h,t,c] / Sk )      sum carried in fp64, which is
 *                  exact for bf16 addends of ordinary magnitude and so independent of order
 *   Ks           = bf16_rne( (float)K - kmean )
 *   sq[b,h,i]    = max |Q[b,h, i*qblk : (i+1)*qblk, :]| / 127     (IEEE fp32 division)
 *   sk[b,h,j]    = max |Ks[b,h, j*kblk : (j+1)*kblk, :]| / 127
 *   Qi8          = clamp(rintf((float)Q / sq), -128, 127)         (IEEE division, ties to even)
 *   Ki8          = clamp(rintf((float)Ks / sk), -128, 127)
 *   absmax == 0  => scale = 0 and every quantised value of the block = 0
 * The last block of a sequence may be short.
 * ------------------------------------------------------------------------------------------ */
static inline int8_t quant1(float x, float s) {
    if (s == 0.f) return 0;
    float r = rintf(x / s);
    if (r > 127.f) r = 127.f;
    if (r < -128.f) r = -128.f;
    return (int8_t)r;
}

int oracle_sage_quant(const uint16_t* Q, const uint16_t* K,
                      int B, int H, int Sq, int Sk, int D, int qblk, int kblk, int smooth_k,
                      float* kmean /*[B,H,D]*/, uint16_t* Ks /*[B,H,Sk,D] or NULL*/,
                      int8_t* Qi8, int8_t* Ki8,
                      float* sq /*[B,H,ceil(Sq/qblk)]*/, float* sk /*[B,H,ceil(Sk/kblk)]*/) {
    if (check_dims(B, H, Sq, Sk, D) || qblk <= 0 || kblk <= 0) return -1;
    const int nqb = (Sq + qblk - 1) / qblk, nkb = (Sk + kblk - 1) / kblk;
    int fail = 0;
#pragma omp parallel for schedule(dynamic, 1)
    for (int bh = 0; bh < B * H; ++bh) {
        const uint16_t* Qh = Q + (size_t)bh * Sq * D;
        const uint16_t* Kh = K + (size_t)bh * Sk * D;
        float* mu = kmean + (size_t)bh * D;
        float* ks = (float*)malloc(sizeof(float) * (size_t)Sk * D);
        if (!ks) { fail = 1; continue; }
        for (int c = 0; c < D; ++c) {
            double acc = 0.0;
            if (smooth_k)
                for (int t = 0; t < Sk; ++t) acc += (double)bf16_to_f32(Kh[(size_t)t * D + c]);
            mu[c] = smooth_k ? (float)(acc / (double)Sk) : 0.f;
        }
        for (int t = 0; t < Sk; ++t)
            for (int c = 0; c < D; ++c) {
                const uint16_t r = f32_to_bf16(bf16_to_f32(Kh[(size_t)t * D + c]) - mu[c]);
                ks[(size_t)t * D + c] = bf16_to_f32(r);
                if (Ks) Ks[((size_t)bh * Sk + t) * D + c] = r;
            }
        for (int ib = 0; ib < nqb; ++ib) {
            const int r0 = ib * qblk, r1 = (r0 + qblk < Sq) ? r0 + qblk : Sq;
            float amax = 0.f;
            for (size_t t = (size_t)r0 * D; t < (size_t)r1 * D; ++t) {
                const float a = fabsf(bf16_to_f32(Qh[t]));
                if (a > amax) amax = a;
            }
            const float s = amax / 127.0f;
            sq[(size_t)bh * nqb + ib] = s;
            for (size_t t = (size_t)r0 * D; t < (size_t)r1 * D; ++t)
                Qi8[(size_t)bh * Sq * D + t] = quant1(bf16_to_f32(Qh[t]), s);
        }
        for (int jb = 0; jb < nkb; ++jb) {
            const int r0 = jb * kblk, r1 = (r0 + kblk < Sk) ? r0 + kblk : Sk;
            float amax = 0.f;
            for (size_t t = (size_t)r0 * D; t < (size_t)r1 * D; ++t) {
                const float a = fabsf(ks[t]);
                if (a > amax) amax = a;
            }
            const float s = amax / 127.0f;
            sk[(size_t)bh * nkb + jb] = s;
            for (size_t t = (size_t)r0 * D; t < (size_t)r1 * D; ++t)
                Ki8[(size_t)bh * Sk * D + t] = quant1(ks[t], s);
        }
        free(ks);
    }
    return fail ? -2 : 0;
}

/*
 * Sage forward from quantised operands:
 *   S_ij = (float)(int32 sum_d Qi8_id Ki8_jd) * (sq[i/qblk] * sk[j/kblk] * scale)
 *   an optional additive fp32 bias [B|1,H|1,Sq,Sk] (element strides, 0 = broadcast) is added to S
 *   (src/sage_attention.rs:126-131); key j is excluded when causal and j > i, or when j >= kv_len[b]
 *   P = softmax(S) in fp32 (naive, materialised); O = P V -> bf16 (O32: the same before rounding).
 *   A row with every key excluded gives O = 0 and LSE = -inf.
 * Only the query rows [row_begin, row_end) of the chosen heads are computed.
 */
int oracle_sage_fwd(const int8_t* Qi8, const int8_t* Ki8, const float* sq, const float* sk,
                    const uint16_t* V, int B, int H, int Sq, int Sk, int D, int qblk, int kblk,
                    float scale, int causal, const int32_t* kv_len,
                    const float* bias, int64_t bsb, int64_t bsh, int64_t bsq, int64_t bsk,
                    int heads_begin, int heads_end, int row_begin, int row_end,
                    uint16_t* O, float* LSE, float* O32) {
    if (check_dims(B, H, Sq, Sk, D) || qblk <= 0 || kblk <= 0) return -1;
    if (row_begin < 0 || row_end > Sq || row_begin > row_end) return -1;
    const int nqb = (Sq + qblk - 1) / qblk, nkb = (Sk + kblk - 1) / kblk;
    int fail = 0;
#pragma omp parallel for schedule(dynamic, 1)
    for (int bh = heads_begin; bh < heads_end; ++bh) {
        const int b = bh / H, hh = bh % H;
        float* v = (float*)malloc(sizeof(float) * (size_t)Sk * D);
        float* row = (float*)malloc(sizeof(float) * (size_t)Sk);
        float* o = (float*)malloc(sizeof(float) * (size_t)D);
        if (!v || !row || !o) {
            fail = 1;
        } else {
            const int8_t* Qh = Qi8 + (size_t)bh * Sq * D;
            const int8_t* Kh = Ki8 + (size_t)bh * Sk * D;
            const uint16_t* Vh = V + (size_t)bh * Sk * D;
            const int klim = kv_len ? (kv_len[b] < Sk ? (kv_len[b] < 0 ? 0 : kv_len[b]) : Sk) : Sk;
            for (size_t t = 0; t < (size_t)Sk * D; ++t) v[t] = bf16_to_f32(Vh[t]);
            for (int i = row_begin; i < row_end; ++i) {
                const float sqi = sq[(size_t)bh * nqb + i / qblk];
                float m = -INFINITY;
                for (int j = 0; j < Sk; ++j) {
                    int32_t acc = 0;
                    for (int d = 0; d < D; ++d)
                        acc += (int32_t)Qh[(size_t)i * D + d] * (int32_t)Kh[(size_t)j * D + d];
                    float s = (float)acc * (sqi * sk[(size_t)bh * nkb + j / kblk] * scale);
                    if (bias) s += bias[b * bsb + hh * bsh + i * bsq + j * bsk];     /* the reference adds its mask to the scores */
                    if ((causal && j > i) || j >= klim) s = -INFINITY;
                    row[j] = s;
                    if (s > m) m = s;
                }
                for (int d = 0; d < D; ++d) o[d] = 0.f;
                float lse = -INFINITY;
                if (m != -INFINITY) {
                    float l = 0.f;
                    for (int j = 0; j < Sk; ++j) { row[j] = expf(row[j] - m); l += row[j]; }
                    for (int j = 0; j < Sk; ++j) {
                        const float p = row[j] / l;
                        if (p == 0.f) continue;
                        for (int d = 0; d < D; ++d) o[d] += p * v[(size_t)j * D + d];
                    }
                    lse = m + logf(l);
                }
                for (int d = 0; d < D; ++d) {
                    const size_t idx = ((size_t)bh * Sq + i) * D + d;
                    O[idx] = f32_to_bf16(o[d]);
                    if (O32) O32[idx] = o[d];
                }
                if (LSE) LSE[(size_t)bh * Sq + i] = lse;
            }
        }
        free(v); free(row); free(o);
    }
    return fail ? -2 : 0;
}
