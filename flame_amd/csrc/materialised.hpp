// The materialised path: attention for the shapes the fused kernels do not serve (head dims that are not multiples
// of 8 or lie above 512, and, above 128, a keep-mask, a bias or the backward).  The reference serves exactly these
// through materialised scores as well (src/sdpa.rs:788-961 forward, src/autograd.rs:801-848 backward): library
// GEMMs for Q K^T, P V and the four backward products, element-wise kernels in between.  Here the GEMMs are
// rocBLAS's (bf16 operands, fp32 accumulation), the element-wise kernels are below, and the scores exist for one
// band of query rows at a time (fp32 logits + bf16 P, in the backward + bf16 dS: 8 bytes per score element of the
// band, as the reference's peak), so that what is kept between forward and backward is still O and the
// log-sum-exp only.  Not a fast path: several passes over the band per step.
#pragma once
#include "attn_common.hpp"

namespace fattn {

struct MatRowsParams {
    float* scores;          // [BH, tq, Sk] fp32: scaled logits in, overwritten only by the caller's next GEMM
    uint16_t* probs;        // [BH, tq, Sk] bf16 out
    float* lse;             // [BH, Sq] (forward: written; backward: read)
    int H, Sq, Sk, tq, q0;  // the band holds query rows [q0, q0 + tq) of every (batch, head)
    MaskArgs m;
    int from_lse;           // 0: forward (row max, sum, LSE, P); 1: backward (P = exp(s - LSE) under the same exclusions)
    int dropout = 0;        // forward only: P is stored dropped and rescaled (the backward drops it in mat_ds_kernel)
};

// s for key j of query row qi of (b, hh), or -inf when the pair is excluded
__device__ __forceinline__ float mat_logit(const MatRowsParams& p, const uint8_t* mbase, const uint8_t* bias_base, int b, int qi,
                                           int j, int klimit, float raw) {
    bool drop = (j >= klimit) | ((p.m.causal != 0) & (j > qi));
    if (!drop && p.m.mask) drop = !mask_attends(p.m, mbase, (int64_t)qi * p.m.sq + (int64_t)j * p.m.sk);
    if (drop) return -INFINITY;
    if (p.m.bias) {
        const int64_t e = (int64_t)qi * p.m.bq + (int64_t)j * p.m.bk;
        raw += p.m.bias_f32 ? reinterpret_cast<const float*>(bias_base)[e]
                            : __builtin_bit_cast(float, (uint32_t)reinterpret_cast<const uint16_t*>(bias_base)[e] << 16);
    }
    return raw;
}

// One workgroup per query row of the band.  Forward: exclusions and bias, row maximum and sum (two passes over the
// row, which sits in L2), LSE = max + ln(sum), P = exp(s - LSE) as bf16; a row without an attended key gets
// LSE = -inf and P = 0; with dropout P is stored as P * f, f = 0 or 1 / (1 - p) per element (drop_factor_at), the
// LSE being that of the undropped row.  Backward: P = exp(s - LSE) from the saved LSE, undropped.
__global__ __launch_bounds__(256) void mat_rows_kernel(const MatRowsParams p) {
    const int row = blockIdx.x;                      // over [BH, tq]
    const int bh = row / p.tq, i = row % p.tq;
    const int qi = p.q0 + i;
    const int b = bh / p.H, hh = bh % p.H;
    const float* s = p.scores + (size_t)row * p.Sk;
    uint16_t* out = p.probs + (size_t)row * p.Sk;
    int klimit = p.Sk;
    if (p.m.kv_len) klimit = min(klimit, max(p.m.kv_len[b], 0));
    const uint8_t* mbase = p.m.mask ? mask_head_base(p.m, b, hh) : nullptr;
    const uint8_t* bias_base = p.m.bias ? static_cast<const uint8_t*>(p.m.bias) + (b * p.m.bb + hh * p.m.bh) * (p.m.bias_f32 ? 4 : 2)
                                        : nullptr;
    __shared__ float red[8];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float lse;
    if (p.from_lse) {
        lse = p.lse[(size_t)bh * p.Sq + qi];
    } else {
        float m = -INFINITY;
        for (int j = tid; j < p.Sk; j += 256) m = fmaxf(m, mat_logit(p, mbase, bias_base, b, qi, j, klimit, s[j]));
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
        if (lane == 0) red[wave] = m;
        __syncthreads();
        m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        __syncthreads();
        float l = 0.f;
        if (m != -INFINITY)
            for (int j = tid; j < p.Sk; j += 256) l += expf(mat_logit(p, mbase, bias_base, b, qi, j, klimit, s[j]) - m);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) l += __shfl_xor(l, off, 64);
        if (lane == 0) red[4 + wave] = l;
        __syncthreads();
        l = (red[4] + red[5]) + (red[6] + red[7]);
        lse = (m == -INFINITY) ? -INFINITY : m + logf(l);
        if (tid == 0 && p.lse) p.lse[(size_t)bh * p.Sq + qi] = lse;
    }
    for (int j = tid; j < p.Sk; j += 256) {
        float pr = 0.f;
        if (lse != -INFINITY) pr = expf(mat_logit(p, mbase, bias_base, b, qi, j, klimit, s[j]) - lse);      // exp(-inf) = 0
        if (p.dropout) pr *= drop_factor_at(p.m, (uint32_t)bh, (uint32_t)qi, (uint32_t)j, (uint32_t)p.Sq, (uint32_t)p.Sk);
        out[j] = (uint16_t)(pack_bf16(pr, 0.f) & 0xffffu);
    }
}

// delta[bh, q] = sum_d dO[b,h,q,d] * O[b,h,q,d] for any head dim: one wavefront per row
struct MatDeltaParams {
    const uint16_t* o;
    const uint16_t* dout;
    Strides os, dos;
    float* delta;           // [BH, Sq]
    int B, H, Sq, dv;
};
__global__ __launch_bounds__(256) void mat_delta_kernel(const MatDeltaParams p) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= (int64_t)p.B * p.H * p.Sq) return;
    const int bh = (int)(row / p.Sq), qi = (int)(row % p.Sq);
    const int b = bh / p.H, hh = bh % p.H;
    const uint16_t* ro = p.o + b * p.os.b + hh * p.os.h + (int64_t)qi * p.os.n;
    const uint16_t* rd = p.dout + b * p.dos.b + hh * p.dos.h + (int64_t)qi * p.dos.n;
    float acc = 0.f;
    for (int d = lane; d < p.dv; d += 64)
        acc += __builtin_bit_cast(float, (uint32_t)ro[d] << 16) * __builtin_bit_cast(float, (uint32_t)rd[d] << 16);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) p.delta[row] = acc;
}

// dS = P * (dP - delta) as bf16, element-wise over the band; delta is per query row.  With dropout (drop.drop_thr
// != 0): dP is the product with the dropped V weights, dS = P * (f dP - delta), and P is overwritten by P * f, the
// weights that multiplied V in the forward, for the dV product that follows.
__global__ __launch_bounds__(256) void mat_ds_kernel(uint16_t* __restrict__ probs, const float* __restrict__ dp,
                                                     const float* __restrict__ delta, uint16_t* __restrict__ ds, int64_t n, int Sk,
                                                     int tq, int Sq, int q0, const MaskArgs drop) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= n) return;
    const int64_t row = e / Sk;
    const int bh = (int)(row / tq), i = (int)(row % tq);
    const float pr = __builtin_bit_cast(float, (uint32_t)probs[e] << 16);
    float g = dp[e];
    if (drop.drop_thr != 0) {
        const float f = drop_factor_at(drop, (uint32_t)bh, (uint32_t)(q0 + i), (uint32_t)(e % Sk), (uint32_t)Sq, (uint32_t)Sk);
        g *= f;
        probs[e] = (uint16_t)(pack_bf16(pr * f, 0.f) & 0xffffu);
    }
    const float v = pr * (g - delta[(size_t)bh * Sq + q0 + i]);
    ds[e] = (uint16_t)(pack_bf16(v, 0.f) & 0xffffu);
}

// fp32 [BH, N, D] contiguous sums -> bf16 tensor through its strides
__global__ __launch_bounds__(256) void mat_store_kernel(const float* __restrict__ src, uint16_t* dst, Strides st, int H, int N, int D,
                                                        int64_t n_elems) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= n_elems) return;
    const int64_t row = e / D;
    const int d = (int)(e % D);
    const int bh = (int)(row / N), n = (int)(row % N);
    const int b = bh / H, hh = bh % H;
    dst[b * st.b + hh * st.h + (int64_t)n * st.n + d] = (uint16_t)(pack_bf16(src[e], 0.f) & 0xffffu);
}

}  // namespace fattn
