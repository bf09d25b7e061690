// SageAttention int8-QK inference forward for gfx950.
//
//   sage_kmean_kernel   kmean[b,h,c] = float( (fp64 sum over tokens of K[b,h,:,c]) / Sk )
//                       the fp64 sum of bf16 addends is exact for ordinary magnitudes, hence
//                       independent of the summation order and bit-identical to a CPU loop
//   sage_quant_kernel   Ks = bf16(float(K) - kmean); per 128-row Q block and per 64-row Ks block:
//                       scale = absmax/127 (IEEE division), code = clamp(rint(x/scale), -128, 127)
//   sage_fwd_kernel     S^T = K^ Q^^T on v_mfma_i32_32x32x32_i8 (int32 accumulate), dequantised with
//                       sq*sk*scale, online softmax in fp32, P -> bf16, O^T = V^T P^T on bf16 MFMA;
//                       same tile walk, LDS-DMA staging and in-wave software pipeline as the bf16
//                       forward kernel (the int8 K tile is half the size, the logit MFMAs half as many)
//
// Quantisation closed form follows the reference's sage_quantize_tensor
// (src/sage_attention.rs:524-541); block granularity, mean smoothing and the int8 MFMA are new.
#pragma once
#include <type_traits>

#include "attn_common.hpp"

namespace fattn {

constexpr int kSageQBlk = 128;
constexpr int kSageKBlk = 64;

struct SageQuantParams {
    const uint16_t* q;
    const uint16_t* k;
    Strides qs, ks;
    int B, H, Sq, Sk;
    int d;           // real head dim: a multiple of 8, at most the compiled D; every tensor written here has rows of D
                     // elements, zero beyond d (zero channels change neither a block's maximum nor a logit)
    int smooth_k;
    float* kmean;    // [B*H, D]
    int8_t* qi8;     // [B*H, Sq, D]
    int8_t* ki8;     // [B*H, Sk, D]
    float* sq;       // [B*H, ceil(Sq/128)]
    float* sk;       // [B*H, ceil(Sk/64)]
    uint16_t* ks_out = nullptr;   // [B*H, Sk, D] bf16 or null: the smoothed K that was quantised, for a backward pass
};

// Channel mean of K, short sequences: one workgroup of 512 threads per (batch, head)
template <int D>
__global__ __launch_bounds__(512) void sage_kmean_kernel(const SageQuantParams p) {
    constexpr int CPR = D / 8;            // 16-byte chunks per row
    constexpr int RG = 512 / CPR;         // row groups
    __shared__ double part[RG][D + 1];
    const int tid = threadIdx.x;
    const int chunk = tid % CPR, rg = tid / CPR;
    const int bh = blockIdx.x;
    const int b = bh / p.H, hh = bh % p.H;
    const uint16_t* kb = p.k + b * p.ks.b + hh * p.ks.h + chunk * 8;
    double acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0;
    if (p.smooth_k) {
        for (int row = rg; row < p.Sk; row += RG) {
            const u32x4 w = ldg16(kb + (int64_t)row * p.ks.n, chunk * 8 < p.d);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[2 * i] += (double)bf16_lo(w[i]);
                acc[2 * i + 1] += (double)bf16_hi(w[i]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) part[rg][chunk * 8 + i] = acc[i];
    __syncthreads();
    if (tid < D) {
        double s = 0.0;
        for (int g = 0; g < RG; ++g) s += part[g][tid];
        p.kmean[(int64_t)bh * D + tid] = p.smooth_k ? (float)(s / (double)p.Sk) : 0.f;
    }
}

// Long sequences: channel mean of K in two steps so that the whole device takes part: workgroup (bh, c) sums the rows
// of chunk c in fp64 and parks its D partial sums in the first bytes of that head's int8 K output
// (overwritten by the quantisation that follows); sage_kmean_final_kernel adds the chunks in order.
// fp64 sums of bf16 values are exact at these lengths, so the result does not depend on the chunking.
template <int D>
__global__ __launch_bounds__(512) void sage_kmean_partial_kernel(const SageQuantParams p, int n_chunks, int rows_per_chunk) {
    constexpr int CPR = D / 8;            // 16-byte chunks per row
    constexpr int RG = 512 / CPR;         // row groups
    __shared__ double part[RG][D + 1];
    const int tid = threadIdx.x;
    const int chunk = tid % CPR, rg = tid / CPR;
    const int bh = blockIdx.x / n_chunks, c = blockIdx.x % n_chunks;
    const int b = bh / p.H, hh = bh % p.H;
    const uint16_t* kb = p.k + b * p.ks.b + hh * p.ks.h + chunk * 8;
    const int r_end = min(p.Sk, (c + 1) * rows_per_chunk);
    double acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0;
    for (int row = c * rows_per_chunk + rg; row < r_end; row += RG) {
        const u32x4 w = ldg16(kb + (int64_t)row * p.ks.n, chunk * 8 < p.d);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[2 * i] += (double)bf16_lo(w[i]);
            acc[2 * i + 1] += (double)bf16_hi(w[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) part[rg][chunk * 8 + i] = acc[i];
    __syncthreads();
    if (tid < D) {
        double s = 0.0;
        for (int g = 0; g < RG; ++g) s += part[g][tid];
        reinterpret_cast<double*>(p.ki8 + (int64_t)bh * p.Sk * D)[c * D + tid] = s;
    }
}

template <int D>
__global__ __launch_bounds__(D) void sage_kmean_final_kernel(const SageQuantParams p, int n_chunks) {
    const int bh = blockIdx.x, tid = threadIdx.x;
    float m = 0.f;
    if (p.smooth_k) {
        const double* scr = reinterpret_cast<const double*>(p.ki8 + (int64_t)bh * p.Sk * D);
        double s = 0.0;
        for (int c = 0; c < n_chunks; ++c) s += scr[c * D + tid];
        m = (float)(s / (double)p.Sk);
    }
    p.kmean[(int64_t)bh * D + tid] = m;
}

// The low byte of the int8 code clamp(rint(x / s), -128, 127) with the IEEE quotient, round half to even, for
// |x| <= 127 s (the block maximum defines s, so the clamp never acts); inv = 1 / s (0 when s is 0).
// x * inv lies within 4e-5 of the correctly rounded quotient (both factors rounded once), so unless it falls within
// 1e-4 of a rounding boundary k + 1/2 the two round to the same integer; only those rare elements (about one in
// 5000) pay for the division itself.  Adding 1.5 * 2^23 rounds to the nearest even integer and leaves the code in
// two's complement in the low mantissa bits.
__device__ __forceinline__ uint32_t quant_code_byte(float x, float s, float inv) {
    constexpr float kMagic = 12582912.0f;
    const float t = x * inv;
    float biased = t + kMagic;
    const float r = biased - kMagic;
    // written so that an infinite or NaN product (a subnormal scale) takes the division as well
    if (__builtin_expect(!(0.5f - fabsf(t - r) >= 1.0e-4f) && s != 0.f, 0)) biased = x / s + kMagic;
    return __float_as_uint(biased) & 0xffu;
}

// grid = B*H*(nqb + ceil(nkb / 2)); one workgroup quantises 128 rows: one Q block, or two neighbouring K blocks
// (rows 0..63 and 64..127 of its range, each with a scale of its own)
template <int D>
__global__ __launch_bounds__(256) void sage_quant_kernel(const SageQuantParams p) {
    constexpr int CPR = D / 8;
    constexpr int RPP = 256 / CPR;            // rows per pass
    constexpr int MAXC = kSageQBlk / RPP;     // chunks per thread for 128 rows; the first half of them are rows 0..63
    static_assert(kSageQBlk == 2 * kSageKBlk && MAXC % 2 == 0, "a workgroup's 128 rows are one Q block or two K blocks");
    __shared__ float red[4][2];
    const int tid = threadIdx.x;
    const int nqb = (p.Sq + kSageQBlk - 1) / kSageQBlk;
    const int nkb = (p.Sk + kSageKBlk - 1) / kSageKBlk;
    const int nkp = (nkb + 1) / 2;
    const int per_bh = nqb + nkp;
    const int bh = blockIdx.x / per_bh;
    const int blk = blockIdx.x % per_bh;
    const bool is_q = blk < nqb;
    const int b = bh / p.H, hh = bh % p.H;
    const int S = is_q ? p.Sq : p.Sk;
    const int r0 = (is_q ? blk : blk - nqb) * kSageQBlk;
    const Strides st = is_q ? p.qs : p.ks;
    const uint16_t* src = (is_q ? p.q : p.k) + b * st.b + hh * st.h;
    const int chunk = tid % CPR;
    const int rsub = tid / CPR;

    float mu[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) mu[i] = 0.f;
    if (!is_q) {
        const f32x4* m = reinterpret_cast<const f32x4*>(p.kmean + (int64_t)bh * D + chunk * 8);
        const f32x4 a = m[0], c = m[1];
        mu[0] = a[0]; mu[1] = a[1]; mu[2] = a[2]; mu[3] = a[3];
        mu[4] = c[0]; mu[5] = c[1]; mu[6] = c[2]; mu[7] = c[3];
    }

    float x[MAXC][8];
    float amax[2] = {0.f, 0.f};               // rows 0..63 / 64..127
    u32x4 raw[MAXC];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {          // all loads first
        const int row = r0 + rsub + RPP * i;
        raw[i] = ldg16(src + (int64_t)row * st.n + chunk * 8, row < S && chunk * 8 < p.d);
    }
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float lo = bf16_lo(raw[i][j]), hi = bf16_hi(raw[i][j]);
            if (!is_q) {   // smoothed K, rounded to bf16 exactly as the checker does
                const uint32_t pk = pack_bf16(lo - mu[2 * j], hi - mu[2 * j + 1]);
                lo = bf16_lo(pk);
                hi = bf16_hi(pk);
            }
            if (r0 + rsub + RPP * i >= S) { lo = 0.f; hi = 0.f; }
            x[i][2 * j] = lo;
            x[i][2 * j + 1] = hi;
            amax[i >= MAXC / 2] = fmaxf(amax[i >= MAXC / 2], fmaxf(fabsf(lo), fabsf(hi)));
        }
    }
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) amax[hf] = fmaxf(amax[hf], __shfl_xor(amax[hf], off, 64));
        if ((tid & 63) == 0) red[tid >> 6][hf] = amax[hf];
    }
    __syncthreads();
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) amax[hf] = fmaxf(fmaxf(red[0][hf], red[1][hf]), fmaxf(red[2][hf], red[3][hf]));
    if (is_q) amax[0] = amax[1] = fmaxf(amax[0], amax[1]);
    float s[2], inv[2];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
        s[hf] = amax[hf] / 127.0f;
        inv[hf] = s[hf] == 0.f ? 0.f : 1.0f / s[hf];
    }
    if (tid == 0) {
        if (is_q) {
            p.sq[(int64_t)bh * nqb + blk] = s[0];
        } else {
            const int kb = 2 * (blk - nqb);
            p.sk[(int64_t)bh * nkb + kb] = s[0];
            if (kb + 1 < nkb) p.sk[(int64_t)bh * nkb + kb + 1] = s[1];
        }
    }
    int8_t* dst = (is_q ? p.qi8 : p.ki8) + (int64_t)bh * S * D;
    uint16_t* ks_dst = (!is_q && p.ks_out) ? p.ks_out + (int64_t)bh * S * D : nullptr;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int row = r0 + rsub + RPP * i;
        if (row >= S) continue;
        if (ks_dst) {       // the values are bf16 already: packing them again is exact
            const u32x4 kw = {pack_bf16(x[i][0], x[i][1]), pack_bf16(x[i][2], x[i][3]), pack_bf16(x[i][4], x[i][5]),
                              pack_bf16(x[i][6], x[i][7])};
            *reinterpret_cast<u32x4*>(ks_dst + (int64_t)row * D + chunk * 8) = kw;
        }
        const float sc = s[i >= MAXC / 2], iv = inv[i >= MAXC / 2];
        uint32_t w0 = 0, w1 = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            w0 |= quant_code_byte(x[i][j], sc, iv) << (8 * j);
            w1 |= quant_code_byte(x[i][4 + j], sc, iv) << (8 * j);
        }
        u32x2 w = {w0, w1};
        *reinterpret_cast<u32x2*>(dst + (int64_t)row * D + chunk * 8) = w;
    }
}

// --------------------------------------------------------------------------------------- forward
struct SageFwdParams {
    const int8_t* qi8;   // [B*H, Sq, D]
    const int8_t* ki8;   // [B*H, Sk, D]
    const float* sq;     // [B*H, ceil(Sq/128)]
    const float* sk;     // [B*H, ceil(Sk/64)]
    const uint16_t* v;
    uint16_t* o;
    float* lse;          // [B*H, Sq] or null
    Strides vs, os;
    int B, H, Sq, Sk;
    int d;               // real head dim of V and O (a multiple of 8, at most the compiled D)
    float scale;
    const int32_t* kv_len;
    int causal;
    // additive bias on the scaled, dequantised logits (natural-log units; -inf excludes), fp32 or bf16, or null
    const void* bias = nullptr;
    int64_t bb = 0, bhs = 0, bq = 0, bk = 0;   // element strides over (b,h,q,k); 0 broadcasts
    int bias_f32 = 1;
    int wg_base = 0;     // the launch covers the problem's workgroups from this one on (problems without exclusions only)
};

template <int D>
struct SageTile {
    static constexpr int BM = 128, BN = 64;
    static constexpr int K_BYTES = BN * D;             // int8 K tile, row-major, swizzled, no padding
    static constexpr int V_BYTES = BN * D * 2;         // bf16 V tile, likewise
    static constexpr int STAGE_BYTES = K_BYTES + V_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static constexpr int K_DMA_PER_WAVE = K_BYTES / 1024 / 4;
    static constexpr int V_DMA_PER_WAVE = V_BYTES / 1024 / 4;
};

// granule swizzle of the int8 K tile (rows of D bytes): 16-byte row reads by 16 adjacent rows hit 16
// distinct bank groups
template <int D>
__device__ __forceinline__ constexpr int swz_i8(int row) {
    return D == 128 ? swz<64>(row) : ((row >> 2) & 3);
}

// NW wavefronts (4 or 8) of 32 queries each per workgroup, as in the bf16 forward kernel.
template <int D, int NW>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void sage_fwd_kernel(const SageFwdParams p) {
    using T = SageTile<D>;
    constexpr int BM = 32 * NW, BN = T::BN;
    constexpr int KC = D / 32;   // int8 contraction chunks (32 per MFMA)
    constexpr int DB = D / 32;   // 32-row blocks of O^T
    constexpr int RS = D;        // V row stride, elements
    constexpr int GPK = D / 16;  // 16-byte granules per K^ row
    constexpr int GPV = D / 8;   // ... per V row
    constexpr int NKD = T::K_DMA_PER_WAVE * 4 / NW, NVD = T::V_DMA_PER_WAVE * 4 / NW;
    static_assert(NKD >= 1 && NVD >= 1, "too many wavefronts for this tile");
    constexpr int PD = 4;
    constexpr int NS = 2 * KC;   // logit MFMAs per tile
    constexpr int NP = 4 * DB;   // PV MFMAs per tile
    static_assert(NS % PD == 0 && NP % PD == 0, "read-ahead depth must divide the fragment counts");
    constexpr int EPS = 32 / NS; // logits per softmax slice
    constexpr int MPS = 32 / NP; // logits per maximum-scan slice
    static_assert(MPS % 2 == 0, "maximum scan takes logits in pairs");

    extern __shared__ __attribute__((aligned(1024))) uint8_t lds8[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;

    const int n_qt = (p.Sq + BM - 1) / BM;
    const int wg = p.kv_len ? xcd_remap_heads(blockIdx.x, gridDim.x, n_qt) : p.wg_base + xcd_remap(blockIdx.x, gridDim.x);
    const int qt = wg % n_qt;
    const int bh = wg / n_qt;
    const int b = bh / p.H, hh = bh % p.H;
    const int q0 = qt * BM;
    const int qw0 = q0 + wave * 32;
    const int nkb = (p.Sk + kSageKBlk - 1) / kSageKBlk;

    const int8_t* qbase = p.qi8 + (int64_t)bh * p.Sq * D;
    const int8_t* kbase = p.ki8 + (int64_t)bh * p.Sk * D;
    const uint16_t* vbase = p.v + b * p.vs.b + hh * p.vs.h;
    uint16_t* obase = p.o + b * p.os.b + hh * p.os.h;
    const float* skb = p.sk + (int64_t)bh * nkb;

    int klimit = p.Sk;
    if (p.kv_len) klimit = min(klimit, max(p.kv_len[b], 0));
    int kend = klimit;
    if (p.causal) kend = min(kend, q0 + BM);
    const int n_tiles = (kend + BN - 1) / BN;

    // Q^ fragments: column = query, 16 consecutive int8 of the contraction per lane
    i32x4 qf[KC];
    {
        const int row = qw0 + n;
        const i32x4 z = {0, 0, 0, 0};
#pragma unroll
        for (int kc = 0; kc < KC; ++kc)
            qf[kc] = row < p.Sq ? *reinterpret_cast<const i32x4*>(qbase + (int64_t)row * D + 32 * kc + 16 * h) : z;
    }
    // the 32 queries of a wavefront lie in one quantisation block of Q (128 rows); fold softmax scale and log2(e)
    const int nqb = (p.Sq + kSageQBlk - 1) / kSageQBlk;
    const float qfac = p.sq[(int64_t)bh * nqb + min(qw0 / kSageQBlk, nqb - 1)] * p.scale * kLog2e;

    // ---- asynchronous tile copies: K^(t) and V(t) live in stage t&1
    const uint32_t lds0 = lds_addr(lds8);
    const int k_row_in = lane / GPK, k_gran = lane % GPK;
    const int v_row_in = lane / GPV, v_gran = lane % GPV;
    constexpr int RPK = 1024 / D, RPV = 1024 / (2 * D);      // rows per 1 KiB copy
    uint32_t k_lane_off[NKD], v_lane_off[NVD];               // bytes
#pragma unroll
    for (int i = 0; i < NKD; ++i) {
        const int row = (wave * NKD + i) * RPK + k_row_in;
        k_lane_off[i] = (uint32_t)(row * D + ((k_gran ^ swz_i8<D>(row)) << 4));
    }
#pragma unroll
    for (int i = 0; i < NVD; ++i) {
        const int row = (wave * NVD + i) * RPV + v_row_in;
        v_lane_off[i] = 2u * (uint32_t)(row * (int)p.vs.n + (src_granule(v_gran ^ swz<D>(row), p.d) << 3));     // columns past d: a valid filler, their O is not stored
    }
    auto k_dst = [&](int t, int i) { return lds0 + (uint32_t)((t & 1) * T::STAGE_BYTES + (wave * NKD + i) * 1024); };
    auto v_dst = [&](int t, int i) { return lds0 + (uint32_t)((t & 1) * T::STAGE_BYTES + T::K_BYTES + (wave * NVD + i) * 1024); };
    auto issue_k = [&](int t) {                              // ragged: rows clamped into the attended range
#pragma unroll
        for (int i = 0; i < NKD; ++i) {
            const int row = (wave * NKD + i) * RPK + k_row_in;
            const int key = min(t * BN + row, klimit - 1);
            dma16(kbase + (int64_t)key * D + ((k_gran ^ swz_i8<D>(row)) << 4), k_dst(t, i));
        }
    };
    auto issue_v = [&](int t) {
#pragma unroll
        for (int i = 0; i < NVD; ++i) {
            const int row = (wave * NVD + i) * RPV + v_row_in;
            const int key = min(t * BN + row, klimit - 1);
            dma16(vbase + (int64_t)key * p.vs.n + (src_granule(v_gran ^ swz<D>(row), p.d) << 3), v_dst(t, i));
        }
    };
    auto issue_full_kv = [&](int tk, int tv) {               // K^ tile tk and V tile tv, both full
        const int8_t* kt = kbase + (int64_t)tk * BN * D;
        const uint16_t* vt = vbase + (int64_t)tv * BN * p.vs.n;
#pragma unroll
        for (int i = 0; i < NKD; ++i) dma16u(kt, k_lane_off[i], k_dst(tk, i));
#pragma unroll
        for (int i = 0; i < NVD; ++i) dma16u(vt, v_lane_off[i], v_dst(tv, i));
    };

    // ---- per-lane LDS read offsets
    int koff[KC];          // bytes: K^ fragment of row n, logical granule 2*kc + h
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) koff[kc] = n * D + (((2 * kc + h) ^ swz_i8<D>(n)) << 4);
    const int tr_r = lane & 15, tr_g16 = (lane >> 4) & 1;
    int voff[2][DB];       // elements: V^T fragment halves, rows 4h + r/4 (+8)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int row = 4 * h + (tr_r >> 2) + 8 * half;
#pragma unroll
        for (int db = 0; db < DB; ++db)
            voff[half][db] = row * RS + (((4 * db + 2 * tr_g16 + ((tr_r & 3) >> 1)) ^ swz<D>(row)) << 3) + 4 * (tr_r & 1);
    }
    auto k_frag = [&](int t, int i) {       // fragment i = (kc, kb) of K^(t); rows 32*kb + n share the swizzle of row n
        const uint8_t* ks = lds8 + (t & 1) * T::STAGE_BYTES;
        return *reinterpret_cast<const u32x4*>(ks + koff[i >> 1] + 32 * (i & 1) * D);
    };
    auto v_frag = [&](int t, int i) {       // fragment i = (cc, db) of V(t)^T
        const uint16_t* vs = reinterpret_cast<const uint16_t*>(lds8 + (t & 1) * T::STAGE_BYTES + T::K_BYTES);
        const int cc = i / DB, db = i % DB;
        const u32x2 lo = lds_read_tr16(vs + voff[0][db] + 16 * cc * RS);
        const u32x2 hi = lds_read_tr16(vs + voff[1][db] + 16 * cc * RS);
        const u32x4 u = {lo[0], lo[1], hi[0], hi[1]};
        return u;
    };

    // ---- running state; m_run is in log2 units of the dequantised, scaled logits
    float m_run = -INFINITY, l_run = 0.f;
    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;

    auto fold_max = [&](float tmax) {        // tmax in log2 units
        tmax = fmaxf(tmax, xhalf(tmax));
        if (__any(tmax > m_run + 8.0f)) {    // the reference maximum may lag the true one by 2^8
            const float m_old = m_run;
            const float m_new = fmaxf(m_old, tmax);
            const float m_to = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = exp2_fast(m_old - m_to);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
        }
    };
    auto zero_tile = [&](i32x16 (&s)[2]) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[kb][r] = 0;
    };
    // int32 accumulators -> dequantised, scaled, masked logits (log2 units), in place; returns their maximum
    const char* bbase = p.bias ? static_cast<const char*>(p.bias) + (b * p.bb + hh * p.bhs) * (p.bias_f32 ? 4 : 2) : nullptr;
    auto finish_masked = [&](i32x16 (&s)[2], int t) {
        const float f = qfac * skb[t];
        const int qi = qw0 + n;
        float tmax = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = t * BN + 32 * kb + acc_row(r, h);
                const bool drop = (key >= klimit) | ((p.causal != 0) & (key > qi));
                float v = (float)s[kb][r] * f;
                if (bbase && !drop && qi < p.Sq) {      // the logits are in log2 units here
                    const int64_t e = (int64_t)qi * p.bq + (int64_t)key * p.bk;
                    const float bv = p.bias_f32 ? reinterpret_cast<const float*>(bbase)[e]
                                                : __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(bbase)[e] << 16);
                    v = fmaf(bv, kLog2e, v);
                }
                v = drop ? -INFINITY : v;
                tmax = fmaxf(tmax, v);
                s[kb][r] = __float_as_int(v);
            }
        return tmax;
    };

    // The logits of the current tile are kept as floats in the accumulator registers: either the plain
    // converted int32 sums, to be multiplied by cur_fac inside the exponential's fused multiply-add
    // (tiles without exclusions), or already scaled and masked values with cur_fac = 1.
    float cur_fac = 1.0f;

    auto step = [&](auto fast_tag, i32x16 (&cur)[2], i32x16 (&nxt)[2], int t) {
        constexpr bool FAST = decltype(fast_tag)::value;
        const bool has_next = FAST || t + 1 < n_tiles;
        if (FAST) {
            issue_full_kv(t + 2, t + 1);
        } else {
            if (t + 2 < n_tiles) issue_k(t + 2);
            if (has_next) issue_v(t + 1);
        }
        const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
        const float fac = cur_fac;
        float rsum0 = 0.f, rsum1 = 0.f;
        bf16x8 pf[4];
        u32x4 fb[PD];
        auto exp_slice = [&](int j) {
#pragma unroll
            for (int e = 0; e < EPS; ++e) {
                const int idx = EPS * j + e, kb = idx >> 4, r = idx & 15;
                const float v = exp2_fast(fmaf(__int_as_float(cur[kb][r]), fac, -m_use));
                cur[kb][r] = __float_as_int(v);
                if (e & 1) rsum1 += v;
                else rsum0 += v;
                if ((idx & 7) == 7) {
                    const int o8 = r - 7;
                    const i32x16& s = cur[kb];
                    pf[idx >> 3] = pack8(__int_as_float(s[o8 + 0]), __int_as_float(s[o8 + 1]), __int_as_float(s[o8 + 2]),
                                         __int_as_float(s[o8 + 3]), __int_as_float(s[o8 + 4]), __int_as_float(s[o8 + 5]),
                                         __int_as_float(s[o8 + 6]), __int_as_float(s[o8 + 7]));
                }
            }
        };
        auto s_mfma = [&](int i) {
            nxt[i & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, fb[i % PD]), qf[i >> 1], nxt[i & 1], 0, 0, 0);
        };
        auto pv_mfma = [&](int i) {
            oacc[i % DB] = mfma32(__builtin_bit_cast(bf16x8, fb[i % PD]), pf[i / DB], oacc[i % DB]);
        };

        if (FAST) {
            const float f_next = qfac * skb[t + 1];
            zero_tile(nxt);
#pragma unroll
            for (int i = 0; i < PD; ++i) {
                fb[i] = k_frag(t + 1, i);
                __builtin_amdgcn_sched_barrier(0);
            }
            // fragments are consumed in pairs, the younger read of a pair first: one s_waitcnt serves two MFMAs
            auto frag_of = [&](int f) { return f < NS ? k_frag(t + 1, f) : v_frag(t, f - NS); };   // f in [0, NS + NP)
#pragma unroll
            for (int i = 0; i < NS; i += 2) {
                s_mfma(i + 1);
                exp_slice(i);
                __builtin_amdgcn_sched_barrier(0);
                s_mfma(i);
                exp_slice(i + 1);
                fb[i % PD] = frag_of(i + PD);
                fb[(i + 1) % PD] = frag_of(i + 1 + PD);
                __builtin_amdgcn_sched_barrier(0);
            }
            l_run += rsum0 + rsum1;
            // O^T += V(t)^T P(t)^T between the int32 -> float conversion and maximum scan of tile t+1
            float tmax = -INFINITY;
            auto scan_slice = [&](int i) {
#pragma unroll
                for (int e = 0; e < MPS; e += 2) {
                    const int i0 = MPS * i + e, i1 = i0 + 1;
                    const float a = (float)nxt[i0 >> 4][i0 & 15], c = (float)nxt[i1 >> 4][i1 & 15];
                    nxt[i0 >> 4][i0 & 15] = __float_as_int(a);
                    nxt[i1 >> 4][i1 & 15] = __float_as_int(c);
                    tmax = fmaxf(fmaxf(tmax, a), c);
                }
            };
#pragma unroll
            for (int i = 0; i < NP; i += 2) {
                pv_mfma(i + 1);
                scan_slice(i);
                __builtin_amdgcn_sched_barrier(0);
                pv_mfma(i);
                scan_slice(i + 1);
                if (i + PD < NP) {
                    fb[i % PD] = frag_of(NS + i + PD);
                    fb[(i + 1) % PD] = frag_of(NS + i + 1 + PD);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            cur_fac = f_next;
            fold_max(tmax * f_next);         // f_next >= 0 and the sums are finite
        } else {
            if (has_next) {
                zero_tile(nxt);
#pragma unroll
                for (int i = 0; i < PD; ++i) {
                    fb[i] = k_frag(t + 1, i);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int i = 0; i < NS; ++i) {
                    s_mfma(i);
                    if (i + PD < NS) fb[i % PD] = k_frag(t + 1, i + PD);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int j = 0; j < NS; ++j) exp_slice(j);
            l_run += rsum0 + rsum1;
#pragma unroll
            for (int i = 0; i < PD; ++i) {
                fb[i] = v_frag(t, i);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                pv_mfma(i);
                if (i + PD < NP) fb[i % PD] = v_frag(t, i + PD);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (has_next) {
                const float tmax = finish_masked(nxt, t + 1);
                cur_fac = 1.0f;
                fold_max(tmax);
            }
        }
        wait_vm0();          // the copies issued by this step have landed
        __syncthreads();     // ... for every wave, and everyone is done reading this step's tiles
    };

    // tiles [0, n_full) need no exclusions for any query of the workgroup
    int n_full = p.bias ? 0 : klimit / BN;       // a bias touches every logit
    if (p.causal) n_full = min(n_full, (q0 + 1) / BN);
    n_full = min(n_full, n_tiles);

    i32x16 sa[2], sb[2];
    if (n_tiles > 0) {
        issue_k(0);
        issue_v(0);
        if (n_tiles > 1) issue_k(1);
        wait_vm0();
        __syncthreads();
        zero_tile(sa);
#pragma unroll
        for (int i = 0; i < NS; ++i)
            sa[i & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, k_frag(0, i)), qf[i >> 1], sa[i & 1], 0, 0, 0);
        fold_max(finish_masked(sa, 0));
        cur_fac = 1.0f;
        __syncthreads();     // every wave has read K^(0) before step 0 starts overwriting it

        const int n_fast = max(0, n_full - 2) & ~1;      // step t is FAST when t + 2 < n_full
        int t = 0;
        for (; t < n_fast; t += 2) {
            step(std::true_type{}, sa, sb, t);
            step(std::true_type{}, sb, sa, t + 1);
        }
        for (; t < n_tiles; t += 2) {
            step(std::false_type{}, sa, sb, t);
            if (t + 1 < n_tiles) step(std::false_type{}, sb, sa, t + 1);
        }
    }

    const int row = qw0 + n;
    const float l = l_run + xhalf(l_run);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    if (row < p.Sq) {
        uint16_t* orow = obase + (int64_t)row * p.os.n;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x16& a = oacc[db];
                u32x2 w = {pack_bf16(a[4 * g] * inv, a[4 * g + 1] * inv), pack_bf16(a[4 * g + 2] * inv, a[4 * g + 3] * inv)};
                if (32 * db + 8 * g + 4 * h < p.d) *reinterpret_cast<u32x2*>(orow + 32 * db + 8 * g + 4 * h) = w;
            }
        if (p.lse && h == 0) p.lse[(int64_t)bh * p.Sq + row] = l > 0.f ? (m_run + log2_fast(l)) * kLn2 : -INFINITY;
    }
}


// ------------------------------------------------------------------- forward, 256-query workgroups
// The same computation as sage_fwd_kernel for workgroups of 256 queries, laid out for one wavefront per
// SIMD like the bf16 fwd_wide_kernel: 4 wavefronts of 64 queries (two 32-query blocks), so that every K^ / V
// fragment read from LDS feeds two MFMAs.  O^T of both blocks lives in the accumulation registers, the Q^
// fragments are pinned there as MFMA B operands, and the int32 logits are produced in architectural registers
// by hand-emitted int8 MFMAs (nothing may touch them until two further MFMAs have been issued).  Four LDS
// stages (K^ tile 64 x D bytes + V tile 64 x D bf16 each), tile t in stage t % 4; step t reads K^(t+1) and V(t)
// and issues the copies of K^(t+3) and V(t+2); one workgroup barrier per step.  The exponentials of tile t are
// threaded between the logit MFMAs of tile t+1 and the first half of the PV products, the maximum
// scan of tile t+1 between the second half.  Serves problems without any
// exclusion (no causal flag, key lengths or bias, Sk a multiple of 64); all others use sage_fwd_kernel.
template <int D>
struct SageWideTile {
    static constexpr int BM = 256, BN = 64;
    static constexpr int K_BYTES = BN * D;
    static constexpr int V_BYTES = BN * D * 2;
    static constexpr int STAGE_BYTES = K_BYTES + V_BYTES;
    static constexpr int NSTAGE = 4;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;
    static constexpr int K_DMA_PER_WAVE = K_BYTES / 1024 / 4;
    static constexpr int V_DMA_PER_WAVE = V_BYTES / 1024 / 4;
};

template <int D>
__global__ __launch_bounds__(256) void sage_fwd_wide_kernel(const SageFwdParams p) {
    using T = SageWideTile<D>;
    constexpr int BN = T::BN, BM = T::BM;
    constexpr int KC = D / 32, DB = D / 32, RS = D;
    constexpr int GPK = D / 16, GPV = D / 8;
    constexpr int NKD = T::K_DMA_PER_WAVE, NVD = T::V_DMA_PER_WAVE;
    static_assert(NKD >= 1 && NVD >= 1, "tile too small for four wavefronts");
    constexpr int PD = 4;
    constexpr int NKF = 2 * KC;          // K^ fragments per tile (kc, kb); two logit MFMAs each
    constexpr int NVF = 4 * DB;          // V^T fragments per tile (16-key chunk, db); two PV MFMAs each
    static_assert(NKF % PD == 0 && NVF % PD == 0, "read-ahead depth must divide the fragment counts");
    static_assert(NKF == 8 || NKF == 4, "softmax slicing assumes 8 or 4 K^ fragments per tile");
    static_assert(DB <= 4, "O^T tuples are pinned four to a query block");

    extern __shared__ __attribute__((aligned(1024))) uint8_t lds8[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;

    const int n_qt = (p.Sq + BM - 1) / BM;
    const int wg = xcd_remap(blockIdx.x, gridDim.x);
    const int qt = wg % n_qt;
    const int bh = wg / n_qt;
    const int b = bh / p.H, hh = bh % p.H;
    const int q0 = qt * BM;
    const int qw0 = q0 + wave * 64;
    const int nkb = (p.Sk + kSageKBlk - 1) / kSageKBlk;

    const int8_t* qbase = p.qi8 + (int64_t)bh * p.Sq * D;
    const int8_t* kbase = p.ki8 + (int64_t)bh * p.Sk * D;
    const uint16_t* vbase = p.v + b * p.vs.b + hh * p.vs.h;
    uint16_t* obase = p.o + b * p.os.b + hh * p.os.h;
    const float* skb = p.sk + (int64_t)bh * nkb;

    const int n_tiles = p.Sk / BN;          // the launcher guarantees Sk % BN == 0 and no exclusions

    // ---- Q^ fragments (B operand of S^T = K^ Q^^T): column = query, 16 consecutive int8; pinned slots qb*KC + kc
    bf16x8 qf[2][KC];
    int qrow[2];
    static_for<2>([&](auto qb_tag) {
        constexpr int qb = decltype(qb_tag)::value;
        qrow[qb] = qw0 + 32 * qb + n;
        const bool ok = qrow[qb] < p.Sq;
        const int8_t* rp = qbase + (int64_t)qrow[qb] * D + 16 * h;
        static_for<KC>([&](auto kc_tag) {
            constexpr int kc = decltype(kc_tag)::value;
            const u32x4 z = {0u, 0u, 0u, 0u};
            qf[qb][kc] = pin_b_fragment<qb * KC + kc>(ok ? *reinterpret_cast<const u32x4*>(rp + 32 * kc) : z);
        });
    });
    // the 64 queries of a wavefront lie in one quantisation block of Q (128 rows); softmax scale and log2(e) folded in
    const int nqb = (p.Sq + kSageQBlk - 1) / kSageQBlk;
    const float qfac = p.sq[(int64_t)bh * nqb + min(qw0 / kSageQBlk, nqb - 1)] * p.scale * kLog2e;

    // ---- asynchronous tile copies: tile t (K^ and V) lives in stage t % 4
    const uint32_t lds0 = lds_addr(lds8);
    const int k_row_in = lane / GPK, k_gran = lane % GPK;
    const int v_row_in = lane / GPV, v_gran = lane % GPV;
    constexpr int RPK = 1024 / D, RPV = 1024 / (2 * D);
    uint32_t k_lane_off[NKD], v_lane_off[NVD];               // bytes
#pragma unroll
    for (int i = 0; i < NKD; ++i) {
        const int row = (wave * NKD + i) * RPK + k_row_in;
        k_lane_off[i] = (uint32_t)(row * D + ((k_gran ^ swz_i8<D>(row)) << 4));
    }
#pragma unroll
    for (int i = 0; i < NVD; ++i) {
        const int row = (wave * NVD + i) * RPV + v_row_in;
        v_lane_off[i] = 2u * (uint32_t)(row * (int)p.vs.n + (src_granule(v_gran ^ swz<D>(row), p.d) << 3));     // columns past d: a valid filler, their O is not stored
    }
    auto k_dst = [&](int stg, int i) { return lds0 + (uint32_t)(stg * T::STAGE_BYTES + (wave * NKD + i) * 1024); };
    auto v_dst = [&](int stg, int i) { return lds0 + (uint32_t)(stg * T::STAGE_BYTES + T::K_BYTES + (wave * NVD + i) * 1024); };
    const int64_t k_tile_stride = (int64_t)BN * D;                       // bytes
    const int64_t v_tile_stride = (int64_t)BN * p.vs.n;                  // elements
    auto issue_whole_k = [&](int t) {
        const int8_t* tb = kbase + (int64_t)min(t, n_tiles - 1) * k_tile_stride;
#pragma unroll
        for (int i = 0; i < NKD; ++i) dma16u(tb, k_lane_off[i], k_dst(t & 3, i));
    };
    auto issue_whole_v = [&](int t) {
        const uint16_t* tb = vbase + (int64_t)min(t, n_tiles - 1) * v_tile_stride;
#pragma unroll
        for (int i = 0; i < NVD; ++i) dma16u(tb, v_lane_off[i], v_dst(t & 3, i));
    };

    // ---- per-lane LDS read offsets, constant over the key loop
    int koff[KC];          // bytes: K^ fragment of row n, logical granule 2*kc + h
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) koff[kc] = n * D + (((2 * kc + h) ^ swz_i8<D>(n)) << 4);
    const int tr_r = lane & 15, tr_g16 = (lane >> 4) & 1;
    int voff[2][DB];       // elements: V^T fragment halves, rows 4h + r/4 (+8)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int row = 4 * h + (tr_r >> 2) + 8 * half;
#pragma unroll
        for (int db = 0; db < DB; ++db)
            voff[half][db] = row * RS + (((4 * db + 2 * tr_g16 + ((tr_r & 3) >> 1)) ^ swz<D>(row)) << 3) + 4 * (tr_r & 1);
    }
    auto k_frag = [&](const uint8_t* stage, int i) {       // fragment i = (kc, kb); rows 32*kb + n share the swizzle of row n
        return *reinterpret_cast<const u32x4*>(stage + koff[i >> 1] + 32 * (i & 1) * D);
    };
    auto v_frag = [&](const uint8_t* stage, int i) {       // fragment i = (cc, db) of V^T
        const uint16_t* vs = reinterpret_cast<const uint16_t*>(stage + T::K_BYTES);
        const int cc = i / DB, db = i % DB;
        const u32x2 lo = lds_read_tr16(vs + voff[0][db] + 16 * cc * RS);
        const u32x2 hi = lds_read_tr16(vs + voff[1][db] + 16 * cc * RS);
        const u32x4 u = {lo[0], lo[1], hi[0], hi[1]};
        return u;
    };

    // ---- running state; m_run is in log2 units of the dequantised, scaled logits
    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
    f32x16 oacc[2][DB];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[qb][db][r] = 0.f;

    auto fold_max = [&](auto qb_tag, float tmax) {           // tmax in log2 units
        constexpr int qb = decltype(qb_tag)::value;
        tmax = fmaxf(tmax, xhalf(tmax));
        if (__any(tmax > m_run[qb] + 8.0f)) {                // the reference maximum may lag the true one by 2^8
            const float m_old = m_run[qb];
            const float m_new = fmaxf(m_old, tmax);
            const float m_to = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = exp2_fast(m_old - m_to);
            m_run[qb] = m_new;
            l_run[qb] *= alpha;
            static_for<DB>([&](auto db_tag) {
                constexpr int db = decltype(db_tag)::value;
                rescale_pinned<4 * qb + db>(oacc[qb][db], alpha);
            });
        }
    };
    // the hand-emitted MFMAs' results become visible 11 issue cycles after issue
    auto settle = [&](i32x16 (&s)[2][2]) {
        asm volatile("s_nop 7\n\ts_nop 7" : "+v"(s[0][0]), "+v"(s[0][1]), "+v"(s[1][0]), "+v"(s[1][1]));
    };

    // The logit accumulators start from the bit pattern of 1.5 * 2^23 instead of zero: an int32 sum s with
    // |s| < 2^22 (here |s| <= 128 * 127^2 < 2^21) added to it is the bit pattern of the float 1.5 * 2^23 + s, exactly,
    // so the int32 -> float conversion costs nothing and the offset folds into the constant of the exponent's fma.
    constexpr int kMagicBits = 0x4B400000;
    constexpr float kMagic = 12582912.0f;
    i32x16 magic16;
#pragma unroll
    for (int r = 0; r < 16; ++r) magic16[r] = kMagicBits;
    asm volatile("" : "+v"(magic16));

    u32x4 fb[PD];
    float cur_fac = 1.0f;          // dequantisation factor of the tile whose logits are current (log2 units per count)
    // One step: P(t) from the logits in `cur` (float bits of 1.5 * 2^23 + the int32 sums), logits of tile t+1 into
    // `nxt`, O += P(t) V(t).  MFMA slot = 2 * fragment + query block.
    auto step = [&](auto stage_tag, i32x16 (&cur)[2][2], i32x16 (&nxt)[2][2], const int8_t* k3_base, const uint16_t* v2_base,
                    float sk_next) {
        constexpr int s0 = decltype(stage_tag)::value;
        constexpr int s1 = (s0 + 1) & 3, s2 = (s0 + 2) & 3, s3 = (s0 + 3) & 3;
        const uint8_t* stage_t = lds8 + s0 * T::STAGE_BYTES;       // V(t)
        const uint8_t* stage_t1 = lds8 + s1 * T::STAGE_BYTES;      // K^(t+1)
        const uint8_t* stage_t2 = lds8 + s2 * T::STAGE_BYTES;      // K^(t+2), landed during this step at the latest
        const float fac = cur_fac;
        float msc[2], rsum0[2] = {0.f, 0.f}, rsum1[2] = {0.f, 0.f};
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) msc[qb] = fmaf(kMagic, fac, (m_run[qb] == -INFINITY) ? 0.f : m_run[qb]);
        u32x4 pw[2][4];                 // P^T operands: [query block][16-key chunk]
        auto exp_elem = [&](int qb, int idx) {
            const int kb = idx >> 4, r = idx & 15;
            cur[qb][kb][r] = __float_as_int(exp2_fast(fmaf(__int_as_float(cur[qb][kb][r]), fac, -msc[qb])));
        };
        auto pack_pair = [&](int qb, int j) {
            const int idx = 2 * j, kb = idx >> 4, r = idx & 15;
            const float a = __int_as_float(cur[qb][kb][r]), c = __int_as_float(cur[qb][kb][r + 1]);
            rsum0[qb] += a;
            rsum1[qb] += c;
            pw[qb][idx >> 3][(idx & 7) >> 1] = pack_bf16(a, c);
        };

        constexpr int NSL = 2 * NKF;             // MFMA slots of the logit phase
        constexpr int NCOPY = NKD + NVD, CS = (NSL - 2) / NCOPY;      // copies of K^(t+3) and V(t+2); copy j goes with slot CS*j + 1
        constexpr int E1 = 16 / NKF, E2 = 32 / NVF;
        static_assert(E1 >= 1 && E2 >= 2 && E2 % 2 == 0 && E1 % 2 == 0, "slicing");
        static_assert(CS >= 2, "copies do not fit the logit phase");
        auto copy_dst = [&](int g) {
            const int j = (g - 1) / CS;
            if (g >= 1 && (g - 1) % CS == 0 && j < NCOPY) dma_set_dst(j < NKD ? k_dst(s3, j) : v_dst(s2, j - NKD));
        };
        auto copy_issue = [&](int g) {
            const int j = (g - 1) / CS;
            if (g >= 1 && (g - 1) % CS == 0 && j < NCOPY) {
                if (j < NKD) dma16u_issue(k3_base, k_lane_off[j]);
                else dma16u_issue(v2_base, v_lane_off[j - NKD]);
            }
        };
        // ---- S(t+1)^T = K^(t+1) Q^^T between the exponentials of the first key block of tile t
        static_for<NKF>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            static_for<2>([&](auto qb_tag) {
                constexpr int qb = decltype(qb_tag)::value;
                constexpr int g = 2 * i + qb;
                copy_dst(g);
                if (qb == 0 && !(i & 1)) {
                    // one wait for the two fragments the ring read together; the pair read after them stays in flight
                    constexpr int younger = (i + 2 < NKF ? 1 : 2) + (i + 3 < NKF ? 1 : 2);
                    wait_lds_reads<younger>();
                }
                mfma32i8_vgpr_bpinned<qb * KC + (i >> 1), (i >> 1) == 0 ? 2 : 1>(nxt[qb][i & 1], fb[i % PD], qf[qb][i >> 1], magic16);
                __builtin_amdgcn_sched_barrier(0);
                copy_issue(g);
#pragma unroll
                for (int e = 0; e < E1; ++e) exp_elem(qb, E1 * i + e);
                if (i > 0) {
#pragma unroll
                    for (int j = E1 * (i - 1) / 2; j < E1 * i / 2; ++j) pack_pair(qb, j);
                }
                if (qb == 1 && (i & 1)) {
#pragma unroll
                    for (int f = i - 1; f <= i; ++f) {
                        if (f + PD < NKF) fb[f % PD] = k_frag(stage_t1, f + PD);
                        else fb[f % PD] = v_frag(stage_t, f + PD - NKF);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        });
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
            for (int j = E1 * (NKF - 1) / 2; j < 8; ++j) pack_pair(qb, j);
        }
        // ---- O^T += V(t)^T P(t)^T, with the rest of the exponentials, then the maximum scan of tile t+1
        float tmax[2];
        static_for<NVF>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            constexpr int cc = i / DB, db = i % DB;
            static_for<2>([&](auto qb_tag) {
                constexpr int qb = decltype(qb_tag)::value;
                if (qb == 0 && !(i & 1)) {
                    constexpr int younger = (i + 2 < NVF ? 2 : 1) + (i + 3 < NVF ? 2 : 1);
                    wait_lds_reads<younger>();
                    __builtin_amdgcn_sched_barrier(0);
                }
                oacc[qb][db] = mfma32(__builtin_bit_cast(bf16x8, fb[i % PD]), __builtin_bit_cast(bf16x8, pw[qb][cc]), oacc[qb][db]);
                __builtin_amdgcn_sched_barrier(0);
                if (i < NVF / 2) {
#pragma unroll
                    for (int e = 0; e < E2; ++e) exp_elem(qb, 16 + E2 * i + e);
                }
                if (i >= 1 && i <= NVF / 2) {
#pragma unroll
                    for (int j = 8 + E2 * (i - 1) / 2; j < 8 + E2 * i / 2; ++j) pack_pair(qb, j);
                }
                if (i >= NVF / 2) {
                    constexpr int MPS = 64 / NVF;     // logits per slot and block
                    constexpr int k = i - NVF / 2;
#pragma unroll
                    for (int e = 0; e < MPS; ++e) {
                        const int idx = MPS * k + e;
                        const float a = __int_as_float(nxt[qb][idx >> 4][idx & 15]);
                        tmax[qb] = (k == 0 && e == 0) ? a : fmaxf(tmax[qb], a);
                    }
                    asm volatile("" : "+v"(tmax[qb]));
                }
                if (qb == 1) {
                    if (i == NVF - PD) {
                        __builtin_amdgcn_sched_barrier(0);
                        // the copies of the step before (K^(t+2), V(t+1)) have landed; this step's may be in flight ...
                        __builtin_amdgcn_s_waitcnt(0x0F70 | (NCOPY & 15) | ((NCOPY >> 4) << 14));
                        __builtin_amdgcn_s_barrier();    // ... for every wave, and every wave is past tile t-1
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    if (i & 1) {
#pragma unroll
                        for (int f = i - 1; f <= i; ++f) {
                            if (f + PD < NVF) fb[f % PD] = v_frag(stage_t, f + PD);
                            else fb[f % PD] = k_frag(stage_t2, f + PD - NVF);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        });
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) l_run[qb] += rsum0[qb] + rsum1[qb];
        const float f_next = qfac * sk_next;
        cur_fac = f_next;
        const float tl0 = (tmax[0] - kMagic) * f_next, tl1 = (tmax[1] - kMagic) * f_next;      // f_next >= 0
        // both lanes of a query hold the same reference maximum, so each may test its own half
        if (__any(tl0 > m_run[0] + 8.0f || tl1 > m_run[1] + 8.0f)) {
            fold_max(std::integral_constant<int, 0>{}, tl0);
            fold_max(std::integral_constant<int, 1>{}, tl1);
        }
    };

    i32x16 sa[2][2], sb[2][2];
    if (n_tiles > 0) {
        // prologue: K^(0..2) and V(0..1) land; logits and maximum of tile 0; the ring starts on K^(1)
        issue_whole_k(0);
        issue_whole_k(1);
        issue_whole_k(2);
        issue_whole_v(0);
        issue_whole_v(1);
        wait_vm0();
        __syncthreads();
        static_for<NKF>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            const u32x4 kfr = k_frag(lds8, i);
            static_for<2>([&](auto qb_tag) {
                constexpr int qb = decltype(qb_tag)::value;
                mfma32i8_vgpr_bpinned<qb * KC + (i >> 1), (i >> 1) == 0 ? 2 : 1>(sa[qb][i & 1], kfr, qf[qb][i >> 1], magic16);
            });
        });
        settle(sa);
        cur_fac = qfac * skb[0];
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
            float tm = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) tm = fmaxf(tm, __int_as_float(sa[qb][kb][r]));
            tm = (tm - kMagic) * cur_fac;
            m_run[qb] = fmaxf(tm, xhalf(tm));
        }
#pragma unroll
        for (int i = 0; i < PD; ++i) fb[i] = k_frag(lds8 + T::STAGE_BYTES, i);

        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        using I3 = std::integral_constant<int, 3>;
        // K^(t+3) and V(t+2) of the step at hand; copies past the last tile re-read the last tile
        const int8_t* k3 = kbase + (int64_t)min(3, n_tiles - 1) * k_tile_stride;
        const uint16_t* v2 = vbase + (int64_t)min(2, n_tiles - 1) * v_tile_stride;
        auto advance = [&](int t) {    // from step t to step t+1
            k3 += (t + 4 < n_tiles) ? k_tile_stride : 0;
            v2 += (t + 3 < n_tiles) ? v_tile_stride : 0;
        };
        // Key-block scales: a load inside the step would have the compiler wait for every outstanding tile copy
        // (vector load) or LDS read (scalar load) along with it.  Instead lane l keeps the scale of tile w + l + 1
        // for a window of 64 steps starting at w, a step picks its own with one v_readlane, and the next
        // window is asked for a window ahead.
        auto load_window = [&](int w) { return skb[min(w + lane + 1, n_tiles - 1)]; };
        float skw = load_window(0), skw_ahead = 0.f;
        asm volatile("" : "+v"(skw));        // landed before the loop, so that no wait for it is placed inside
        auto fnext = [&](int t) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(skw), t & 63)); };
        for (int t = 0; t < n_tiles; t += 4) {
            if ((t & 63) == 0) {
                if (t > 0) skw = skw_ahead;
                skw_ahead = load_window(t + 64);
            }
            step(I0{}, sa, sb, k3, v2, fnext(t));
            if (t + 1 >= n_tiles) break;
            advance(t);
            step(I1{}, sb, sa, k3, v2, fnext(t + 1));
            if (t + 2 >= n_tiles) break;
            advance(t + 1);
            step(I2{}, sa, sb, k3, v2, fnext(t + 2));
            if (t + 3 >= n_tiles) break;
            advance(t + 2);
            step(I3{}, sb, sa, k3, v2, fnext(t + 3));
            advance(t + 3);
        }
        wait_vm0();          // no copy may land after the workgroup has gone
    }

    // ---- epilogue
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
        const int row = qrow[qb];
        const float l = l_run[qb] + xhalf(l_run[qb]);
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        if (row < p.Sq) {
            uint16_t* orow = obase + (int64_t)row * p.os.n;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const f32x16& a = oacc[qb][db];
                    u32x2 w = {pack_bf16(a[4 * g] * inv, a[4 * g + 1] * inv),
                               pack_bf16(a[4 * g + 2] * inv, a[4 * g + 3] * inv)};
                    if (32 * db + 8 * g + 4 * h < p.d) *reinterpret_cast<u32x2*>(orow + 32 * db + 8 * g + 4 * h) = w;
                }
            if (p.lse && h == 0) p.lse[(int64_t)bh * p.Sq + row] = l > 0.f ? (m_run[qb] + log2_fast(l)) * kLn2 : -INFINITY;
        }
    }
}

}  // namespace fattn
