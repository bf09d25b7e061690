// SageAttention int8-QK inference forward for gfx950.
//
//   sage_kmean_kernel   kmean[b,h,c] = float( (fp64 sum over tokens of K[b,h,:,c]) / Sk )
//                       the fp64 sum of bf16 addends is exact for ordinary magnitudes, hence
//                       independent of the summation order and bit-identical to a CPU loop
//   sage_quant_kernel   Ks = bf16(float(K) - kmean); per 128-row Q block and per 64-row Ks block:
//                       scale = absmax/127 (IEEE division), code = clamp(rint(x/scale), -128, 127)
//   sage_fwd_kernel     S^T = K^ Q^^T on v_mfma_i32_32x32x32_i8 (int32 accumulate), dequantised with
//                       sq*sk*scale, online softmax in fp32, P -> bf16, O^T = V^T P^T on bf16 MFMA
//
// Quantisation closed form follows the reference's sage_quantize_tensor
// (src/sage_attention.rs:524-541); block granularity, mean smoothing and the int8 MFMA are new.
#pragma once
#include "attn_common.hpp"

namespace fattn {

constexpr int kSageQBlk = 128;
constexpr int kSageKBlk = 64;

struct SageQuantParams {
    const uint16_t* q;
    const uint16_t* k;
    Strides qs, ks;
    int B, H, Sq, Sk;
    int smooth_k;
    float* kmean;    // [B*H, D]
    int8_t* qi8;     // [B*H, Sq, D]
    int8_t* ki8;     // [B*H, Sk, D]
    float* sq;       // [B*H, ceil(Sq/128)]
    float* sk;       // [B*H, ceil(Sk/64)]
};

// one workgroup of 512 threads per (batch, head)
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
            const u32x4 w = *reinterpret_cast<const u32x4*>(kb + (int64_t)row * p.ks.n);
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

__device__ __forceinline__ int quant_code(float x, float s) {
    if (s == 0.f) return 0;
    float r = __builtin_rintf(x / s);      // IEEE division, round half to even
    r = fminf(fmaxf(r, -128.f), 127.f);
    return (int)r;
}

// grid = B*H*(nqb + nkb); one workgroup quantises one block
template <int D>
__global__ __launch_bounds__(256) void sage_quant_kernel(const SageQuantParams p) {
    constexpr int CPR = D / 8;
    constexpr int RPP = 256 / CPR;            // rows per pass
    constexpr int MAXC = kSageQBlk / RPP;     // chunks per thread for a 128-row block
    __shared__ float red[4];
    const int tid = threadIdx.x;
    const int nqb = (p.Sq + kSageQBlk - 1) / kSageQBlk;
    const int nkb = (p.Sk + kSageKBlk - 1) / kSageKBlk;
    const int per_bh = nqb + nkb;
    const int bh = blockIdx.x / per_bh;
    const int blk = blockIdx.x % per_bh;
    const bool is_q = blk < nqb;
    const int b = bh / p.H, hh = bh % p.H;
    const int rows_blk = is_q ? kSageQBlk : kSageKBlk;
    const int S = is_q ? p.Sq : p.Sk;
    const int r0 = (is_q ? blk : blk - nqb) * rows_blk;
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
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int row = r0 + rsub + RPP * i;
        const bool ok = (rsub + RPP * i) < rows_blk && row < S;
        const u32x4 w = ldg16(src + (int64_t)row * st.n + chunk * 8, ok);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float lo = bf16_lo(w[j]), hi = bf16_hi(w[j]);
            if (!is_q) {   // smoothed K, rounded to bf16 exactly as the checker does
                const uint32_t pk = pack_bf16(lo - mu[2 * j], hi - mu[2 * j + 1]);
                lo = bf16_lo(pk);
                hi = bf16_hi(pk);
            }
            if (!ok) { lo = 0.f; hi = 0.f; }
            x[i][2 * j] = lo;
            x[i][2 * j + 1] = hi;
            amax = fmaxf(amax, fmaxf(fabsf(lo), fabsf(hi)));
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float s = amax / 127.0f;
    if (tid == 0) {
        if (is_q) p.sq[(int64_t)bh * nqb + blk] = s;
        else p.sk[(int64_t)bh * nkb + (blk - nqb)] = s;
    }
    int8_t* dst = (is_q ? p.qi8 : p.ki8) + (int64_t)bh * S * D;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int row = r0 + rsub + RPP * i;
        const bool ok = (rsub + RPP * i) < rows_blk && row < S;
        if (!ok) continue;
        uint32_t w0 = 0, w1 = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            w0 |= (uint32_t)(quant_code(x[i][j], s) & 0xff) << (8 * j);
            w1 |= (uint32_t)(quant_code(x[i][4 + j], s) & 0xff) << (8 * j);
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
    float scale;
    const int32_t* kv_len;
    int causal;
};

template <int D>
struct SageTile {
    static constexpr int BM = 128, BN = 64;
    static constexpr int KSB = D + 16;            // bytes per row of the int8 K tile
    static constexpr int VS = D + 32;             // elements per row of the bf16 V tile (transposing reads)
    static constexpr int K_BYTES = BN * KSB;
    static constexpr int V_BYTES = BN * VS * 2;
    static constexpr int STAGE_BYTES = K_BYTES + V_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static constexpr int NKC = BN * (D / 16) / 256;   // 16-byte int8 chunks per thread (D=128: 2, D=64: 1)
    static constexpr int NVC = BN * (D / 8) / 256;    // 16-byte bf16 chunks per thread
};

template <int D>
__global__ __launch_bounds__(256) void sage_fwd_kernel(const SageFwdParams p) {
    using T = SageTile<D>;
    constexpr int BM = T::BM, BN = T::BN, KSB = T::KSB, VS = T::VS;
    constexpr int DC = D / 32;   // int8 contraction chunks (32 per MFMA)
    constexpr int DB = D / 32;

    extern __shared__ __attribute__((aligned(16))) uint8_t lds8[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, h = lane >> 5;

    const int n_qt = (p.Sq + BM - 1) / BM;
    const int wg = xcd_remap(blockIdx.x, gridDim.x);
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
    i32x4 qf[DC];
    {
        const int row = qw0 + n;
        const i32x4 z = {0, 0, 0, 0};
#pragma unroll
        for (int dc = 0; dc < DC; ++dc)
            qf[dc] = row < p.Sq ? *reinterpret_cast<const i32x4*>(qbase + (int64_t)row * D + 32 * dc + 16 * h) : z;
    }
    // one quantisation block of Q per workgroup (BM == 128); fold softmax scale and log2(e)
    const float qfac = p.sq[(int64_t)bh * n_qt + qt] * p.scale * kLog2e;

    u32x4 kreg[T::NKC], vreg[T::NVC];
    auto load_tile = [&](int t) {
        const int key0 = t * BN;
#pragma unroll
        for (int i = 0; i < T::NKC; ++i) {
            const int c = tid + 256 * i;
            const int row = c / (D / 16), col = c % (D / 16);
            const int key = key0 + row;
            const u32x4 z = {0u, 0u, 0u, 0u};
            kreg[i] = key < p.Sk ? *reinterpret_cast<const u32x4*>(kbase + (int64_t)key * D + col * 16) : z;
        }
#pragma unroll
        for (int i = 0; i < T::NVC; ++i) {
            const int c = tid + 256 * i;
            const int row = c / (D / 8), col = c % (D / 8);
            const int key = key0 + row;
            vreg[i] = ldg16(vbase + (int64_t)key * p.vs.n + col * 8, key < klimit);
        }
    };
    auto store_tile = [&](int buf) {
        uint8_t* ks = lds8 + buf * T::STAGE_BYTES;
        uint16_t* vs = reinterpret_cast<uint16_t*>(ks + T::K_BYTES);
#pragma unroll
        for (int i = 0; i < T::NKC; ++i) {
            const int c = tid + 256 * i;
            const int row = c / (D / 16), col = c % (D / 16);
            *reinterpret_cast<u32x4*>(ks + row * KSB + col * 16) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < T::NVC; ++i) {
            const int c = tid + 256 * i;
            const int row = c / (D / 8), col = c % (D / 8);
            *reinterpret_cast<u32x4*>(vs + row * VS + col * 8) = vreg[i];
        }
    };

    float m_run = -INFINITY, l_run = 0.f;    // m_run in log2 units of the dequantised, scaled logits
    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;

    if (n_tiles > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();

    for (int t = 0; t < n_tiles; ++t) {
        const int buf = t & 1;
        const bool more = (t + 1) < n_tiles;
        if (more) load_tile(t + 1);
        const uint8_t* ks = lds8 + buf * T::STAGE_BYTES;
        const uint16_t* vs = reinterpret_cast<const uint16_t*>(ks + T::K_BYTES);
        const int key0 = t * BN;

        i32x16 iacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) iacc[kb][r] = 0;
#pragma unroll
        for (int dc = 0; dc < DC; ++dc)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const i32x4 ka = *reinterpret_cast<const i32x4*>(ks + (32 * kb + n) * KSB + 32 * dc + 16 * h);
                iacc[kb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ka, qf[dc], iacc[kb], 0, 0, 0);
            }

        const float f = qfac * skb[t];       // one K quantisation block per 64-key tile
        f32x16 sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[kb][r] = (float)iacc[kb][r] * f;

        const bool tail = key0 + BN > klimit;
        const bool diag = p.causal && (key0 + BN - 1 > qw0);
        if (tail || diag) {
            const int qi = qw0 + n;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = key0 + 32 * kb + acc_row(r, h);
                    const bool drop = key >= klimit || (p.causal && key > qi);
                    sacc[kb][r] = drop ? -INFINITY : sacc[kb][r];
                }
        }

        float tmax = sacc[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, sacc[kb][r]);
        tmax = fmaxf(tmax, xhalf(tmax));
        const float m_new = fmaxf(m_run, tmax);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = exp2_fast(m_run - m_use);
        m_run = m_new;
        float rsum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float e = exp2_fast(sacc[kb][r] - m_use);
                sacc[kb][r] = e;
                rsum += e;
            }
        l_run = l_run * alpha + rsum;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;

#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            const int kb = cc >> 1, o8 = 8 * (cc & 1);
            const f32x16& s = sacc[kb];
            const bf16x8 pf = pack8(s[o8], s[o8 + 1], s[o8 + 2], s[o8 + 3], s[o8 + 4], s[o8 + 5], s[o8 + 6], s[o8 + 7]);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const bf16x8 va = lds_tr_frag(vs, VS, 16 * cc, 32 * db, lane);
                oacc[db] = mfma32(va, pf, oacc[db]);
            }
        }

        if (more) store_tile(buf ^ 1);
        __syncthreads();
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
                *reinterpret_cast<u32x2*>(orow + 32 * db + 8 * g + 4 * h) = w;
            }
        if (p.lse && h == 0) p.lse[(int64_t)bh * p.Sq + row] = l > 0.f ? (m_run + log2_fast(l)) * kLn2 : -INFINITY;
    }
}

}  // namespace fattn
