// Tiled QK^T -> online softmax -> PV forward for gfx950.  Writes O (bf16) and, when asked, the
// per-row log-sum-exp of the scaled logits; the Sq x Sk score matrix never leaves registers.
//
// One workgroup = 4 wavefronts = 128*NWQ query rows of one (batch, head); each wavefront owns
// 32*NWQ rows whose Q fragments stay in registers.  K/V tiles of 64 keys are staged through LDS
// (double buffered, register prefetch), both row-major.  The logits are produced transposed, S^T = K Q^T, so that
// every lane holds values of a single query: row max / row sum are in-lane reductions plus one
// exchange between the wave halves, the bf16 P^T values are already in the B-operand layout of the
// second MFMA (O^T = V^T P^T), and the running rescale of O is a per-lane scalar.  The V^T operand
// of that MFMA is gathered from the row-major V tile with the transposing LDS read.
#pragma once
#include "attn_common.hpp"

namespace fattn {

struct FwdParams {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* o;
    float* lse;          // contiguous [B*H, Sq] or null
    Strides qs, ks, vs, os;
    int B, H, Sq, Sk;
    float scale;
    MaskArgs m;
};

template <int D>
struct FwdTile {
    static constexpr int BN = 64;            // keys per tile
    static constexpr int KS = D + 8;         // LDS row stride of the K tile, elements
    static constexpr int VS = D + 8;         // LDS row stride of the V tile, elements
    static constexpr int K_ELEMS = BN * KS;
    static constexpr int V_ELEMS = BN * VS;
    static constexpr int STAGE_ELEMS = K_ELEMS + V_ELEMS;
    static constexpr int LDS_BYTES = 2 * STAGE_ELEMS * 2;
    static constexpr int NKC = BN * (D / 8) / 256;   // 16-byte chunks per thread and tensor
};

template <int D, int NWQ>
__global__ __launch_bounds__(256) void fwd_kernel(const FwdParams p) {
    using T = FwdTile<D>;
    constexpr int BN = T::BN, KS = T::KS, VS = T::VS;
    constexpr int BM = 128 * NWQ;
    constexpr int DC = D / 16;   // contraction chunks of QK^T
    constexpr int DB = D / 32;   // 32-row blocks of O^T

    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, h = lane >> 5;

    const int n_qt = (p.Sq + BM - 1) / BM;
    const int qt = blockIdx.x % n_qt;
    const int bh = blockIdx.x / n_qt;
    const int b = bh / p.H, hh = bh % p.H;
    const int q0 = qt * BM;
    const int qw0 = q0 + wave * 32 * NWQ;

    const uint16_t* qbase = p.q + b * p.qs.b + hh * p.qs.h;
    const uint16_t* kbase = p.k + b * p.ks.b + hh * p.ks.h;
    const uint16_t* vbase = p.v + b * p.vs.b + hh * p.vs.h;
    uint16_t* obase = p.o + b * p.os.b + hh * p.os.h;

    int klimit = p.Sk;
    if (p.m.kv_len) klimit = min(klimit, max(p.m.kv_len[b], 0));
    int kend = klimit;
    if (p.m.causal) kend = min(kend, q0 + BM);
    const int n_tiles = (kend + BN - 1) / BN;
    const uint8_t* mbase = p.m.mask ? p.m.mask + b * p.m.sb + hh * p.m.sh : nullptr;

    // ---- Q fragments (B operand of S^T = K Q^T): column = query, 8 consecutive d
    bf16x8 qf[NWQ][DC];
#pragma unroll
    for (int qb = 0; qb < NWQ; ++qb) {
        const int row = qw0 + 32 * qb + n;
        const bool ok = row < p.Sq;
        const uint16_t* rp = qbase + (int64_t)row * p.qs.n + 8 * h;
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) qf[qb][dc] = __builtin_bit_cast(bf16x8, ldg16(rp + 16 * dc, ok));
    }

    // ---- staging assignment
    u32x4 kreg[T::NKC];
    u32x4 vreg[T::NKC];

    auto load_tile = [&](int t) {
        const int key0 = t * BN;
#pragma unroll
        for (int i = 0; i < T::NKC; ++i) {
            const int c = tid + 256 * i;
            const int row = c / (D / 8), col = c % (D / 8);
            const int key = key0 + row;
            kreg[i] = ldg16(kbase + (int64_t)key * p.ks.n + col * 8, key < p.Sk);
            vreg[i] = ldg16(vbase + (int64_t)key * p.vs.n + col * 8, key < klimit);
        }
    };
    auto store_tile = [&](int buf) {
        uint16_t* ks = lds + buf * T::STAGE_ELEMS;
        uint16_t* vs = ks + T::K_ELEMS;
#pragma unroll
        for (int i = 0; i < T::NKC; ++i) {
            const int c = tid + 256 * i;
            const int row = c / (D / 8), col = c % (D / 8);
            *reinterpret_cast<u32x4*>(ks + row * KS + col * 8) = kreg[i];
            *reinterpret_cast<u32x4*>(vs + row * VS + col * 8) = vreg[i];
        }
    };

    // ---- running state; each lane serves query column n of every block qb
    const float c_log2 = p.scale * kLog2e;
    float m_run[NWQ], l_run[NWQ];
    f32x16 oacc[NWQ][DB];
#pragma unroll
    for (int qb = 0; qb < NWQ; ++qb) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[qb][db][r] = 0.f;
    }

    if (n_tiles > 0) {
        load_tile(0);
        store_tile(0);
    }
    __syncthreads();

    for (int t = 0; t < n_tiles; ++t) {
        const int buf = t & 1;
        const bool more = (t + 1) < n_tiles;
        if (more) load_tile(t + 1);

        const uint16_t* ks = lds + buf * T::STAGE_ELEMS;
        const uint16_t* vs = ks + T::K_ELEMS;
        const int key0 = t * BN;

        // ---- S^T = K Q^T : rows = keys (two blocks of 32), columns = queries
        f32x16 sacc[NWQ][2];
#pragma unroll
        for (int qb = 0; qb < NWQ; ++qb)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[qb][kb][r] = 0.f;
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const bf16x8 ka = *reinterpret_cast<const bf16x8*>(ks + (32 * kb + n) * KS + 16 * dc + 8 * h);
#pragma unroll
                for (int qb = 0; qb < NWQ; ++qb) sacc[qb][kb] = mfma32(ka, qf[qb][dc], sacc[qb][kb]);
            }
        }

        // ---- exclusions: ragged tail / key length, causal, explicit keep-mask
        const bool tail = key0 + BN > klimit;
        const bool diag = p.m.causal && (key0 + BN - 1 > qw0);
        if (tail || diag || mbase) {
#pragma unroll
            for (int qb = 0; qb < NWQ; ++qb) {
                const int qi = qw0 + 32 * qb + n;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int key = key0 + 32 * kb + acc_row(r, h);
                        bool drop = key >= klimit;
                        if (p.m.causal) drop = drop || key > qi;
                        if (mbase && !drop && qi < p.Sq)
                            drop = mbase[(int64_t)qi * p.m.sq + (int64_t)key * p.m.sk] == 0;
                        if (drop) sacc[qb][kb][r] = -INFINITY;
                    }
            }
        }

        // ---- online softmax, one query per lane
        bf16x8 pf[NWQ][4];
#pragma unroll
        for (int qb = 0; qb < NWQ; ++qb) {
            float tmax = sacc[qb][0][0];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, sacc[qb][kb][r]);
            tmax = fmaxf(tmax, xhalf(tmax));
            const float m_new = fmaxf(m_run[qb], tmax);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = exp2_fast((m_run[qb] - m_use) * c_log2);
            m_run[qb] = m_new;
            const float msc = m_use * c_log2;
            float rsum = 0.f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float e = exp2_fast(fmaf(sacc[qb][kb][r], c_log2, -msc));
                    sacc[qb][kb][r] = e;
                    rsum += e;
                }
            l_run[qb] = l_run[qb] * alpha + rsum;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[qb][db][r] *= alpha;
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
                const int kb = cc >> 1, o8 = 8 * (cc & 1);
                const f32x16& s = sacc[qb][kb];
                pf[qb][cc] = pack8(s[o8 + 0], s[o8 + 1], s[o8 + 2], s[o8 + 3], s[o8 + 4], s[o8 + 5], s[o8 + 6],
                                   s[o8 + 7]);
            }
        }

        // ---- O^T += V^T P^T : rows = d, columns = queries, contraction over the 64 keys
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const bf16x8 va = lds_tr_frag(vs, VS, 16 * cc, 32 * db, lane);
#pragma unroll
                for (int qb = 0; qb < NWQ; ++qb) oacc[qb][db] = mfma32(va, pf[qb][cc], oacc[qb][db]);
            }
        }

        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue
#pragma unroll
    for (int qb = 0; qb < NWQ; ++qb) {
        const int row = qw0 + 32 * qb + n;
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
                    *reinterpret_cast<u32x2*>(orow + 32 * db + 8 * g + 4 * h) = w;
                }
            if (p.lse && h == 0) {
                const float v = l > 0.f ? (m_run[qb] * c_log2 + log2_fast(l)) * kLn2 : -INFINITY;
                p.lse[(int64_t)bh * p.Sq + row] = v;
            }
        }
    }
}

}  // namespace fattn
