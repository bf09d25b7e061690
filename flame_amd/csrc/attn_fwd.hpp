// Tiled QK^T -> online softmax -> PV forward for gfx950.  Writes O (bf16) and, when asked, the
// per-row log-sum-exp of the scaled logits; the Sq x Sk score matrix never leaves registers.
//
// One workgroup = 4 wavefronts = 128*NWQ query rows of one (batch, head); each wavefront owns
// 32*NWQ rows whose Q fragments stay in registers.  K/V tiles of 64 keys are copied global -> LDS
// by the asynchronous LDS-DMA loads (no staging registers), double buffered, row-major with an XOR
// swizzle of the 16-byte granules so that both the row reads of K and the transposing reads of V are
// free of bank conflicts without padding.  The logits are produced transposed, S^T = K Q^T, so that
// every lane holds values of a single query: row max / row sum are in-lane reductions plus one
// exchange between the wave halves, the bf16 P^T values are already in the B-operand layout of the
// second MFMA (O^T = V^T P^T), and the running rescale of O is a per-lane scalar that is skipped
// while the running maximum stays within 2^8 of the reference maximum in use.
#pragma once
#include <type_traits>

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
    static constexpr int BN = 64;                   // keys per tile
    static constexpr int RS = D;                    // LDS row stride, elements
    static constexpr int TILE_ELEMS = BN * D;       // one K or V tile
    static constexpr int STAGE_ELEMS = 2 * TILE_ELEMS;
    static constexpr int LDS_BYTES = 2 * STAGE_ELEMS * 2;
    static constexpr int ROWS_PER_DMA = 1024 / (D * 2);          // rows covered by one 64-lane x 16-byte copy
    static constexpr int DMA_PER_WAVE = BN / ROWS_PER_DMA / 4;   // copies per wave and tensor
};

template <int D, int NWQ, bool HASMASK>
__global__ __launch_bounds__(256, (NWQ == 1 ? 2 : 1)) void fwd_kernel(const FwdParams p) {
    using T = FwdTile<D>;
    constexpr int BN = T::BN, RS = T::RS;
    constexpr int BM = 128 * NWQ;
    constexpr int DC = D / 16;   // contraction chunks of QK^T
    constexpr int DB = D / 32;   // 32-row blocks of O^T
    constexpr int GPR = D / 8;   // 16-byte granules per row

    extern __shared__ __attribute__((aligned(1024))) uint16_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, h = lane >> 5;

    const int n_qt = (p.Sq + BM - 1) / BM;
    const int wg = xcd_remap(blockIdx.x, gridDim.x);
    const int qt = wg % n_qt;
    const int bh = wg / n_qt;
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
    const uint8_t* mbase = HASMASK ? p.m.mask + b * p.m.sb + hh * p.m.sh : nullptr;

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

    // ---- asynchronous tile copies.  Full tiles: uniform tile base + a per-lane 32-bit offset that
    //      never changes; the ragged last tile clamps its rows into the attended range.
    const int dma_row_in = lane / GPR;                       // row inside one 1 KiB copy
    const int dma_gran = lane % GPR;                         // physical granule written by this lane
    int k_lane_off[T::DMA_PER_WAVE], v_lane_off[T::DMA_PER_WAVE];
#pragma unroll
    for (int i = 0; i < T::DMA_PER_WAVE; ++i) {
        const int row = (wave * T::DMA_PER_WAVE + i) * T::ROWS_PER_DMA + dma_row_in;
        const int c = dma_gran ^ swz<D>(row);
        k_lane_off[i] = row * (int)p.ks.n + c * 8;
        v_lane_off[i] = row * (int)p.vs.n + c * 8;
    }
    auto issue_tile = [&](int t, int buf) {
        uint16_t* kdst = lds + buf * T::STAGE_ELEMS;
        uint16_t* vdst = kdst + T::TILE_ELEMS;
#pragma unroll
        for (int i = 0; i < T::DMA_PER_WAVE; ++i) {
            const int ji = wave * T::DMA_PER_WAVE + i;
            const int row = ji * T::ROWS_PER_DMA + dma_row_in;
            const int key = min(t * BN + row, klimit - 1);   // tail rows re-read the last attended key
            const int c = dma_gran ^ swz<D>(row);
            dma16(kbase + (int64_t)key * p.ks.n + c * 8, kdst + ji * 512);
            dma16(vbase + (int64_t)key * p.vs.n + c * 8, vdst + ji * 512);
        }
    };
    auto issue_full_tile = [&](int t, int buf) {
        uint16_t* kdst = lds + buf * T::STAGE_ELEMS;
        uint16_t* vdst = kdst + T::TILE_ELEMS;
        const uint16_t* kt = kbase + (int64_t)t * BN * p.ks.n;
        const uint16_t* vt = vbase + (int64_t)t * BN * p.vs.n;
#pragma unroll
        for (int i = 0; i < T::DMA_PER_WAVE; ++i) {
            const int ji = wave * T::DMA_PER_WAVE + i;
            dma16u(kt, 2u * k_lane_off[i], kdst + ji * 512);
            dma16u(vt, 2u * v_lane_off[i], vdst + ji * 512);
        }
    };

    // ---- per-lane LDS read offsets (elements), constant over the key loop
    int koff[DC];          // K fragment: row 32*kb + n, logical granule 2*dc + h
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) koff[dc] = n * RS + (((2 * dc + h) ^ swz<D>(n)) << 3);
    const int tr_r = lane & 15, tr_g16 = (lane >> 4) & 1;
    int voff[2][DB];       // V^T fragment halves: rows 4h + r/4 (+8), logical granule 4*db + 2*g16 + (r&3)/2
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int row = 4 * h + (tr_r >> 2) + 8 * half;
#pragma unroll
        for (int db = 0; db < DB; ++db)
            voff[half][db] = row * RS + (((4 * db + 2 * tr_g16 + ((tr_r & 3) >> 1)) ^ swz<D>(row)) << 3) + 4 * (tr_r & 1);
    }

    // ---- running state; each lane serves query column n of every block qb
    const float c_log2 = p.scale * kLog2e;
    const float stale_ok = 8.0f / c_log2;     // the reference maximum may lag the true one by 2^8
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

    if (n_tiles > 0) issue_tile(0, 0);
    wait_vm0();
    __syncthreads();

    // One key tile.  MASKED: the tile needs per-element exclusions (ragged tail, causal diagonal,
    // explicit mask).  COPY: 1 = the next tile is a full one (straight-line copies), 2 = decide at run time.
    auto tile_step = [&](auto masked_tag, auto copy_tag, int t) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        constexpr int COPY = decltype(copy_tag)::value;
        const int buf = t & 1;
        if (COPY == 1) issue_full_tile(t + 1, buf ^ 1);
        else if (t + 1 < n_tiles) issue_tile(t + 1, buf ^ 1);

        const uint16_t* ks = lds + buf * T::STAGE_ELEMS;
        const uint16_t* vs = ks + T::TILE_ELEMS;
        const int key0 = t * BN;

        // ---- S^T = K Q^T : rows = keys (two blocks of 32), columns = queries.  K fragments are read
        //      PD ahead of the MFMAs that consume them.
        f32x16 sacc[NWQ][2];
#pragma unroll
        for (int qb = 0; qb < NWQ; ++qb)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[qb][kb][r] = 0.f;
        {
            constexpr int NF = 2 * DC, PD = 4;
            bf16x8 fb[PD];
            auto rd = [&](int i) { return *reinterpret_cast<const bf16x8*>(ks + koff[i >> 1] + 32 * (i & 1) * RS); };
#pragma unroll
            for (int i = 0; i < PD; ++i) {
                fb[i] = rd(i);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < NF; ++i) {
                const int dc = i >> 1, kb = i & 1;
#pragma unroll
                for (int qb = 0; qb < NWQ; ++qb) sacc[qb][kb] = mfma32(fb[i % PD], qf[qb][dc], sacc[qb][kb]);
                if (i + PD < NF) fb[i % PD] = rd(i + PD);
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        // ---- exclusions: ragged tail / key length, causal, explicit keep-mask
        if (MASKED) {
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
                        if (HASMASK) {
                            if (!drop && qi < p.Sq) drop = mbase[(int64_t)qi * p.m.sq + (int64_t)key * p.m.sk] == 0;
                        }
                        sacc[qb][kb][r] = drop ? -INFINITY : sacc[qb][kb][r];   // select, not a divergent store
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
            // move the reference maximum (and rescale the running sums) only when some lane's tile
            // maximum exceeds it by more than 2^8 in the exponent domain; wave-uniform branch
            if (__any(tmax > m_run[qb] + stale_ok)) {
                const float m_old = m_run[qb];
                const float m_new = fmaxf(m_old, tmax);
                const float m_to = (m_new == -INFINITY) ? 0.f : m_new;
                const float alpha = exp2_fast((m_old - m_to) * c_log2);
                m_run[qb] = m_new;
                l_run[qb] *= alpha;
                if constexpr (NWQ > 1) {
#pragma unroll
                    for (int db = 0; db < DB; ++db) scale_acc_agpr(oacc[qb][db], alpha);
                } else {
#pragma unroll
                    for (int db = 0; db < DB; ++db)
#pragma unroll
                        for (int r = 0; r < 16; ++r) oacc[qb][db][r] *= alpha;
                }
            }
            const float m_use = (m_run[qb] == -INFINITY) ? 0.f : m_run[qb];
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
            l_run[qb] += rsum;
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
                const int kb = cc >> 1, o8 = 8 * (cc & 1);
                const f32x16& s = sacc[qb][kb];
                pf[qb][cc] = pack8(s[o8 + 0], s[o8 + 1], s[o8 + 2], s[o8 + 3], s[o8 + 4], s[o8 + 5], s[o8 + 6],
                                   s[o8 + 7]);
            }
        }

        // ---- O^T += V^T P^T : rows = d, columns = queries, contraction over the 64 keys
        {
            constexpr int NF = 4 * DB, PD = 4;
            bf16x8 fb[PD];
            auto rd = [&](int i) {
                const int cc = i / DB, db = i % DB;
                const u32x2 lo = lds_read_tr16(vs + voff[0][db] + 16 * cc * RS);
                const u32x2 hi = lds_read_tr16(vs + voff[1][db] + 16 * cc * RS);
                const u32x4 u = {lo[0], lo[1], hi[0], hi[1]};
                return __builtin_bit_cast(bf16x8, u);
            };
#pragma unroll
            for (int i = 0; i < PD; ++i) {
                fb[i] = rd(i);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < NF; ++i) {
                const int cc = i / DB, db = i % DB;
#pragma unroll
                for (int qb = 0; qb < NWQ; ++qb) oacc[qb][db] = mfma32(fb[i % PD], pf[qb][cc], oacc[qb][db]);
                if (i + PD < NF) fb[i % PD] = rd(i + PD);
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        wait_vm0();          // next tile has landed in the other buffer
        __syncthreads();     // ... for every wave, and everyone is done reading this one
    };

    // Tiles [0, n_full) need no exclusions for any query of the workgroup; the rest (ragged tail, causal
    // diagonal, or everything under an explicit mask) run the specialised masked body.
    int n_full = HASMASK ? 0 : klimit / BN;
    if (p.m.causal) n_full = min(n_full, (q0 + 1) / BN);
    n_full = min(n_full, n_tiles);
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    for (int t = 0; t < n_full - 1; ++t) tile_step(std::false_type{}, I1{}, t);
    if (n_full > 0) tile_step(std::false_type{}, I2{}, n_full - 1);
    for (int t = n_full; t < n_tiles; ++t) tile_step(std::true_type{}, I2{}, t);

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
