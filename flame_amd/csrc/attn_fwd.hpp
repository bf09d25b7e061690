// Tiled QK^T -> online softmax -> PV forward for gfx950.  Writes O (bf16) and, when asked, the
// per-row log-sum-exp of the scaled logits; the Sq x Sk score matrix never leaves registers.
//
// One workgroup = NW wavefronts (4 or 8) = 32*NW query rows of one (batch, head); each wavefront owns
// 32 rows whose Q fragments stay in registers.  Eight wavefronts share each K/V tile among twice as
// many queries (half the copy traffic per MFMA) and are used when the query count fills such
// workgroups; either way two wavefronts are resident per SIMD.  K/V tiles of 64 keys are copied global -> LDS
// by the asynchronous LDS-DMA loads (no staging registers), double buffered, row-major with an XOR
// swizzle of the 16-byte granules so that both the row reads of K and the transposing reads of V are
// free of bank conflicts without padding.  The logits are produced transposed, S^T = K Q^T, so that
// every lane holds values of a single query: row max / row sum are in-lane reductions plus one
// exchange between the wave halves, the bf16 P^T values are already in the B-operand layout of the
// second MFMA (O^T = V^T P^T), and the running rescale of O is a per-lane scalar that is skipped
// while the running maximum stays within 2^8 of the reference maximum in use.
//
// The key loop is software-pipelined inside each wavefront: a wavefront issues at most one
// instruction every four cycles, and the matrix pipe and the vector ALU only run side by side when
// their instructions alternate in that stream.  Step t therefore threads the exponentials of tile t
// between the MFMAs that produce the logits of tile t+1, and the row-maximum scan of tile t+1 between
// the MFMAs of O += P(t) V(t).  The K tile in LDS runs one tile ahead of the V tile.
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
    int d;               // real head dim of Q and K: a multiple of 8, at most the compiled D
    int dv;              // real head dim of V and O, likewise
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

// VECMASK (with HASMASK): the only exclusions besides key lengths and the causal flag come from a keep-mask
// whose rows are contiguous and 16-byte aligned, Sk is a multiple of the tile and there is no bias; the
// general exclusion code (per-element loads, bias) is then not compiled in, which frees the registers
// that made the general masked kernel spill.
// DROPOUT: the probabilities that multiply V are dropped and rescaled element by element (drop_factor); the row sums,
// and with them the log-sum-exp, stay those of the undropped softmax.
template <int D, bool HASMASK, int NW, bool VECMASK = false, bool DROPOUT = false>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void fwd_kernel(const FwdParams p) {
    static_assert(!VECMASK || HASMASK, "VECMASK is a special case of HASMASK");
    using T = FwdTile<D>;
    constexpr int BN = T::BN, RS = T::RS;
    constexpr int BM = 32 * NW;  // query rows per workgroup
    constexpr int DC = D / 16;   // contraction chunks of QK^T
    constexpr int DB = D / 32;   // 32-row blocks of O^T
    constexpr int GPR = D / 8;   // 16-byte granules per row
    constexpr int NDMA = T::DMA_PER_WAVE * 4 / NW;
    constexpr int PD = 4;        // LDS read-ahead depth, in fragments
    // Tile t lives in stage t % 2; K runs 2 tiles and V 1 tile ahead of use, one barrier per step.
    // (Measured: four stages with deeper prefetch, or a barrier only every second step, are slower.)
    constexpr int NSTAGE = 2;
    constexpr int KD = NSTAGE / 2 + 1, VD = NSTAGE / 2;      // prefetch distances, in tiles
    static_assert((2 * DC) % PD == 0 && (4 * DB) % PD == 0, "read-ahead depth must divide the fragment counts");
    static_assert(2 * DC == 16 || 2 * DC == 8, "softmax slicing assumes 16 or 8 logit MFMAs per tile");

    extern __shared__ __attribute__((aligned(1024))) uint16_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;

    const int n_qt = (p.Sq + BM - 1) / BM;
    const int wg = p.m.kv_len ? xcd_remap_heads(blockIdx.x, gridDim.x, n_qt) : xcd_remap(blockIdx.x, gridDim.x);
    int qt = wg % n_qt, bh = wg / n_qt;
    if (p.m.causal && !p.m.kv_len) causal_longest_first(wg, n_qt, gridDim.x, qt, bh);
    const int b = bh / p.H, hh = bh % p.H;
    const int q0 = qt * BM;
    const int qw0 = q0 + wave * 32;

    const uint16_t* qbase = p.q + b * p.qs.b + hh * p.qs.h;
    const uint16_t* kbase = p.k + b * p.ks.b + hh * p.ks.h;
    const uint16_t* vbase = p.v + b * p.vs.b + hh * p.vs.h;
    uint16_t* obase = p.o + b * p.os.b + hh * p.os.h;

    int klimit = p.Sk;
    if (p.m.kv_len) klimit = min(klimit, max(p.m.kv_len[b], 0));
    int kend = klimit;
    if (p.m.causal) kend = min(kend, q0 + BM);
    const int n_tiles = (kend + BN - 1) / BN;
    const uint8_t* mbase = (HASMASK && p.m.mask) ? mask_head_base(p.m, b, hh) : nullptr;
    const char* bbase = (HASMASK && p.m.bias)
                            ? static_cast<const char*>(p.m.bias) + (b * p.m.bb + hh * p.m.bh) * (p.m.bias_f32 ? 4 : 2)
                            : nullptr;

    // ---- Q fragments (B operand of S^T = K Q^T): column = query, 8 consecutive d
    bf16x8 qf[DC];
    {
        const int row = qw0 + n;
        const bool ok = row < p.Sq;
        const uint16_t* rp = qbase + (int64_t)row * p.qs.n + 8 * h;
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) qf[dc] = __builtin_bit_cast(bf16x8, ldg16(rp + 16 * dc, ok && 16 * dc + 8 * h < p.d));
    }

    // ---- asynchronous tile copies.  K(t) and V(t) live in stage t&1.  Full tiles: uniform tile base
    //      + a per-lane 32-bit byte offset that never changes; ragged tiles clamp their rows into the
    //      attended range.
    const uint32_t lds0 = lds_addr(lds);
    const int dma_row_in = lane / GPR;                       // row inside one 1 KiB copy
    const int dma_gran = lane % GPR;                         // physical granule written by this lane
    uint32_t k_lane_off[NDMA], v_lane_off[NDMA];
#pragma unroll
    for (int i = 0; i < NDMA; ++i) {
        const int row = (wave * NDMA + i) * T::ROWS_PER_DMA + dma_row_in;
        const int c = dma_gran ^ swz<D>(row);
        k_lane_off[i] = 2u * (uint32_t)(row * (int)p.ks.n + src_granule(c, p.d) * 8);
        v_lane_off[i] = 2u * (uint32_t)(row * (int)p.vs.n + src_granule(c, p.dv) * 8);
    }
    auto dst_of = [&](int t, int which, int i) {             // LDS byte address of copy i of this wave
        return lds0 + 2u * (uint32_t)((t & (NSTAGE - 1)) * T::STAGE_ELEMS + which * T::TILE_ELEMS + (wave * NDMA + i) * 512);
    };
    auto issue_ragged = [&](const uint16_t* base, int64_t row_stride, int t, int which) {
#pragma unroll
        for (int i = 0; i < NDMA; ++i) {
            const int row = (wave * NDMA + i) * T::ROWS_PER_DMA + dma_row_in;
            const int key = min(t * BN + row, klimit - 1);   // tail rows re-read the last attended key
            const int c = src_granule(dma_gran ^ swz<D>(row), which ? p.dv : p.d);
            dma16(base + (int64_t)key * row_stride + c * 8, dst_of(t, which, i));
        }
    };
    auto issue_k = [&](int t) { issue_ragged(kbase, p.ks.n, t, 0); };
    auto issue_v = [&](int t) { issue_ragged(vbase, p.vs.n, t, 1); };
    auto issue_full_kv = [&](int tk, int tv) {               // K tile tk and V tile tv, both full
        const uint16_t* kt = kbase + (int64_t)tk * BN * p.ks.n;
        const uint16_t* vt = vbase + (int64_t)tv * BN * p.vs.n;
#pragma unroll
        for (int i = 0; i < NDMA; ++i) {
            dma16u(kt, k_lane_off[i], dst_of(tk, 0, i));
            dma16u(vt, v_lane_off[i], dst_of(tv, 1, i));
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
    auto k_frag = [&](int t, int i) {       // fragment i = (dc, kb) of K(t)
        const uint16_t* ks = lds + (t & (NSTAGE - 1)) * T::STAGE_ELEMS;
        return *reinterpret_cast<const bf16x8*>(ks + koff[i >> 1] + 32 * (i & 1) * RS);
    };
    auto v_frag = [&](int t, int i) {       // fragment i = (cc, db) of V(t)^T
        const uint16_t* vs = lds + (t & (NSTAGE - 1)) * T::STAGE_ELEMS + T::TILE_ELEMS;
        const int cc = i / DB, db = i % DB;
        const u32x2 lo = lds_read_tr16(vs + voff[0][db] + 16 * cc * RS);
        const u32x2 hi = lds_read_tr16(vs + voff[1][db] + 16 * cc * RS);
        const u32x4 u = {lo[0], lo[1], hi[0], hi[1]};
        return __builtin_bit_cast(bf16x8, u);
    };

    // ---- running state; each lane serves query column n
    const float c_log2 = p.scale * kLog2e;
    const float stale_ok = 8.0f / c_log2;     // the reference maximum may lag the true one by 2^8
    float m_run = -INFINITY, l_run = 0.f;
    f32x16 oacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;

    constexpr int NS = 2 * DC;     // logit MFMAs per tile
    constexpr int NP = 4 * DB;     // PV MFMAs per tile
    constexpr int EPS = 32 / NS;   // logits handled per softmax slice

    // flat index (mod 2^32) of this lane's query row in the [B*H, Sq, Sk] probability tensor
    const uint32_t drop_qi = (uint32_t)(qw0 + n);
    (void)drop_qi;
    // exclusions of tile t: ragged tail / key length, causal, explicit keep-mask
    auto apply_mask = [&](f32x16 (&s)[2], int t) {
        const int qi = qw0 + n;
        if constexpr (VECMASK) {
            MaskRow64 mrow;
            mrow.load(mbase + (int64_t)min(qi, p.Sq - 1) * p.m.sq + t * BN);
            // the key length and the causal diagonal cut few tiles: there they are folded into the mask bytes,
            // so that the per-element test is the mask byte alone
            const int lim = (p.m.causal ? min(klimit, qi + 1) : klimit) - t * BN;
            if (__any(lim < BN)) mrow.restrict_to(lim);
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) s[kb][r] = mrow.keep(kb, r, h) ? s[kb][r] : -INFINITY;
            return;
        }
        // a lane's 64 keep-mask bytes of the tile in four 16-byte loads where the layout allows it (each
        // lane owns a query row, so byte loads would touch one cache line per lane and element)
        const bool vec_mask = HASMASK && mbase && p.m.rows16 && t * BN + BN <= p.Sk;
        MaskRow64 mrow;
        if (vec_mask) mrow.load(mbase + (int64_t)min(qi, p.Sq - 1) * p.m.sq + t * BN);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = t * BN + 32 * kb + acc_row(r, h);
                bool drop = (key >= klimit) | ((p.m.causal != 0) & (key > qi));     // bitwise: selects, not branches
                float val = s[kb][r];
                if (HASMASK) {
                    if (vec_mask) drop = drop || !mrow.keep(kb, r, h);
                    else if (mbase && !drop && qi < p.Sq) drop = !mask_attends(p.m, mbase, (int64_t)qi * p.m.sq + (int64_t)key * p.m.sk);
                    if (bbase) {      // scale * (s + bias / scale) = scale * s + bias
                        float bv = 0.f;
                        if (!drop && qi < p.Sq) {
                            const int64_t e = (int64_t)qi * p.m.bq + (int64_t)key * p.m.bk;
                            bv = p.m.bias_f32 ? reinterpret_cast<const float*>(bbase)[e]
                                              : __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(bbase)[e] << 16);
                        }
                        val = fmaf(bv, p.m.inv_scale, val);
                    }
                }
                s[kb][r] = drop ? -INFINITY : val;   // select, not a divergent store
            }
    };
    // Fold the maximum of a freshly computed tile into the running state.  The reference maximum
    // moves (and the running sums are rescaled) only when some lane's tile maximum exceeds it by more
    // than 2^8 in the exponent domain; the branch is wave-uniform.
    auto fold_max = [&](float tmax) {
        tmax = fmaxf(tmax, xhalf(tmax));
        if (__any(tmax > m_run + stale_ok)) {
            const float m_old = m_run;
            const float m_new = fmaxf(m_old, tmax);
            const float m_to = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = exp2_fast((m_old - m_to) * c_log2);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
        }
    };
    auto zero_tile = [&](f32x16 (&s)[2]) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[kb][r] = 0.f;
    };

    // One step: P(t) from the logits in `cur`, logits of tile t+1 into `nxt`, O += P(t) V(t).
    // FAST: tile t+1 needs no exclusions and K(t+KD), V(t+VD) are full tiles (straight-line copies and
    // the interleaved instruction stream).  Otherwise every decision is taken at run time and the
    // phases run one after the other.
    auto step = [&](auto fast_tag, f32x16 (&cur)[2], f32x16 (&nxt)[2], int t) {
        constexpr bool FAST = decltype(fast_tag)::value;
        const bool has_next = FAST || t + 1 < n_tiles;
        if (FAST) {
            issue_full_kv(t + KD, t + VD);
        } else {
            if (t + KD < n_tiles) issue_k(t + KD);
            if (t + VD < n_tiles) issue_v(t + VD);
        }
        const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
        const float msc = m_use * c_log2;
        float rsum0 = 0.f, rsum1 = 0.f;
        bf16x8 pf[4];
        bf16x8 fb[PD];
        // P(t): slice j covers logits [EPS*j, EPS*j + EPS) of the tile in (kb, r) order
        auto exp_slice = [&](int j) {
#pragma unroll
            for (int e = 0; e < EPS; ++e) {
                const int idx = EPS * j + e, kb = idx >> 4, r = idx & 15;
                const float v = exp2_fast(fmaf(cur[kb][r], c_log2, -msc));
                if (e & 1) rsum1 += v;
                else rsum0 += v;
                if constexpr (DROPOUT) {
                    const uint32_t key = (uint32_t)(t * BN + 32 * kb + acc_row(r, h));
                    cur[kb][r] = v * drop_factor_at(p.m, (uint32_t)bh, drop_qi, key, (uint32_t)p.Sq, (uint32_t)p.Sk);
                } else {
                    cur[kb][r] = v;
                }
                if ((idx & 7) == 7) {
                    const int o8 = r - 7;
                    const f32x16& s = cur[kb];
                    pf[idx >> 3] = pack8(s[o8 + 0], s[o8 + 1], s[o8 + 2], s[o8 + 3], s[o8 + 4], s[o8 + 5], s[o8 + 6], s[o8 + 7]);
                }
            }
        };

        if (FAST) {
            // ---- S(t+1)^T = K(t+1) Q^T between the exponentials of tile t
            zero_tile(nxt);
#pragma unroll
            for (int i = 0; i < PD; ++i) {
                fb[i] = k_frag(t + 1, i);
                __builtin_amdgcn_sched_barrier(0);
            }
            // Fragments are consumed in pairs, the younger read of a pair first: LDS returns in order, so
            // the wait for it also covers its partner and one s_waitcnt serves two MFMAs.  The two reads
            // that refill the ring are issued together at the end of the pair.
            auto frag_of = [&](int f) { return f < NS ? k_frag(t + 1, f) : v_frag(t, f - NS); };   // f in [0, NS + NP)
#pragma unroll
            for (int i = 0; i < NS; i += 2) {
                nxt[1] = mfma32(fb[(i + 1) % PD], qf[i >> 1], nxt[1]);
                exp_slice(i);
                __builtin_amdgcn_sched_barrier(0);
                nxt[0] = mfma32(fb[i % PD], qf[i >> 1], nxt[0]);
                exp_slice(i + 1);
                fb[i % PD] = frag_of(i + PD);
                fb[(i + 1) % PD] = frag_of(i + 1 + PD);
                __builtin_amdgcn_sched_barrier(0);
            }
            l_run += rsum0 + rsum1;
            // ---- O^T += V(t)^T P(t)^T between the row-maximum scan of tile t+1
            float tmax = nxt[0][0];
            constexpr int MPS = 32 / NP;
            auto max_slice = [&](int i) {
#pragma unroll
                for (int e = 0; e < MPS; e += 2) {
                    const int idx = MPS * i + e;
                    tmax = fmaxf(fmaxf(tmax, nxt[idx >> 4][idx & 15]), nxt[(idx + 1) >> 4][(idx + 1) & 15]);
                }
            };
#pragma unroll
            for (int i = 0; i < NP; i += 2) {
                oacc[(i + 1) % DB] = mfma32(fb[(i + 1) % PD], pf[(i + 1) / DB], oacc[(i + 1) % DB]);
                max_slice(i);
                __builtin_amdgcn_sched_barrier(0);
                oacc[i % DB] = mfma32(fb[i % PD], pf[i / DB], oacc[i % DB]);
                max_slice(i + 1);
                if (i + PD < NP) {
                    fb[i % PD] = frag_of(NS + i + PD);
                    fb[(i + 1) % PD] = frag_of(NS + i + 1 + PD);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            fold_max(tmax);
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
                    nxt[i & 1] = mfma32(fb[i % PD], qf[i >> 1], nxt[i & 1]);
                    if (i + PD < NS) fb[i % PD] = k_frag(t + 1, i + PD);
                    __builtin_amdgcn_sched_barrier(0);
                }
                apply_mask(nxt, t + 1);
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
                oacc[i % DB] = mfma32(fb[i % PD], pf[i / DB], oacc[i % DB]);
                if (i + PD < NP) fb[i % PD] = v_frag(t, i + PD);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (has_next) {
                float tmax = nxt[0][0];
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, nxt[kb][r]);
                fold_max(tmax);
            }
        }
        wait_vm0();          // the copies issued by this step have landed
        __syncthreads();     // ... for every wave, and everyone is done reading this step's tiles
    };

    // Tiles [0, n_full) need no exclusions for any query of the workgroup; the rest (ragged tail, causal
    // diagonal, or everything under an explicit mask) carry per-element exclusions.
    int n_full = HASMASK ? 0 : klimit / BN;
    if (p.m.causal) n_full = min(n_full, (q0 + 1) / BN);
    n_full = min(n_full, n_tiles);

    f32x16 sa[2], sb[2];
    if (n_tiles > 0) {
        // prologue: the first KD tiles of K and VD tiles of V land; logits and maximum of tile 0
#pragma unroll
        for (int i = 0; i < KD; ++i) {
            if (i < n_tiles) issue_k(i);
            if (i < VD && i < n_tiles) issue_v(i);
        }
        wait_vm0();
        __syncthreads();
        zero_tile(sa);
#pragma unroll
        for (int i = 0; i < NS; ++i) sa[i & 1] = mfma32(k_frag(0, i), qf[i >> 1], sa[i & 1]);
        if (n_full < 1) apply_mask(sa, 0);
        float tmax = sa[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, sa[kb][r]);
        fold_max(tmax);
        __syncthreads();     // every wave has read K(0) before step 0 starts overwriting it

        // step t is FAST when t + KD < n_full; an even number of them keeps `sa` the current tile
        const int n_fast = max(0, n_full - KD) & ~1;
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

    // ---- epilogue
    {
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
                    u32x2 w = {pack_bf16(a[4 * g] * inv, a[4 * g + 1] * inv),
                               pack_bf16(a[4 * g + 2] * inv, a[4 * g + 3] * inv)};
                    if (32 * db + 8 * g + 4 * h < p.dv) *reinterpret_cast<u32x2*>(orow + 32 * db + 8 * g + 4 * h) = w;
                }
            if (p.lse && h == 0) {
                const float v = l > 0.f ? (m_run * c_log2 + log2_fast(l)) * kLn2 : -INFINITY;
                p.lse[(int64_t)bh * p.Sq + row] = v;
            }
        }
    }
}

// ------------------------------------------------------------------- forward, 256-query workgroups
// The same computation as fwd_kernel for workgroups of 256 queries, laid out for one wavefront per
// SIMD: 4 wavefronts of 64 queries (two 32-query blocks) each, so that every K / V fragment read from
// LDS feeds two MFMAs and the LDS reads and waits per MFMA halve.  O^T of both blocks and the Q
// fragments live in the accumulation registers (Q as pinned MFMA B operands), the logits in
// architectural registers through hand-emitted MFMAs (see mfma32_vgpr_bacc): nothing may touch them until
// two further MFMAs have been issued.  Four LDS stages, K(t) and V(t) in stage t % 4: step t reads
// K(t+1) and V(t) and issues the copies of K(t+3) and V(t+2), each into a slot whose previous tile was
// last read two barriers ago, and each with more than a full step to land; one workgroup barrier
// per step, placed just before the fragment ring first reads K(t+2); the ring runs on across steps.
// Every step is the pipelined one: the kernel serves problems without any exclusion (no causal
// flag, key lengths, keep-mask or bias, Sk a multiple of 64); all others use fwd_kernel.  Copies past the
// last tile re-read the last tile, and the logits "of the tile after the last" are never used.  A
// kernel of this size must not spill: scratch memory per wavefront limits how many workgroups the
// device keeps resident, which halved the throughput of a version with a general slow path.
template <int D>
struct FwdWideTile {
    static constexpr int BM = 256;
    static constexpr int BN = 64;
    static constexpr int RS = D;
    static constexpr int TILE_ELEMS = BN * D;
    static constexpr int STAGE_ELEMS = 2 * TILE_ELEMS;
    static constexpr int NSTAGE = 4;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_ELEMS * 2;
    static constexpr int ROWS_PER_DMA = 1024 / (D * 2);
    static constexpr int DMA_PER_WAVE = BN / ROWS_PER_DMA / 4;
};

template <int D>
__global__ __launch_bounds__(256) void fwd_wide_kernel(const FwdParams p) {
    using T = FwdWideTile<D>;
    constexpr int BN = T::BN, RS = T::RS, BM = T::BM;
    constexpr int DC = D / 16, DB = D / 32, GPR = D / 8;
    constexpr int NDMA = T::DMA_PER_WAVE;
    constexpr int PD = 4;
    constexpr int NKF = 2 * DC;          // K fragments per tile (dc, kb); two logit MFMAs each
    constexpr int NVF = 4 * DB;          // V^T fragments per tile (16-key chunk, db); two PV MFMAs each
    static_assert(NKF % PD == 0 && NVF % PD == 0, "read-ahead depth must divide the fragment counts");
    static_assert(NKF == 16 || NKF == 8, "softmax slicing assumes 16 or 8 K fragments per tile");
    static_assert(DB <= 4, "O^T tuples are pinned four to a query block");

    extern __shared__ __attribute__((aligned(1024))) uint16_t lds[];

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

    const uint16_t* qbase = p.q + b * p.qs.b + hh * p.qs.h;
    const uint16_t* kbase = p.k + b * p.ks.b + hh * p.ks.h;
    const uint16_t* vbase = p.v + b * p.vs.b + hh * p.vs.h;
    uint16_t* obase = p.o + b * p.os.b + hh * p.os.h;

    const int n_tiles = p.Sk / BN;          // the launcher guarantees Sk % BN == 0 and no exclusions

    // ---- Q fragments (B operand of S^T = K Q^T): column = query, 8 consecutive d; pinned slots qb*DC + dc
    bf16x8 qf[2][DC];
    int qrow[2];
    static_for<2>([&](auto qb_tag) {
        constexpr int qb = decltype(qb_tag)::value;
        qrow[qb] = qw0 + 32 * qb + n;
        const bool ok = qrow[qb] < p.Sq;
        const uint16_t* rp = qbase + (int64_t)qrow[qb] * p.qs.n + 8 * h;
        static_for<DC>([&](auto dc_tag) {
            constexpr int dc = decltype(dc_tag)::value;
            qf[qb][dc] = pin_b_fragment<qb * DC + dc>(ldg16(rp + 16 * dc, ok && 16 * dc + 8 * h < p.d));
        });
    });

    // ---- asynchronous tile copies: tile t (K and V) lives in stage t % 4
    const uint32_t lds0 = lds_addr(lds);
    const int dma_row_in = lane / GPR, dma_gran = lane % GPR;
    uint32_t k_lane_off[NDMA], v_lane_off[NDMA];
#pragma unroll
    for (int i = 0; i < NDMA; ++i) {
        const int row = (wave * NDMA + i) * T::ROWS_PER_DMA + dma_row_in;
        const int c = dma_gran ^ swz<D>(row);
        k_lane_off[i] = 2u * (uint32_t)(row * (int)p.ks.n + src_granule(c, p.d) * 8);
        v_lane_off[i] = 2u * (uint32_t)(row * (int)p.vs.n + src_granule(c, p.dv) * 8);
    }
    auto dst_of = [&](int stg, int which, int i) {
        return lds0 + 2u * (uint32_t)(stg * T::STAGE_ELEMS + which * T::TILE_ELEMS + (wave * NDMA + i) * 512);
    };
    // whole tile t (clamped to the last one) of K or V into stage t % 4, all copies at once (prologue)
    auto issue_whole = [&](const uint16_t* base, int64_t row_stride, const uint32_t (&lane_off)[NDMA], int t, int which) {
        const uint16_t* tb = base + (int64_t)min(t, n_tiles - 1) * BN * row_stride;
#pragma unroll
        for (int i = 0; i < NDMA; ++i) dma16u(tb, lane_off[i], dst_of(t & 3, which, i));
    };

    // ---- per-lane LDS read offsets (elements), constant over the key loop
    int koff[DC];
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) koff[dc] = n * RS + (((2 * dc + h) ^ swz<D>(n)) << 3);
    const int tr_r = lane & 15, tr_g16 = (lane >> 4) & 1;
    int voff[2][DB];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int row = 4 * h + (tr_r >> 2) + 8 * half;
#pragma unroll
        for (int db = 0; db < DB; ++db)
            voff[half][db] = row * RS + (((4 * db + 2 * tr_g16 + ((tr_r & 3) >> 1)) ^ swz<D>(row)) << 3) + 4 * (tr_r & 1);
    }
    auto k_frag = [&](const uint16_t* stage, int i) {       // fragment i = (dc, kb)
        return *reinterpret_cast<const bf16x8*>(stage + koff[i >> 1] + 32 * (i & 1) * RS);
    };
    auto v_frag = [&](const uint16_t* stage, int i) {       // fragment i = (cc, db) of V^T
        const uint16_t* vs = stage + T::TILE_ELEMS;
        const int cc = i / DB, db = i % DB;
        const u32x2 lo = lds_read_tr16(vs + voff[0][db] + 16 * cc * RS);
        const u32x2 hi = lds_read_tr16(vs + voff[1][db] + 16 * cc * RS);
        const u32x4 u = {lo[0], lo[1], hi[0], hi[1]};
        return __builtin_bit_cast(bf16x8, u);
    };

    // ---- running state; each lane serves query column n of both blocks
    const float c_log2 = p.scale * kLog2e;
    const float stale_ok = 8.0f / c_log2;
    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
    f32x16 oacc[2][DB];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[qb][db][r] = 0.f;

    // Fold the tile maximum of one query block into its running state (see fwd_kernel).  O^T of block
    // qb is pinned to a[64 qb : 64 qb + 63] for the rescale.
    auto fold_max = [&](auto qb_tag, float tmax) {
        constexpr int qb = decltype(qb_tag)::value;
        tmax = fmaxf(tmax, xhalf(tmax));
        if (__any(tmax > m_run[qb] + stale_ok)) {
            const float m_old = m_run[qb];
            const float m_new = fmaxf(m_old, tmax);
            const float m_to = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = exp2_fast((m_old - m_to) * c_log2);
            m_run[qb] = m_new;
            l_run[qb] *= alpha;
            static_for<DB>([&](auto db_tag) {
                constexpr int db = decltype(db_tag)::value;
                rescale_pinned<4 * qb + db>(oacc[qb][db], alpha);
            });
        }
    };
    // the first tile: nothing accumulated yet
    auto first_max = [&](int qb, float tmax) { m_run[qb] = fmaxf(tmax, xhalf(tmax)); };
    // the hand-emitted MFMAs' results become visible 11 issue cycles after issue; the logits pass through
    // the statement so that nothing that reads them can be scheduled ahead of it
    auto settle = [&](f32x16 (&s)[2][2]) {
        asm volatile("s_nop 7\n\ts_nop 7" : "+v"(s[0][0]), "+v"(s[0][1]), "+v"(s[1][0]), "+v"(s[1][1]));
    };
    // S(t)^T of both query blocks from the K tile in `stage`, no overlap (prologue and slow steps)
    auto logits_plain = [&](f32x16 (&s)[2][2], const uint16_t* stage) {
        static_for<NKF>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            const bf16x8 kfr = k_frag(stage, i);
            static_for<2>([&](auto qb_tag) {
                constexpr int qb = decltype(qb_tag)::value;
                mfma32_vgpr_bpinned<qb * DC + (i >> 1), (i >> 1) == 0 ? 0 : 1>(s[qb][i & 1], kfr, qf[qb][i >> 1], s[qb][i & 1]);
            });
        });
        settle(s);
    };
    auto tile_max = [&](const f32x16 (&s)[2]) {
        float tmax = s[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, s[kb][r]);
        return tmax;
    };

    bf16x8 fb[PD];
    // One step: P(t) from the logits in `cur`, logits of tile t+1 into `nxt`, O += P(t) V(t).  MFMA slot
    // = 2 * fragment + query block.  The exponentials of the first key block of tile t are threaded between
    // the logit MFMAs of tile t+1; those of the second key block (needed from the middle of the PV products
    // on) between the first half of the MFMAs of O += P(t) V(t), the row-maximum scan of tile t+1 between
    // the second half: the wavefront is bound by instruction issue, so every slot gets its share.
    // STAGE: stage of tile t (0 .. 3).  k3_base / v2_base: tiles t+3 of K and t+2 of V (clamped).
    auto step = [&](auto stage_tag, f32x16 (&cur)[2][2], f32x16 (&nxt)[2][2], const uint16_t* k3_base,
                    const uint16_t* v2_base) {
        constexpr int s0 = decltype(stage_tag)::value;
        constexpr int s1 = (s0 + 1) & 3, s2 = (s0 + 2) & 3, s3 = (s0 + 3) & 3;
        const uint16_t* stage_t = lds + s0 * T::STAGE_ELEMS;       // V(t)
        const uint16_t* stage_t1 = lds + s1 * T::STAGE_ELEMS;      // K(t+1)
        const uint16_t* stage_t2 = lds + s2 * T::STAGE_ELEMS;      // K(t+2), landed during this step at the latest
        float msc[2], rsum0[2] = {0.f, 0.f}, rsum1[2] = {0.f, 0.f};
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) msc[qb] = ((m_run[qb] == -INFINITY) ? 0.f : m_run[qb]) * c_log2;
        u32x4 pw[2][4];                 // P^T operands: [query block][16-key chunk]
        // exponential of logit idx (in (kb, r) order) of query block qb
        auto exp_elem = [&](int qb, int idx) {
            const int kb = idx >> 4, r = idx & 15;
            cur[qb][kb][r] = exp2_fast(fmaf(cur[qb][kb][r], c_log2, -msc[qb]));
        };
        // Sums and packs a pair one slot after its exponentials, so that nothing waits on the transcendental
        // unit.  (The row sum is taken over the unrounded values: summing the packed pair with one
        // v_dot2_f32_bf16 would save an instruction per pair, but moves the logsumexp of a row that one key
        // dominates by up to 2^-9.)
        auto pack_pair = [&](int qb, int j) {
            const int idx = 2 * j, kb = idx >> 4, r = idx & 15;
            rsum0[qb] += cur[qb][kb][r];
            rsum1[qb] += cur[qb][kb][r + 1];
            pw[qb][idx >> 3][(idx & 7) >> 1] = pack_bf16(cur[qb][kb][r], cur[qb][kb][r + 1]);
        };

        {
            constexpr int NSL = 2 * NKF;             // MFMA slots of the logit phase
            static_assert(NSL == 32 || NSL == 16, "slicing");
            // copies of K(t+3) and V(t+2); copy j goes with slot CS*j + 1
            constexpr int NCOPY = 2 * NDMA, CS = (NSL - 2) / NCOPY;
            // exponentials per slot and query block: the first key block's in the logit phase, the second's
            // in the first half of the other phase, whose slots have the vector unit to spare
            constexpr int E1 = 16 / NKF, E2 = 32 / NVF;
            static_assert(E1 >= 1 && E2 >= 2 && E2 % 2 == 0, "slicing");
            static_assert(CS >= 2, "copies do not fit the logit phase");
            auto copy_dst = [&](int g) {
                const int j = (g - 1) / CS;
                if (g >= 1 && (g - 1) % CS == 0 && j < NCOPY) dma_set_dst(dst_of(j < NDMA ? s3 : s2, j / NDMA, j % NDMA));
            };
            auto copy_issue = [&](int g) {
                const int j = (g - 1) / CS;
                if (g >= 1 && (g - 1) % CS == 0 && j < NCOPY) {
                    if (j < NDMA) dma16u_issue(k3_base, k_lane_off[j]);
                    else dma16u_issue(v2_base, v_lane_off[j - NDMA]);
                }
            };
            // ---- S(t+1)^T = K(t+1) Q^T between the exponentials of tile t
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
                    mfma32_vgpr_bpinned<qb * DC + (i >> 1), (i >> 1) == 0 ? 0 : 1>(nxt[qb][i & 1], fb[i % PD], qf[qb][i >> 1], nxt[qb][i & 1]);
                    __builtin_amdgcn_sched_barrier(0);
                    copy_issue(g);
                    // slot g: exponentials of E1 logits of the first key block of query block qb, packing of
                    // the pairs that were complete a slot ago
#pragma unroll
                    for (int e = 0; e < E1; ++e) exp_elem(qb, E1 * i + e);
                    if (i > 0) {
#pragma unroll
                        for (int j = E1 * (i - 1) / 2; j < E1 * i / 2; ++j) pack_pair(qb, j);
                    }
                    // the ring is refilled two fragments at a time, so that one wait covers both
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
            // ---- O^T += V(t)^T P(t)^T, with the rest of the exponentials and the row-maximum scan of tile t+1
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
                    oacc[qb][db] = mfma32(fb[i % PD], __builtin_bit_cast(bf16x8, pw[qb][cc]), oacc[qb][db]);
                    __builtin_amdgcn_sched_barrier(0);
                    if (i < NVF / 2) {
                        // first half: the exponentials of the second key block, due at slot NVF / 2
#pragma unroll
                        for (int e = 0; e < E2; ++e) exp_elem(qb, 16 + E2 * i + e);
                    }
                    if (i >= 1 && i <= NVF / 2) {
#pragma unroll
                        for (int j = 8 + E2 * (i - 1) / 2; j < 8 + E2 * i / 2; ++j) pack_pair(qb, j);
                    }
                    if (i >= NVF / 2) {
                        // second half: row maximum of tile t+1 (its logits may be touched from slot 2 on)
                        constexpr int MPS = 64 / NVF;     // logits per slot and block
                        constexpr int k = i - NVF / 2;
                        if (k == 0) tmax[qb] = nxt[qb][0][0];
#pragma unroll
                        for (int e = 0; e < MPS; ++e) {
                            const int idx = MPS * k + e;
                            tmax[qb] = fmaxf(tmax[qb], nxt[qb][idx >> 4][idx & 15]);
                        }
                        // the scan feeds nothing before the end of the step: keep this slot's part in this slot
                        asm volatile("" : "+v"(tmax[qb]));
                    }
                    if (qb == 1) {
                        if (i == NVF - PD) {
                            __builtin_amdgcn_sched_barrier(0);
                            // the copies of the step before (K(t+2), V(t+1)) have landed; this step's may be in flight ...
                            __builtin_amdgcn_s_waitcnt(0x0F70 | ((2 * NDMA) & 15) | (((2 * NDMA) >> 4) << 14));
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
            // Both lanes of a query hold the same reference maximum, so each may test its own half; the
            // exchange between the halves and the rescale stay inside the rarely taken branch.
            if (__any(tmax[0] > m_run[0] + stale_ok || tmax[1] > m_run[1] + stale_ok)) {
                fold_max(std::integral_constant<int, 0>{}, tmax[0]);
                fold_max(std::integral_constant<int, 1>{}, tmax[1]);
            }
        }
    };

    f32x16 sa[2][2], sb[2][2];
    if (n_tiles > 0) {
        // prologue: K(0..2) and V(0..1) land; logits and maximum of tile 0; the ring starts on K(1)
        issue_whole(kbase, p.ks.n, k_lane_off, 0, 0);
        issue_whole(kbase, p.ks.n, k_lane_off, 1, 0);
        issue_whole(kbase, p.ks.n, k_lane_off, 2, 0);
        issue_whole(vbase, p.vs.n, v_lane_off, 0, 1);
        issue_whole(vbase, p.vs.n, v_lane_off, 1, 1);
        wait_vm0();
        __syncthreads();
        logits_plain(sa, lds);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) first_max(qb, tile_max(sa[qb]));
#pragma unroll
        for (int i = 0; i < PD; ++i) fb[i] = k_frag(lds + T::STAGE_ELEMS, i);

        const int64_t k_tile_stride = (int64_t)BN * p.ks.n, v_tile_stride = (int64_t)BN * p.vs.n;
        using I0 = std::integral_constant<int, 0>;
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        using I3 = std::integral_constant<int, 3>;
        // Tile t sits in stage t % 4 and its logits in `sa` when t is even: four step bodies.
        // K(t+3) and V(t+2) of the step at hand; copies past the last tile re-read the last tile
        const uint16_t* k3 = kbase + (int64_t)min(3, n_tiles - 1) * k_tile_stride;
        const uint16_t* v2 = vbase + (int64_t)min(2, n_tiles - 1) * v_tile_stride;
        auto advance = [&](int t) {    // from step t to step t+1
            k3 += (t + 4 < n_tiles) ? k_tile_stride : 0;
            v2 += (t + 3 < n_tiles) ? v_tile_stride : 0;
        };
        for (int t = 0; t < n_tiles; t += 4) {
            step(I0{}, sa, sb, k3, v2);
            if (t + 1 >= n_tiles) break;
            advance(t);
            step(I1{}, sb, sa, k3, v2);
            if (t + 2 >= n_tiles) break;
            advance(t + 1);
            step(I2{}, sa, sb, k3, v2);
            if (t + 3 >= n_tiles) break;
            advance(t + 2);
            step(I3{}, sb, sa, k3, v2);
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
                    if (32 * db + 8 * g + 4 * h < p.dv) *reinterpret_cast<u32x2*>(orow + 32 * db + 8 * g + 4 * h) = w;
                }
            if (p.lse && h == 0) {
                const float v = l > 0.f ? (m_run[qb] * c_log2 + log2_fast(l)) * kLn2 : -INFINITY;
                p.lse[(int64_t)bh * p.Sq + row] = v;
            }
        }
    }
}

}  // namespace fattn
