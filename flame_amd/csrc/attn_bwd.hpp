// Backward of the tiled attention for gfx950: recomputes P tile by tile from Q, K and the saved
// log-sum-exp, never materialising the Sq x Sk matrix.
//
//   dq       one workgroup owns 128 queries (32 per wavefront, two wavefronts per SIMD) or, when the
//            problem fills them, 256 queries (64 per wavefront, one wavefront per SIMD), and walks over
//            the key tiles (64 keys), with the logits transposed (lane = query): S^T = K Q^T, dP^T = V dO^T,
//            dS^T = P^T (dP^T - delta) and dQ^T += K^T dS^T accumulated in fp32 registers for the whole
//            walk, dS^T going into the last MFMA straight from the accumulators.  Runs first and also
//            leaves -delta_i = -sum_d dO_id * O_id and LSE_i * log2(e) (fp32, one value per query row)
//            in the workspace for the next kernel.
//   dkdv     one workgroup owns 128 keys (32 per wavefront) of one (batch, head) and walks over the
//            query tiles (64 rows): S = Q K^T, dP = dO V^T, P = exp2(S*c - LSE*log2e),
//            dS = P * (dP - delta); dV^T += dO^T P and dK^T += Q^T dS stay in fp32 registers for the
//            whole walk (P and dS are used as MFMA operands straight from the accumulators), and so do
//            the wavefront's K and V fragments (in the accumulation registers).  When the
//            key blocks do not fill the last scheduling round, the blocks of that round are split
//            along the walk and their fp32 partial sums are combined by the merge kernel.
// Accumulating dQ from the dkdv walk with fp32 atomics was measured at about one lane-atomic per
// clock per CU, more than the whole MFMA time of the backward; recomputing S and dP in a second,
// query-major kernel costs 2 extra GEMMs out of 7 and no atomics, no fp32 scratch and no convert pass.
//
// Tiles are copied global -> LDS by asynchronous LDS-DMA loads (two stages where two wavefronts share a
// SIMD, three where one wavefront runs alone and nobody would cover a drained pipeline), row-major with an XOR swizzle of the 16-byte granules; their
// transposed MFMA operands (Q^T, dO^T) and the dS operand come from transposing LDS reads, so no tile
// is stored twice and no access pattern has bank conflicts.  One workgroup barrier per step.
#pragma once
#include <type_traits>

#include "attn_common.hpp"

namespace fattn {

struct BwdParams {
    // dK/dV grid: workgroups [0, n_whole) walk every query tile of one key block; the remaining key
    // blocks are served by split_parts workgroups each, every one walking a slice of the query tiles
    // and leaving fp32 partial sums in split_ws for bwd_dkdv_merge_kernel.  n_whole < 0: no splitting.
    int n_whole = -1;
    int split_parts = 1;
    int rows_ready = 0;            // -delta and lse2 are in the workspace already (bwd_rows_kernel ran): read, do not form
    int joint_n_dq = 0;            // bwd_joint_kernel: the first joint_n_dq workgroups are dQ workgroups
    float* split_ws = nullptr;
    size_t split_ws_bytes = 0;     // host side only
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    const uint16_t* o;
    const uint16_t* dout;
    const float* lse;     // contiguous [B*H, Sq]
    uint16_t* dq;
    uint16_t* dk;
    uint16_t* dv;
    float* ndelta;        // workspace, [B*H, Sq]: -rowsum(dO * O)
    float* lse2;          // workspace, [B*H, Sq]: LSE * log2(e), +inf where LSE = -inf
    Strides qs, ks, vs, os, dos, dqs, dks, dvs;
    int B, H, Sq, Sk;
    int d;                // real head dim: a multiple of 8, at most the compiled D
    float scale;
    MaskArgs m;
    unsigned long long* phase_cycles;   // profiling aid: per-phase cycle sums of wave 0 of every workgroup, or null
};

// ------------------------------------------------------------------------------------------ dkdv
template <int D>
struct BwdTile {
    static constexpr int BM = 64;                   // query rows per step
    static constexpr int BN = 128;                  // keys per workgroup
    static constexpr int RS = D;                    // LDS row stride of the Q / dO / K / V tiles (swizzled, unpadded)
    static constexpr int Q_ELEMS = BM * RS;
    static constexpr int STAGE_ELEMS = 2 * Q_ELEMS;               // Q tile + dO tile (also one 128-row tile)
    static constexpr int ROW_FLOATS = 2 * BM;                     // lse2 and -delta of one step
    static constexpr int NSTAGE = 3;
    // [3 stages of Q,dO][3 x (lse2, -delta)]
    static constexpr int LDS_BYTES = NSTAGE * STAGE_ELEMS * 2 + NSTAGE * ROW_FLOATS * 4;
    // with a keep-mask staged through LDS: [3 x (64 queries x 128 keys) mask bytes] behind the rest
    static constexpr int MASK_STAGE_BYTES = BM * BN;
    static constexpr int LDS_BYTES_VECMASK = LDS_BYTES + NSTAGE * MASK_STAGE_BYTES;
    static constexpr int ROWS_PER_DMA = 1024 / (D * 2);
    static constexpr int DMA_PER_WAVE = BM / ROWS_PER_DMA / 4;    // 1 KiB copies per wave and tensor
};

template <int D>
__device__ __forceinline__ void dkdv_store(const BwdParams& p, const f32x16 (&dkacc)[D / 32], const f32x16 (&dvacc)[D / 32],
                                           int b, int hh, int krow, int h);

// VECMASK (with HASMASK): the keep-mask rows are contiguous and 16-byte aligned, Sq is a multiple of 64, Sk
// of 128, and there is no causal flag.  The 64 x 128 mask bytes of a step then travel to LDS with the step's other copies (two more
// 1 KiB copies per wavefront) and every lane reads the bytes of its key a few elements ahead of use,
// instead of fetching 32 bytes from global memory into 32 registers at the start of every step; with the
// registers back, the walk runs the same straight-line steps as the unmasked one.
// DROPOUT: dV takes the dropped and rescaled probabilities, dP = f (dO V^T) with the same factor f (drop_factor), and
// -delta is added per element instead of seeding the dP accumulators.
// block / nblocks: this workgroup's index in the dK/dV grid and the size of that grid (the kernel's own launch, or
// the dK/dV part of bwd_joint_kernel's).
template <int D, bool HASMASK, bool TIMING, bool VECMASK = false, bool DROPOUT = false>
__device__ __forceinline__ void bwd_dkdv_body(const BwdParams& p, const int block, const int nblocks) {
    static_assert(!VECMASK || HASMASK, "VECMASK is a special case of HASMASK");
    using T = BwdTile<D>;
    constexpr int BM = T::BM, BN = T::BN, RS = T::RS;
    constexpr int DC = D / 16;     // contraction chunks over the head dim
    constexpr int DB = D / 32;     // 32-row blocks of dK^T / dV^T
    constexpr int GPR = D / 8;     // 16-byte granules per row
    constexpr int RPD = T::ROWS_PER_DMA, NDQ = T::DMA_PER_WAVE;

    extern __shared__ __attribute__((aligned(1024))) uint16_t lds[];
    uint16_t* stage0 = lds;                                        // [3][Q tile | dO tile]
    float* rows0 = reinterpret_cast<float*>(lds + T::NSTAGE * T::STAGE_ELEMS);   // [3][lse2 | -delta]
    const uint8_t* mask0 = reinterpret_cast<const uint8_t*>(lds) + T::LDS_BYTES;  // [3][64 x 128] mask bytes (VECMASK)

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;

    const int n_kt = (p.Sk + BN - 1) / BN;
    int wg, part = 0, nparts = 1;
    if (p.n_whole < 0) {
        wg = p.m.kv_len ? xcd_remap_heads(block, nblocks, n_kt) : xcd_remap(block, nblocks);
    } else if (block < p.n_whole) {
        wg = xcd_remap(block, p.n_whole);
    } else {          // the split key blocks come last in dispatch order and fill the final, partial round
        const int e = block - p.n_whole;
        nparts = p.split_parts;
        wg = p.n_whole + e / nparts;
        part = e % nparts;
    }
    const int kt = wg % n_kt;
    const int bh = wg / n_kt;
    const int b = bh / p.H, hh = bh % p.H;
    const int k0 = kt * BN;
    const int kw0 = k0 + 32 * wave;

    const uint16_t* qbase = p.q + b * p.qs.b + hh * p.qs.h;
    const uint16_t* kbase = p.k + b * p.ks.b + hh * p.ks.h;
    const uint16_t* vbase = p.v + b * p.vs.b + hh * p.vs.h;
    const uint16_t* dobase = p.dout + b * p.dos.b + hh * p.dos.h;
    const float* lsebase = p.lse2 + (int64_t)bh * p.Sq;
    const float* ndeltabase = p.ndelta + (int64_t)bh * p.Sq;

    int klimit = p.Sk;
    if (p.m.kv_len) klimit = min(klimit, max(p.m.kv_len[b], 0));
    const uint8_t* mbase = HASMASK ? mask_head_base(p.m, b, hh) : nullptr;

    const int n_qt = (p.Sq + BM - 1) / BM;
    int qt_begin = p.m.causal ? (k0 / BM) : 0;
    if (k0 >= klimit || (p.m.causal && k0 >= p.Sq)) {
        // Nothing attends to these keys (past the key length, or past the last query under the causal flag):
        // dK = dV = 0, written at once.  Padded batches launch many such workgroups; they must not cost a
        // prologue each.
        f32x16 zero[D / 32];
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) zero[db][r] = 0.f;
        dkdv_store<D>(p, zero, zero, b, hh, kw0 + n, h);
        return;
    }
    const int n_it = n_qt - qt_begin;
    // The walk visits the query tiles that need per-element exclusions first (all of them when an explicit
    // mask is given, else the causal diagonal tiles and a partial last tile) and the fully attended ones afterwards, so that each of the two loops runs one
    // specialised, branch-free body.  The order of the tiles does not matter to the sums.
    // (A key block that the key length cuts needs none: a lane owns one key, its column of dK^T / dV^T
    // depends on no other key's P or dS, and the columns of the keys past the length are zeroed before the store.)
    const bool all_masked = HASMASK;
    int lead_end = qt_begin;
    if (n_it > 0) {
        if (all_masked) lead_end = n_qt;
        else if (p.m.causal) lead_end = max(qt_begin, min(n_qt, (k0 + BN - 2) / BM + 1));
    }
    const int n_lead = lead_end - qt_begin;
    const int tail_extra = (n_it > 0 && !all_masked && (p.Sq % BM) != 0 && lead_end < n_qt) ? 1 : 0;
    const int n_masked = n_lead + tail_extra;
    auto tile_of = [&](int it) {
        if (it < n_lead) return qt_begin + it;
        if (it < n_masked) return n_qt - 1;
        return lead_end + (it - n_masked);
    };
    // ---- per-lane LDS offsets (elements), constant over the walk
    int roff[DC];          // 16-byte row reads: row (32*blk + n), logical granule 2*dc + h
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) roff[dc] = n * RS + (((2 * dc + h) ^ swz<D>(n)) << 3);
    const int tr_r = lane & 15, tr_g16 = (lane >> 4) & 1;
    int toff[2][DB];       // transposing reads of a D-wide tile: rows 4h + r/4 (+8), granule 4*db + 2*g16 + (r&3)/2
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int row = 4 * h + (tr_r >> 2) + 8 * half;
#pragma unroll
        for (int db = 0; db < DB; ++db)
            toff[half][db] = row * RS + (((4 * db + 2 * tr_g16 + ((tr_r & 3) >> 1)) ^ swz<D>(row)) << 3) + 4 * (tr_r & 1);
    }
    auto tr_frag = [&](const uint16_t* tile, int o0, int o1) {
        const u32x2 lo = lds_read_tr16(tile + o0);
        const u32x2 hi = lds_read_tr16(tile + o1);
        const u32x4 u = {lo[0], lo[1], hi[0], hi[1]};
        return __builtin_bit_cast(bf16x8, u);
    };

    const int dma_row_in = lane / GPR, dma_gran = lane % GPR;
    const uint32_t lds0 = lds_addr(lds);
    const uint32_t rows_lds0 = lds0 + 2u * T::NSTAGE * T::STAGE_ELEMS;   // byte address of rows0

    // ---- prologue: the K and V fragments of this wavefront's 32 keys are held in registers for the whole walk
    bf16x8 kf[DC], vf[DC];
    {
        constexpr int NDMA = BN / RPD / 4;     // 1 KiB copies per wave for a 128-row tile
#pragma unroll
        for (int i = 0; i < NDMA; ++i) {
            const int ji = wave * NDMA + i;
            const int row = ji * RPD + dma_row_in;
            const int key = max(min(k0 + row, klimit - 1), 0);   // rows past the attended range re-read a valid row
            const int c = src_granule(dma_gran ^ swz<D>(row), p.d);
            dma16(kbase + (int64_t)key * p.ks.n + c * 8, lds0 + 2u * (T::STAGE_ELEMS + ji * 512));
            dma16(vbase + (int64_t)key * p.vs.n + c * 8, lds0 + 2u * (ji * 512));
        }
        wait_vm0();
        __syncthreads();
        if (p.d < D) {      // padded head dim: S and dP must not see the copies' filler, so it is zeroed in LDS
            const u32x4 z = {0u, 0u, 0u, 0u};
            for (int idx = tid; idx < BN * GPR; idx += 256) {
                const int row = idx / GPR, gl = idx % GPR;
                if (gl * 8 >= p.d) {
                    const int off = row * RS + ((gl ^ swz<D>(row)) << 3);
                    *reinterpret_cast<u32x4*>(stage0 + off) = z;
                    *reinterpret_cast<u32x4*>(stage0 + T::STAGE_ELEMS + off) = z;
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
            kf[dc] = *reinterpret_cast<const bf16x8*>(stage0 + T::STAGE_ELEMS + roff[dc] + 32 * wave * RS);
            vf[dc] = *reinterpret_cast<const bf16x8*>(stage0 + roff[dc] + 32 * wave * RS);
        }
        __syncthreads();
    }

    // ---- asynchronous staging of the 64-row Q / dO tiles and their lse2 / -delta rows, three stages.
    //      Address = uniform tile base + a per-lane 32-bit offset that never changes.
    uint32_t q_lane_off[NDQ], do_lane_off[NDQ];     // bytes
#pragma unroll
    for (int i = 0; i < NDQ; ++i) {
        const int row = (wave * NDQ + i) * RPD + dma_row_in;
        const int c = src_granule(dma_gran ^ swz<D>(row), p.d);
        q_lane_off[i] = 2u * (uint32_t)(row * (int)p.qs.n + c * 8);
        do_lane_off[i] = 2u * (uint32_t)(row * (int)p.dos.n + c * 8);
    }
    auto q_dst = [&](int stg, int which, int i) {    // LDS byte address of copy i of this wave (which: 0 = Q, 1 = dO)
        return lds0 + 2u * (uint32_t)(stg * T::STAGE_ELEMS + which * T::Q_ELEMS + (wave * NDQ + i) * 512);
    };
    auto rows_dst = [&](int stg) { return rows_lds0 + 4u * (uint32_t)(stg * T::ROW_FLOATS + wave * BM); };
    // keep-mask tile of a step: 8 copies of 8 rows x 128 bytes, two per wavefront
    uint32_t m_lane_off[2] = {0u, 0u};
    if (VECMASK) {
#pragma unroll
        for (int jm = 0; jm < 2; ++jm)
            m_lane_off[jm] = (uint32_t)(((wave * 2 + jm) * 8 + (lane >> 3)) * (int)p.m.sq + 16 * (lane & 7));
    }
    auto mask_dst = [&](int stg, int jm) {
        return lds0 + (uint32_t)(T::LDS_BYTES + stg * T::MASK_STAGE_BYTES + (wave * 2 + jm) * 1024);
    };
    auto mask_tile = [&](int qt) { return mbase + (int64_t)qt * BM * p.m.sq + k0; };
    auto issue_q_tile = [&](int qt, int stg) {
        const int q0 = qt * BM;
        if (q0 + BM <= p.Sq) {
            const uint16_t* qt_base = qbase + (int64_t)q0 * p.qs.n;
            const uint16_t* dot_base = dobase + (int64_t)q0 * p.dos.n;
#pragma unroll
            for (int i = 0; i < NDQ; ++i) {
                dma16u(qt_base, q_lane_off[i], q_dst(stg, 0, i));
                dma16u(dot_base, do_lane_off[i], q_dst(stg, 1, i));
            }
            if (wave < 2) dma4((wave == 0 ? lsebase : ndeltabase) + q0 + lane, rows_dst(stg));
            if (VECMASK) {
#pragma unroll
                for (int jm = 0; jm < 2; ++jm) dma16u(mask_tile(qt), m_lane_off[jm], mask_dst(stg, jm));
            }
        } else {   // last, partial tile: rows past the end re-read the last valid row
#pragma unroll
            for (int i = 0; i < NDQ; ++i) {
                const int ji = wave * NDQ + i;
                const int row = ji * RPD + dma_row_in;
                const int qi = min(q0 + row, p.Sq - 1);
                const int c = src_granule(dma_gran ^ swz<D>(row), p.d);
                dma16(qbase + (int64_t)qi * p.qs.n + c * 8, q_dst(stg, 0, i));
                dma16(dobase + (int64_t)qi * p.dos.n + c * 8, q_dst(stg, 1, i));
            }
            if (wave < 2) {
                const int qi = min(q0 + lane, p.Sq - 1);
                dma4((wave == 0 ? lsebase : ndeltabase) + qi, rows_dst(stg));
            }
        }
    };

    f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            dkacc[db][r] = 0.f;
            dvacc[db][r] = 0.f;
        }

    const float c_log2 = p.scale * kLog2e;
    const int key = kw0 + n;
    // VECMASK: a mask byte excludes its element when it is <= this: 0 for an attended key, 255 for one past the key length
    const uint32_t dead_thr = key >= klimit ? 0xffu : 0u;

    unsigned long long ph[6] = {0, 0, 0, 0, 0, 0};
    unsigned long long tprev = TIMING ? __builtin_readcyclecounter() : 0ull;
    const unsigned long long wall0 = TIMING ? wall_clock64() : 0ull;
#define FATTN_PHASE(i)                                                  \
    if (TIMING) {                                                       \
        const unsigned long long tnow = __builtin_readcyclecounter();   \
        ph[i] += tnow - tprev;                                          \
        tprev = tnow;                                                   \
    }

    // One step of the walk handles one 64-query tile as two 32-query blocks in four phases of NS MFMAs:
    //   A0: S,dP(block 0)          | issue of the next tile's copies
    //   A1: S,dP(block 1)          | P,dS(block 0)
    //   B0: dV,dK += (block 0)     | P,dS(block 1)
    //   B1: dV,dK += (block 1)
    // written as an explicit software pipeline for a single wavefront per SIMD: the MFMA pipe and the
    // vector ALU run side by side only when their instructions alternate in the instruction stream, so
    // the per-element arithmetic of one block is threaded between the MFMAs of its neighbour, one
    // accumulator register per MFMA.  The G = 4 NS operand fragments of a step come from LDS through one
    // ring of PD registers that runs PD fragments ahead of the MFMAs, across the phases and on into the
    // next step; the scheduling barriers keep the compiler from undoing either interleave.
    //
    // Three LDS stages, one workgroup barrier per step, placed just before the ring first reads the next
    // stage: by then every wave's copies of the next tile have landed, and every wave has finished the
    // previous step, whose stage the next step's copies overwrite.  No wave ever drains its pipeline.
    //
    // dP accumulates on top of -delta (loaded from LDS straight into the accumulator registers), so
    // dS = P * dP' needs no subtraction.
    constexpr int NS = 2 * DC;      // MFMAs per phase
    constexpr int G = 4 * NS;       // MFMAs = operand fragments per step
    constexpr int PD = 4;           // read-ahead depth of the fragment ring
    static_assert(2 * DC == 4 * DB, "all phases must have the same number of MFMA slots");
    constexpr int NCOPY = 2 * NDQ + 1 + (VECMASK ? 2 : 0);     // copies per wavefront and step: Q, dO, a row, mask
    static_assert(NS % PD == 0 && 4 * (NCOPY - 1) + 1 < G - PD, "ring depth / copy slices do not fit");
    f32x16 dpacc[2];
    bf16x8 fb[PD];
    // fragment g of a step: [0, 2 NS) 16-byte row reads (block, dc, Q | dO); [2 NS, 4 NS) transposing
    // reads (block, 16-query chunk, db, dO^T | Q^T)
    auto frag = [&](const uint16_t* Qs, int g) {
        const uint16_t* dOs = Qs + T::Q_ELEMS;
        const int qb = (g / NS) & 1, i = g % NS;
        if (g < 2 * NS) {
            const int dc = i >> 1;
            return *reinterpret_cast<const bf16x8*>(((i & 1) ? dOs : Qs) + roff[dc] + 32 * qb * RS);
        }
        const int c = i / (2 * DB), db = (i >> 1) % DB, cc = 2 * qb + c;
        return tr_frag((i & 1) ? Qs : dOs, toff[0][db] + 16 * cc * RS, toff[1][db] + 16 * cc * RS);
    };
    // -delta of queries 8*g4 + 4h .. +3 of block qb -> the dP accumulator registers of those rows
    auto ndelta_rows = [&](const float* rows, int qb, int g4) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(rows + BM + 32 * qb + 8 * g4 + 4 * h);
#pragma unroll
        for (int t = 0; t < 4; ++t) dpacc[qb][4 * g4 + t] = DROPOUT ? 0.f : v[t];
    };

    // this workgroup's slice [it_lo, it_hi) of the walk
    const int it_lo = (int)((int64_t)part * n_it / nparts);
    const int it_hi = (int)((int64_t)(part + 1) * n_it / nparts);
    // The stages are numbered so that the steps which need exclusions (they come first and take their
    // stage from a run-time counter) leave the counter at 0 for the main loop, whose three unrolled
    // steps have their stages fixed at compile time.
    const int n_masked_here = max(min(n_masked, it_hi) - it_lo, 0);
    // (VECMASK: every step needs exclusions and the straight-line loop comes first, so it starts in stage 0)
    int st = VECMASK ? 0 : (3 - n_masked_here % 3) % 3;        // LDS stage of the step about to run
    if (it_hi > it_lo) {
        issue_q_tile(tile_of(it_lo), st);
        wait_vm0();
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PD; ++i) fb[i] = frag(stage0 + st * T::STAGE_ELEMS, i);
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) ndelta_rows(rows0 + st * T::ROW_FLOATS, 0, g4);
    }

    // COPY: 0 = this is the last step, 1 = the next tile is a full one (straight-line copies),
    //       2 = decide at run time (used by the few steps that need exclusions)
    // STAGE: LDS stage that holds this step's tile (0 / 1 / 2), or -1 to take it from `st`.
    auto step = [&](auto masked_tag, auto copy_tag, auto stage_tag, int st, int it, int qt, int qt_next,
                    const uint16_t* nq_base, const uint16_t* ndo_base, const float* nrow_base) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        constexpr int COPY = decltype(copy_tag)::value;
        constexpr int STAGE = decltype(stage_tag)::value;
        const int cur = STAGE >= 0 ? STAGE : st;
        const int nxt = STAGE >= 0 ? (STAGE + 1) % 3 : (st == 2 ? 0 : st + 1);
        const int q0 = qt * BM;
        const bool have_next = COPY == 1 || (COPY == 2 && it + 1 < it_hi);

        const uint16_t* Qs = stage0 + cur * T::STAGE_ELEMS;
        const uint16_t* Qn = stage0 + nxt * T::STAGE_ELEMS;
        const float* rows_c = rows0 + cur * T::ROW_FLOATS;      // [lse2 | -delta] of this step's queries
        const float* rows_n = rows0 + nxt * T::ROW_FLOATS;

        f32x16 sacc[2];
        bf16x8 pf[2][2], dsf[2][2];
        f32x4 l4, l4n;
        // keep-mask bytes of this lane's key for the 64 queries of the tile, fetched up front in one batch
        // (a load per element inside the pipelined slices would wait out a memory round trip each time)
        uint32_t mk[2][16];
        if (HASMASK && !VECMASK && MASKED) {
            const int64_t mkey = (int64_t)min(key, p.Sk - 1) * p.m.sk;
#pragma unroll
            for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int qi = q0 + 32 * qb + 8 * (r >> 2) + 4 * h + (r & 3);
                    mk[qb][r] = mask_attends(p.m, mbase, mkey + (int64_t)min(qi, p.Sq - 1) * p.m.sq) ? 1u : 0u;
                }
        }
        // lse2 is read one group of four queries ahead of its use, so that waiting for it never drains
        // the fragment reads that were issued in between
        // (VECMASK: and with it the four mask bytes of this lane's key for those queries)
        const uint8_t* mask_c = mask0 + cur * T::MASK_STAGE_BYTES + (4 * h) * BN + 32 * wave + n;
        const uint8_t* nm_base = VECMASK ? mask_tile(qt_next) : nullptr;
        uint32_t m4[4], m4n[4];
        f32x4 nd4, nd4n;                 // DROPOUT: -delta of the same four queries
        auto rows_ahead = [&](int qb, int g) {
            l4n = *reinterpret_cast<const f32x4*>(rows_c + 32 * qb + 8 * g + 4 * h);
            if (DROPOUT) nd4n = *reinterpret_cast<const f32x4*>(rows_c + BM + 32 * qb + 8 * g + 4 * h);
            if (VECMASK) {
#pragma unroll
                for (int t = 0; t < 4; ++t) m4n[t] = mask_c[(32 * qb + 8 * g + t) * BN];
            }
        };

        // element r of block qb: P = exp2(S*c - lse2), dS = P*(dP - delta); pack after 8 and 16.
        // The product for element r is issued with the exponential of element r + 1, so that no
        // instruction waits on the transcendental unit.
        auto ds_mul = [&](int qb, int r) {
            if (!DROPOUT) dpacc[qb][r] = sacc[qb][r] * dpacc[qb][r];       // DROPOUT: elem() has formed dS already
            if ((r & 7) == 7) {
                const int c = r >> 3, o8 = 8 * c;
                const f32x16& d = dpacc[qb];
                dsf[qb][c] = pack8(d[o8], d[o8 + 1], d[o8 + 2], d[o8 + 3], d[o8 + 4], d[o8 + 5], d[o8 + 6], d[o8 + 7]);
            }
        };
        auto elem = [&](int qb, int r) {
            const int g = r >> 2, t = r & 3;
            if (t == 0) {
                l4 = l4n;
                if (DROPOUT) nd4 = nd4n;
                if (VECMASK) {
#pragma unroll
                    for (int u = 0; u < 4; ++u) m4[u] = m4n[u];
                }
                if (g < 3) rows_ahead(qb, g + 1);
                else if (qb == 0) rows_ahead(1, 0);
            }
            float pr = exp2_fast(fmaf(sacc[qb][r], c_log2, -l4[t]));
            if (r > 0) ds_mul(qb, r - 1);
            if (MASKED) {
                const int qi = q0 + 32 * qb + 8 * g + 4 * h + t;
                bool drop;
                if constexpr (VECMASK) {
                    drop = m4[t] <= dead_thr;       // whole tiles, no causal flag: the mask byte decides, one compare
                } else {
                    // bitwise, not short-circuit: one select per element instead of a chain of branches
                    drop = (key >= klimit) | (qi >= p.Sq) | ((p.m.causal != 0) & (key > qi));
                    if (HASMASK) drop |= mk[qb][r] == 0;
                }
                pr = drop ? 0.f : pr;
            }
            if constexpr (DROPOUT) {
                const uint32_t qi = (uint32_t)(q0 + 32 * qb + 8 * g + 4 * h + t);
                const float f = drop_factor_at(p.m, (uint32_t)bh, qi, (uint32_t)key, (uint32_t)p.Sq, (uint32_t)p.Sk);
                dpacc[qb][r] = pr * fmaf(f, dpacc[qb][r], nd4[t]);       // dS = P (f dP - delta)
                pr *= f;                                                  // what multiplied V in the forward
            }
            sacc[qb][r] = pr;
            if ((r & 7) == 7) {
                const int c = r >> 3, o8 = 8 * c;
                const f32x16& s = sacc[qb];
                pf[qb][c] = pack8(s[o8], s[o8 + 1], s[o8 + 2], s[o8 + 3], s[o8 + 4], s[o8 + 5], s[o8 + 6], s[o8 + 7]);
            }
        };
        // slice s (of NS per block) of the element-wise work: one logit register for D = 128, two for D = 64;
        // slice NS is the last product
        auto elem_slot = [&](int qb, int s) {
            if (s == NS) ds_mul(qb, 15);
            else if (NS == 16) elem(qb, s);
            else { elem(qb, 2 * s); elem(qb, 2 * s + 1); }
        };

        // copies of the next tile, one instruction at a time (full tiles: uniform base + lane offset), each
        // in two halves around an MFMA: destination into M0, then the copy.  nq_base / ndo_base / nrow_base
        // are the wave-uniform addresses of the next tile's Q rows, dO rows and lse2 (even waves) or
        // -delta (odd waves) rows; waves 2 and 3 repeat the row copies of waves 0 and 1.
        const bool next_full = COPY == 1 || (qt_next * BM + BM) <= p.Sq;
        const bool copying = COPY == 1 || (COPY == 2 && have_next && next_full);
        auto copy_dst_of = [&](int j) {
            return j < 2 * NDQ ? q_dst(nxt, j & 1, j >> 1) : rows_lds0 + 4u * (uint32_t)(nxt * T::ROW_FLOATS + (wave & 1) * BM);
        };
        // Copy j goes with MFMA slot 4j + 1.  In straight-line steps, while that MFMA is a hand-emitted one
        // (phases A0 and A1), the copy is split around it.
        auto copy_dst = [&](int g) {
            const int j = g / 4;
            if (COPY == 1 && g % 4 == 1 && j <= 2 * NDQ && g < 2 * NS) dma_set_dst(copy_dst_of(j));
        };
        auto copy_issue = [&](int g) {
            const int j = g / 4;
            if (COPY == 0 || g % 4 != 1 || j >= NCOPY) return;
            if (COPY == 1 && g < 2 * NS) {
                if (j == 2 * NDQ) dma4u_issue(nrow_base, 4u * (uint32_t)lane);
                else if (j & 1) dma16u_issue(ndo_base, do_lane_off[j >> 1]);
                else dma16u_issue(nq_base, q_lane_off[j >> 1]);
            } else if (copying) {          // destination and copy in one piece
                if (j > 2 * NDQ) dma16u(nm_base, m_lane_off[j - 2 * NDQ - 1], mask_dst(nxt, j - 2 * NDQ - 1));
                else if (j == 2 * NDQ) dma4(nrow_base + lane, copy_dst_of(j));
                else if (j & 1) dma16u(ndo_base, do_lane_off[j >> 1], copy_dst_of(j));
                else dma16u(nq_base, q_lane_off[j >> 1], copy_dst_of(j));
            }
        };
        if (COPY == 2 && have_next && !next_full) issue_q_tile(qt_next, nxt);   // partial tile: slow path, all at once

        // The element-wise work of a block trails the hand-emitted MFMAs that produced its S and dP by
        // LAG MFMA slots (see mfma32_vgpr_bacc), so its last LAG slices run at the start of the phase after.
        constexpr int LAG = 2;
        auto side = [&](int g) {
            const int phase = g / NS, i = g % NS;
            copy_issue(g);
            if (phase == 0) {
                if (i >= NS - 4) ndelta_rows(rows_c, 1, i - (NS - 4));
                if (i == NS - 1) rows_ahead(0, 0);
            } else if (phase == 1) {
                if (i >= LAG) elem_slot(0, i - LAG);
            } else if (phase == 2) {
                if (i <= LAG) elem_slot(0, NS - LAG + i);
                if (i >= LAG) elem_slot(1, i - LAG);
            } else {
                if (i <= LAG) elem_slot(1, NS - LAG + i);
            }
        };
        auto refill = [&](int g) {
            const int ng = g + PD;
            if (ng < G) fb[g % PD] = frag(Qs, ng);
            else if (COPY == 1 || (COPY == 2 && have_next)) fb[g % PD] = frag(Qn, ng - G);
        };

        // fragments are consumed in pairs, the younger read first: one s_waitcnt serves two MFMAs
        auto run_phase = [&](auto phase_tag) {
            constexpr int PHASE = decltype(phase_tag)::value;
#pragma unroll
            for (int i = 0; i < NS; i += 2) {
                const int g = PHASE * NS + i;
                if constexpr (PHASE < 2) {      // S = Q K^T and dP = dO V^T - delta, rows = queries of block qb, columns = this wave's keys
                    const int qb = PHASE, dc = i >> 1;
                    // the dropout builds: the allocator splits the accumulators around the longer element arithmetic
                    // and moves parts of them back right before these statements
                    mfma32_vgpr_bacc<DROPOUT>(dpacc[qb], fb[(g + 1) % PD], vf[dc]);
                    side(g);
                    __builtin_amdgcn_sched_barrier(0);
                    copy_dst(g + 1);
                    if (i == 0) mfma32_vgpr_first_bacc<DROPOUT>(sacc[qb], fb[g % PD], kf[dc]);
                    else mfma32_vgpr_bacc<DROPOUT>(sacc[qb], fb[g % PD], kf[dc]);
                    side(g + 1);
                } else {              // dV^T += dO^T P, dK^T += Q^T dS: rows = d, columns = keys, contraction over queries
                    const int qb = PHASE - 2, c = i / (2 * DB), db = (i >> 1) % DB;
                    dkacc[db] = mfma32(fb[(g + 1) % PD], dsf[qb][c], dkacc[db]);
                    side(g);
                    __builtin_amdgcn_sched_barrier(0);
                    dvacc[db] = mfma32(fb[g % PD], pf[qb][c], dvacc[db]);
                    side(g + 1);
                }
                if (g == G - PD && COPY != 0) {
                    if (COPY == 1 || have_next) {
                        __builtin_amdgcn_sched_barrier(0);
                        FATTN_PHASE(3)
                        wait_vm0();                          // this wave's copies of the next tile have landed
                        __builtin_amdgcn_s_barrier();        // ... everyone's have, and everyone is past the previous step
                        FATTN_PHASE(4)
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int g4 = 0; g4 < 4; ++g4) ndelta_rows(rows_n, 0, g4);
                    }
                }
                refill(g);
                refill(g + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (PHASE < 3) { FATTN_PHASE(PHASE) }
        };
        run_phase(std::integral_constant<int, 0>{});
        run_phase(std::integral_constant<int, 1>{});
        run_phase(std::integral_constant<int, 2>{});
        run_phase(std::integral_constant<int, 3>{});
    };

    using IM = std::integral_constant<int, -1>;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    const int64_t q_tile_stride = (int64_t)BM * p.qs.n, do_tile_stride = (int64_t)BM * p.dos.n;
    const float* rowbase = (wave & 1) ? ndeltabase : lsebase;
    int it_m = it_lo;
    if constexpr (VECMASK) {
        // Every tile needs exclusions, all are whole and consecutive: the same three straight-line steps
        // with fixed stages as the unmasked loop below.
        int qt = qt_begin + it_m;
        const uint16_t* nq = qbase + (qt + 1) * q_tile_stride;
        const uint16_t* ndo = dobase + (qt + 1) * do_tile_stride;
        const float* nrow = rowbase + (qt + 1) * BM;
        for (; it_m + 3 <= it_hi - 1; it_m += 3, qt += 3) {
            step(std::true_type{}, I1{}, I0{}, 0, it_m, qt, qt + 1, nq, ndo, nrow);
            nq += q_tile_stride, ndo += do_tile_stride, nrow += BM;
            step(std::true_type{}, I1{}, I1{}, 1, it_m + 1, qt + 1, qt + 2, nq, ndo, nrow);
            nq += q_tile_stride, ndo += do_tile_stride, nrow += BM;
            step(std::true_type{}, I1{}, I2{}, 2, it_m + 2, qt + 2, qt + 3, nq, ndo, nrow);
            nq += q_tile_stride, ndo += do_tile_stride, nrow += BM;
        }
    }
    for (int it = it_m; it < n_masked_here + it_lo; ++it) {
        const int qn = it + 1 < it_hi ? tile_of(it + 1) : 0;
        step(std::true_type{}, I2{}, IM{}, st, it, tile_of(it), qn, qbase + qn * q_tile_stride, dobase + qn * do_tile_stride,
             rowbase + qn * BM);
        st = st == 2 ? 0 : st + 1;
    }
    // every tile after the first n_masked is a full, fully attended one, and they are consecutive;
    // the stage counter is 0 here
    {
        int it = max(n_masked, it_lo);
        int qt = lead_end + (it - n_masked);
        const uint16_t* nq = qbase + (qt + 1) * q_tile_stride;     // the tile after the current one
        const uint16_t* ndo = dobase + (qt + 1) * do_tile_stride;
        const float* nrow = rowbase + (qt + 1) * BM;
        auto advance = [&]() {
            nq += q_tile_stride;
            ndo += do_tile_stride;
            nrow += BM;
        };
        for (; it + 3 <= it_hi - 1; it += 3, qt += 3) {
            step(std::false_type{}, I1{}, I0{}, 0, it, qt, qt + 1, nq, ndo, nrow);
            advance();
            step(std::false_type{}, I1{}, I1{}, 1, it + 1, qt + 1, qt + 2, nq, ndo, nrow);
            advance();
            step(std::false_type{}, I1{}, I2{}, 2, it + 2, qt + 2, qt + 3, nq, ndo, nrow);
            advance();
        }
        for (; it < it_hi - 1; ++it, ++qt) {
            step(std::false_type{}, I1{}, IM{}, st, it, qt, qt + 1, nq, ndo, nrow);
            advance();
            st = st == 2 ? 0 : st + 1;
        }
        if (it < it_hi) step(std::false_type{}, I0{}, IM{}, st, it, qt, qt, nq, ndo, nrow);
    }

    if (TIMING && p.phase_cycles && tid == 0) {
        ph[5] = wall_clock64() - wall0;      // 100 MHz
#pragma unroll
        for (int i = 0; i < 6; ++i) p.phase_cycles[(size_t)block * 6 + i] = ph[i];
    }
#undef FATTN_PHASE

    // ---- epilogue
    if (nparts > 1) {
        // fp32 partial sums of this slice, in accumulator order: [tensor][thread][db][16]
        float* dst = p.split_ws + ((size_t)(wg - p.n_whole) * nparts + part) * (size_t)(2 * BN * D);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x16& a = dkacc[db];
                const f32x16& c = dvacc[db];
                const f32x4 wk = {a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
                const f32x4 wv = {c[4 * g], c[4 * g + 1], c[4 * g + 2], c[4 * g + 3]};
                *reinterpret_cast<f32x4*>(dst + ((size_t)tid * DB + db) * 16 + 4 * g) = wk;
                *reinterpret_cast<f32x4*>(dst + (size_t)BN * D + ((size_t)tid * DB + db) * 16 + 4 * g) = wv;
            }
        return;
    }
    if (key >= klimit) {          // nothing attends to this lane's key
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                dkacc[db][r] = 0.f;
                dvacc[db][r] = 0.f;
            }
    }
    dkdv_store<D>(p, dkacc, dvacc, b, hh, kw0 + n, h);
}

template <int D, bool HASMASK, bool TIMING, bool VECMASK = false, bool DROPOUT = false>
__global__ __launch_bounds__(256) void bwd_dkdv_kernel(const BwdParams p) {
    bwd_dkdv_body<D, HASMASK, TIMING, VECMASK, DROPOUT>(p, (int)blockIdx.x, (int)gridDim.x);
}

// dK^T / dV^T accumulators (rows = d, column = this lane's key) -> bf16 rows of dK (scaled) and dV
template <int D>
__device__ __forceinline__ void dkdv_store(const BwdParams& p, const f32x16 (&dkacc)[D / 32], const f32x16 (&dvacc)[D / 32],
                                           int b, int hh, int krow, int h) {
    constexpr int DB = D / 32;
    if (krow < p.Sk) {
        uint16_t* dkrow = p.dk + b * p.dks.b + hh * p.dks.h + (int64_t)krow * p.dks.n;
        uint16_t* dvrow = p.dv + b * p.dvs.b + hh * p.dvs.h + (int64_t)krow * p.dvs.n;
        const float s = p.scale;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x16& a = dkacc[db];
                const f32x16& c = dvacc[db];
                u32x2 wk = {pack_bf16(a[4 * g] * s, a[4 * g + 1] * s), pack_bf16(a[4 * g + 2] * s, a[4 * g + 3] * s)};
                u32x2 wv = {pack_bf16(c[4 * g], c[4 * g + 1]), pack_bf16(c[4 * g + 2], c[4 * g + 3])};
                if (32 * db + 8 * g + 4 * h < p.d) *reinterpret_cast<u32x2*>(dkrow + 32 * db + 8 * g + 4 * h) = wk;
                if (32 * db + 8 * g + 4 * h < p.d) *reinterpret_cast<u32x2*>(dvrow + 32 * db + 8 * g + 4 * h) = wv;
            }
    }
}

// Sums the fp32 partials that the split workgroups of one key block left behind and writes dK, dV.
// One workgroup per (split key block, 32-wide block of d); the thread layout mirrors the accumulators.
template <int D>
__global__ __launch_bounds__(256) void bwd_dkdv_merge_kernel(const BwdParams p) {
    constexpr int BN = BwdTile<D>::BN, DB = D / 32;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, h = lane >> 5;
    const int n_kt = (p.Sk + BN - 1) / BN;
    const int sb = (int)blockIdx.x / DB, db = (int)blockIdx.x % DB;
    const int wg = p.n_whole + sb;
    const int kt = wg % n_kt;
    const int bh = wg / n_kt;
    const int b = bh / p.H, hh = bh % p.H;
    f32x4 ak[4], av[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        ak[g] = f32x4{0.f, 0.f, 0.f, 0.f};
        av[g] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    for (int part = 0; part < p.split_parts; ++part) {
        const float* src = p.split_ws + ((size_t)sb * p.split_parts + part) * (size_t)(2 * BN * D) + ((size_t)tid * DB + db) * 16;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            ak[g] += *reinterpret_cast<const f32x4*>(src + 4 * g);
            av[g] += *reinterpret_cast<const f32x4*>(src + (size_t)BN * D + 4 * g);
        }
    }
    const int krow = kt * BN + 32 * wave + n;
    if (krow < p.Sk) {
        uint16_t* dkrow = p.dk + b * p.dks.b + hh * p.dks.h + (int64_t)krow * p.dks.n;
        uint16_t* dvrow = p.dv + b * p.dvs.b + hh * p.dvs.h + (int64_t)krow * p.dvs.n;
        const float s = p.scale;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 wk = {pack_bf16(ak[g][0] * s, ak[g][1] * s), pack_bf16(ak[g][2] * s, ak[g][3] * s)};
            u32x2 wv = {pack_bf16(av[g][0], av[g][1]), pack_bf16(av[g][2], av[g][3])};
            if (32 * db + 8 * g + 4 * h < p.d) *reinterpret_cast<u32x2*>(dkrow + 32 * db + 8 * g + 4 * h) = wk;
            if (32 * db + 8 * g + 4 * h < p.d) *reinterpret_cast<u32x2*>(dvrow + 32 * db + 8 * g + 4 * h) = wv;
        }
    }
}

// -------------------------------------------------------------------------------------------- dq
template <int D>
struct BwdDqTile {
    static constexpr int BM = 128;                  // query rows per workgroup (32 per wavefront)
    static constexpr int BN = 64;                   // keys per tile
    static constexpr int RS = D;
    static constexpr int TILE_ELEMS = BN * D;
    static constexpr int STAGE_ELEMS = 2 * TILE_ELEMS;            // K tile + V tile
    static constexpr int LDS_BYTES = 2 * STAGE_ELEMS * 2;
    static constexpr int ROWS_PER_DMA = 1024 / (D * 2);
    static constexpr int DMA_PER_WAVE = BN / ROWS_PER_DMA / 4;
};

// NW wavefronts of 32 queries each per workgroup, two per SIMD (the library instantiates NW = 4; problems
// that fill 256-query workgroups go to bwd_dq_wide_kernel below).
// VECMASK (with HASMASK): the keep-mask rows are contiguous and 16-byte aligned and Sk is a multiple of the
// tile, so the per-element mask loads are not compiled in and the kernel fits two workgroups per unit again.
template <int D, bool HASMASK, int NW, bool VECMASK = false, bool DROPOUT = false>
__global__ __launch_bounds__(64 * NW, (NW == 4 && (!HASMASK || VECMASK)) ? 2 : 1) void bwd_dq_kernel(const BwdParams p) {
    static_assert(!VECMASK || HASMASK, "VECMASK is a special case of HASMASK");
    using T = BwdDqTile<D>;
    constexpr int BM = 32 * NW, BN = T::BN, RS = T::RS;
    constexpr int DC = D / 16;
    constexpr int DB = D / 32;
    constexpr int GPR = D / 8;

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
    const uint16_t* dobase = p.dout + b * p.dos.b + hh * p.dos.h;

    int klimit = p.Sk;
    if (p.m.kv_len) klimit = min(klimit, max(p.m.kv_len[b], 0));
    int kend = klimit;
    if (p.m.causal) kend = min(kend, q0 + BM);
    const int n_tiles = (kend + BN - 1) / BN;
    const uint8_t* mbase = HASMASK ? mask_head_base(p.m, b, hh) : nullptr;

    // ---- Q and dO fragments (B operands: column = query, 8 consecutive d), per-query scalars
    const int qrow = qw0 + n;
    const bool qok = qrow < p.Sq;
    bf16x8 qf[DC], dof[DC];
    {
        const uint16_t* rq = qbase + (int64_t)qrow * p.qs.n + 8 * h;
        const uint16_t* rd = dobase + (int64_t)qrow * p.dos.n + 8 * h;
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
            const bool in_d = qok && 16 * dc + 8 * h < p.d;
            qf[dc] = __builtin_bit_cast(bf16x8, ldg16(rq + 16 * dc, in_d));
            dof[dc] = __builtin_bit_cast(bf16x8, ldg16(rd + 16 * dc, in_d));
        }
    }
    // Per-query scalars, formed here and also left in the workspace for the dK/dV kernel that runs next:
    //   delta = rowsum(dO * O)   (the bf16 O that the forward saved)
    //   lse2  = LSE * log2(e), +inf for fully excluded rows and rows past the end (P = exp2(s - inf) = 0)
    float lse2 = INFINITY, delta = 0.f;
    {
        const uint16_t* ro = p.o + b * p.os.b + hh * p.os.h + (int64_t)qrow * p.os.n + 8 * h;
        float part = 0.f;
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
            const u32x4 ov = ldg16(ro + 16 * dc, qok && 16 * dc + 8 * h < p.d);
            const u32x4 dv = __builtin_bit_cast(u32x4, dof[dc]);
#pragma unroll
            for (int i = 0; i < 4; ++i) part += bf16_lo(dv[i]) * bf16_lo(ov[i]) + bf16_hi(dv[i]) * bf16_hi(ov[i]);
        }
        part += xhalf(part);
        if (qok) {
            const float l = p.lse[(int64_t)bh * p.Sq + qrow];
            lse2 = (l == -INFINITY) ? INFINITY : l * kLog2e;
            delta = part;
            if (h == 0) {
                p.ndelta[(int64_t)bh * p.Sq + qrow] = -delta;
                p.lse2[(int64_t)bh * p.Sq + qrow] = lse2;
            }
        }
    }

    const int dma_row_in = lane / GPR, dma_gran = lane % GPR;
    constexpr int NDMA = T::DMA_PER_WAVE * 4 / NW;
    const uint32_t lds0 = lds_addr(lds);
    uint32_t k_lane_off[NDMA], v_lane_off[NDMA];     // bytes
#pragma unroll
    for (int i = 0; i < NDMA; ++i) {
        const int row = (wave * NDMA + i) * T::ROWS_PER_DMA + dma_row_in;
        const int c = src_granule(dma_gran ^ swz<D>(row), p.d);
        k_lane_off[i] = 2u * (uint32_t)(row * (int)p.ks.n + c * 8);
        v_lane_off[i] = 2u * (uint32_t)(row * (int)p.vs.n + c * 8);
    }
    auto dst_of = [&](int buf, int which, int i) {    // LDS byte address of copy i of this wave (which: 0 = K, 1 = V)
        return lds0 + 2u * (uint32_t)(buf * T::STAGE_ELEMS + which * T::TILE_ELEMS + (wave * NDMA + i) * 512);
    };
    auto issue_tile = [&](int t, int buf) {
#pragma unroll
        for (int i = 0; i < NDMA; ++i) {
            const int row = (wave * NDMA + i) * T::ROWS_PER_DMA + dma_row_in;
            const int key = min(t * BN + row, klimit - 1);   // tail rows re-read the last attended key
            const int c = src_granule(dma_gran ^ swz<D>(row), p.d);
            dma16(kbase + (int64_t)key * p.ks.n + c * 8, dst_of(buf, 0, i));
            dma16(vbase + (int64_t)key * p.vs.n + c * 8, dst_of(buf, 1, i));
        }
    };
    auto issue_full_tile = [&](int t, int buf) {
        const uint16_t* kt = kbase + (int64_t)t * BN * p.ks.n;
        const uint16_t* vt = vbase + (int64_t)t * BN * p.vs.n;
#pragma unroll
        for (int i = 0; i < NDMA; ++i) {
            dma16u(kt, k_lane_off[i], dst_of(buf, 0, i));
            dma16u(vt, v_lane_off[i], dst_of(buf, 1, i));
        }
    };

    int koff[DC];          // 16-byte row reads of K / V: row 32*kb + n, logical granule 2*dc + h
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) koff[dc] = n * RS + (((2 * dc + h) ^ swz<D>(n)) << 3);
    const int tr_r = lane & 15, tr_g16 = (lane >> 4) & 1;
    int toff[2][DB];       // transposing reads of K: rows 4h + r/4 (+8), logical granule 4*db + 2*g16 + (r&3)/2
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int row = 4 * h + (tr_r >> 2) + 8 * half;
#pragma unroll
        for (int db = 0; db < DB; ++db)
            toff[half][db] = row * RS + (((4 * db + 2 * tr_g16 + ((tr_r & 3) >> 1)) ^ swz<D>(row)) << 3) + 4 * (tr_r & 1);
    }

    const float c_log2 = p.scale * kLog2e;
    f32x16 dqacc[DB];      // dQ^T: rows = d, column = this lane's query
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dqacc[db][r] = 0.f;

    if (n_tiles > 0) issue_tile(0, 0);
    MaskRow64 mnext;          // keep-mask bytes of this lane's query row for the next tile (vector-load layouts only)
#pragma unroll
    for (int j = 0; j < 4; ++j) mnext.w[j] = u32x4{0u, 0u, 0u, 0u};
    if (HASMASK && !VECMASK && p.m.rows16 && n_tiles > 0 && BN <= p.Sk) mnext.load(mbase + (int64_t)min(qrow, p.Sq - 1) * p.m.sq);
    wait_vm0();
    __syncthreads();

    // One tile of 64 keys = two blocks of 32.  The phases of the two blocks are staggered so that the
    // element-wise work of one phase is threaded between the MFMAs of the next, two logits per MFMA:
    //   S(0) | dP(0) + P(0) | S(1) + dS(0) | dP(1) + P(1) | dQ(0) + dS(1) | dQ(1)
    // with one ring of LDS fragments, read PD ahead, running through all 48 operand fetches.
    // BUF: stage that holds this tile (0 / 1), or -1 to take it from the parity of t.
    auto tile_step = [&](auto masked_tag, auto copy_tag, auto buf_tag, int t) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        constexpr int COPY = decltype(copy_tag)::value;
        constexpr int BUF = decltype(buf_tag)::value;
        constexpr int PD = 4;
        static_assert(DC % PD == 0 && (2 * DB) % PD == 0, "read-ahead depth must divide the fragment counts");
        const int buf = BUF >= 0 ? BUF : (t & 1);
        if (COPY == 1) issue_full_tile(t + 1, buf ^ 1);
        else if (t + 1 < n_tiles) issue_tile(t + 1, buf ^ 1);
        const uint16_t* ks = lds + buf * T::STAGE_ELEMS;
        const uint16_t* vs = ks + T::TILE_ELEMS;
        const int key0 = t * BN;

        // operand fetch f of the tile, in consumption order
        constexpr int NROW = 4 * DC;                // row-read fragments: S(0), dP(0), S(1), dP(1)
        constexpr int NALL = NROW + 4 * DB;         // + the transposed K fragments of dQ(0), dQ(1)
        auto fetch = [&](int f) {
            if (f < NROW) {
                const int phase = f / DC, dc = f % DC;            // phase: 0 S(0), 1 dP(0), 2 S(1), 3 dP(1)
                return *reinterpret_cast<const bf16x8*>(((phase & 1) ? vs : ks) + koff[dc] + 32 * (phase >> 1) * RS);
            }
            const int g = f - NROW, cc = g / DB, db = g % DB;      // cc = 16-key chunk of the tile
            const u32x2 lo = lds_read_tr16(ks + toff[0][db] + 16 * cc * RS);
            const u32x2 hi = lds_read_tr16(ks + toff[1][db] + 16 * cc * RS);
            const u32x4 u = {lo[0], lo[1], hi[0], hi[1]};
            return __builtin_bit_cast(bf16x8, u);
        };
        bf16x8 fb[PD];
#pragma unroll
        for (int i = 0; i < PD; ++i) {
            fb[i] = fetch(i);
            __builtin_amdgcn_sched_barrier(0);
        }

        f32x16 sacc[2], dpacc[2];
        bf16x8 dsf[2][2];
        // a lane's 64 keep-mask bytes of the tile in four 16-byte loads where the layout allows it, fetched
        // one tile ahead
        const bool vec_mask = HASMASK && MASKED && p.m.rows16 && key0 + BN <= p.Sk;
        MaskRow64 mrow = mnext;
        if constexpr (VECMASK) {
            // two workgroups per unit: the other wavefront of the SIMD covers the load, and a second row in
            // registers would spill
            mrow.load(mbase + (int64_t)min(qrow, p.Sq - 1) * p.m.sq + key0);
            // the key length and the causal diagonal cut few tiles: there they are folded into the mask bytes,
            // so that the per-element test is the mask byte alone
            const int lim = (p.m.causal ? min(klimit, qrow + 1) : klimit) - key0;
            if (__any(lim < BN)) mrow.restrict_to(lim);
        } else if (HASMASK && MASKED && p.m.rows16 && key0 + 2 * BN <= p.Sk && t + 1 < n_tiles) {
            mnext.load(mbase + (int64_t)min(qrow, p.Sq - 1) * p.m.sq + key0 + BN);
        }
        auto p_elem = [&](int kb, int r) {          // P^T: one query per lane, so LSE is a per-lane scalar
            float pr = exp2_fast(fmaf(sacc[kb][r], c_log2, -lse2));
            if constexpr (VECMASK) {
                pr = mrow.keep(kb, r, h) ? pr : 0.f;
            } else if (MASKED) {
                const int key = key0 + 32 * kb + acc_row(r, h);
                bool drop = (key >= klimit) | ((p.m.causal != 0) & (key > qrow));     // bitwise: selects, not branches
                if (HASMASK) {
                    if (vec_mask) drop = drop || !mrow.keep(kb, r, h);
                    else if (!drop && qok) drop = !mask_attends(p.m, mbase, (int64_t)qrow * p.m.sq + (int64_t)key * p.m.sk);
                }
                pr = drop ? 0.f : pr;
            }
            sacc[kb][r] = pr;
        };
        auto ds_elem = [&](int kb, int r) {         // dS^T = P^T (dP^T - delta), packed after 8 and 16
            if constexpr (DROPOUT) {
                // O = (P f) V with f = 0 or 1 / (1 - p): dP = f (dO V^T), and rowsum(dP P) is still rowsum(dO O)
                const uint32_t key = (uint32_t)(key0 + 32 * kb + acc_row(r, h));
                const float f = drop_factor_at(p.m, (uint32_t)bh, (uint32_t)qrow, key, (uint32_t)p.Sq, (uint32_t)p.Sk);
                dpacc[kb][r] = sacc[kb][r] * fmaf(f, dpacc[kb][r], -delta);
            } else {
                dpacc[kb][r] = sacc[kb][r] * (dpacc[kb][r] - delta);
            }
            if ((r & 7) == 7) {
                const int o8 = r - 7;
                const f32x16& d = dpacc[kb];
                dsf[kb][r >> 3] = pack8(d[o8], d[o8 + 1], d[o8 + 2], d[o8 + 3], d[o8 + 4], d[o8 + 5], d[o8 + 6], d[o8 + 7]);
            }
        };
        constexpr int EPM = 16 / DC;                // logits per MFMA slot in the row phases
        constexpr int EPQ = 16 / (2 * DB);          // ... and in the dQ phases
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                sacc[kb][r] = 0.f;
                dpacc[kb][r] = 0.f;
            }
        auto row_phase = [&](auto phase_tag) {
            constexpr int PH = decltype(phase_tag)::value, KB = PH >> 1;
#pragma unroll
            for (int dc = 0; dc < DC; ++dc) {
                constexpr int F0 = PH * DC;
                const int f = F0 + dc;
                if (PH & 1) dpacc[KB] = mfma32(fb[f % PD], dof[dc], dpacc[KB]);
                else sacc[KB] = mfma32(fb[f % PD], qf[dc], sacc[KB]);
                fb[f % PD] = fetch(f + PD);
#pragma unroll
                for (int e = 0; e < EPM; ++e) {
                    const int r = EPM * dc + e;
                    if (PH == 1) p_elem(0, r);
                    if (PH == 2) ds_elem(0, r);
                    if (PH == 3) p_elem(1, r);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        auto dq_phase = [&](auto kb_tag) {
            constexpr int KB = decltype(kb_tag)::value;
#pragma unroll
            for (int g = 0; g < 2 * DB; ++g) {
                const int f = NROW + 2 * DB * KB + g, c = g / DB, db = g % DB;
                dqacc[db] = mfma32(fb[f % PD], dsf[KB][c], dqacc[db]);
                if (f + PD < NALL) fb[f % PD] = fetch(f + PD);
                if (KB == 0) {
#pragma unroll
                    for (int e = 0; e < EPQ; ++e) ds_elem(1, EPQ * g + e);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        row_phase(std::integral_constant<int, 0>{});
        row_phase(std::integral_constant<int, 1>{});
        row_phase(std::integral_constant<int, 2>{});
        row_phase(std::integral_constant<int, 3>{});
        dq_phase(std::integral_constant<int, 0>{});
        dq_phase(std::integral_constant<int, 1>{});

        wait_vm0();
        __syncthreads();
    };

    int n_full = HASMASK ? 0 : klimit / BN;
    if (p.m.causal) n_full = min(n_full, (q0 + 1) / BN);
    n_full = min(n_full, n_tiles);
    using IM = std::integral_constant<int, -1>;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    {
        int t = 0;
        for (; t + 2 < n_full; t += 2) {      // tiles t+1 and t+2 are full: straight-line copies, fixed stages
            tile_step(std::false_type{}, I1{}, I0{}, t);
            tile_step(std::false_type{}, I1{}, I1{}, t + 1);
        }
        for (; t < n_full; ++t) tile_step(std::false_type{}, I2{}, IM{}, t);
        for (; t < n_tiles; ++t) tile_step(std::true_type{}, I2{}, IM{}, t);
    }

    // ---- epilogue: dQ = scale * dQ^T, bf16
    if (qok) {
        uint16_t* dqrow = p.dq + b * p.dqs.b + hh * p.dqs.h + (int64_t)qrow * p.dqs.n;
        const float s = p.scale;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x16& a = dqacc[db];
                u32x2 w = {pack_bf16(a[4 * g] * s, a[4 * g + 1] * s), pack_bf16(a[4 * g + 2] * s, a[4 * g + 3] * s)};
                if (32 * db + 8 * g + 4 * h < p.d) *reinterpret_cast<u32x2*>(dqrow + 32 * db + 8 * g + 4 * h) = w;
            }
    }
}

// ---------------------------------------------------------------------------- dq, 256-query workgroups
// The same computation as bwd_dq_kernel for workgroups of 256 queries, laid out for one wavefront per
// SIMD: 4 wavefronts of 64 queries (two 32-query blocks) each.  Every K / V fragment read from LDS then
// feeds two MFMAs (one per query block), which halves the LDS reads and waits per MFMA; the register
// file of a lone wavefront holds dQ^T of both blocks and the Q / dO fragments in the accumulation
// registers (Q / dO as MFMA B operands), and S^T / dP^T in architectural registers through hand-emitted
// MFMAs (see mfma32_vgpr_bacc).  dP^T starts from -delta, so dS^T = P^T * dP'^T is one multiply.
// Three LDS stages of K / V tiles, one barrier per tile, one ring of fragment reads that runs on into
// the next tile, copies split around MFMAs and spread over the tile: as in bwd_dkdv_kernel.
// No explicit keep-mask variant: such problems use bwd_dq_kernel.
template <int D>
struct BwdDqWideTile {
    static constexpr int BM = 256;                  // query rows per workgroup (64 per wavefront)
    static constexpr int BN = 64;                   // keys per tile
    static constexpr int RS = D;
    static constexpr int TILE_ELEMS = BN * D;
    static constexpr int STAGE_ELEMS = 2 * TILE_ELEMS;            // K tile + V tile
    static constexpr int NSTAGE = 3;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_ELEMS * 2;
    static constexpr int ROWS_PER_DMA = 1024 / (D * 2);
    static constexpr int DMA_PER_WAVE = BN / ROWS_PER_DMA / 4;    // 1 KiB copies per wave and tensor
};

template <int D>
__device__ __forceinline__ void bwd_dq_wide_body(const BwdParams& p, const int block, const int nblocks) {
    using T = BwdDqWideTile<D>;
    constexpr int BM = T::BM, BN = T::BN, RS = T::RS;
    constexpr int DC = D / 16;
    constexpr int DB = D / 32;
    constexpr int GPR = D / 8;
    constexpr int NDMA = T::DMA_PER_WAVE;

    extern __shared__ __attribute__((aligned(1024))) uint16_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;

    const int n_qt = (p.Sq + BM - 1) / BM;
    const int wg = p.m.kv_len ? xcd_remap_heads(block, nblocks, n_qt) : xcd_remap(block, nblocks);
    int qt = wg % n_qt, bh = wg / n_qt;
    if (p.m.causal && !p.m.kv_len) causal_longest_first(wg, n_qt, nblocks, qt, bh);
    const int b = bh / p.H, hh = bh % p.H;
    const int q0 = qt * BM;
    const int qw0 = q0 + wave * 64;

    const uint16_t* qbase = p.q + b * p.qs.b + hh * p.qs.h;
    const uint16_t* kbase = p.k + b * p.ks.b + hh * p.ks.h;
    const uint16_t* vbase = p.v + b * p.vs.b + hh * p.vs.h;
    const uint16_t* dobase = p.dout + b * p.dos.b + hh * p.dos.h;

    int klimit = p.Sk;
    if (p.m.kv_len) klimit = min(klimit, max(p.m.kv_len[b], 0));
    int kend = klimit;
    if (p.m.causal) kend = min(kend, q0 + BM);
    const int n_tiles = (kend + BN - 1) / BN;

    // ---- Q and dO fragments (B operands: column = query, 8 consecutive d) and the per-query scalars of
    //      both query blocks; -delta and lse2 are also left in the workspace for the dK/dV kernel
    bf16x8 qf[2][DC], dof[2][DC];          // pinned to accumulation registers: slots qb*DC + dc and 16 + qb*DC + dc
    float lse2[2];
    f32x16 ndelta16[2];
    int qrow[2];
    static_for<2>([&](auto qb_tag) {
        constexpr int qb = decltype(qb_tag)::value;
        qrow[qb] = qw0 + 32 * qb + n;
        const bool qok = qrow[qb] < p.Sq;
        const uint16_t* rq = qbase + (int64_t)qrow[qb] * p.qs.n + 8 * h;
        const uint16_t* rd = dobase + (int64_t)qrow[qb] * p.dos.n + 8 * h;
        const uint16_t* ro = p.o + b * p.os.b + hh * p.os.h + (int64_t)qrow[qb] * p.os.n + 8 * h;
        float part = 0.f;
        static_for<DC>([&](auto dc_tag) {
            constexpr int dc = decltype(dc_tag)::value;
            const bool in_d = qok && 16 * dc + 8 * h < p.d;
            qf[qb][dc] = pin_b_fragment<qb * DC + dc>(ldg16(rq + 16 * dc, in_d));
            const u32x4 dv = ldg16(rd + 16 * dc, in_d);
            dof[qb][dc] = pin_b_fragment<16 + qb * DC + dc>(dv);
            if (!p.rows_ready) {
                const u32x4 ov = ldg16(ro + 16 * dc, in_d);
#pragma unroll
                for (int i = 0; i < 4; ++i) part += bf16_lo(dv[i]) * bf16_lo(ov[i]) + bf16_hi(dv[i]) * bf16_hi(ov[i]);
            }
        });
        lse2[qb] = INFINITY;
        float nd = 0.f;
        if (p.rows_ready) {       // bwd_rows_kernel has left both rows in the workspace
            if (qok) {
                nd = p.ndelta[(int64_t)bh * p.Sq + qrow[qb]];
                lse2[qb] = p.lse2[(int64_t)bh * p.Sq + qrow[qb]];
            }
        } else {
            part += xhalf(part);
            if (qok) {
                const float l = p.lse[(int64_t)bh * p.Sq + qrow[qb]];
                lse2[qb] = (l == -INFINITY) ? INFINITY : l * kLog2e;
                nd = -part;
                if (h == 0) {
                    p.ndelta[(int64_t)bh * p.Sq + qrow[qb]] = nd;
                    p.lse2[(int64_t)bh * p.Sq + qrow[qb]] = lse2[qb];
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) ndelta16[qb][r] = nd;
    });

    // ---- asynchronous staging of the K / V tiles
    const int dma_row_in = lane / GPR, dma_gran = lane % GPR;
    const uint32_t lds0 = lds_addr(lds);
    uint32_t k_lane_off[NDMA], v_lane_off[NDMA];     // bytes
#pragma unroll
    for (int i = 0; i < NDMA; ++i) {
        const int row = (wave * NDMA + i) * T::ROWS_PER_DMA + dma_row_in;
        const int c = src_granule(dma_gran ^ swz<D>(row), p.d);
        k_lane_off[i] = 2u * (uint32_t)(row * (int)p.ks.n + c * 8);
        v_lane_off[i] = 2u * (uint32_t)(row * (int)p.vs.n + c * 8);
    }
    auto dst_of = [&](int stg, int which, int i) {    // LDS byte address of copy i of this wave (which: 0 = K, 1 = V)
        return lds0 + 2u * (uint32_t)(stg * T::STAGE_ELEMS + which * T::TILE_ELEMS + (wave * NDMA + i) * 512);
    };
    auto issue_tile = [&](int t, int stg) {          // any tile: rows past the attended range re-read the last attended key
#pragma unroll
        for (int i = 0; i < NDMA; ++i) {
            const int row = (wave * NDMA + i) * T::ROWS_PER_DMA + dma_row_in;
            const int key = max(min(t * BN + row, klimit - 1), 0);
            const int c = src_granule(dma_gran ^ swz<D>(row), p.d);
            dma16(kbase + (int64_t)key * p.ks.n + c * 8, dst_of(stg, 0, i));
            dma16(vbase + (int64_t)key * p.vs.n + c * 8, dst_of(stg, 1, i));
        }
    };

    int koff[DC];          // 16-byte row reads of K / V: row 32*kb + n, logical granule 2*dc + h
#pragma unroll
    for (int dc = 0; dc < DC; ++dc) koff[dc] = n * RS + (((2 * dc + h) ^ swz<D>(n)) << 3);
    const int tr_r = lane & 15, tr_g16 = (lane >> 4) & 1;
    int toff[2][DB];       // transposing reads of K: rows 4h + r/4 (+8), logical granule 4*db + 2*g16 + (r&3)/2
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int row = 4 * h + (tr_r >> 2) + 8 * half;
#pragma unroll
        for (int db = 0; db < DB; ++db)
            toff[half][db] = row * RS + (((4 * db + 2 * tr_g16 + ((tr_r & 3) >> 1)) ^ swz<D>(row)) << 3) + 4 * (tr_r & 1);
    }

    const float c_log2 = p.scale * kLog2e;
    f32x16 dqacc[2][DB];      // dQ^T: rows = d, column = this lane's query of block qb
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) dqacc[qb][db][r] = 0.f;

    // Operand fragments of a tile, in consumption order; each feeds two MFMAs (query blocks 0 and 1):
    //   [0, DC) K rows of key block 0 (S), [DC, 2DC) V rows of block 0 (dP), then the same for block 1,
    //   [4DC, 4DC + 2DB) K^T of key block 0 by (16-key chunk, db) (dQ), then of block 1
    constexpr int NROW = 4 * DC, NF = NROW + 4 * DB;
    constexpr int PD = 4;                            // read-ahead depth of the fragment ring
    static_assert(DC % PD == 0 && (2 * DB) % PD == 0, "read-ahead depth must divide the fragment counts");
    auto fetch = [&](const uint16_t* ks, int f) {
        const uint16_t* vs = ks + T::TILE_ELEMS;
        if (f < NROW) {
            const int phase = f / DC, dc = f % DC;            // phase: 0 S(0), 1 dP(0), 2 S(1), 3 dP(1)
            return *reinterpret_cast<const bf16x8*>(((phase & 1) ? vs : ks) + koff[dc] + 32 * (phase >> 1) * RS);
        }
        const int g = f - NROW, cc = g / DB, db = g % DB;      // cc = 16-key chunk of the tile
        const u32x2 lo = lds_read_tr16(ks + toff[0][db] + 16 * cc * RS);
        const u32x2 hi = lds_read_tr16(ks + toff[1][db] + 16 * cc * RS);
        const u32x4 u = {lo[0], lo[1], hi[0], hi[1]};
        return __builtin_bit_cast(bf16x8, u);
    };
    bf16x8 fb[PD];
    if (n_tiles > 0) {
        issue_tile(0, 0);
        wait_vm0();
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PD; ++i) fb[i] = fetch(lds, i);
    }

    // One tile of 64 keys = two key blocks of 32, six phases of 2 DC MFMAs (MFMA slot = 2 * fragment +
    // query block).  The element-wise work of a phase is threaded between the MFMAs of the next one:
    //   S(0) | dP(0) + P(0) | S(1) + dS(0) | dP(1) + P(1) | dQ(0) + dS(1) | dQ(1)
    // Element e of query block 0 goes with slot e of its phase, that of query block 1 with slot e + 1
    // (its S / dP are complete one MFMA later), the sixteenth spilling into the first slot of the
    // next phase: every hand-emitted MFMA result is first touched two MFMAs after it was issued.
    // COPY: 1 = the next tile is a full one (copies split around the MFMAs), 2 = decide at run time.
    // STAGE: LDS stage that holds this tile (0 / 1 / 2), or -1 to take it from st.
    auto tile_step = [&](auto masked_tag, auto copy_tag, auto stage_tag, int st, int t, const uint16_t* nk_base,
                         const uint16_t* nv_base) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        constexpr int COPY = decltype(copy_tag)::value;
        constexpr int STAGE = decltype(stage_tag)::value;
        const int cur = STAGE >= 0 ? STAGE : st;
        const int nxt = STAGE >= 0 ? (STAGE + 1) % 3 : (st == 2 ? 0 : st + 1);
        const bool have_next = COPY == 1 || t + 1 < n_tiles;
        if (COPY == 2 && have_next) issue_tile(t + 1, nxt);
        const uint16_t* ks = lds + cur * T::STAGE_ELEMS;
        const uint16_t* kn = lds + nxt * T::STAGE_ELEMS;
        const int key0 = t * BN;

        f32x16 sacc[2][2], dpacc[2][2];             // [query block][key block]
        u32x4 dsw[2][2][2];                         // dS^T operands: [query block][key block][16-key chunk]

        auto p_elem = [&](int qb, int kb, int r) {  // P^T: one query per lane, so LSE is a per-lane scalar
            float pr = exp2_fast(fmaf(sacc[qb][kb][r], c_log2, -lse2[qb]));
            if (MASKED) {
                const int key = key0 + 32 * kb + acc_row(r, h);
                const bool drop = (key >= klimit) | ((p.m.causal != 0) & (key > qrow[qb]));     // bitwise: selects, not branches
                pr = drop ? 0.f : pr;
            }
            sacc[qb][kb][r] = pr;
        };
        auto ds_elem = [&](int qb, int kb, int r) { // dS^T = P^T * (dP^T - delta), packed in pairs
            f32x16& d = dpacc[qb][kb];
            d[r] = sacc[qb][kb][r] * d[r];
            if (r & 1) dsw[qb][kb][r >> 3][(r & 7) >> 1] = pack_bf16(d[r - 1], d[r]);
        };
        // element-wise work that goes with MFMA slot i of phase ph
        constexpr int NSL = 2 * DC;                 // MFMA slots per phase
        static_assert(NSL == 16 || NSL == 8, "element schedule written for 16 or 8 slots per phase");
        auto elems_of = [&](int ph, int i, auto fn) {      // fn(qb, e) for the elements scheduled at (ph, i)
            // query block 0: elements [EL*i, EL*(i+1)) at slot i; query block 1: one slot later
            constexpr int EL = 16 / NSL;            // 1 or 2 elements per slot and block
#pragma unroll
            for (int e = 0; e < EL; ++e) fn(0, EL * i + e);
            if (i > 0) {
#pragma unroll
                for (int e = 0; e < EL; ++e) fn(1, EL * (i - 1) + e);
            }
        };
        auto spill_of = [&](auto fn) {               // the last elements of query block 1, in slot 0 of the next phase
            constexpr int EL = 16 / NSL;
#pragma unroll
            for (int e = 0; e < EL; ++e) fn(1, EL * (NSL - 1) + e);
        };
        // copies of the next tile: copy j goes with MFMA slot CS * j + 1 of the S / dP phases
        constexpr int NCOPY = 2 * NDMA;
        constexpr int CS = (4 * NSL - 2) / NCOPY;
        static_assert(CS >= 2, "copies do not fit the S / dP phases");
        auto copy_dst = [&](int g) {
            const int j = (g - 1) / CS;
            if (COPY == 1 && g >= 1 && (g - 1) % CS == 0 && j < NCOPY) dma_set_dst(dst_of(nxt, j & 1, j >> 1));
        };
        auto copy_issue = [&](int g) {
            const int j = (g - 1) / CS;
            if (COPY == 1 && g >= 1 && (g - 1) % CS == 0 && j < NCOPY) {
                if (j & 1) dma16u_issue(nv_base, v_lane_off[j >> 1]);
                else dma16u_issue(nk_base, k_lane_off[j >> 1]);
            }
        };
        auto refill = [&](int f) {
            const int nf = f + PD;
            if (nf < NF) fb[f % PD] = fetch(ks, nf);
            else if (have_next) fb[f % PD] = fetch(kn, nf - NF);
        };
        auto side = [&](int ph, int i) {
            if (ph == 1) elems_of(ph, i, [&](int qb, int e) { p_elem(qb, 0, e); });
            if (ph == 2) {
                if (i == 0) spill_of([&](int qb, int e) { p_elem(qb, 0, e); });
                elems_of(ph, i, [&](int qb, int e) { ds_elem(qb, 0, e); });
            }
            if (ph == 3) {
                if (i == 0) spill_of([&](int qb, int e) { ds_elem(qb, 0, e); });
                elems_of(ph, i, [&](int qb, int e) { p_elem(qb, 1, e); });
            }
            if (ph == 4) {
                if (i == 0) spill_of([&](int qb, int e) { p_elem(qb, 1, e); });
                elems_of(ph, i, [&](int qb, int e) { ds_elem(qb, 1, e); });
            }
            if (ph == 5 && i == 0) spill_of([&](int qb, int e) { ds_elem(qb, 1, e); });
        };

        auto row_phase = [&](auto phase_tag) {      // S^T(kb) = K Q^T or dP^T(kb) = V dO^T - delta
            constexpr int PH = decltype(phase_tag)::value, KB = PH >> 1;
            static_for<DC>([&](auto dc_tag) {
                constexpr int dc = decltype(dc_tag)::value;
                constexpr int f = PH * DC + dc;
                static_for<2>([&](auto qb_tag) {
                    constexpr int qb = decltype(qb_tag)::value;
                    constexpr int i = 2 * dc + qb, g = PH * NSL + i;
                    constexpr int SLOT = ((PH & 1) ? 16 : 0) + qb * DC + dc;      // Q fragments first, then dO
                    copy_dst(g);
                    if constexpr (PH & 1)
                        mfma32_vgpr_bpinned<SLOT, dc == 0 ? 2 : 1>(dpacc[qb][KB], fb[f % PD], dof[qb][dc], ndelta16[qb]);
                    else
                        mfma32_vgpr_bpinned<SLOT, dc == 0 ? 0 : 1>(sacc[qb][KB], fb[f % PD], qf[qb][dc], ndelta16[qb]);
                    __builtin_amdgcn_sched_barrier(0);      // the element-wise work below must not move above this MFMA
                    copy_issue(g);
                    side(PH, i);
                    if (qb == 1) refill(f);
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
        };
        auto dq_phase = [&](auto kb_tag) {          // dQ^T += K^T(kb) dS^T(kb)
            constexpr int KB = decltype(kb_tag)::value;
#pragma unroll
            for (int g = 0; g < 2 * DB; ++g) {
                const int f = NROW + 2 * DB * KB + g, c = g / DB, db = g % DB;
#pragma unroll
                for (int qb = 0; qb < 2; ++qb) {
                    dqacc[qb][db] = mfma32(fb[f % PD], __builtin_bit_cast(bf16x8, dsw[qb][KB][c]), dqacc[qb][db]);
                    __builtin_amdgcn_sched_barrier(0);
                    side(4 + KB, 2 * g + qb);
                    if (qb == 1) {
                        if (f == NF - PD && have_next) {
                            __builtin_amdgcn_sched_barrier(0);
                            wait_vm0();                          // this wave's copies of the next tile have landed
                            __builtin_amdgcn_s_barrier();        // ... everyone's have, and everyone is past the previous tile
                            __builtin_amdgcn_sched_barrier(0);
                        }
                        refill(f);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        row_phase(std::integral_constant<int, 0>{});
        row_phase(std::integral_constant<int, 1>{});
        row_phase(std::integral_constant<int, 2>{});
        row_phase(std::integral_constant<int, 3>{});
        dq_phase(std::integral_constant<int, 0>{});
        dq_phase(std::integral_constant<int, 1>{});
    };

    int n_full = klimit / BN;
    if (p.m.causal) n_full = min(n_full, (q0 + 1) / BN);
    n_full = min(n_full, n_tiles);
    using IM = std::integral_constant<int, -1>;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    {
        const int64_t k_tile_stride = (int64_t)BN * p.ks.n, v_tile_stride = (int64_t)BN * p.vs.n;
        const uint16_t* nk = kbase + k_tile_stride;      // the tile after the current one
        const uint16_t* nv = vbase + v_tile_stride;
        int t = 0, st = 0;
        for (; t + 3 < n_full; t += 3) {      // tiles t+1 .. t+3 are full: straight-line copies, fixed stages
            tile_step(std::false_type{}, I1{}, I0{}, 0, t, nk, nv);
            nk += k_tile_stride, nv += v_tile_stride;
            tile_step(std::false_type{}, I1{}, I1{}, 1, t + 1, nk, nv);
            nk += k_tile_stride, nv += v_tile_stride;
            tile_step(std::false_type{}, I1{}, I2{}, 2, t + 2, nk, nv);
            nk += k_tile_stride, nv += v_tile_stride;
        }
        for (; t < n_full; ++t) {
            tile_step(std::false_type{}, I2{}, IM{}, st, t, nk, nv);
            st = st == 2 ? 0 : st + 1;
        }
        for (; t < n_tiles; ++t) {
            tile_step(std::true_type{}, I2{}, IM{}, st, t, nk, nv);
            st = st == 2 ? 0 : st + 1;
        }
    }

    // ---- epilogue: dQ = scale * dQ^T, bf16
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
        if (qrow[qb] < p.Sq) {
            uint16_t* dqrow = p.dq + b * p.dqs.b + hh * p.dqs.h + (int64_t)qrow[qb] * p.dqs.n;
            const float s = p.scale;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const f32x16& a = dqacc[qb][db];
                    u32x2 w = {pack_bf16(a[4 * g] * s, a[4 * g + 1] * s), pack_bf16(a[4 * g + 2] * s, a[4 * g + 3] * s)};
                    if (32 * db + 8 * g + 4 * h < p.d) *reinterpret_cast<u32x2*>(dqrow + 32 * db + 8 * g + 4 * h) = w;
                }
        }
}

template <int D>
__global__ __launch_bounds__(256) void bwd_dq_wide_kernel(const BwdParams p) {
    bwd_dq_wide_body<D>(p, (int)blockIdx.x, (int)gridDim.x);
}

// ------------------------------------------------------------------------------- per-query rows
// -delta_i = -sum_d dO_id * O_id and LSE_i * log2(e) (+inf where LSE = -inf) for every query row, as a pass of its
// own: with both rows in the workspace beforehand (BwdParams::rows_ready) the dQ and dK/dV walks no longer depend
// on each other and can share one grid.  D / 8 lanes per row, one 16-byte granule of O and of dO each.
template <int D>
__global__ __launch_bounds__(256) void bwd_rows_kernel(const BwdParams p) {
    constexpr int LPR = D / 8;                       // lanes per row
    constexpr int ROWS = 256 / LPR;                  // rows per workgroup
    const int tid = threadIdx.x;
    const int g = tid % LPR;
    const int64_t row = (int64_t)blockIdx.x * ROWS + tid / LPR;       // over [B*H, Sq]
    const int64_t n_rows = (int64_t)p.B * p.H * p.Sq;
    const bool ok = row < n_rows;
    const int64_t rr = ok ? row : 0;
    const int bh = (int)(rr / p.Sq), qi = (int)(rr % p.Sq);
    const int b = bh / p.H, hh = bh % p.H;
    const bool in_d = ok && 8 * g < p.d;
    const u32x4 ov = ldg16(p.o + b * p.os.b + hh * p.os.h + (int64_t)qi * p.os.n + 8 * g, in_d);
    const u32x4 dv = ldg16(p.dout + b * p.dos.b + hh * p.dos.h + (int64_t)qi * p.dos.n + 8 * g, in_d);
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) part += bf16_lo(dv[i]) * bf16_lo(ov[i]) + bf16_hi(dv[i]) * bf16_hi(ov[i]);
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, 64);
    if (ok && g == 0) {
        const float l = p.lse[row];
        p.ndelta[row] = -part;
        p.lse2[row] = (l == -INFINITY) ? INFINITY : l * kLog2e;
    }
}

// ------------------------------------------------------------------------ dQ and dK/dV in one grid
// For problems whose walks are all equally long (no causal flag, key lengths or mask) and fill 256-query
// workgroups: the dQ workgroups (the longer ones) come first in dispatch order, the whole dK/dV key blocks next,
// the split ones last, so that compute units freed by one kind of workgroup go on with the next and only the
// short split pieces make up the tail.  Needs the per-query rows beforehand (bwd_rows_kernel).
template <int D>
__global__ __launch_bounds__(256) void bwd_joint_kernel(const BwdParams p) {
    const int block = (int)blockIdx.x;
    if (block < p.joint_n_dq) bwd_dq_wide_body<D>(p, block, p.joint_n_dq);
    else bwd_dkdv_body<D, false, false>(p, block - p.joint_n_dq, (int)gridDim.x - p.joint_n_dq);
}

}  // namespace fattn
