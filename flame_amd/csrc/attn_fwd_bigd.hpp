// Forward for head dims above 128 (up to 512): the reference's entry points take any head dim and serve these
// through their materialised path (src/sdpa.rs:483-587, :788-961; e.g. the single-head attention of a VAE mid block,
// D = 512).  Same algorithm and outputs as fwd_kernel (S^T = K Q^T, online softmax in fp32, O^T += V^T P^T, O and
// LSE), with the head dim cut into NC chunks of 128 that are laid out in LDS exactly like the 128-wide tiles of the
// other kernels, so fragment reads, swizzle and copies are the same per chunk:
//   * one wavefront per SIMD, 32 queries per wavefront; the Q fragments of all chunks (32 NC registers) and the
//     wavefront's part of O^T (64 NC registers for the whole head dim) stay in registers.  Up to D = 256 that is
//     4 wavefronts x 32 queries per workgroup.  Above (SPLIT), the full O^T would not fit beside Q in 512 registers,
//     so two wavefronts share 32 queries: both form the same S^T and P^T, and each accumulates one half of the
//     output head dim (two of the four 32-wide column blocks of every chunk): 64 queries per workgroup, 1.5x the
//     MFMA work of the unsplit form instead of register spills in the inner loop;
//     NW = wavefronts per workgroup; the library launches NW = 4 only: a wavefront's time does not depend on how
//     many share its K/V tiles, so smaller workgroups make nothing faster (measured: a single D = 512 head of 4096
//     positions 0.234 ms with NW = 4, 0.273 ms with NW = 2, which issues twice the copies per wavefront);
//   * 32-key tiles (K and V: 8 KiB per chunk each), two LDS stages of K and two of V, one workgroup barrier per tile;
//   * a software pipeline one tile deep: step t = [S^T of tile t+1, with the copies of V(t+1) and K(t+2) issued
//     between its MFMAs] [PV of tile t, with the softmax of tile t+1 (maximum, exponentials, bf16 packing) threaded
//     between its MFMAs] [the rare rescale of O^T].  LDS fragments are read one chunk ahead of the MFMAs that use
//     them (one wavefront per SIMD: nothing else hides the latency);
//   * S^T accumulates in architectural registers and O^T in accumulation registers pinned to a[0:127], both emitted
//     by hand: a kernel whose accumulators a conditional rescale also touches otherwise moves them through
//     architectural registers every tile.  The Q fragments of the first two chunks are pinned to a[128:191]: left
//     unpinned, the register allocator moved them into place before each use, and a hand-emitted MFMA directly
//     behind such a move read the old contents (the compiler spaces its own MFMAs two wait states from a vector-ALU
//     write of their operands; the hand-emitted forms used here carry those wait states themselves).
// Exclusions: causal flag, key lengths, ragged last tile.  Head dims that are not a multiple of 128 are zero-padded
// on the way in (as in the other kernels) and not stored on the way out.
#pragma once
#include "attn_fwd.hpp"

namespace fattn {

template <int NC, bool SPLIT, int NW>
struct FwdBigDTile {
    static_assert(NW == 4 || NW == 2 || (NW == 1 && !SPLIT), "wavefronts per workgroup (the library launches 4)");
    static constexpr int BM = (SPLIT ? 16 : 32) * NW, BN = 32;
    static constexpr int NDB = SPLIT ? 2 : 4;                  // 32-wide output column blocks per chunk and wavefront
    static constexpr int SUB_ELEMS = BN * 128;                 // one chunk of one tensor: 32 rows x 128
    static constexpr int TENSOR_STAGE_ELEMS = NC * SUB_ELEMS;  // one tile of K or of V
    static constexpr int LDS_BYTES = 4 * TENSOR_STAGE_ELEMS * 2; // two stages of K, two of V
    static constexpr int COPIES_PER_WAVE = NC * 8 / NW;        // 1 KiB copies (4 rows of one chunk) per tensor and wave
};

// A problem with few query tiles leaves most compute units idle; then key_splits workgroups share a query tile, each
// walks a contiguous slice of its key tiles and writes a normalised fp32 partial output with its log-sum-exp, and
// fwd_bigd_merge_kernel combines them (the partial sums of flash decoding).
struct FwdBigDParams : FwdParams {
    int key_splits;      // 1: no split, O and LSE are written directly
    float* part_o;       // [key_splits][B*H*Sq][dv]
    float* part_lse;     // [key_splits][B*H*Sq], natural log, -inf for a slice without an attended key
};

// the other of the two LDS stages, as a constant where the stage is one
template <int P>
__device__ constexpr std::integral_constant<int, 1 - P> other_stage(std::integral_constant<int, P>) { return {}; }
__device__ inline int other_stage(int stage) { return stage ^ 1; }

template <int NC, bool SPLIT, int NW>
__global__ __launch_bounds__(64 * NW) void fwd_bigd_kernel(const FwdBigDParams p) {
    using T = FwdBigDTile<NC, SPLIT, NW>;
    constexpr int BN = T::BN, BM = T::BM, NDB = T::NDB;
    constexpr int NCP = T::COPIES_PER_WAVE;

    extern __shared__ __attribute__((aligned(1024))) uint16_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;

    const int n_qt = (p.Sq + BM - 1) / BM;
    const int n_bh = p.B * p.H;
    const int wg_all = xcd_remap(blockIdx.x, gridDim.x);
    const int slice = wg_all / (n_qt * n_bh);         // which slice of the key tiles (0 without a split)
    const int wg = wg_all % (n_qt * n_bh);
    const int qt = wg % n_qt, bh = wg / n_qt;
    const int b = bh / p.H, hh = bh % p.H;
    const int q0 = qt * BM;
    const int qgroup = SPLIT ? wave >> 1 : wave;      // which 32 queries of the workgroup
    const int db0 = SPLIT ? 2 * (wave & 1) : 0;       // first output column block of this wavefront
    const int qw0 = q0 + qgroup * 32;
    const int qi = qw0 + n;

    const uint16_t* qbase = p.q + b * p.qs.b + hh * p.qs.h;
    const uint16_t* kbase = p.k + b * p.ks.b + hh * p.ks.h;
    const uint16_t* vbase = p.v + b * p.vs.b + hh * p.vs.h;
    uint16_t* obase = p.o + b * p.os.b + hh * p.os.h;

    int klimit = p.Sk;
    if (p.m.kv_len) klimit = min(klimit, max(p.m.kv_len[b], 0));
    int kend = klimit;
    if (p.m.causal) kend = min(kend, q0 + BM);
    const int n_tiles_all = (kend + BN - 1) / BN;
    const int tiles_per_slice = (n_tiles_all + p.key_splits - 1) / p.key_splits;
    const int t_lo = slice * tiles_per_slice;                    // this workgroup walks tiles t_lo .. n_tiles - 1
    const int n_tiles = min(n_tiles_all, t_lo + tiles_per_slice);

    // ---- Q fragments of every chunk (B operand of S^T = K Q^T): column = query, 8 consecutive d
    bf16x8 qf[NC][8];
    {
        const bool ok = qi < p.Sq;
        const uint16_t* rp = qbase + (int64_t)qi * p.qs.n + 8 * h;
        // the fragments of the first two chunks are pinned to accumulation registers a[128:191] (beside O^T in
        // a[0:127]); left to the register allocator they are moved into place before every use, and a hand-emitted
        // MFMA right behind such a move reads the old contents
        static_for<NC * 8>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            constexpr int c = i / 8, dc = i % 8;
            const u32x4 w = ldg16(rp + 128 * c + 16 * dc, ok && 128 * c + 16 * dc + 8 * h < p.d);
            if constexpr (c < 2) qf[c][dc] = pin_b_fragment<i>(w);
            else qf[c][dc] = __builtin_bit_cast(bf16x8, w);
        });
    }

    // ---- tile copies: copy j of a wavefront moves 4 rows of one chunk (1 KiB); lane = (row in copy, physical granule).
    //      Source = wave-uniform address of the tile + a 32-bit per-lane byte offset (row strides are below 2^24
    //      elements, so 31 rows fit).  For a tile that lies whole below the key limit the offsets are loop constants,
    //      kept in 2 NCP registers (FULL); for the last, ragged tile rows past the attended range re-read the last
    //      attended key and the offsets are formed per copy.
    //      LDS: K stages 0 and 1, then V stages 0 and 1 (tile t in stage (t - t_lo) & 1 of its tensor;
    //      the stage is passed along as a constant where the loop is unrolled by two, as a value elsewhere).
    const uint32_t lds0 = lds_addr(lds);
    const int cp_row_in = lane >> 4;
    const int cp_gl = (lane & 15) ^ (cp_row_in << 2);            // physical granule ^ the lane's part of the swizzle
    auto copy_offset = [&](int which, int j, int rmax) -> uint32_t {
        const int64_t row_stride = which ? p.vs.n : p.ks.n;
        const int cj = wave * NCP + j;                           // 0 .. 8 NC - 1, wave-uniform
        const int row = min(4 * (cj & 7) + cp_row_in, rmax);
        const int g = cp_gl ^ (cj & 3);                          // logical granule: swz<128>(row) = (row & 3) << 2 | (row >> 2) & 3
        int dk = 128 * (cj >> 3) + 8 * g;
        dk = dk < p.d ? dk : 0;                                  // p.dv == p.d in this kernel
        return 2u * (uint32_t)(row * (int)row_stride + dk);
    };
    uint32_t cp_off[2][NCP];
    static_for<2 * NCP>([&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        cp_off[i / NCP][i % NCP] = copy_offset(i / NCP, i % NCP, BN - 1);
    });
    auto issue_copy = [&](auto which_tag, auto full_tag, int t, auto j_tag, auto stage_of_t) {        // which: 0 = K, 1 = V
        const int stage = stage_of_t;
        constexpr int which = decltype(which_tag)::value;
        constexpr bool FULL = decltype(full_tag)::value;
        constexpr int j = decltype(j_tag)::value;
        const int64_t row_stride = which ? p.vs.n : p.ks.n;
        const uint16_t* tb = (which ? vbase : kbase) + (int64_t)t * BN * row_stride;
        const int cj = wave * NCP + j;
        const uint32_t dst = lds0 + 2u * (uint32_t)((2 * which + stage) * T::TENSOR_STAGE_ELEMS + (cj >> 3) * T::SUB_ELEMS + (cj & 7) * 512);
        if constexpr (FULL) dma16u(tb, cp_off[which][j], dst);
        else dma16u(tb, copy_offset(which, j, klimit - 1 - t * BN), dst);          // rmax >= 0 for every tile that is copied
    };
    using KTag = std::integral_constant<int, 0>;
    using VTag = std::integral_constant<int, 1>;

    // ---- per-lane LDS read offsets inside a chunk (elements), as in the 128-wide kernels
    int koff[8];
#pragma unroll
    for (int dc = 0; dc < 8; ++dc) koff[dc] = n * 128 + (((2 * dc + h) ^ swz<128>(n)) << 3);
    const int tr_r = lane & 15, tr_g16 = (lane >> 4) & 1;
    int voff[2][NDB];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int row = 4 * h + (tr_r >> 2) + 8 * half;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
            voff[half][db] = row * 128 + (((4 * (db0 + db) + 2 * tr_g16 + ((tr_r & 3) >> 1)) ^ swz<128>(row)) << 3) + 4 * (tr_r & 1);
    }

    const float c_log2 = p.scale * kLog2e;
    const float stale_ok = 8.0f / c_log2;     // the reference maximum may lag the true one by 2^8
    float m_run = -INFINITY, l_run = 0.f;
    f32x16 oacc[NC][NDB];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[c][db][r] = 0.f;

    // ---- the phases of a tile
    // S^T (32 keys x 32 queries) of tile t1 over all chunks, emitted by hand with the accumulator in architectural
    // registers (O^T is pinned to the accumulation registers).  The K fragments of chunk c + 1 are read while the MFMAs
    // of chunk c run: with one wavefront per SIMD nothing else hides the LDS latency.  COPIES: the copies of V tile t1
    // and of K tile t1 + 1 are issued between the MFMAs, one (NW = 1: two) per MFMA from the first on.
    constexpr int CPS = (2 * NCP + 8 * NC - 1) / (8 * NC);       // copies per MFMA slot
    auto logits = [&](auto copies_tag, auto full_tag, int t1, f32x16& s, auto stage_of_t1) {
        constexpr bool COPIES = decltype(copies_tag)::value;
        const int stage1 = stage_of_t1;
        const uint16_t* ks = lds + stage1 * T::TENSOR_STAGE_ELEMS;
        const bool more_k = t1 + 1 < n_tiles;
        bf16x8 kf[2][8];
        auto read_k = [&](int c, bf16x8 (&dst)[8]) {
#pragma unroll
            for (int dc = 0; dc < 8; ++dc) dst[dc] = *reinterpret_cast<const bf16x8*>(ks + c * T::SUB_ELEMS + koff[dc]);
        };
        read_k(0, kf[0]);
        static_for<NC>([&](auto c_tag) {
            constexpr int c = decltype(c_tag)::value;
            if constexpr (c + 1 < NC) read_k(c + 1, kf[(c + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            static_for<8>([&](auto dc_tag) {
                constexpr int dc = decltype(dc_tag)::value;
                // Q fragments of the first two chunks live in the accumulation registers beside O^T (at most
                // 128 + 64), those of the others in architectural registers
                if constexpr (c < 2) mfma32_vgpr_bpinned<c * 8 + dc, (c == 0 && dc == 0) ? 0 : 1>(s, kf[c & 1][dc], qf[c][dc], s);
                else mfma32_vgpr(s, kf[c & 1][dc], qf[c][dc]);
                if constexpr (COPIES) {
                    static_for<CPS>([&](auto u_tag) {
                        constexpr int idx = (c * 8 + dc) * CPS + decltype(u_tag)::value;
                        if constexpr (idx < NCP) issue_copy(VTag{}, full_tag, t1, std::integral_constant<int, idx>{}, stage_of_t1);
                        else if constexpr (idx < 2 * NCP) {      // FULL says that K tile t1 + 1 exists, too
                            if (decltype(full_tag)::value || more_k) issue_copy(KTag{}, full_tag, t1 + 1, std::integral_constant<int, idx - NCP>{}, other_stage(stage_of_t1));
                        }
                    });
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // Exclusions and the running maximum of tile t1; returns each lane's factor for the accumulated O^T and sets
    // `rescale` (wave-uniform) when some lane's is not 1: the reference maximum may lag the true one by 2^8.
    auto fold_max = [&](int t1, f32x16& s, bool& rescale) -> float {
        const bool edge = (t1 + 1) * BN > klimit || (p.m.causal && (t1 + 1) * BN > qw0 + 1);
        if (edge) {
            const int key_limit = p.m.causal ? min(klimit, qi + 1) : klimit;      // keys below it are attended
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = t1 * BN + acc_row(r, h) >= key_limit ? -INFINITY : s[r];
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, s[r]);
        asm volatile("" : "+v"(tmax));       // the scan stays in its slot
        tmax = fmaxf(tmax, xhalf(tmax));
        float alpha = 1.0f;
        rescale = __any(tmax > m_run + stale_ok);
        if (rescale) {
            const float m_new = fmaxf(m_run, tmax);
            const float m_to = (m_new == -INFINITY) ? 0.f : m_new;
            alpha = exp2_fast((m_run - m_to) * c_log2);
            m_run = m_new;
            l_run *= alpha;
        }
        return alpha;
    };
    auto exps = [&](f32x16& s, int lo, int hi, float msc) {
#pragma unroll
        for (int r = lo; r < hi; ++r) {
            float e = exp2_fast(fmaf(s[r], c_log2, -msc));
            asm volatile("" : "+v"(e));      // computed here, between the MFMAs, not where the compiler would sink it
            s[r] = e;
            l_run += e;
        }
    };
    auto rescale_all = [&](float alpha) {
        static_for<NC * NDB>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            mfma32_apinned_settle<i, i == 0>(oacc[i / NDB][i % NDB]);
        });
        static_for<NC * NDB>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            rescale_pinned<i>(oacc[i / NDB][i % NDB], alpha);
        });
    };
    // O^T += V^T P^T of tile t (accumulators pinned: see mfma32_apinned), V^T fragments read one chunk ahead.  SOFTMAX:
    // the softmax of the next tile's logits s is threaded between the MFMAs: nothing for the first two (the logits
    // were written by hand-emitted MFMAs just before), the maximum after the third, the exponentials after the others,
    // and the bf16 P^T operands of the next tile come out in pn.
    constexpr int NM = 2 * NC * NDB;                             // PV MFMAs per tile
    constexpr int NE = NM - 3;                                   // of which carry exponentials
    auto pv = [&](auto softmax_tag, int t, const bf16x8 (&pf)[2], f32x16& s, bf16x8 (&pn)[2], float& alpha, bool& rescale, auto stage_of_t) {
        constexpr bool SOFTMAX = decltype(softmax_tag)::value;
        const int stage = stage_of_t;
        const uint16_t* vs = lds + (2 + stage) * T::TENSOR_STAGE_ELEMS;
        bf16x8 vf[2][2 * NDB];
        auto read_v = [&](int c, bf16x8 (&dst)[2 * NDB]) {
#pragma unroll
            for (int cc = 0; cc < 2; ++cc)
#pragma unroll
                for (int db = 0; db < NDB; ++db) {
                    const uint16_t* vsub = vs + c * T::SUB_ELEMS + 16 * cc * 128;
                    const u32x2 lo = lds_read_tr16(vsub + voff[0][db]);
                    const u32x2 hi = lds_read_tr16(vsub + voff[1][db]);
                    const u32x4 u = {lo[0], lo[1], hi[0], hi[1]};
                    dst[cc * NDB + db] = __builtin_bit_cast(bf16x8, u);
                }
        };
        float msc = 0.f;
        read_v(0, vf[0]);
        static_for<NC>([&](auto c_tag) {
            constexpr int c = decltype(c_tag)::value;
            if constexpr (c + 1 < NC) read_v(c + 1, vf[(c + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            static_for<2 * NDB>([&](auto f_tag) {                // 16 keys cc, then column block db: neighbours are independent
                constexpr int f = decltype(f_tag)::value;
                constexpr int cc = f / NDB, db = f % NDB, i = c * NDB + db, m = c * 2 * NDB + f;
                mfma32_apinned<i>(oacc[c][db], vf[c & 1][f], pf[cc]);
                if constexpr (SOFTMAX) {
                    if constexpr (m == 2) {
                        alpha = fold_max(t + 1, s, rescale);
                        msc = ((m_run == -INFINITY) ? 0.f : m_run) * c_log2;
                    }
                    if constexpr (m >= 3) exps(s, ((m - 3) * 16) / NE, ((m - 2) * 16) / NE, msc);
                    if constexpr (m == NM - 1) {
                        pn[0] = pack8(s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7]);
                        pn[1] = pack8(s[8], s[9], s[10], s[11], s[12], s[13], s[14], s[15]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    using Yes = std::integral_constant<bool, true>;
    using No = std::integral_constant<bool, false>;

    // ---- the walk over the key tiles.  Tile t's logits and softmax run one step ahead of its PV products: step t is
    //      [S^T of tile t+1 with the copies of V(t+1) and K(t+2) between its MFMAs] [PV of tile t with the softmax of
    //      tile t+1 between its MFMAs] [the rare rescale of O^T] [all copies landed, one workgroup barrier].
    if (n_tiles > t_lo) {
        f32x16 s;
        bf16x8 pf[2], pn[2];
        float alpha = 1.0f;
        bool rescale = false;
        using S0 = std::integral_constant<int, 0>;
        using S1 = std::integral_constant<int, 1>;
        static_for<NCP>([&](auto j_tag) { issue_copy(KTag{}, No{}, t_lo, j_tag, S0{}); });
        static_for<NCP>([&](auto j_tag) { issue_copy(VTag{}, No{}, t_lo, j_tag, S0{}); });
        if (n_tiles > t_lo + 1) static_for<NCP>([&](auto j_tag) { issue_copy(KTag{}, No{}, t_lo + 1, j_tag, S1{}); });
        wait_vm0();
        __syncthreads();
        logits(No{}, No{}, t_lo, s, S0{});
        mfma32_vgpr_settle(s);
        (void)fold_max(t_lo, s, rescale);                        // nothing accumulated yet: no rescale
        exps(s, 0, 16, ((m_run == -INFINITY) ? 0.f : m_run) * c_log2);
        pf[0] = pack8(s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7]);
        pf[1] = pack8(s[8], s[9], s[10], s[11], s[12], s[13], s[14], s[15]);
        auto step = [&](auto full_tag, int t, auto stage_of_t) {
            logits(Yes{}, full_tag, t + 1, s, other_stage(stage_of_t));
            pv(Yes{}, t, pf, s, pn, alpha, rescale, stage_of_t);
            if (rescale) rescale_all(alpha);
            pf[0] = pn[0];
            pf[1] = pn[1];
            wait_vm0();            // the copies issued in this step have landed ...
            __syncthreads();       // ... everyone's, and everyone is done with the stages they go to next
        };
        // While the tiles copied in a step, V(t + 1) and K(t + 2), are both walked and lie whole below the key limit:
        // constant copy offsets, no test per copy, and (up to D = 256) two steps per trip so that the LDS stages are
        // constants, too.
        // The last steps (two to four) form their offsets and stages.
        int t = t_lo;
        const int t_whole_end = min(n_tiles, klimit / BN) - 2;
        if constexpr (NC <= 2) {
            for (; t + 1 < t_whole_end; t += 2) {
                step(Yes{}, t, S0{});
                step(Yes{}, t + 1, S1{});
            }
        } else {           // measured: no gain with three chunks; with four the second set of LDS addresses spills
            for (; t < t_whole_end; ++t) step(Yes{}, t, (t - t_lo) & 1);
        }
        for (; t + 1 < n_tiles; ++t) step(No{}, t, (t - t_lo) & 1);
        pv(No{}, n_tiles - 1, pf, s, pn, alpha, rescale, (n_tiles - 1 - t_lo) & 1);
    }

    // ---- epilogue
    static_for<NC * NDB>([&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        mfma32_apinned_settle<i, i == 0>(oacc[i / NDB][i % NDB]);
    });
    const float l = l_run + xhalf(l_run);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    const float lse_val = l > 0.f ? (m_run * c_log2 + log2_fast(l)) * kLn2 : -INFINITY;
    if (p.key_splits > 1) {
        if (qi < p.Sq) {
            const int64_t prow_i = ((int64_t)slice * n_bh + bh) * p.Sq + qi;
            float* prow = p.part_o + prow_i * p.dv;
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int db = 0; db < NDB; ++db)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int d0 = 128 * c + 32 * (db0 + db) + 8 * g + 4 * h;
                        if (d0 < p.dv) {
                            const f32x16& a = oacc[c][db];
                            const f32x4 w = {a[4 * g] * inv, a[4 * g + 1] * inv, a[4 * g + 2] * inv, a[4 * g + 3] * inv};
                            *reinterpret_cast<f32x4*>(prow + d0) = w;
                        }
                    }
            if (h == 0 && db0 == 0) p.part_lse[prow_i] = lse_val;
        }
        return;
    }
    if (qi < p.Sq) {
        uint16_t* orow = obase + (int64_t)qi * p.os.n;
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int d0 = 128 * c + 32 * (db0 + db) + 8 * g + 4 * h;
                    if (d0 < p.dv) {
                        const f32x16& a = oacc[c][db];
                        u32x2 w = {pack_bf16(a[4 * g] * inv, a[4 * g + 1] * inv), pack_bf16(a[4 * g + 2] * inv, a[4 * g + 3] * inv)};
                        *reinterpret_cast<u32x2*>(orow + d0) = w;
                    }
                }
        if (p.lse && h == 0 && db0 == 0) p.lse[(int64_t)bh * p.Sq + qi] = lse_val;
    }
}

// Combines the partial outputs of a key split: LSE = log sum_s exp(LSE_s), O = sum_s exp(LSE_s - LSE) O_s.  One lane
// per query row and 4 output columns.
__global__ __launch_bounds__(256) void fwd_bigd_merge_kernel(const FwdBigDParams p) {
    const int groups = p.dv >> 2;
    const int64_t rows = (int64_t)p.B * p.H * p.Sq;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows * groups) return;
    const int64_t row = idx / groups;
    const int g = (int)(idx % groups);
    float m = -INFINITY;
    for (int s = 0; s < p.key_splits; ++s) m = fmaxf(m, p.part_lse[s * rows + row]);
    float sum = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    if (m != -INFINITY) {
        for (int s = 0; s < p.key_splits; ++s) {
            const float w = expf(p.part_lse[s * rows + row] - m);
            const f32x4 v = *reinterpret_cast<const f32x4*>(p.part_o + (s * rows + row) * p.dv + 4 * g);
            sum += w;
            acc[0] = fmaf(w, v[0], acc[0]); acc[1] = fmaf(w, v[1], acc[1]);
            acc[2] = fmaf(w, v[2], acc[2]); acc[3] = fmaf(w, v[3], acc[3]);
        }
    }
    const float inv = sum > 0.f ? 1.0f / sum : 0.f;
    const int64_t bh = row / p.Sq, qi = row % p.Sq;
    uint16_t* orow = p.o + (bh / p.H) * p.os.b + (bh % p.H) * p.os.h + qi * p.os.n;
    const u32x2 w = {pack_bf16(acc[0] * inv, acc[1] * inv), pack_bf16(acc[2] * inv, acc[3] * inv)};
    *reinterpret_cast<u32x2*>(orow + 4 * g) = w;
    if (p.lse && g == 0) p.lse[row] = sum > 0.f ? m + logf(sum) : -INFINITY;
}

}  // namespace fattn
