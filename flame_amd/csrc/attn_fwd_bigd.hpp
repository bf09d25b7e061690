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
//   * 32-key tiles (K and V: 8 KiB per chunk each), two LDS stages, the copies of tile t+1 in flight while tile t
//     is computed, one workgroup barrier per tile; inside a tile the LDS fragments are read one chunk ahead of the
//     MFMAs that use them;
//   * S^T accumulates in architectural registers and O^T in accumulation registers pinned to a[0:127], both emitted
//     by hand: a kernel whose accumulators a conditional rescale also touches otherwise moves them through
//     architectural registers every tile.
// Exclusions: causal flag, key lengths, ragged last tile.  Head dims that are not a multiple of 128 are zero-padded
// on the way in (as in the other kernels) and not stored on the way out.
#pragma once
#include "attn_fwd.hpp"

namespace fattn {

template <int NC, bool SPLIT>
struct FwdBigDTile {
    static constexpr int BM = SPLIT ? 64 : 128, BN = 32;
    static constexpr int NDB = SPLIT ? 2 : 4;                  // 32-wide output column blocks per chunk and wavefront
    static constexpr int SUB_ELEMS = BN * 128;                 // one chunk of one tensor: 32 rows x 128
    static constexpr int STAGE_ELEMS = 2 * NC * SUB_ELEMS;     // K chunks, then V chunks
    static constexpr int LDS_BYTES = 2 * STAGE_ELEMS * 2;
    static constexpr int COPIES_PER_WAVE = NC * 8 / 4;         // 1 KiB copies (4 rows of one chunk) per tensor and wave
};

template <int NC, bool SPLIT>
__global__ __launch_bounds__(256) void fwd_bigd_kernel(const FwdParams p) {
    using T = FwdBigDTile<NC, SPLIT>;
    constexpr int BN = T::BN, BM = T::BM, NDB = T::NDB;
    constexpr int NCP = T::COPIES_PER_WAVE;

    extern __shared__ __attribute__((aligned(1024))) uint16_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, h = lane >> 5;

    const int n_qt = (p.Sq + BM - 1) / BM;
    const int wg = xcd_remap(blockIdx.x, gridDim.x);
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
    const int n_tiles = (kend + BN - 1) / BN;

    // ---- Q fragments of every chunk (B operand of S^T = K Q^T): column = query, 8 consecutive d
    bf16x8 qf[NC][8];
    {
        const bool ok = qi < p.Sq;
        const uint16_t* rp = qbase + (int64_t)qi * p.qs.n + 8 * h;
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int dc = 0; dc < 8; ++dc)
                qf[c][dc] = __builtin_bit_cast(bf16x8, ldg16(rp + 128 * c + 16 * dc, ok && 128 * c + 16 * dc + 8 * h < p.d));
    }

    // ---- tile copies: copy j of a wavefront moves 4 rows of one chunk (1 KiB); lane = (row in copy, physical granule).
    //      Source = wave-uniform address of the tile + a 32-bit per-lane byte offset (rows past the attended range
    //      re-read the last attended key; row strides are below 2^24 elements, so 31 rows fit).  The offsets are formed
    //      again for every tile from two lane constants: kept per copy across the loop they would take 4 NC registers
    //      that the Q fragments and O^T need (a spill reload in the loop waits on vmcnt, that is, on the copies).
    const uint32_t lds0 = lds_addr(lds);
    const int cp_row_in = lane >> 4;
    const int cp_gl = (lane & 15) ^ (cp_row_in << 2);            // physical granule ^ the lane's part of the swizzle
    auto issue_tile = [&](int t) {
        const uint32_t stage = lds0 + 2u * (uint32_t)((t & 1) * T::STAGE_ELEMS);
        const uint16_t* kt = kbase + (int64_t)t * BN * p.ks.n;
        const uint16_t* vt = vbase + (int64_t)t * BN * p.vs.n;
        const int rmax = klimit - 1 - t * BN;                    // >= 0 for every tile of the loop
        int row_in = cp_row_in, gl = cp_gl;
        asm volatile("" : "+v"(row_in), "+v"(gl));               // opaque: nothing below is hoisted out of the key loop
#pragma unroll
        for (int j = 0; j < NCP; ++j) {
            const int cj = wave * NCP + j;                       // 0 .. 8 NC - 1, wave-uniform
            const int chunk = cj >> 3;
            const int row = min(4 * (cj & 7) + row_in, rmax);
            const int g = gl ^ (cj & 3);                         // logical granule: swz<128>(row) = (row & 3) << 2 | (row >> 2) & 3
            int dk = 128 * chunk + 8 * g;
            dk = dk < p.d ? dk : 0;                              // p.dv == p.d in this kernel
            const uint32_t dst = stage + 2u * (uint32_t)(chunk * T::SUB_ELEMS + (cj & 7) * 512);
            dma16u(kt, 2u * (uint32_t)(row * (int)p.ks.n + dk), dst);
            dma16u(vt, 2u * (uint32_t)(row * (int)p.vs.n + dk), dst + 2u * (uint32_t)(NC * T::SUB_ELEMS));
        }
    };

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

    if (n_tiles > 0) {
        issue_tile(0);
        wait_vm0();
        __syncthreads();
    }
    for (int t = 0; t < n_tiles; ++t) {
        if (t + 1 < n_tiles) issue_tile(t + 1);
        const uint16_t* ks = lds + (t & 1) * T::STAGE_ELEMS;
        const uint16_t* vs = ks + NC * T::SUB_ELEMS;
        // ---- S^T (32 keys x 32 queries) over all chunks
        //      (emitted by hand with the accumulator in architectural registers: O^T below is pinned to the
        //      accumulation registers).  The K fragments of chunk c + 1 are read while the MFMAs of chunk c run:
        //      with one wavefront per SIMD nothing else hides the LDS latency.
        f32x16 s;
        {
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
#pragma unroll
                for (int dc = 0; dc < 8; ++dc) {
                    // Q fragments of the first two chunks live in the accumulation registers beside O^T (at most
                    // 128 + 64), those of the others in architectural registers
                    if (c == 0 && dc == 0) mfma32_vgpr_first_bacc(s, kf[c & 1][dc], qf[c][dc]);
                    else if (c < 2) mfma32_vgpr_bacc(s, kf[c & 1][dc], qf[c][dc]);
                    else mfma32_vgpr(s, kf[c & 1][dc], qf[c][dc]);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        }
        mfma32_vgpr_settle(s);
        // ---- exclusions and the tile maximum
        const bool edge = (t + 1) * BN > klimit || (p.m.causal && (t + 1) * BN > qw0 + 1);
        float tmax = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            if (edge) {
                const int key = t * BN + acc_row(r, h);
                const bool drop = (key >= klimit) | ((p.m.causal != 0) & (key > qi));
                s[r] = drop ? -INFINITY : s[r];
            }
            tmax = fmaxf(tmax, s[r]);
        }
        tmax = fmaxf(tmax, xhalf(tmax));
        if (__any(tmax > m_run + stale_ok)) {
            const float m_new = fmaxf(m_run, tmax);
            const float m_to = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = exp2_fast((m_run - m_to) * c_log2);
            m_run = m_new;
            l_run *= alpha;
            static_for<NC * NDB>([&](auto i_tag) {
                constexpr int i = decltype(i_tag)::value;
                rescale_pinned<i>(oacc[i / NDB][i % NDB], alpha);
            });
        }
        // ---- P^T in the B-operand layout of the second product
        const float msc = ((m_run == -INFINITY) ? 0.f : m_run) * c_log2;
        float rsum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            s[r] = exp2_fast(fmaf(s[r], c_log2, -msc));
            rsum += s[r];
        }
        l_run += rsum;
        const bf16x8 pf[2] = {pack8(s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7]),
                              pack8(s[8], s[9], s[10], s[11], s[12], s[13], s[14], s[15])};
        // ---- O^T += V^T P^T (accumulators pinned: see mfma32_apinned), V^T fragments read one chunk ahead
        {
            bf16x8 vf[2][2 * NDB];
            auto read_v = [&](int c, bf16x8 (&dst)[2 * NDB]) {
#pragma unroll
                for (int db = 0; db < NDB; ++db)
#pragma unroll
                    for (int cc = 0; cc < 2; ++cc) {
                        const uint16_t* vsub = vs + c * T::SUB_ELEMS + 16 * cc * 128;
                        const u32x2 lo = lds_read_tr16(vsub + voff[0][db]);
                        const u32x2 hi = lds_read_tr16(vsub + voff[1][db]);
                        const u32x4 u = {lo[0], lo[1], hi[0], hi[1]};
                        dst[2 * db + cc] = __builtin_bit_cast(bf16x8, u);
                    }
            };
            read_v(0, vf[0]);
            static_for<NC>([&](auto c_tag) {
                constexpr int c = decltype(c_tag)::value;
                if constexpr (c + 1 < NC) read_v(c + 1, vf[(c + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);
                static_for<NDB>([&](auto db_tag) {
                    constexpr int db = decltype(db_tag)::value;
                    constexpr int i = c * NDB + db;
                    mfma32_apinned<i, i == 0>(oacc[c][db], vf[c & 1][2 * db], pf[0]);
                    mfma32_apinned<i, i == 0>(oacc[c][db], vf[c & 1][2 * db + 1], pf[1]);
                });
                __builtin_amdgcn_sched_barrier(0);
            });
        }
        wait_vm0();            // the copies of tile t+1 have landed ...
        __syncthreads();       // ... everyone's, and everyone is done reading tile t
    }

    // ---- epilogue
    static_for<NC * NDB>([&](auto i_tag) {
        constexpr int i = decltype(i_tag)::value;
        mfma32_apinned_settle<i, i == 0>(oacc[i / NDB][i % NDB]);
    });
    const float l = l_run + xhalf(l_run);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
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
        if (p.lse && h == 0 && db0 == 0) p.lse[(int64_t)bh * p.Sq + qi] = l > 0.f ? (m_run * c_log2 + log2_fast(l)) * kLn2 : -INFINITY;
    }
}

}  // namespace fattn
