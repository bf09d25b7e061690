// Fused input preparation for joint attention: per-head RMS normalisation over the head dim
// (optional learned scale), interleaved-pair rotary embedding from per-position cos/sin tables, and
// the [B,N,H,D] -> [B,H,N,D] layout change, in one HBM-bound pass: every element is read once and
// written once.
//
// Arithmetic follows the reference's two kernels run back to back, including the bf16 rounding
// between them:
//   v[i]    = bf16( x[i] * (1 / sqrt(mean_i(x^2) + eps)) * w[i] )       (fused_rms_norm.cu:26-86)
//   y[2p]   = bf16( v[2p] * cos[n,p] - v[2p+1] * sin[n,p] )             (bf16_ops.rs:361-394)
//   y[2p+1] = bf16( v[2p] * sin[n,p] + v[2p+1] * cos[n,p] )
//
// One row (D elements) is served by D/8 adjacent lanes, 8 elements = 4 rotation pairs per lane, so
// loads and stores are 16 bytes per lane and the mean of squares is a butterfly over D/8 lanes; the same
// lanes serve that position in several heads, which share its table entries.
#pragma once
#include "attn_common.hpp"

namespace fattn {

struct PrepParams {
    const uint16_t* x;
    const uint16_t* w;       // [D] bf16 or null (no learned scale)
    const void* cos_t;       // [N, D/2] fp32 or bf16, or null (no rotation)
    const void* sin_t;
    uint16_t* y;
    Strides xs, ys;          // element strides over (B, H, N); D stride is 1
    int B, H, N;
    float eps;
    int norm;                // apply the RMS normalisation
    int table_f32;           // tables are fp32 (else bf16)
};

// Heads served by one thread: the rotation tables depend on the position only, so a thread loads its
// four (cos, sin) pairs once and applies them to the same 8 elements of kPrepHeadsPerThread heads.
constexpr int kPrepHeadsPerThread = 4;

template <int D>
__global__ __launch_bounds__(256) void prep_qk_kernel(const PrepParams p) {
    constexpr int LPR = D / 8;              // lanes per row
    constexpr int RPB = 256 / LPR;          // (position, head group) items per workgroup
    constexpr int HPT = kPrepHeadsPerThread;
    const int tid = threadIdx.x;
    const int sub = tid % LPR;
    const int hgroups = (p.H + HPT - 1) / HPT;
    const int64_t item = (int64_t)blockIdx.x * RPB + tid / LPR;     // index over (b, n, head group)
    const int64_t items = (int64_t)p.B * p.N * hgroups;
    if (item >= items) return;              // no barriers or cross-row exchanges follow (the butterfly stays inside a row's lanes,
                                            // which leave together)
    const int hg = (int)(item % hgroups);
    const int64_t bn = item / hgroups;
    const int n = (int)(bn % p.N), b = (int)(bn / p.N);

    u32x4 wraw = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};      // bf16 ones
    if (p.norm && p.w) wraw = *reinterpret_cast<const u32x4*>(p.w + 8 * sub);
    float c[4], sn[4];
    if (p.cos_t) {
        const int64_t t0 = (int64_t)n * (D / 2) + 4 * sub;
        if (p.table_f32) {
            const f32x4 cv = *reinterpret_cast<const f32x4*>(static_cast<const float*>(p.cos_t) + t0);
            const f32x4 sv = *reinterpret_cast<const f32x4*>(static_cast<const float*>(p.sin_t) + t0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                c[i] = cv[i];
                sn[i] = sv[i];
            }
        } else {
            const u32x2 cv = *reinterpret_cast<const u32x2*>(static_cast<const uint16_t*>(p.cos_t) + t0);
            const u32x2 sv = *reinterpret_cast<const u32x2*>(static_cast<const uint16_t*>(p.sin_t) + t0);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                c[2 * i] = bf16_lo(cv[i]);
                c[2 * i + 1] = bf16_hi(cv[i]);
                sn[2 * i] = bf16_lo(sv[i]);
                sn[2 * i + 1] = bf16_hi(sv[i]);
            }
        }
    }

    // all loads first, so that they are in flight together
    u32x4 raw[HPT];
#pragma unroll
    for (int k = 0; k < HPT; ++k) {
        const int hh = min(hg * HPT + k, p.H - 1);
        raw[k] = *reinterpret_cast<const u32x4*>(p.x + b * p.xs.b + hh * p.xs.h + (int64_t)n * p.xs.n + 8 * sub);
    }
#pragma unroll
    for (int k = 0; k < HPT; ++k) {
        const int hh = hg * HPT + k;
        float v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = bf16_lo(raw[k][i]);
            v[2 * i + 1] = bf16_hi(raw[k][i]);
        }
        if (p.norm) {
            // The sum of squares is carried in fp64: squares of bf16 values are exact there and so, for any realistic
            // spread of magnitudes, is their sum, which makes the mean independent of the summation order and equal to
            // a CPU restatement's; it is rounded to fp32 once.  Square root and division are the correctly rounded
            // fp32 ones (not the hardware's approximate reciprocal square root), so every step is IEEE arithmetic.
            double ss = 0.0;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += (double)v[i] * (double)v[i];
#pragma unroll
            for (int off = LPR / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
            const float ms = (float)(ss / (double)D);
            // __builtin_sqrtf and the division operator are the correctly rounded ones under hipcc's default
            // -fhip-fp32-correctly-rounded-divide-sqrt (the __fsqrt_rn intrinsic is the approximate native one here)
            const float rs = 1.0f / __builtin_sqrtf(ms + p.eps);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma clang fp contract(off)
                // round to bf16 as the stand-alone normalisation kernel would, then carry on in fp32
                const uint32_t packed = pack_bf16(v[2 * i] * rs * bf16_lo(wraw[i]), v[2 * i + 1] * rs * bf16_hi(wraw[i]));
                v[2 * i] = bf16_lo(packed);
                v[2 * i + 1] = bf16_hi(packed);
            }
        }
        u32x4 out;
        if (p.cos_t) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // plain fp32 arithmetic, every product and sum rounded on its own: no contraction into
                // fused multiply-adds, so that the result does not depend on which product gets fused
#pragma clang fp contract(off)
                const float e = v[2 * i], o = v[2 * i + 1];
                const float ec = e * c[i], os = o * sn[i], es = e * sn[i], oc = o * c[i];
                out[i] = pack_bf16(ec - os, es + oc);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) out[i] = pack_bf16(v[2 * i], v[2 * i + 1]);
        }
        if (hh < p.H) *reinterpret_cast<u32x4*>(p.y + b * p.ys.b + hh * p.ys.h + (int64_t)n * p.ys.n + 8 * sub) = out;
    }
}

}  // namespace fattn
