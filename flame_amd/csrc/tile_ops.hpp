// Element-wise primitives on score tiles: the stand-alone entry points that the reference's chunked host
// loops call between their GEMMs (reference: src/kernels/sdpa_kernels.cu:34-403, declared for Rust in
// src/cuda/ffi.rs:349-422).  The fused attention kernels of this library need none of them; they exist so
// that host code written against these symbols (the dropout path among them) links and computes the same
// values.  All of them are bound by memory traffic: every lane moves 16 bytes per access where the row length
// and the alignment allow it, a tile row never straddles two lanes' vectors, and scores that a mask does not
// touch are neither read nor written.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <float.h>

#include "attn_common.hpp"

namespace fattn {

constexpr float kScoreMasked = -1.0e9f;     // value the [B,H,Q,K] mask kernels store (sdpa_kernels.cu:57, :76)
constexpr float kTileNegInf = -1.0e30f;     // finite stand-in for -inf that the tile kernel adds (sdpa_kernels.cu:8-10)

// scores[b,h,q,k] = -1e9 where k_offset + k > q_offset + q.  VEC consecutive keys per lane (K % VEC == 0).
template <int VEC>
__global__ __launch_bounds__(256) void tile_causal_mask_kernel(float* scores, int64_t n_vec, int Q, int K, int q_offset, int k_offset) {
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v >= n_vec) return;
    const int64_t e = v * VEC;
    const int k = (int)(e % K);
    const int q = (int)((e / K) % Q);
    const int first_masked = q_offset + q - k_offset + 1;     // keys k >= first_masked are in the future
    if (k + VEC <= first_masked) return;
    if constexpr (VEC == 4) {
        if (k >= first_masked) {
            const float4 m = {kScoreMasked, kScoreMasked, kScoreMasked, kScoreMasked};
            *reinterpret_cast<float4*>(scores + e) = m;
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i)
        if (k + i >= first_masked) scores[e + i] = kScoreMasked;
}

// scores[i] = -1e9 where mask[i] == 0 (one mask byte per score)
template <int VEC>
__global__ __launch_bounds__(256) void tile_attn_mask_kernel(float* scores, const uint8_t* mask, int64_t n_vec) {
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v >= n_vec) return;
    const int64_t e = v * VEC;
    if constexpr (VEC == 4) {
        const uint32_t m = *reinterpret_cast<const uint32_t*>(mask + e);
        // a byte is zero iff its bit 7 comes out set here
        const uint32_t zero = ~(((m & 0x7f7f7f7fu) + 0x7f7f7f7fu) | m) & 0x80808080u;
        if (zero == 0) return;
        if (zero == 0x80808080u) {
            const float4 f = {kScoreMasked, kScoreMasked, kScoreMasked, kScoreMasked};
            *reinterpret_cast<float4*>(scores + e) = f;
            return;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (zero & (0x80u << (8 * i))) scores[e + i] = kScoreMasked;
    } else {
        if (mask[e] == 0) scores[e] = kScoreMasked;
    }
}

struct TileMaskParams {
    float* logits;
    const uint8_t* user_bool;
    const float* user_add;
    int q_t, k_t, q_abs_start, k_abs_start, bool_rank, add_rank, k_total;
    int zero_is_mask, causal;
};

// logits[bh,qi,kj] += delta, delta = ((0 + add) + (masked ? -1e30 : nothing)) + (future ? -1e30 : nothing), in that
// order (sdpa_kernels.cu:98-137).  Rank 3 operands are tile-shaped, rank 2 operands are [BH, k_total] rows
// indexed by the absolute key.
template <int VEC>
__global__ __launch_bounds__(256) void tile_add_mask_kernel(const TileMaskParams p, int64_t n_vec) {
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v >= n_vec) return;
    const int64_t e = v * VEC;
    const int kj = (int)(e % p.k_t);
    const int qi = (int)((e / p.k_t) % p.q_t);
    const int64_t bh = e / ((int64_t)p.k_t * p.q_t);
    float x[VEC], add[VEC];
    uint8_t mv[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        add[i] = 0.0f;
        mv[i] = 1;
    }
    const bool has_add = p.user_add && (p.add_rank == 3 || p.add_rank == 2);
    const bool has_bool = p.user_bool && (p.bool_rank == 3 || p.bool_rank == 2);
    const int64_t row2 = bh * p.k_total + p.k_abs_start + kj;       // index into a rank 2 operand
    if constexpr (VEC == 4) {
        const float4 f = *reinterpret_cast<const float4*>(p.logits + e);
        x[0] = f.x; x[1] = f.y; x[2] = f.z; x[3] = f.w;
        // tile-shaped operands share the logits' index: one vector access each where their base allows it
        if (has_add && p.add_rank == 3 && (reinterpret_cast<uintptr_t>(p.user_add) & 15) == 0) {
            const float4 a = *reinterpret_cast<const float4*>(p.user_add + e);
            add[0] = a.x; add[1] = a.y; add[2] = a.z; add[3] = a.w;
        } else if (has_add) {
#pragma unroll
            for (int i = 0; i < 4; ++i) add[i] = p.add_rank == 3 ? p.user_add[e + i] : p.user_add[row2 + i];
        }
        if (has_bool && p.bool_rank == 3 && (reinterpret_cast<uintptr_t>(p.user_bool) & 3) == 0) {
            const uint32_t m = *reinterpret_cast<const uint32_t*>(p.user_bool + e);
#pragma unroll
            for (int i = 0; i < 4; ++i) mv[i] = (uint8_t)(m >> (8 * i));
        } else if (has_bool) {
#pragma unroll
            for (int i = 0; i < 4; ++i) mv[i] = p.bool_rank == 3 ? p.user_bool[e + i] : p.user_bool[row2 + i];
        }
    } else {
        x[0] = p.logits[e];
        if (has_add) add[0] = p.add_rank == 3 ? p.user_add[e] : p.user_add[row2];
        if (has_bool) mv[0] = p.bool_rank == 3 ? p.user_bool[e] : p.user_bool[row2];
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        const int k_abs = p.k_abs_start + kj + i;
        float delta = 0.0f;
        if (has_add) delta += add[i];
        if (has_bool && (p.zero_is_mask ? mv[i] == 0 : mv[i] != 0)) delta += kTileNegInf;
        if (p.causal && k_abs > p.q_abs_start + qi) delta += kTileNegInf;
        x[i] += delta;
    }
    if constexpr (VEC == 4) {
        const float4 f = {x[0], x[1], x[2], x[3]};
        *reinterpret_cast<float4*>(p.logits + e) = f;
    } else {
        p.logits[e] = x[0];
    }
}

// probs[bh,qi,kj] = bf16(exp(logits - lse[bh,qi]))
template <int VEC>
__global__ __launch_bounds__(256) void tile_softmax_from_lse_kernel(const float* logits, const float* lse_row, uint16_t* probs,
                                                                    int64_t n_vec, int k_t) {
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v >= n_vec) return;
    const int64_t e = v * VEC;
    const float lse = lse_row[e / k_t];
    if constexpr (VEC == 8) {
        const float4 a = *reinterpret_cast<const float4*>(logits + e);
        const float4 b = *reinterpret_cast<const float4*>(logits + e + 4);
        u32x4 w;
        w[0] = pack_bf16(__expf(a.x - lse), __expf(a.y - lse));
        w[1] = pack_bf16(__expf(a.z - lse), __expf(a.w - lse));
        w[2] = pack_bf16(__expf(b.x - lse), __expf(b.y - lse));
        w[3] = pack_bf16(__expf(b.z - lse), __expf(b.w - lse));
        *reinterpret_cast<u32x4*>(probs + e) = w;
    } else {
        probs[e] = (uint16_t)(pack_bf16(__expf(logits[e] - lse), 0.f) & 0xffffu);
    }
}

// out[bh,qi] = log(sum_k exp(logits - max_k)) + max_k, one wavefront per row, the maximum starting from
// -FLT_MAX as in the reference (an empty or all -inf row gives -inf: exp(-inf + FLT_MAX) = 0, log(0) = -inf).
__global__ __launch_bounds__(256) void tile_lse_from_logits_kernel(const float* logits, float* out, int64_t rows, int k_t) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* x = logits + row * k_t;
    const bool vec = (k_t % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
    // one pass: every lane keeps a running maximum and the sum of exp(x - that maximum), rescaled when the maximum
    // moves; the lanes are combined at the end
    float mx = -FLT_MAX, sum = 0.f;
    auto take4 = [&](const float4 f) {
        const float m4 = fmaxf(fmaxf(f.x, f.y), fmaxf(f.z, f.w));
        if (m4 > mx) {
            sum *= __expf(mx - m4);
            mx = m4;
        }
        sum += (__expf(f.x - mx) + __expf(f.y - mx)) + (__expf(f.z - mx) + __expf(f.w - mx));
    };
    if (vec) {
        int k = 4 * lane;
        for (; k + 768 < k_t; k += 1024) {              // four loads in flight per lane
            const float4 f0 = *reinterpret_cast<const float4*>(x + k);
            const float4 f1 = *reinterpret_cast<const float4*>(x + k + 256);
            const float4 f2 = *reinterpret_cast<const float4*>(x + k + 512);
            const float4 f3 = *reinterpret_cast<const float4*>(x + k + 768);
            take4(f0);
            take4(f1);
            take4(f2);
            take4(f3);
        }
        for (; k < k_t; k += 256) take4(*reinterpret_cast<const float4*>(x + k));
    } else {
        for (int k = lane; k < k_t; k += 64) {
            const float v = x[k];
            if (v > mx) {
                sum *= __expf(mx - v);
                mx = v;
            }
            sum += __expf(v - mx);
        }
    }
    float all = mx;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) all = fmaxf(all, __shfl_xor(all, off));
    sum *= __expf(mx - all);          // a lane that saw nothing has sum 0
    mx = all;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0) out[row] = __logf(sum) + mx;
}

// lse[i] = log(exp(lse[i]) + exp(tile[i])), max-shifted; two -inf give -inf (the reference's expression is NaN there,
// its callers use the finite -1e30 instead of -inf)
__global__ __launch_bounds__(256) void tile_lse_merge_kernel(float* lse_row, const float* tile_lse_row, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float a = lse_row[i], b = tile_lse_row[i];
    const float m = fmaxf(a, b);
    lse_row[i] = (m == -INFINITY) ? -INFINITY : m + __logf(__expf(a - m) + __expf(b - m));
}

__device__ __forceinline__ uint32_t tile_xorshift32(uint32_t x) {
    x ^= x << 13;
    x ^= x >> 17;
    x ^= x << 5;
    return x;
}

// the reference's counter-based uniform in [0,1): 24 bits of one xorshift32 round of a hash of (seed, bh, qi, kj)
// (sdpa_kernels.cu:18-33); qi and kj are the coordinates inside the tile
__device__ __forceinline__ float tile_uniform01(uint64_t seed, int bh, int qi, int kj) {
    const uint32_t s = (uint32_t)seed ^ (1103515245u * (((uint32_t)bh * 73856093u) ^ ((uint32_t)qi * 19349663u) ^ ((uint32_t)kj * 83492791u)));
    return (float)(tile_xorshift32(s) & 0x00FFFFFFu) / 16777216.0f;
}

// probs = u < p ? 0 : bf16(float(probs) * (1 / (1 - p))), in place
template <int VEC>
__global__ __launch_bounds__(256) void tile_dropout_kernel(uint16_t* probs, float p, float scale, uint64_t seed, int64_t n_vec, int q_t, int k_t) {
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v >= n_vec) return;
    const int64_t e = v * VEC;
    const int kj = (int)(e % k_t);
    const int qi = (int)((e / k_t) % q_t);
    const int bh = (int)(e / ((int64_t)k_t * q_t));
    auto one = [&](uint16_t bits, int i) -> float {
        const float val = __uint_as_float((uint32_t)bits << 16);
        return tile_uniform01(seed, bh, qi, kj + i) < p ? 0.0f : val * scale;
    };
    if constexpr (VEC == 8) {
        u32x4 w = *reinterpret_cast<const u32x4*>(probs + e);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            w[j] = pack_bf16(one((uint16_t)(w[j] & 0xffffu), 2 * j), one((uint16_t)(w[j] >> 16), 2 * j + 1));
        *reinterpret_cast<u32x4*>(probs + e) = w;
    } else {
        probs[e] = (uint16_t)(pack_bf16(one(probs[e], 0), 0.f) & 0xffffu);
    }
}

}  // namespace fattn
