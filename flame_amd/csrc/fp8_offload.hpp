// BF16 <-> FP8 E4M3 conversion of saved activations on their way to and from pinned host memory: the pair the
// reference's activation offload pool runs on its transfer stream (src/cuda/fp8_quant.cu:19-72,
// src/cuda/fp8_dequant.cu:10-39; used by src/activation_offload.rs:536-586, :678-700 with the fixed scale 8/448).
// Byte work bound by HBM: 3 bytes move per element in either direction.  16 elements per lane and step (two 16-byte
// loads, one 16-byte store, or the reverse), grid-stride over the tensor, scalar code for the last n % 16 elements
// and for pointers that are not 16-byte aligned.
//
// The codes are the reference's, bit for bit, including where they differ from OCP E4M3:
//   * encode(x) = code of |x * inv_scale| after clamping to 448, sign bit from `product < 0`;
//   * the 3-bit mantissa is rounded half up in magnitude (not to even);
//   * products of 256 and above all give 0x7F: the encoder saturates one binade early (biased exponent >= 15), so
//     the codes 0x78..0x7E are never written, and the decoder reads 0x7F as 480 (it has no NaN), not 448;
//   * below 2^-6 the mantissa is floor(product * 512 + 0.5) in fp32, capped at 7 (a product that rounds up to the
//     smallest normal stays at the largest subnormal);
//   * the reference is compiled with flush-to-zero (build.rs:261, :295 pass --use_fast_math): denormal inputs and
//     denormal products count as +0 in the encoder (code 0x00 even for negative inputs), and a denormal product in
//     the decoder becomes a zero with the code's sign;
//   * -0.0 encodes as 0x00 (`-0.0 < 0` is false); NaN is not specified by the reference (it reads the exponent
//     frexpf leaves unset) and gives sign | 0x7F here.
// The arithmetic is done on the bit patterns: for a normal product the reference's frexpf / round / carry sequence
// equals adding half a step (1 << 19) to the 23-bit fraction and letting the carry run into the exponent.
// The host passes scales that are themselves below 2^-126 as zero (flush-to-zero applies to both operands).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fattn {

// Branch-free: every element costs the same dozen vector instructions whatever its range.
//   normal range (product >= 2^-6): (bits + half a mantissa step) >> 20 is exponent and rounded 3-bit mantissa in one
//   number, a carry out of the mantissa raising the exponent; minus the bias difference (127 - 7) << 3.  Everything
//   from 0x78 up (248 and above after rounding, the clamp to 448, infinity, NaN) is 0x7F.
//   below 2^-6: floor(product * 512 + 0.5) with the sum rounded once in fp32, capped at 7.
//   a product below 2^-126 (or a denormal input) is zero, without a sign.
__device__ __forceinline__ uint32_t fp8_encode_bf16(uint32_t bf16_bits, float inv_scale) {
    const uint32_t pu = __float_as_uint(__uint_as_float(bf16_bits << 16) * inv_scale);
    const uint32_t u = pu & 0x7fffffffu;
    uint32_t code_n = ((u + (1u << 19)) >> 20) - (120u << 3);
    code_n = code_n >= 0x78u ? 0x7fu : code_n;
    const uint32_t code_s = min((uint32_t)(__uint_as_float(u) * 512.0f + 0.5f), 7u);
    const uint32_t code = (u >= 0x3c800000u ? code_n : code_s) | ((pu >> 24) & 0x80u);
    const bool zero = (u < 0x00800000u) | ((bf16_bits & 0x7f80u) == 0);
    return zero ? 0u : code;
}

__device__ __forceinline__ uint32_t f32_to_bf16_rne(float f) {
    const uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ uint32_t fp8_decode_bf16(uint32_t code, float scale) {
    const uint32_t sign = (code & 0x80u) << 24;
    const uint32_t exp = (code >> 3) & 0xfu, mant = code & 7u;
    float v;
    if (exp == 0) v = (float)mant * 0.001953125f;                // mant / 8 * 2^-6
    else v = __uint_as_float(((exp + 120u) << 23) | (mant << 20));
    float p = __uint_as_float(__float_as_uint(v) | sign) * scale;
    if ((__float_as_uint(p) & 0x7f800000u) == 0) p = __uint_as_float(__float_as_uint(p) & 0x80000000u);   // flushed
    return f32_to_bf16_rne(p);
}

struct Fp8Params {
    const void* in;
    void* out;
    float scale;        // inv_scale for the encoder, scale for the decoder
    size_t n;
};

template <bool VEC>
__global__ __launch_bounds__(256) void bf16_to_fp8_kernel(const Fp8Params p) {
    const uint16_t* in = static_cast<const uint16_t*>(p.in);
    uint8_t* out = static_cast<uint8_t*>(p.out);
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t nthreads = (size_t)gridDim.x * blockDim.x;
    size_t done = 0;
    if (VEC) {
        const size_t nvec = p.n / 16;
        for (size_t i = tid; i < nvec; i += nthreads) {
            const uint4 a = reinterpret_cast<const uint4*>(in)[2 * i];
            const uint4 b = reinterpret_cast<const uint4*>(in)[2 * i + 1];
            const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t c0 = fp8_encode_bf16(w[2 * j] & 0xffffu, p.scale), c1 = fp8_encode_bf16(w[2 * j] >> 16, p.scale);
                const uint32_t c2 = fp8_encode_bf16(w[2 * j + 1] & 0xffffu, p.scale), c3 = fp8_encode_bf16(w[2 * j + 1] >> 16, p.scale);
                o[j] = c0 | (c1 << 8) | (c2 << 16) | (c3 << 24);
            }
            reinterpret_cast<uint4*>(out)[i] = make_uint4(o[0], o[1], o[2], o[3]);
        }
        done = nvec * 16;
    }
    for (size_t i = done + tid; i < p.n; i += nthreads) out[i] = (uint8_t)fp8_encode_bf16(in[i], p.scale);
}

// The decoder reads a 256-entry table of finished bf16 values that each workgroup builds for the launch's scale (one
// entry per lane): one LDS read per element in place of the decode arithmetic.
template <bool VEC>
__global__ __launch_bounds__(256) void fp8_to_bf16_kernel(const Fp8Params p) {
    __shared__ uint16_t lut[256];
    lut[threadIdx.x] = (uint16_t)fp8_decode_bf16(threadIdx.x, p.scale);
    __syncthreads();
    const uint8_t* in = static_cast<const uint8_t*>(p.in);
    uint16_t* out = static_cast<uint16_t*>(p.out);
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t nthreads = (size_t)gridDim.x * blockDim.x;
    size_t done = 0;
    if (VEC) {
        const size_t nvec = p.n / 16;
        for (size_t i = tid; i < nvec; i += nthreads) {
            const uint4 a = reinterpret_cast<const uint4*>(in)[i];
            const uint32_t w[4] = {a.x, a.y, a.z, a.w};
            uint32_t o[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                o[2 * j] = (uint32_t)lut[w[j] & 0xffu] | ((uint32_t)lut[(w[j] >> 8) & 0xffu] << 16);
                o[2 * j + 1] = (uint32_t)lut[(w[j] >> 16) & 0xffu] | ((uint32_t)lut[w[j] >> 24] << 16);
            }
            reinterpret_cast<uint4*>(out)[2 * i] = make_uint4(o[0], o[1], o[2], o[3]);
            reinterpret_cast<uint4*>(out)[2 * i + 1] = make_uint4(o[4], o[5], o[6], o[7]);
        }
        done = nvec * 16;
    }
    for (size_t i = done + tid; i < p.n; i += nthreads) out[i] = lut[in[i]];
}

}  // namespace fattn
