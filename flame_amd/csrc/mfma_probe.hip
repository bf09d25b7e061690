// Measurement aid, not part of the attention library: a kernel that does nothing but bf16 MFMAs
// (v_mfma_f32_32x32x16_bf16, the instruction the attention kernels are built on) on operands taken from the
// caller's data, one or two wavefronts per SIMD on every compute unit.  bench.py --mfma-ceiling runs it with the
// MFMA count of each attention kernel: the time it takes is what the matrix pipe alone allows for that work at the
// clock the board grants such a load, which is the ceiling the attention kernels are compared with.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Each wavefront: `iters` rounds of 8 MFMAs on 4 independent accumulators and 8 operand fragments read once from
// `data` (16 bytes per lane and fragment; the values decide how many bits toggle, hence the power drawn).
__global__ __launch_bounds__(512) void mfma_loop_kernel(const u32x4* __restrict__ data, float* __restrict__ sink, int iters) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) & 1023;
    bf16x8 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i] = __builtin_bit_cast(bf16x8, data[(size_t)(wave * 8 + i) * 64 + lane]);
        b[i] = __builtin_bit_cast(bf16x8, data[(size_t)(wave * 8 + 4 + i) * 64 + lane]);
    }
    f32x16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j], b[j], acc[j], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(j + 1) & 3], b[(j + 2) & 3], acc[j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[j][r];
    if (s == 12345.678f) sink[0] = s;      // keeps the loop alive; never true for these inputs in practice
}

extern "C" {

// data: at least 1024 * 8 * 64 * 16 bytes (8 MiB) of bf16 values on the device.  workgroups x waves_per_wg wavefronts
// run iters x 8 MFMAs each.  Returns 0, -1 for bad arguments, else the hipError_t of the launch.
int flame_probe_mfma_loop(const void* data, void* sink, int workgroups, int waves_per_wg, int iters, void* stream) {
    if (!data || !sink || workgroups <= 0 || iters <= 0 || waves_per_wg <= 0 || waves_per_wg > 8) return -1;
    hipLaunchKernelGGL(mfma_loop_kernel, dim3((unsigned)workgroups), dim3(64u * (unsigned)waves_per_wg), 0,
                       static_cast<hipStream_t>(stream), static_cast<const u32x4*>(data), static_cast<float*>(sink), iters);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

size_t flame_probe_mfma_data_bytes(void) { return (size_t)1024 * 8 * 64 * 16; }

}  // extern "C"
