// Shared device helpers for the gfx950 (CDNA4) attention kernels: 64-lane wavefronts,
// v_mfma_f32_32x32x16_bf16 fragments, bf16 packing.  Compiled for gfx950 only.
#pragma once
#include <type_traits>
#include <utility>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fattn {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---------------------------------------------------------------------------------------------
// v_mfma_f32_32x32x16_bf16:  D[32x32] += A[32x16] * B[16x32]
//   lane l, half h = l/32, n = l%32
//   A operand: 8 bf16 = A[n][8h .. 8h+7]        (row n, eight consecutive k)
//   B operand: 8 bf16 = B[8h .. 8h+7][n]        (column n, eight consecutive k)
//   C/D      : 16 f32, register r holds D[8*(r/4) + 4h + (r%4)][n]
// Because the k positions of A and B only have to agree with each other, any fixed permutation of
// the contraction index may be applied to both operands.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// The same MFMA with the accumulator pinned to the architectural VGPRs, for kernels that also keep
// long-lived accumulators in the accumulation registers: the compiler picks one MFMA form per function,
// and with the accumulation form every value the vector ALU wants to read costs a v_accvgpr_read.
// Emitted by hand, so the compiler's hazard bookkeeping does not see it.  The caller must keep at
// least two other MFMAs between the last of these writing an accumulator and the first vector-ALU
// instruction that touches it (the result of an 8-pass MFMA is visible 11 issue cycles after issue).
// The B operand is held in the accumulation registers: operands that live for a whole kernel (a
// workgroup's own K / V fragments) then cost no architectural VGPRs.
// GUARD: two wait states in front, for kernel variants in which the register allocator moves an operand (part of an
// accumulator it has split, a fragment) into place right before the statement: an MFMA may read a register the vector
// ALU wrote two wait states later at the earliest, and the compiler keeps that distance only for its own MFMAs.
template <bool GUARD = false>
__device__ __forceinline__ void mfma32_vgpr_first_bacc(f32x16& acc, bf16x8 a, bf16x8 b) {
    if constexpr (GUARD) asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "a"(b));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "a"(b));
}
template <bool GUARD = false>
__device__ __forceinline__ void mfma32_vgpr_bacc(f32x16& acc, bf16x8 a, bf16x8 b) {
    if constexpr (GUARD) asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(b));
    else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(b));
}
// Both operands in architectural registers (a kernel whose B fragments are too many for the accumulation file's
// free part).  After the last MFMA of a chain, mfma32_vgpr_settle spends the 11 wait states before its result may be
// read, for kernels that have no other MFMAs to put there.
// The two wait states in front: an operand the register allocator moved into place just before the statement was
// written by the vector ALU, and an MFMA may read such a register two wait states later at the earliest (the compiler
// keeps that distance for its own MFMAs, not for these).
__device__ __forceinline__ void mfma32_vgpr(f32x16& acc, bf16x8 a, bf16x8 b) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma32_vgpr_settle(f32x16& acc) {
    asm volatile("s_nop 11" : "+v"(acc));
}
// ---------------------------------------------------------------------------------------------
// Fixed accumulation registers.  Inline assembly can only name a physical register by a literal, so the two
// register maps are written out once, here, and every statement below is generated from them; each row is checked
// against the rule it follows at compile time, so a wrong number does not build.
//   B slots:    slot s holds a 16-byte MFMA operand in a[128 + 4 s : 131 + 4 s]
//   acc tuples: tuple t holds a 32x32 fp32 accumulator block in a[16 t : 16 t + 15]
// ---------------------------------------------------------------------------------------------
#define FATTN_B_SLOTS(X) \
    X(0, 128, 129, 130, 131) \
    X(1, 132, 133, 134, 135) \
    X(2, 136, 137, 138, 139) \
    X(3, 140, 141, 142, 143) \
    X(4, 144, 145, 146, 147) \
    X(5, 148, 149, 150, 151) \
    X(6, 152, 153, 154, 155) \
    X(7, 156, 157, 158, 159) \
    X(8, 160, 161, 162, 163) \
    X(9, 164, 165, 166, 167) \
    X(10, 168, 169, 170, 171) \
    X(11, 172, 173, 174, 175) \
    X(12, 176, 177, 178, 179) \
    X(13, 180, 181, 182, 183) \
    X(14, 184, 185, 186, 187) \
    X(15, 188, 189, 190, 191) \
    X(16, 192, 193, 194, 195) \
    X(17, 196, 197, 198, 199) \
    X(18, 200, 201, 202, 203) \
    X(19, 204, 205, 206, 207) \
    X(20, 208, 209, 210, 211) \
    X(21, 212, 213, 214, 215) \
    X(22, 216, 217, 218, 219) \
    X(23, 220, 221, 222, 223) \
    X(24, 224, 225, 226, 227) \
    X(25, 228, 229, 230, 231) \
    X(26, 232, 233, 234, 235) \
    X(27, 236, 237, 238, 239) \
    X(28, 240, 241, 242, 243) \
    X(29, 244, 245, 246, 247) \
    X(30, 248, 249, 250, 251) \
    X(31, 252, 253, 254, 255)
#define FATTN_ACC_TUPLES(X) \
    X(0, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15) \
    X(1, 16, 17, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28, 29, 30, 31) \
    X(2, 32, 33, 34, 35, 36, 37, 38, 39, 40, 41, 42, 43, 44, 45, 46, 47) \
    X(3, 48, 49, 50, 51, 52, 53, 54, 55, 56, 57, 58, 59, 60, 61, 62, 63) \
    X(4, 64, 65, 66, 67, 68, 69, 70, 71, 72, 73, 74, 75, 76, 77, 78, 79) \
    X(5, 80, 81, 82, 83, 84, 85, 86, 87, 88, 89, 90, 91, 92, 93, 94, 95) \
    X(6, 96, 97, 98, 99, 100, 101, 102, 103, 104, 105, 106, 107, 108, 109, 110, 111) \
    X(7, 112, 113, 114, 115, 116, 117, 118, 119, 120, 121, 122, 123, 124, 125, 126, 127)
#define FATTN_STR_(x) #x
#define FATTN_STR(x) FATTN_STR_(x)
#define FATTN_AREG(r) "a" FATTN_STR(r)
#define FATTN_ARANGE(lo, hi) "{a[" FATTN_STR(lo) ":" FATTN_STR(hi) "]}"
#define FATTN_CHECK_B_SLOT(I, R0, R1, R2, R3) \
    static_assert(R0 == 128 + 4 * I && R1 == R0 + 1 && R2 == R0 + 2 && R3 == R0 + 3, "row of FATTN_B_SLOTS")
#define FATTN_CHECK_ACC_TUPLE(I, R0, R1, R2, R3, R4, R5, R6, R7, R8, R9, R10, R11, R12, R13, R14, R15)                          \
    static_assert(R0 == 16 * I && R1 == R0 + 1 && R2 == R0 + 2 && R3 == R0 + 3 && R4 == R0 + 4 && R5 == R0 + 5 && R6 == R0 + 6 && \
                  R7 == R0 + 7 && R8 == R0 + 8 && R9 == R0 + 9 && R10 == R0 + 10 && R11 == R0 + 11 && R12 == R0 + 12 &&           \
                  R13 == R0 + 13 && R14 == R0 + 14 && R15 == R0 + 15, "row of FATTN_ACC_TUPLES")

// The same with the B operand pinned to accumulation registers a[128 + 4 SLOT : 131 + 4 SLOT], for a
// kernel whose 32 resident B fragments must stay put there (left to itself the register allocator
// homes some of them in architectural registers and copies them over before every use).
// MODE 0: acc = a b; 1: acc += a b; 2: acc = c + a b.
template <int SLOT, int MODE>
__device__ __forceinline__ void mfma32_vgpr_bpinned(f32x16& acc, bf16x8 a, bf16x8 b, const f32x16& c) {
    static_assert(SLOT >= 0 && SLOT < 32, "32 pinned fragments");
#define FATTN_PIN(I, R0, R1, R2, R3)                                                                                                        \
    FATTN_CHECK_B_SLOT(I, R0, R1, R2, R3);                                                                                                  \
    if constexpr (SLOT == I) {                                                                                                              \
        if constexpr (MODE == 0) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), FATTN_ARANGE(R0, R3)(b));     \
        if constexpr (MODE == 1) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), FATTN_ARANGE(R0, R3)(b));     \
        if constexpr (MODE == 2) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(acc) : "v"(a), FATTN_ARANGE(R0, R3)(b), "v"(c)); \
    }
    FATTN_B_SLOTS(FATTN_PIN)
#undef FATTN_PIN
}

// The int8 counterpart (v_mfma_i32_32x32x32_i8: D[32x32] += A[32x32] * B[32x32], 16 consecutive int8 of the
// contraction per lane and operand, int32 accumulators in architectural VGPRs), same pinned B slots; the B
// value is the 128-bit carrier that pin_b_fragment returned.
template <int SLOT, int MODE>
__device__ __forceinline__ void mfma32i8_vgpr_bpinned(i32x16& acc, u32x4 a, bf16x8 b, const i32x16& c) {
    static_assert(SLOT >= 0 && SLOT < 32, "32 pinned fragments");
#define FATTN_PIN(I, R0, R1, R2, R3)                                                                                                      \
    if constexpr (SLOT == I) {                                                                                                            \
        if constexpr (MODE == 0) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), FATTN_ARANGE(R0, R3)(b));     \
        if constexpr (MODE == 1) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc) : "v"(a), FATTN_ARANGE(R0, R3)(b));     \
        if constexpr (MODE == 2) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %3" : "=&v"(acc) : "v"(a), FATTN_ARANGE(R0, R3)(b), "v"(c)); \
    }
    FATTN_B_SLOTS(FATTN_PIN)
#undef FATTN_PIN
}

// Moves a fragment into its pinned accumulation registers (the value the MFMAs above are given).
template <int SLOT>
__device__ __forceinline__ bf16x8 pin_b_fragment(u32x4 w) {
    bf16x8 out;
#define FATTN_PIN(I, R0, R1, R2, R3)                                                                                       \
    if constexpr (SLOT == I)                                                                                               \
        asm volatile("v_accvgpr_write_b32 " FATTN_AREG(R0) ", %1\n\tv_accvgpr_write_b32 " FATTN_AREG(R1) ", %2\n\t"        \
                     "v_accvgpr_write_b32 " FATTN_AREG(R2) ", %3\n\tv_accvgpr_write_b32 " FATTN_AREG(R3) ", %4"             \
                     : "=" FATTN_ARANGE(R0, R3)(out) : "v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3]));
    FATTN_B_SLOTS(FATTN_PIN)
#undef FATTN_PIN
    return out;
}

// acc *= alpha for an accumulator tuple pinned to a[16 IDX : 16 IDX + 15], one register at a time through a
// single architectural register: rescaling accumulators that live in the accumulation registers
// through compiler-generated copies needs dozens of temporaries and ended in scratch spills.
template <int IDX>
__device__ __forceinline__ void rescale_pinned(f32x16& acc, float alpha) {
    static_assert(IDX >= 0 && IDX < 8, "eight pinned accumulator tuples");
    float tmp;
    // one register: read, multiply, one wait state, write back
#define FATTN_RS(r) "v_accvgpr_read_b32 %1, " FATTN_AREG(r) "\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 " FATTN_AREG(r) ", %1"
#define FATTN_PIN(I, R0, R1, R2, R3, R4, R5, R6, R7, R8, R9, R10, R11, R12, R13, R14, R15)                                      \
    FATTN_CHECK_ACC_TUPLE(I, R0, R1, R2, R3, R4, R5, R6, R7, R8, R9, R10, R11, R12, R13, R14, R15);                             \
    if constexpr (IDX == I)                                                                                                     \
        asm volatile(FATTN_RS(R0) "\n\t" FATTN_RS(R1) "\n\t" FATTN_RS(R2) "\n\t" FATTN_RS(R3) "\n\t" FATTN_RS(R4) "\n\t"        \
                     FATTN_RS(R5) "\n\t" FATTN_RS(R6) "\n\t" FATTN_RS(R7) "\n\t" FATTN_RS(R8) "\n\t" FATTN_RS(R9) "\n\t"        \
                     FATTN_RS(R10) "\n\t" FATTN_RS(R11) "\n\t" FATTN_RS(R12) "\n\t" FATTN_RS(R13) "\n\t" FATTN_RS(R14) "\n\t"   \
                     FATTN_RS(R15)                                                                                              \
                     : "+" FATTN_ARANGE(R0, R15)(acc), "=&v"(tmp) : "v"(alpha));
    FATTN_ACC_TUPLES(FATTN_PIN)
#undef FATTN_PIN
#undef FATTN_RS
}

// acc += a b with the accumulator pinned to a[16 IDX : 16 IDX + 15] (the tuples rescale_pinned works on) and both
// operands in architectural registers, emitted by hand: given the same fixed registers at every use, the accumulator
// never moves (left to the compiler's MFMA form, accumulators that a conditional rescale also touches travelled
// through architectural registers once per key tile).  Two wait states in front, as in mfma32_vgpr: the B operand may
// have been written, or moved into place, by the vector ALU just before.  mfma32_apinned_settle<IDX, WAIT> is the fence before the
// accumulators are read after the last tile: the one with WAIT spends the 11 wait states, and since volatile
// statements keep their order, fencing every accumulator after it orders all their reads behind that wait.
template <int IDX>
__device__ __forceinline__ void mfma32_apinned(f32x16& acc, bf16x8 a, bf16x8 b) {
    static_assert(IDX >= 0 && IDX < 8, "eight pinned accumulator tuples");
#define FATTN_PIN(I, R0, R1, R2, R3, R4, R5, R6, R7, R8, R9, R10, R11, R12, R13, R14, R15)                          \
    if constexpr (IDX == I) {                                                                                       \
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+" FATTN_ARANGE(R0, R15)(acc) : "v"(a), "v"(b)); \
    }
    FATTN_ACC_TUPLES(FATTN_PIN)
#undef FATTN_PIN
}
template <int IDX, bool WAIT>
__device__ __forceinline__ void mfma32_apinned_settle(f32x16& acc) {
    static_assert(IDX >= 0 && IDX < 8, "eight pinned accumulator tuples");
#define FATTN_PIN(I, R0, R1, R2, R3, R4, R5, R6, R7, R8, R9, R10, R11, R12, R13, R14, R15)     \
    if constexpr (IDX == I) {                                                                  \
        if constexpr (WAIT) asm volatile("s_nop 11" : "+" FATTN_ARANGE(R0, R15)(acc));         \
        else asm volatile("" : "+" FATTN_ARANGE(R0, R15)(acc));                                \
    }
    FATTN_ACC_TUPLES(FATTN_PIN)
#undef FATTN_PIN
}

// compile-time loop: f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int, N - 1>{})
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// row index inside a 32x32 accumulator block for register r of a lane in half h
__device__ __forceinline__ constexpr int acc_row(int r, int h) { return 8 * (r >> 2) + 4 * h + (r & 3); }

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 v = {lo, hi};
    bf16x2 b = __builtin_convertvector(v, bf16x2);   // v_cvt_pk_bf16_f32, round-to-nearest-even
    return __builtin_bit_cast(uint32_t, b);
}

// Waits until at most N of this wavefront's LDS reads are outstanding (they return in order); the vector
// memory and export counters are left alone.
template <int N>
__device__ __forceinline__ void wait_lds_reads() {
    static_assert(N >= 0 && N < 16, "lgkmcnt is a 4-bit field");
    __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8));
}

__device__ __forceinline__ bf16x8 pack8(float a0, float a1, float a2, float a3, float a4, float a5, float a6,
                                        float a7) {
    u32x4 u = {pack_bf16(a0, a1), pack_bf16(a2, a3), pack_bf16(a4, a5), pack_bf16(a6, a7)};
    return __builtin_bit_cast(bf16x8, u);
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }   // v_exp_f32
__device__ __forceinline__ float log2_fast(float x) { return __builtin_amdgcn_logf(x); }    // v_log_f32

// exchange with the lane 32 positions away (the other half of the wave)
__device__ __forceinline__ float xhalf(float x) { return __shfl_xor(x, 32, 64); }

// 16-byte global load of 8 bf16, zero when the predicate is false
__device__ __forceinline__ u32x4 ldg16(const uint16_t* p, bool ok) {
    u32x4 z = {0u, 0u, 0u, 0u};
    return ok ? *reinterpret_cast<const u32x4*>(p) : z;
}

typedef short s16x4 __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i receives element (i%4) of the four
// 8-byte rows addressed by lanes i/4, i/4+4, i/4+8, i/4+12 of the group.  When lane r of a group
// points at &X[k0 + r/4][c0 + 4*(r%4)] of a row-major tile X, lane i therefore receives
// X[k0+0..3][c0+i]: the group transposes a 4(k) x 16(column) block so that every lane ends up with
// four consecutive contraction elements of its own column.
__device__ __forceinline__ u32x2 lds_read_tr16(const uint16_t* p) {
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
    return __builtin_bit_cast(u32x2, v);
}

// 16-byte-granule XOR swizzle of a row-major bf16 tile whose rows are D*2 bytes (no padding).
// 16 consecutive rows get distinct bank groups for the same logical granule, and 4 consecutive rows
// land in 4 disjoint 64-byte bank groups: both access patterns used by the kernels (16-byte row
// reads, transposing 8-byte reads of a 4-row x 64-byte block) are conflict-free on the 64-bank LDS.
template <int D>
__device__ __forceinline__ constexpr int swz(int row) {
    return D == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
}

// One wave-wide asynchronous copy global -> LDS: lane l delivers 16 (or 4) bytes to lds_dst + 16*l (4*l).
// The destination must be wave-uniform (it travels in M0).  Completion is tracked by vmcnt only, and
// the caller waits explicitly (wait_vm0 + barrier) before anyone reads the destination.
// The instruction is emitted by hand: when the compiler knows of a pending LDS-DMA it turns every
// following LDS-read wait into a full drain (lgkmcnt(0)), which defeats the read-ahead pipelines of
// the kernels.  Hidden from its wait-count bookkeeping, LDS reads of *other* buffers keep their exact
// counts.  Compiler-issued vmcnt waits stay correct: extra outstanding operations only make a
// counted wait stricter.
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)p);
}
// destination given as a wave-uniform LDS byte address
__device__ __forceinline__ void dma16(const void* gsrc, uint32_t lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(lds_byte_addr), "v"(gsrc) : "m0", "memory");
}
__device__ __forceinline__ void dma4(const void* gsrc, uint32_t lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" :: "s"(lds_byte_addr), "v"(gsrc) : "m0", "memory");
}
// ... and the source split into a wave-uniform base and a non-negative per-lane byte offset
__device__ __forceinline__ void dma16u(const void* gbase_wave_uniform, uint32_t lane_byte_off, uint32_t lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_byte_addr), "v"(lane_byte_off), "s"(gbase_wave_uniform) : "m0", "memory");
}
// The same copies in two halves, for software pipelines that place another instruction (an MFMA)
// between them instead of the s_nop: writing M0 and reading it in an LDS-DMA need one wait state.
// Nothing that writes M0 may come between the two halves.
__device__ __forceinline__ void dma_set_dst(uint32_t lds_byte_addr) {
    asm volatile("s_mov_b32 m0, %0" :: "s"(lds_byte_addr) : "m0");
}
__device__ __forceinline__ void dma16u_issue(const void* gbase_wave_uniform, uint32_t lane_byte_off) {
    asm volatile("global_load_lds_dwordx4 %0, %1" :: "v"(lane_byte_off), "s"(gbase_wave_uniform) : "memory");
}
__device__ __forceinline__ void dma4u_issue(const void* gbase_wave_uniform, uint32_t lane_byte_off) {
    asm volatile("global_load_lds_dword %0, %1" :: "v"(lane_byte_off), "s"(gbase_wave_uniform) : "memory");
}
// destination given as a pointer into LDS (wave-uniform)
__device__ __forceinline__ void dma16(const void* gsrc, void* lds_dst) { dma16(gsrc, lds_addr(lds_dst)); }
__device__ __forceinline__ void dma4(const void* gsrc, void* lds_dst) { dma4(gsrc, lds_addr(lds_dst)); }
__device__ __forceinline__ void dma16u(const void* gbase_wave_uniform, uint32_t lane_byte_off, void* lds_dst) {
    dma16u(gbase_wave_uniform, lane_byte_off, lds_addr(lds_dst));
}
__device__ __forceinline__ void wait_vm0() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0) only

// Workgroups are dealt to the 8 XCDs (each with its own L2) round-robin by linear id.  Remap the id
// so that XCD x works on the contiguous range [x*total/8, (x+1)*total/8) of tiles: all tiles of one
// (batch, head) then share one L2 and its K/V (forward) or Q/dO (backward) stay resident there.
__device__ __forceinline__ int xcd_remap(int linear, int total) {
    constexpr int kXcd = 8;
    return (total % kXcd == 0) ? (linear % kXcd) * (total / kXcd) + linear / kXcd : linear;
}
// The same for batches whose sequences differ in length (per-batch key lengths): contiguous ranges would hand
// whole batches, the long ones and the short ones, to different XCDs.  Here XCD x takes the (batch, head)
// slices x, x + 8, x + 16, ...: every slice still stays in one L2, and the heads of one batch are spread
// over all XCDs.  `per_head`: tiles per (batch, head) slice; the id runs slice-major.
__device__ __forceinline__ int xcd_remap_heads(int linear, int total, int per_head) {
    constexpr int kXcd = 8;
    const int n_heads = total / per_head;
    if (n_heads % kXcd != 0) return xcd_remap(linear, total);
    const int x = linear % kXcd, j = linear / kXcd;
    return ((j / per_head) * kXcd + x) * per_head + j % per_head;
}

// Causal problems: the key walk of query unit qt grows with qt, and workgroups start in id order, so the longest
// walks must come first or they finish alone at the end.  Within the contiguous range of units that one XCD
// works through (whole heads where the counts allow), the order becomes: last unit of every head, then the
// units before them, and so on.  `wg`: unit id after xcd_remap, head-major; returns (qt, head) through refs.
__device__ __forceinline__ void causal_longest_first(int wg, int n_qt, int total, int& qt, int& bh) {
    const int per_xcd = (total % 8 == 0) ? total / 8 : total;
    if (per_xcd % n_qt == 0) {
        const int heads = per_xcd / n_qt;
        const int base = wg / per_xcd * per_xcd, j = wg - base;
        qt = n_qt - 1 - j / heads;
        bh = base / n_qt + j % heads;
    } else {
        qt = n_qt - 1 - wg % n_qt;
        bh = wg / n_qt;
    }
}

struct Strides {
    int64_t b, h, n;   // element strides of a [B,H,N,D] bf16 view; the D stride is 1
};

// Head dims below the compiled one (any multiple of 8, e.g. 96 on the 128-wide kernels) run zero-padded:
// fragments loaded straight from global memory are zero past the real head dim, tile copies re-read
// granule 0 of their row there (finite values that only ever meet those zero operands, or land in
// output rows past the real head dim, which are not stored), and stores skip those rows.
__device__ __forceinline__ int src_granule(int c, int d_real) { return c * 8 < d_real ? c : 0; }

// The 64 keep-mask bytes of one query row over a 64-key tile, as loaded by the kernels whose lanes own
// a query: keep(kb, r) is the byte of key 32*kb + acc_row(r, h).
struct MaskRow64 {
    u32x4 w[4];
    __device__ __forceinline__ void load(const uint8_t* row_tile) {
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = *reinterpret_cast<const u32x4*>(row_tile + 16 * j);
    }
    // Clears the bytes of the keys at or past `limit` (relative to the first key of the tile): key-length and
    // causal exclusions then need no test of their own per element.  Meant for the few tiles they cut.
    __device__ __forceinline__ void restrict_to(int limit) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int c = min(max(limit - 4 * i, 0), 4);                  // bytes of dword i that stay
            const uint32_t m = c >= 4 ? 0xffffffffu : ((1u << (8 * c)) - 1u);
            w[i >> 2][i & 3] &= m;
        }
    }
    __device__ __forceinline__ bool keep(int kb, int r, int h) const {      // kb, r compile-time; h per lane
        const int d0 = 8 * kb + 2 * (r >> 2);                               // dword of the even half
        const uint32_t lo = w[d0 >> 2][d0 & 3], hi = w[(d0 + 1) >> 2][(d0 + 1) & 3];
        const uint32_t word = h ? hi : lo;
        return (word & (0xffu << (8 * (r & 3)))) != 0;
    }
};

enum MaskMode : int {
    kMaskU8 = 0,             // uint8, non-zero attends
    kMaskBf16Keep = 1,       // bf16, a value below 0.5 excludes (the public keep-mask convention of the reference)
    kMaskBf16Drop = 2,       // bf16, a value above 0.5 excludes (the convention of the reference's streaming entry point)
};

struct MaskArgs {
    const int32_t* kv_len;   // [B] or null
    const uint8_t* mask;     // explicit mask or null; element type and meaning per mask_mode
    int64_t sb, sh, sq, sk;  // element strides over (b,h,q,k); 0 broadcasts
    int causal;              // key j > query i is excluded
    int rows16 = 0;          // uint8 keep-mask rows are contiguous along keys and 16-byte aligned (vector loads allowed)
    int mask_mode = kMaskU8;
    // additive bias on the scaled logits (forward only), fp32 or bf16, or null
    const void* bias = nullptr;
    int64_t bb = 0, bh = 0, bq = 0, bk = 0;   // element strides over (b,h,q,k); 0 broadcasts
    int bias_f32 = 1;
    float inv_scale = 1.f;   // 1 / softmax scale: the bias is folded into the raw scores as bias / scale
    // dropout of the probabilities (kernels instantiated with DROPOUT only): see drop_factor
    uint32_t drop_seed = 0;  // low 32 bits of the seed
    uint32_t drop_thr = 0;   // ceil(p * 2^24): an element is kept when its 24-bit uniform is >= this
    float drop_scale = 1.f;  // 1 / (1 - p)
    uint32_t drop_cq = 0, drop_ck = 0;   // tiles of a chunked draw along queries and keys; drop_cq = 0: one draw over the tensor
};

// Factor that dropout applies to the probability of flat element index idx of the [B*H, Sq, Sk] probability tensor
// (low 32 bits): 0 or 1 / (1 - p).  The uniform is the reference's (src/rng/mod.rs:14-24, drawn over the whole
// tensor by src/autograd_v4/ops/sdpa.rs:229-231, :604-649): u = (xorshift32(seed ^ idx) >> 8) / 2^24, kept when
// u >= p, which in integers is (xorshift32(seed ^ idx) >> 8) >= ceil(p * 2^24).
__device__ __forceinline__ float drop_factor(const MaskArgs& m, uint32_t idx) {
    uint32_t s = m.drop_seed ^ idx;
    s ^= s << 13;
    s ^= s >> 17;
    s ^= s << 5;
    return (s >> 8) >= m.drop_thr ? m.drop_scale : 0.f;
}

// The same for element (bh, qi, key) when the reference's operator is chunked (src/autograd_v4/ops/sdpa.rs:180-199,
// :444): it draws per tile of drop_cq x drop_ck (the last ones shorter) over the tile's own [B*H, q_t, k_t] tensor,
// under the seed derive_tile_seed gives (:600-602), whose low word is seed + k_offset (the query offset is shifted
// out of it).  drop_cq = 0 is the draw over the whole tensor.
__device__ __forceinline__ float drop_factor_at(const MaskArgs& m, uint32_t bh, uint32_t qi, uint32_t key, uint32_t Sq, uint32_t Sk) {
    if (m.drop_cq == 0) return drop_factor(m, (bh * Sq + qi) * Sk + key);
    const uint32_t qo = qi / m.drop_cq * m.drop_cq, ko = key / m.drop_ck * m.drop_ck;
    const uint32_t qt = min(m.drop_cq, Sq - qo), kt = min(m.drop_ck, Sk - ko);
    uint32_t s = (m.drop_seed + ko) ^ ((bh * qt + (qi - qo)) * kt + (key - ko));
    s ^= s << 13;
    s ^= s >> 17;
    s ^= s << 5;
    return (s >> 8) >= m.drop_thr ? m.drop_scale : 0.f;
}

// one element of an explicit mask, addressed in elements from the (batch, head) base: does it attend?
__device__ __forceinline__ bool mask_attends(const MaskArgs& m, const uint8_t* base, int64_t elem) {
    if (m.mask_mode == kMaskU8) return base[elem] != 0;
    const float v = __builtin_bit_cast(float, (uint32_t)reinterpret_cast<const uint16_t*>(base)[elem] << 16);
    return m.mask_mode == kMaskBf16Keep ? !(v < 0.5f) : !(v > 0.5f);
}
// (batch, head) base of an explicit mask
__device__ __forceinline__ const uint8_t* mask_head_base(const MaskArgs& m, int b, int hh) {
    return m.mask + (b * m.sb + hh * m.sh) * (m.mask_mode == kMaskU8 ? 1 : 2);
}

}  // namespace fattn
