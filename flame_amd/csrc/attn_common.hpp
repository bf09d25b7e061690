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
// The same with the B operand pinned to accumulation registers a[128 + 4 SLOT : 131 + 4 SLOT], for a
// kernel whose 32 resident B fragments must stay put there (left to itself the register allocator
// homes some of them in architectural registers and copies them over before every use).
// MODE 0: acc = a b; 1: acc += a b; 2: acc = c + a b.
template <int SLOT, int MODE>
__device__ __forceinline__ void mfma32_vgpr_bpinned(f32x16& acc, bf16x8 a, bf16x8 b, const f32x16& c) {
    static_assert(SLOT >= 0 && SLOT < 32, "32 pinned fragments");
#define FATTN_PIN(I, R)                                                                                                  \
    if constexpr (SLOT == I) {                                                                                           \
        if constexpr (MODE == 0) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), R(b));     \
        if constexpr (MODE == 1) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), R(b));     \
        if constexpr (MODE == 2) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(acc) : "v"(a), R(b), "v"(c)); \
    }
    FATTN_PIN(0, "{a[128:131]}")
    FATTN_PIN(1, "{a[132:135]}")
    FATTN_PIN(2, "{a[136:139]}")
    FATTN_PIN(3, "{a[140:143]}")
    FATTN_PIN(4, "{a[144:147]}")
    FATTN_PIN(5, "{a[148:151]}")
    FATTN_PIN(6, "{a[152:155]}")
    FATTN_PIN(7, "{a[156:159]}")
    FATTN_PIN(8, "{a[160:163]}")
    FATTN_PIN(9, "{a[164:167]}")
    FATTN_PIN(10, "{a[168:171]}")
    FATTN_PIN(11, "{a[172:175]}")
    FATTN_PIN(12, "{a[176:179]}")
    FATTN_PIN(13, "{a[180:183]}")
    FATTN_PIN(14, "{a[184:187]}")
    FATTN_PIN(15, "{a[188:191]}")
    FATTN_PIN(16, "{a[192:195]}")
    FATTN_PIN(17, "{a[196:199]}")
    FATTN_PIN(18, "{a[200:203]}")
    FATTN_PIN(19, "{a[204:207]}")
    FATTN_PIN(20, "{a[208:211]}")
    FATTN_PIN(21, "{a[212:215]}")
    FATTN_PIN(22, "{a[216:219]}")
    FATTN_PIN(23, "{a[220:223]}")
    FATTN_PIN(24, "{a[224:227]}")
    FATTN_PIN(25, "{a[228:231]}")
    FATTN_PIN(26, "{a[232:235]}")
    FATTN_PIN(27, "{a[236:239]}")
    FATTN_PIN(28, "{a[240:243]}")
    FATTN_PIN(29, "{a[244:247]}")
    FATTN_PIN(30, "{a[248:251]}")
    FATTN_PIN(31, "{a[252:255]}")
#undef FATTN_PIN
}

// The int8 counterpart (v_mfma_i32_32x32x32_i8: D[32x32] += A[32x32] * B[32x32], 16 consecutive int8 of the
// contraction per lane and operand, int32 accumulators in architectural VGPRs), same pinned B slots; the B
// value is the 128-bit carrier that pin_b_fragment returned.
template <int SLOT, int MODE>
__device__ __forceinline__ void mfma32i8_vgpr_bpinned(i32x16& acc, u32x4 a, bf16x8 b, const i32x16& c) {
    static_assert(SLOT >= 0 && SLOT < 32, "32 pinned fragments");
#define FATTN_PIN(I, R)                                                                                                  \
    if constexpr (SLOT == I) {                                                                                           \
        if constexpr (MODE == 0) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), R(b));     \
        if constexpr (MODE == 1) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc) : "v"(a), R(b));     \
        if constexpr (MODE == 2) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %3" : "=&v"(acc) : "v"(a), R(b), "v"(c)); \
    }
    FATTN_PIN(0, "{a[128:131]}")
    FATTN_PIN(1, "{a[132:135]}")
    FATTN_PIN(2, "{a[136:139]}")
    FATTN_PIN(3, "{a[140:143]}")
    FATTN_PIN(4, "{a[144:147]}")
    FATTN_PIN(5, "{a[148:151]}")
    FATTN_PIN(6, "{a[152:155]}")
    FATTN_PIN(7, "{a[156:159]}")
    FATTN_PIN(8, "{a[160:163]}")
    FATTN_PIN(9, "{a[164:167]}")
    FATTN_PIN(10, "{a[168:171]}")
    FATTN_PIN(11, "{a[172:175]}")
    FATTN_PIN(12, "{a[176:179]}")
    FATTN_PIN(13, "{a[180:183]}")
    FATTN_PIN(14, "{a[184:187]}")
    FATTN_PIN(15, "{a[188:191]}")
    FATTN_PIN(16, "{a[192:195]}")
    FATTN_PIN(17, "{a[196:199]}")
    FATTN_PIN(18, "{a[200:203]}")
    FATTN_PIN(19, "{a[204:207]}")
    FATTN_PIN(20, "{a[208:211]}")
    FATTN_PIN(21, "{a[212:215]}")
    FATTN_PIN(22, "{a[216:219]}")
    FATTN_PIN(23, "{a[220:223]}")
    FATTN_PIN(24, "{a[224:227]}")
    FATTN_PIN(25, "{a[228:231]}")
    FATTN_PIN(26, "{a[232:235]}")
    FATTN_PIN(27, "{a[236:239]}")
    FATTN_PIN(28, "{a[240:243]}")
    FATTN_PIN(29, "{a[244:247]}")
    FATTN_PIN(30, "{a[248:251]}")
    FATTN_PIN(31, "{a[252:255]}")
#undef FATTN_PIN
}

// Moves a fragment into its pinned accumulation registers (the value the MFMAs above are given).
template <int SLOT>
__device__ __forceinline__ bf16x8 pin_b_fragment(u32x4 w) {
    bf16x8 out;
#define FATTN_PIN(I, C, R0, R1, R2, R3)                                                                        \
    if constexpr (SLOT == I)                                                                                   \
        asm volatile("v_accvgpr_write_b32 " R0 ", %1\n\tv_accvgpr_write_b32 " R1 ", %2\n\t"                    \
                     "v_accvgpr_write_b32 " R2 ", %3\n\tv_accvgpr_write_b32 " R3 ", %4"                         \
                     : C(out) : "v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3]));
    FATTN_PIN(0, "={a[128:131]}", "a128", "a129", "a130", "a131")
    FATTN_PIN(1, "={a[132:135]}", "a132", "a133", "a134", "a135")
    FATTN_PIN(2, "={a[136:139]}", "a136", "a137", "a138", "a139")
    FATTN_PIN(3, "={a[140:143]}", "a140", "a141", "a142", "a143")
    FATTN_PIN(4, "={a[144:147]}", "a144", "a145", "a146", "a147")
    FATTN_PIN(5, "={a[148:151]}", "a148", "a149", "a150", "a151")
    FATTN_PIN(6, "={a[152:155]}", "a152", "a153", "a154", "a155")
    FATTN_PIN(7, "={a[156:159]}", "a156", "a157", "a158", "a159")
    FATTN_PIN(8, "={a[160:163]}", "a160", "a161", "a162", "a163")
    FATTN_PIN(9, "={a[164:167]}", "a164", "a165", "a166", "a167")
    FATTN_PIN(10, "={a[168:171]}", "a168", "a169", "a170", "a171")
    FATTN_PIN(11, "={a[172:175]}", "a172", "a173", "a174", "a175")
    FATTN_PIN(12, "={a[176:179]}", "a176", "a177", "a178", "a179")
    FATTN_PIN(13, "={a[180:183]}", "a180", "a181", "a182", "a183")
    FATTN_PIN(14, "={a[184:187]}", "a184", "a185", "a186", "a187")
    FATTN_PIN(15, "={a[188:191]}", "a188", "a189", "a190", "a191")
    FATTN_PIN(16, "={a[192:195]}", "a192", "a193", "a194", "a195")
    FATTN_PIN(17, "={a[196:199]}", "a196", "a197", "a198", "a199")
    FATTN_PIN(18, "={a[200:203]}", "a200", "a201", "a202", "a203")
    FATTN_PIN(19, "={a[204:207]}", "a204", "a205", "a206", "a207")
    FATTN_PIN(20, "={a[208:211]}", "a208", "a209", "a210", "a211")
    FATTN_PIN(21, "={a[212:215]}", "a212", "a213", "a214", "a215")
    FATTN_PIN(22, "={a[216:219]}", "a216", "a217", "a218", "a219")
    FATTN_PIN(23, "={a[220:223]}", "a220", "a221", "a222", "a223")
    FATTN_PIN(24, "={a[224:227]}", "a224", "a225", "a226", "a227")
    FATTN_PIN(25, "={a[228:231]}", "a228", "a229", "a230", "a231")
    FATTN_PIN(26, "={a[232:235]}", "a232", "a233", "a234", "a235")
    FATTN_PIN(27, "={a[236:239]}", "a236", "a237", "a238", "a239")
    FATTN_PIN(28, "={a[240:243]}", "a240", "a241", "a242", "a243")
    FATTN_PIN(29, "={a[244:247]}", "a244", "a245", "a246", "a247")
    FATTN_PIN(30, "={a[248:251]}", "a248", "a249", "a250", "a251")
    FATTN_PIN(31, "={a[252:255]}", "a252", "a253", "a254", "a255")
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
    if constexpr (IDX == 0)
        asm volatile("v_accvgpr_read_b32 %1, a0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a0, %1\n\tv_accvgpr_read_b32 %1, a1\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a1, %1\n\tv_accvgpr_read_b32 %1, a2\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a2, %1\n\tv_accvgpr_read_b32 %1, a3\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a3, %1\n\tv_accvgpr_read_b32 %1, a4\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a4, %1\n\tv_accvgpr_read_b32 %1, a5\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a5, %1\n\tv_accvgpr_read_b32 %1, a6\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a6, %1\n\tv_accvgpr_read_b32 %1, a7\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a7, %1\n\tv_accvgpr_read_b32 %1, a8\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a8, %1\n\tv_accvgpr_read_b32 %1, a9\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a9, %1\n\tv_accvgpr_read_b32 %1, a10\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a10, %1\n\tv_accvgpr_read_b32 %1, a11\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a11, %1\n\tv_accvgpr_read_b32 %1, a12\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a12, %1\n\tv_accvgpr_read_b32 %1, a13\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a13, %1\n\tv_accvgpr_read_b32 %1, a14\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a14, %1\n\tv_accvgpr_read_b32 %1, a15\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a15, %1" : "+{a[0:15]}"(acc), "=&v"(tmp) : "v"(alpha));
    if constexpr (IDX == 1)
        asm volatile("v_accvgpr_read_b32 %1, a16\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a16, %1\n\tv_accvgpr_read_b32 %1, a17\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a17, %1\n\tv_accvgpr_read_b32 %1, a18\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a18, %1\n\tv_accvgpr_read_b32 %1, a19\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a19, %1\n\tv_accvgpr_read_b32 %1, a20\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a20, %1\n\tv_accvgpr_read_b32 %1, a21\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a21, %1\n\tv_accvgpr_read_b32 %1, a22\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a22, %1\n\tv_accvgpr_read_b32 %1, a23\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a23, %1\n\tv_accvgpr_read_b32 %1, a24\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a24, %1\n\tv_accvgpr_read_b32 %1, a25\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a25, %1\n\tv_accvgpr_read_b32 %1, a26\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a26, %1\n\tv_accvgpr_read_b32 %1, a27\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a27, %1\n\tv_accvgpr_read_b32 %1, a28\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a28, %1\n\tv_accvgpr_read_b32 %1, a29\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a29, %1\n\tv_accvgpr_read_b32 %1, a30\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a30, %1\n\tv_accvgpr_read_b32 %1, a31\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a31, %1" : "+{a[16:31]}"(acc), "=&v"(tmp) : "v"(alpha));
    if constexpr (IDX == 2)
        asm volatile("v_accvgpr_read_b32 %1, a32\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a32, %1\n\tv_accvgpr_read_b32 %1, a33\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a33, %1\n\tv_accvgpr_read_b32 %1, a34\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a34, %1\n\tv_accvgpr_read_b32 %1, a35\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a35, %1\n\tv_accvgpr_read_b32 %1, a36\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a36, %1\n\tv_accvgpr_read_b32 %1, a37\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a37, %1\n\tv_accvgpr_read_b32 %1, a38\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a38, %1\n\tv_accvgpr_read_b32 %1, a39\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a39, %1\n\tv_accvgpr_read_b32 %1, a40\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a40, %1\n\tv_accvgpr_read_b32 %1, a41\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a41, %1\n\tv_accvgpr_read_b32 %1, a42\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a42, %1\n\tv_accvgpr_read_b32 %1, a43\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a43, %1\n\tv_accvgpr_read_b32 %1, a44\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a44, %1\n\tv_accvgpr_read_b32 %1, a45\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a45, %1\n\tv_accvgpr_read_b32 %1, a46\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a46, %1\n\tv_accvgpr_read_b32 %1, a47\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a47, %1" : "+{a[32:47]}"(acc), "=&v"(tmp) : "v"(alpha));
    if constexpr (IDX == 3)
        asm volatile("v_accvgpr_read_b32 %1, a48\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a48, %1\n\tv_accvgpr_read_b32 %1, a49\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a49, %1\n\tv_accvgpr_read_b32 %1, a50\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a50, %1\n\tv_accvgpr_read_b32 %1, a51\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a51, %1\n\tv_accvgpr_read_b32 %1, a52\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a52, %1\n\tv_accvgpr_read_b32 %1, a53\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a53, %1\n\tv_accvgpr_read_b32 %1, a54\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a54, %1\n\tv_accvgpr_read_b32 %1, a55\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a55, %1\n\tv_accvgpr_read_b32 %1, a56\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a56, %1\n\tv_accvgpr_read_b32 %1, a57\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a57, %1\n\tv_accvgpr_read_b32 %1, a58\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a58, %1\n\tv_accvgpr_read_b32 %1, a59\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a59, %1\n\tv_accvgpr_read_b32 %1, a60\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a60, %1\n\tv_accvgpr_read_b32 %1, a61\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a61, %1\n\tv_accvgpr_read_b32 %1, a62\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a62, %1\n\tv_accvgpr_read_b32 %1, a63\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a63, %1" : "+{a[48:63]}"(acc), "=&v"(tmp) : "v"(alpha));
    if constexpr (IDX == 4)
        asm volatile("v_accvgpr_read_b32 %1, a64\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a64, %1\n\tv_accvgpr_read_b32 %1, a65\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a65, %1\n\tv_accvgpr_read_b32 %1, a66\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a66, %1\n\tv_accvgpr_read_b32 %1, a67\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a67, %1\n\tv_accvgpr_read_b32 %1, a68\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a68, %1\n\tv_accvgpr_read_b32 %1, a69\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a69, %1\n\tv_accvgpr_read_b32 %1, a70\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a70, %1\n\tv_accvgpr_read_b32 %1, a71\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a71, %1\n\tv_accvgpr_read_b32 %1, a72\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a72, %1\n\tv_accvgpr_read_b32 %1, a73\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a73, %1\n\tv_accvgpr_read_b32 %1, a74\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a74, %1\n\tv_accvgpr_read_b32 %1, a75\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a75, %1\n\tv_accvgpr_read_b32 %1, a76\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a76, %1\n\tv_accvgpr_read_b32 %1, a77\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a77, %1\n\tv_accvgpr_read_b32 %1, a78\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a78, %1\n\tv_accvgpr_read_b32 %1, a79\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a79, %1" : "+{a[64:79]}"(acc), "=&v"(tmp) : "v"(alpha));
    if constexpr (IDX == 5)
        asm volatile("v_accvgpr_read_b32 %1, a80\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a80, %1\n\tv_accvgpr_read_b32 %1, a81\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a81, %1\n\tv_accvgpr_read_b32 %1, a82\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a82, %1\n\tv_accvgpr_read_b32 %1, a83\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a83, %1\n\tv_accvgpr_read_b32 %1, a84\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a84, %1\n\tv_accvgpr_read_b32 %1, a85\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a85, %1\n\tv_accvgpr_read_b32 %1, a86\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a86, %1\n\tv_accvgpr_read_b32 %1, a87\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a87, %1\n\tv_accvgpr_read_b32 %1, a88\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a88, %1\n\tv_accvgpr_read_b32 %1, a89\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a89, %1\n\tv_accvgpr_read_b32 %1, a90\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a90, %1\n\tv_accvgpr_read_b32 %1, a91\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a91, %1\n\tv_accvgpr_read_b32 %1, a92\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a92, %1\n\tv_accvgpr_read_b32 %1, a93\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a93, %1\n\tv_accvgpr_read_b32 %1, a94\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a94, %1\n\tv_accvgpr_read_b32 %1, a95\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a95, %1" : "+{a[80:95]}"(acc), "=&v"(tmp) : "v"(alpha));
    if constexpr (IDX == 6)
        asm volatile("v_accvgpr_read_b32 %1, a96\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a96, %1\n\tv_accvgpr_read_b32 %1, a97\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a97, %1\n\tv_accvgpr_read_b32 %1, a98\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a98, %1\n\tv_accvgpr_read_b32 %1, a99\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a99, %1\n\tv_accvgpr_read_b32 %1, a100\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a100, %1\n\tv_accvgpr_read_b32 %1, a101\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a101, %1\n\tv_accvgpr_read_b32 %1, a102\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a102, %1\n\tv_accvgpr_read_b32 %1, a103\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a103, %1\n\tv_accvgpr_read_b32 %1, a104\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a104, %1\n\tv_accvgpr_read_b32 %1, a105\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a105, %1\n\tv_accvgpr_read_b32 %1, a106\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a106, %1\n\tv_accvgpr_read_b32 %1, a107\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a107, %1\n\tv_accvgpr_read_b32 %1, a108\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a108, %1\n\tv_accvgpr_read_b32 %1, a109\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a109, %1\n\tv_accvgpr_read_b32 %1, a110\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a110, %1\n\tv_accvgpr_read_b32 %1, a111\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a111, %1" : "+{a[96:111]}"(acc), "=&v"(tmp) : "v"(alpha));
    if constexpr (IDX == 7)
        asm volatile("v_accvgpr_read_b32 %1, a112\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a112, %1\n\tv_accvgpr_read_b32 %1, a113\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a113, %1\n\tv_accvgpr_read_b32 %1, a114\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a114, %1\n\tv_accvgpr_read_b32 %1, a115\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a115, %1\n\tv_accvgpr_read_b32 %1, a116\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a116, %1\n\tv_accvgpr_read_b32 %1, a117\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a117, %1\n\tv_accvgpr_read_b32 %1, a118\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a118, %1\n\tv_accvgpr_read_b32 %1, a119\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a119, %1\n\tv_accvgpr_read_b32 %1, a120\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a120, %1\n\tv_accvgpr_read_b32 %1, a121\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a121, %1\n\tv_accvgpr_read_b32 %1, a122\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a122, %1\n\tv_accvgpr_read_b32 %1, a123\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a123, %1\n\tv_accvgpr_read_b32 %1, a124\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a124, %1\n\tv_accvgpr_read_b32 %1, a125\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a125, %1\n\tv_accvgpr_read_b32 %1, a126\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a126, %1\n\tv_accvgpr_read_b32 %1, a127\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 a127, %1" : "+{a[112:127]}"(acc), "=&v"(tmp) : "v"(alpha));
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
#define FATTN_PIN(I, R)                                                                                        \
    if constexpr (IDX == I) {                                                                                  \
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : R(acc) : "v"(a), "v"(b));          \
    }
    FATTN_PIN(0, "+{a[0:15]}")
    FATTN_PIN(1, "+{a[16:31]}")
    FATTN_PIN(2, "+{a[32:47]}")
    FATTN_PIN(3, "+{a[48:63]}")
    FATTN_PIN(4, "+{a[64:79]}")
    FATTN_PIN(5, "+{a[80:95]}")
    FATTN_PIN(6, "+{a[96:111]}")
    FATTN_PIN(7, "+{a[112:127]}")
#undef FATTN_PIN
}
template <int IDX, bool WAIT>
__device__ __forceinline__ void mfma32_apinned_settle(f32x16& acc) {
    static_assert(IDX >= 0 && IDX < 8, "eight pinned accumulator tuples");
#define FATTN_PIN(I, R)                                                                                        \
    if constexpr (IDX == I) {                                                                                  \
        if constexpr (WAIT) asm volatile("s_nop 11" : R(acc));                                                 \
        else asm volatile("" : R(acc));                                                                        \
    }
    FATTN_PIN(0, "+{a[0:15]}")
    FATTN_PIN(1, "+{a[16:31]}")
    FATTN_PIN(2, "+{a[32:47]}")
    FATTN_PIN(3, "+{a[48:63]}")
    FATTN_PIN(4, "+{a[64:79]}")
    FATTN_PIN(5, "+{a[80:95]}")
    FATTN_PIN(6, "+{a[96:111]}")
    FATTN_PIN(7, "+{a[112:127]}")
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
