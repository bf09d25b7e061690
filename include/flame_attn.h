/* placeholder while the kernels come up; replaced by the full header */
#ifndef FLAME_ATTN_H
#define FLAME_ATTN_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif
#define FLAME_ATTN_OK 0
#define FLAME_ATTN_ERR_INVALID (-1)
#define FLAME_ATTN_ERR_UNSUPPORTED (-2)
enum { FLAME_ATTN_KERNEL_FWD = 0, FLAME_ATTN_KERNEL_BWD_PREP = 1, FLAME_ATTN_KERNEL_BWD_DKDV = 2,
       FLAME_ATTN_KERNEL_BWD_DQ = 3, FLAME_ATTN_KERNEL_SAGE_KMEAN = 4, FLAME_ATTN_KERNEL_SAGE_QUANT = 5,
       FLAME_ATTN_KERNEL_SAGE_FWD = 6, FLAME_ATTN_N_KERNEL_KINDS = 8 };
typedef struct { double total_ms[FLAME_ATTN_N_KERNEL_KINDS]; int launches[FLAME_ATTN_N_KERNEL_KINDS]; } FlameAttnKernelTimes;
int flame_attn_profiling_enable(int on);
int flame_attn_profiling_read(FlameAttnKernelTimes* out);
int flame_attn_fwd_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                        int B, int H, int N_q, int N_kv, int D, float scale,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides,
                        int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                        int causal, const int32_t* kv_len,
                        const uint8_t* keep_mask, const int64_t* mask_strides,
                        void* stream);
int flame_sage_quant_qk_int8(const void* Q, const void* K, int B, int H, int N_q, int N_kv, int D,
                             const int64_t* q_strides, const int64_t* k_strides, int64_t q_off, int64_t k_off,
                             int smooth_k, void* Qi8, void* Ki8, void* q_scales, void* k_scales, void* k_mean,
                             void* stream);
int flame_sage_attn_fwd_int8(const void* Qi8, const void* Ki8, const void* q_scales, const void* k_scales,
                             const void* V, void* O, void* LSE, int B, int H, int N_q, int N_kv, int D,
                             float scale, const int64_t* v_strides, const int64_t* o_strides,
                             int64_t v_off, int64_t o_off, int causal, const int32_t* kv_len, void* stream);
size_t flame_attn_bwd_workspace_bytes(int B, int H, int N_q, int D);
int flame_attn_bwd_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                        const void* LSE, void* dQ, void* dK, void* dV,
                        int B, int H, int N_q, int N_kv, int D, float scale,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                        const int64_t* dk_strides, const int64_t* dv_strides,
                        int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                        int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                        int causal, const int32_t* kv_len,
                        const uint8_t* keep_mask, const int64_t* mask_strides,
                        void* workspace, size_t workspace_bytes, void* stream);
#ifdef __cplusplus
}
#endif
#endif
