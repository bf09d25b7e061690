/* placeholder while the kernels come up; replaced by the full header */
#ifndef FLAME_ATTN_H
#define FLAME_ATTN_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif
#define FLAME_ATTN_OK 0
#define FLAME_ATTN_ERR_INVALID (-1)
#define FLAME_ATTN_ERR_UNSUPPORTED (-2)
int flame_attn_fwd_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                        int B, int H, int N_q, int N_kv, int D, float scale,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides,
                        int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                        int causal, const int32_t* kv_len,
                        const uint8_t* keep_mask, const int64_t* mask_strides,
                        void* stream);
#ifdef __cplusplus
}
#endif
#endif
