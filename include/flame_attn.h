/*
 * flame_attn.h -- C ABI of libflame_attn_hip.so, the gfx950 (MI355X) implementation of the
 * activation-memory-saving attention path of flame-core.
 *
 * What the library is: tiled QK^T -> online softmax -> PV forward that writes O and the per-row
 * log-sum-exp (never the Sq x Sk matrix), a backward that recomputes P tile by tile to form
 * dQ, dK, dV, and a SageAttention int8-QK inference forward.  Hand-written HIP for gfx950 only.
 *
 * Conventions shared by every entry point
 *   - tensors are device pointers owned by the caller; nothing is retained or freed by the callee
 *   - bf16 tensors are 4-D [B, H, N, D]; `*_strides` are four ELEMENT strides in (B, H, N, D) order,
 *     `*_off` / `*_offset_elems` are element offsets added to the base pointer.  The D stride must
 *     be 1, the other strides and the offsets multiples of 8 (16-byte rows), N strides below 2^24.
 *     This admits the DiT view reshape([B,N,H,D]).permute(0,2,1,3) without a copy
 *     (reference: src/sdpa.rs:607-621, :646-651).
 *   - D (head dim) is any multiple of 8 up to 128.  The kernels are compiled for 64 and 128 (the
 *     reference's production sizes, with 96: src/sdpa.rs:149, src/cuda/flash_attention_fwd.cu:307-324);
 *     other sizes, 96 included, run zero-padded to the next compiled size inside the tile loads and
 *     stores, at that size's cost.  The forward entry points also take multiples of 8 above 128, up
 *     to 512 (the reference serves those through its materialised path, src/sdpa.rs:483-587; e.g. the
 *     one-head D = 512 attention of a VAE mid block), in chunks of 128, when there is no keep-mask,
 *     bias or dropout and V has the head dim of Q; the backward does not (recompute through a
 *     materialised path there).  On a small problem at these head dims (at most 128 query-tile workgroups, at least
 *     512 keys) the keys can be split over workgroups, which needs room for fp32 partial outputs (at most 67 MB):
 *     flame_attn_fwd_ws_bf16 takes it from the caller (flame_attn_fwd_workspace_bytes), flame_attn_fwd_bf16 has no
 *     such argument and does not split, the reference-named entry points use a buffer the library keeps per
 *     (device, stream), as stated for flame_cudnn_sdpa_bwd_bf16.
 *     Anything else returns FLAME_ATTN_ERR_UNSUPPORTED.  The Sage and
 *     input-preparation entry points take 64 or 128 only.
 *   - LSE / Stats: fp32, contiguous [B*H, N_q] (== [B,H,N_q,1] with strides [H*N_q, N_q, 1, 1]),
 *     value = max_j s_ij + ln(sum_j exp(s_ij - max)), s = scale * Q K^T, natural log
 *     (reference: src/cuda/cudnn_sdpa.cpp:271-279, src/sdpa.rs:715-722).  A row with no attended
 *     key has LSE = -inf, O = 0 and zero gradients.
 *   - exclusions: `causal` excludes key j > query i (absolute indices, reference
 *     kernels/sdpa_kernels.cu:129-135); `kv_len` (int32 [B] on the device, may be null) excludes keys
 *     j >= kv_len[b]; `keep_mask` (uint8 on the device, may be null, non-zero = attend, reference
 *     src/sdpa.rs:458-470) is addressed with four element strides over (b, h, q, k), 0 = broadcast.
 *   - `stream` is a hipStream_t passed as void*; null = the default stream.  Every call only
 *     enqueues kernels: no host synchronisation, and no allocation except where stated.
 *   - return value: 0 on success, FLAME_ATTN_ERR_INVALID (-1) for null pointers / non-positive
 *     sizes / non-positive scale (reference: src/cuda/cudnn_sdpa.cpp:326-328),
 *     FLAME_ATTN_ERR_UNSUPPORTED (-2) for layouts or head sizes that are not built, otherwise the
 *     positive hipError_t of a failed launch.  Nothing is printed and nothing is thrown.
 */
#ifndef FLAME_ATTN_H
#define FLAME_ATTN_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLAME_ATTN_OK 0
#define FLAME_ATTN_ERR_INVALID (-1)
#define FLAME_ATTN_ERR_UNSUPPORTED (-2)
#define FLAME_ATTN_ERR_TOO_LARGE (-3)   /* flame_attn_bwd_bf16_noalloc only: more query rows than its fixed scratch holds */

/* Status enum of the reference's flame_* / fc_* family (cuda/include/flame_cuda_status.h:7-12). */
typedef enum {
    FLAME_ATTN_STATUS_OK = 0,
    FLAME_ATTN_STATUS_ERR_INVALID = 1,
    FLAME_ATTN_STATUS_ERR_UNSUPPORTED = 2,
    FLAME_ATTN_STATUS_ERR_HIP = 3
} FlameAttnStatus;

/* ------------------------------------------------------------------------------------------------
 * Primary entry points (extensions of the reference trio: causal flag, key lengths, keep-mask,
 * caller-provided workspace).
 * ---------------------------------------------------------------------------------------------- */

/* Forward.  LSE may be null (inference).  Replaces flame_cudnn_sdpa_bf16 /
 * flame_cudnn_sdpa_bf16_train_fwd (src/cuda/ffi.rs:609-666), flame_flash_attention_bf16
 * (src/cuda/ffi.rs:584-595) and the streaming / chunked fallbacks (src/cuda_ops_ffi.rs:199-221,
 * src/ffi/cuda_ffi.h:98-115, cuda/streaming_attn_bf16.h:7-17). */
int flame_attn_fwd_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                        int B, int H, int N_q, int N_kv, int D, float scale,
                        const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                        const int64_t* o_strides,
                        int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                        int causal, const int32_t* kv_len,
                        const uint8_t* keep_mask, const int64_t* mask_strides,
                        void* stream);

/* The same forward with a caller workspace (16-byte aligned device memory, used only during the call; null or too
 * small is accepted).  Only the forward for head dims above 128 on a grid that leaves compute units idle uses it, for
 * the fp32 partial outputs of workgroups that share a query tile and walk slices of the keys; with less room than
 * flame_attn_fwd_workspace_bytes returns it uses fewer slices, with none it runs unsplit.  Never allocates, so a first
 * call can be captured into a HIP graph (the reference's contract for code on the backward path:
 * src/cuda_graph.rs:11-18).  No counterpart in the reference's FFI. */
size_t flame_attn_fwd_workspace_bytes(int B, int H, int N_q, int N_kv, int D);
int flame_attn_fwd_ws_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                           int B, int H, int N_q, int N_kv, int D, float scale,
                           const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                           const int64_t* o_strides,
                           int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                           int causal, const int32_t* kv_len,
                           const uint8_t* keep_mask, const int64_t* mask_strides,
                           void* workspace, size_t workspace_bytes, void* stream);

/* Forward with an additive bias on the scaled logits: softmax(scale * Q K^T + bias) V, fp32 softmax.
 * bias: fp32 (FLAME_ATTN_DTYPE_F32) or bf16 device tensor read through four element strides over
 * (B,H,N_q,N_kv); a stride of 0 broadcasts that dimension ([1,H,Q,K] relative-position biases).
 * keep_mask may be given as well.  Inference only: there is no backward for the bias.
 * Replaces sdpa::forward_with_bias / attention::sdpa_with_bias (src/sdpa.rs:232-328,
 * src/attention/sdpa.rs:542-558), which materialise the fp32 score matrix. */
int flame_attn_fwd_bias_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                             int B, int H, int N_q, int N_kv, int D, float scale,
                             const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                             const int64_t* o_strides,
                             int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                             const void* bias, int bias_dtype, const int64_t* bias_strides,
                             const uint8_t* keep_mask, const int64_t* mask_strides,
                             void* stream);

/* Forward with dropout of the attention probabilities, as the reference's autograd_v4 operator draws it when it is
 * not chunked (SdpaConfig::dropout_p / dropout_seed, src/autograd_v4/ops/sdpa.rs:25-26, :229-231, :604-649; generator
 * src/rng/mod.rs:14-24): every element of the [B*H, N_q, N_kv] probability tensor with flat index i is kept when
 * (xorshift32(seed ^ i) >> 8) / 2^24 >= dropout_p (seed and i in their low 32 bits) and then multiplied by
 * 1 / (1 - dropout_p); the kept set is bit-identical to the reference's for the same seed.  O = (P * factor) V; LSE is
 * that of the undropped softmax, as the reference saves it.  0 <= dropout_p < 1 (else -1).
 * Arguments otherwise as flame_attn_fwd_bf16.  No counterpart in the reference's FFI: there the operator is a chain of
 * tensor operations. */
int flame_attn_fwd_dropout_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                int B, int H, int N_q, int N_kv, int D, float scale,
                                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                const int64_t* o_strides,
                                int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                                int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                float dropout_p, uint64_t dropout_seed, void* stream);
/* Its backward: dV = (P * factor)^T dO, dS = P * (factor * (dO V^T) - rowsum(dO * O)), dQ = scale dS K,
 * dK = scale dS^T Q with the same kept set, i.e. the derivative of the forward above (the reference's own backward,
 * src/autograd_v4/ops/sdpa.rs:756-772, forms dS without the factor P and is not reproduced).  O is the output of
 * flame_attn_fwd_dropout_bf16 with the same dropout_p and dropout_seed.  Arguments otherwise as flame_attn_bwd_bf16. */
int flame_attn_bwd_dropout_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                                const void* LSE, void* dQ, void* dK, void* dV,
                                int B, int H, int N_q, int N_kv, int D, float scale,
                                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                                const int64_t* dk_strides, const int64_t* dv_strides,
                                int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                                int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                                int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                float dropout_p, uint64_t dropout_seed,
                                void* workspace, size_t workspace_bytes, void* stream);
/* The same pair with the kept set the operator draws when it is chunked (save = SaveLSE and chunk_q < N_q or chunk_kv <
 * N_kv, src/autograd_v4/ops/sdpa.rs:180-199, :444): one draw per tile of draw_chunk_q x draw_chunk_kv (the last tiles
 * shorter) over the tile's own [B*H, q_t, k_t] tensor, under the seed derive_tile_seed gives (:600-602), whose low word
 * is dropout_seed + k_offset.  0, or a chunk of at least the sequence length, means the whole axis; with both whole this
 * is the pair above.  The attention itself is not chunked: only the kept set depends on the tiles.
 * Parity unpinned for one case: a seed whose low word is 0 (in the pair above: dropout_seed itself; here: the derived
 * seed of some tile, dropout_seed + k_offset wrapping to 0) makes the reference draw from its process-global generator
 * instead (src/rng/mod.rs:139-143, :187-193), so no fixed kept set exists for it there; this library draws with the 0. */
int flame_attn_fwd_dropout_tiled_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                      int B, int H, int N_q, int N_kv, int D, float scale,
                                      const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                      const int64_t* o_strides,
                                      int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                                      int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                      float dropout_p, uint64_t dropout_seed, int draw_chunk_q, int draw_chunk_kv, void* stream);
int flame_attn_bwd_dropout_tiled_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                                      const void* LSE, void* dQ, void* dK, void* dV,
                                      int B, int H, int N_q, int N_kv, int D, float scale,
                                      const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                      const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                                      const int64_t* dk_strides, const int64_t* dv_strides,
                                      int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                                      int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                                      int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                      float dropout_p, uint64_t dropout_seed, int draw_chunk_q, int draw_chunk_kv,
                                      void* workspace, size_t workspace_bytes, void* stream);

/* Recommended bytes of device scratch for the backward: two fp32 values per query row (required),
 * plus one 128-key block of fp32 dK/dV partial sums per compute unit of the current device
 * (optional: lets the dK/dV kernel split the key blocks of its last, partly filled scheduling round
 * over the idle compute units).  A workspace that only covers the row part is accepted. */
size_t flame_attn_bwd_workspace_bytes(int B, int H, int N_q, int D);

/* Backward from Q, K, V, the saved O and LSE, and the upstream gradient dO (bf16).  Writes bf16
 * dQ [B,H,N_q,D], dK, dV [B,H,N_kv,D] through their own strides.  `workspace` is 16-byte aligned
 * device memory, ideally of flame_attn_bwd_workspace_bytes(...) bytes, used only during the call.
 * Replaces flame_cudnn_sdpa_bwd_bf16 (src/cuda/ffi.rs:682-716) and the materialising recompute
 * attention_backward_recompute (src/autograd.rs:801-848); follows the arithmetic of
 * tests/cudnn_sdpa_bwd_parity.rs:31-98 with D_i = rowsum(dO * O). */
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

/* The same backward for callers that cannot allocate device memory and have no workspace to hand over:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart
 * in the reference.  The scratch is a fixed array in device memory that every GPU the library runs on
 * holds until the process ends (40 MiB: two fp32 rows for up to FLAME_ATTN_NOALLOC_MAX_ROWS query rows,
 * 32 MiB of fp32 dK/dV partial sums); the call allocates and frees nothing.
 * B * H * N_q above FLAME_ATTN_NOALLOC_MAX_ROWS returns FLAME_ATTN_ERR_TOO_LARGE and launches nothing.
 * All calls on one GPU share that array: calls that overlap on one GPU (different streams, or host
 * threads on different streams) race; calls on one stream are ordered and safe.  Nothing in the array
 * has to start at zero and nothing is kept between calls.  Results are bit-identical to
 * flame_attn_bwd_bf16 with a workspace of flame_attn_bwd_workspace_bytes(...) bytes. */
#define FLAME_ATTN_NOALLOC_MAX_ROWS (1 << 20)
int flame_attn_bwd_noalloc_max_rows(void);
int flame_attn_bwd_bf16_noalloc(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                                const void* LSE, void* dQ, void* dK, void* dV,
                                int B, int H, int N_q, int N_kv, int D, float scale,
                                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                                const int64_t* dk_strides, const int64_t* dv_strides,
                                int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                                int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                                int causal, const int32_t* kv_len,
                                const uint8_t* keep_mask, const int64_t* mask_strides, void* stream);

/* ------------------------------------------------------------------------------------------------
 * The materialised path: every shape the fused kernels refuse.  Any head dim D >= 1 (no multiple-of-8 rule, no
 * upper limit, D stride 1 and non-negative strides as the only layout rules), a value head dim Dv of its own,
 * causal flag, key lengths, keep-mask and (forward) additive bias as in the primary entry points, and the
 * backward for all of them.  It is what the reference does for these shapes (materialised scores through
 * library GEMMs: src/sdpa.rs:483-587, :788-961; backward src/autograd.rs:801-848): rocBLAS bf16 GEMMs with fp32
 * accumulation for Q K^T, P V and the four backward products (rocBLAS is loaded with dlopen on the first call,
 * which makes these two the only entry points that need it; FLAME_ATTN_ERR_UNSUPPORTED when it cannot be loaded),
 * this library's element-wise kernels in between.  The scores exist for one band of query rows at a time, in the
 * caller's workspace (8 bytes per score element of the band in the backward, 6 in the forward); what is kept
 * between forward and backward is O and LSE, as everywhere else.  flame_attn_materialised_workspace_bytes returns
 * the size with which the whole problem is one band or, for large problems, bands of about 512 MiB; any workspace
 * that holds 16 query rows is accepted (more bands).  The first call creates a rocBLAS handle per device, which
 * allocates: these entry points are not meant for graph capture.  Several times slower than the fused kernels
 * where both apply.  dropout_p, dropout_seed, draw_chunk_q, draw_chunk_kv: dropout of the probabilities as in
 * flame_attn_fwd_dropout_bf16 / flame_attn_fwd_dropout_tiled_bf16 (dropout_p = 0: none; draw_chunk_* = 0: one draw
 * over the whole tensor), the same kept set, the backward with the values the forward had.
 * ---------------------------------------------------------------------------------------------- */
size_t flame_attn_materialised_workspace_bytes(int B, int H, int N_q, int N_kv, int D, int Dv, int backward);
int flame_attn_fwd_materialised_bf16(const void* Q, const void* K, const void* V, void* O, void* LSE,
                                     int B, int H, int N_q, int N_kv, int D, int Dv, float scale,
                                     const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                     const int64_t* o_strides,
                                     int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t lse_off,
                                     int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                     const void* bias, int bias_dtype, const int64_t* bias_strides,
                                     float dropout_p, uint64_t dropout_seed, int draw_chunk_q, int draw_chunk_kv,
                                     void* workspace, size_t workspace_bytes, void* stream);
int flame_attn_bwd_materialised_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                                     const void* LSE, void* dQ, void* dK, void* dV,
                                     int B, int H, int N_q, int N_kv, int D, int Dv, float scale,
                                     const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                     const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                                     const int64_t* dk_strides, const int64_t* dv_strides,
                                     int64_t q_off, int64_t k_off, int64_t v_off, int64_t o_off, int64_t do_off,
                                     int64_t lse_off, int64_t dq_off, int64_t dk_off, int64_t dv_off,
                                     int causal, const int32_t* kv_len, const uint8_t* keep_mask, const int64_t* mask_strides,
                                     float dropout_p, uint64_t dropout_seed, int draw_chunk_q, int draw_chunk_kv,
                                     void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------
 * SageAttention int8-QK inference variant (API shape: src/sage_attention.rs:21-65; quantiser closed
 * form: src/sage_attention.rs:524-541; block granularity, K mean smoothing and int8 MFMA are new).
 * ---------------------------------------------------------------------------------------------- */

/* k_mean[b,h,c] = float(fp64 sum_t K[b,h,t,c] / N_kv) (0 when smooth_k == 0);
 * Ks = bf16(float(K) - k_mean);  per 128-row block of Q and per 64-row block of Ks:
 * scale = absmax / 127 (IEEE fp32 division), code = clamp(rint(x / scale), -128, 127), scale 0 -> 0.
 * Outputs are contiguous: Qi8 [B,H,N_q,Dr], Ki8 [B,H,N_kv,Dr] int8; q_scales [B,H,ceil(N_q/128)],
 * k_scales [B,H,ceil(N_kv/64)], k_mean [B,H,Dr] fp32.  D: any multiple of 8 up to 128.  Dr is the row length the
 * forward below reads: 64 for D <= 64, else 128 (so Dr = D for the two compiled sizes); elements D .. Dr-1 of
 * every row are written as zero, which changes neither a block's maximum nor a logit. */
int flame_sage_quant_qk_int8(const void* Q, const void* K, int B, int H, int N_q, int N_kv, int D,
                             const int64_t* q_strides, const int64_t* k_strides, int64_t q_off, int64_t k_off,
                             int smooth_k, void* Qi8, void* Ki8, void* q_scales, void* k_scales, void* k_mean,
                             void* stream);

/* The same, and also writes the smoothed K that was quantised, Ks = bf16(float(K) - k_mean), contiguous bf16
 * [B,H,N_kv,Dr] (K_smoothed may be null; a backward reads it as a [B,H,N_kv,D] view with row stride Dr).  The reference saves this tensor for the backward of its Sage
 * operator (src/sage_attention.rs:138-144, key_smoothed); see flame_host.hpp sage_attention_backward. */
int flame_sage_quant_qk_int8_ks(const void* Q, const void* K, int B, int H, int N_q, int N_kv, int D,
                                const int64_t* q_strides, const int64_t* k_strides, int64_t q_off, int64_t k_off,
                                int smooth_k, void* Qi8, void* Ki8, void* q_scales, void* k_scales, void* k_mean,
                                void* K_smoothed, void* stream);

/* S = float(int32 Q^ K^^T) * sq * sk * scale on int8 MFMA, online softmax fp32, P bf16, O = P V
 * on bf16 MFMA.  LSE may be null.  Qi8 / Ki8 as the quantiser above wrote them (rows of Dr elements);
 * V and O are bf16 views of head dim D. */
int flame_sage_attn_fwd_int8(const void* Qi8, const void* Ki8, const void* q_scales, const void* k_scales,
                             const void* V, void* O, void* LSE, int B, int H, int N_q, int N_kv, int D,
                             float scale, const int64_t* v_strides, const int64_t* o_strides,
                             int64_t v_off, int64_t o_off, int causal, const int32_t* kv_len, void* stream);

/* The same with an additive bias on the dequantised, scaled logits (fp32 or bf16, four element strides
 * over (B,H,N_q,N_kv), 0 = broadcast; -inf excludes a position): the attention_mask argument of the
 * reference's SageAttention::forward, which it adds to the scores before the softmax
 * (src/sage_attention.rs:126-131). */
int flame_sage_attn_fwd_bias_int8(const void* Qi8, const void* Ki8, const void* q_scales, const void* k_scales,
                                  const void* V, void* O, void* LSE, int B, int H, int N_q, int N_kv, int D,
                                  float scale, const int64_t* v_strides, const int64_t* o_strides,
                                  int64_t v_off, int64_t o_off, int causal, const int32_t* kv_len,
                                  const void* bias, int bias_dtype, const int64_t* bias_strides, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Entry points with the reference's own names and argument lists: drop-in symbols for the
 * declarations in src/cuda/ffi.rs, src/cuda_ops_ffi.rs, src/ffi/cuda_ffi.h and
 * cuda/streaming_attn_bf16.h.  All are shims onto the primary entry points above.
 * ---------------------------------------------------------------------------------------------- */

/* src/cuda/ffi.rs:609-629 (implementation replaced: src/cuda/cudnn_sdpa.cpp:314-395). */
int flame_cudnn_sdpa_bf16(const void* Q, const void* K, const void* V, void* O,
                          int B, int H, int N_q, int N_kv, int D, float scale,
                          const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                          const int64_t* o_strides,
                          int64_t q_offset_elems, int64_t k_offset_elems, int64_t v_offset_elems,
                          int64_t o_offset_elems, void* stream);

/* src/cuda/ffi.rs:644-666 (src/cuda/cudnn_sdpa.cpp:405-484). */
int flame_cudnn_sdpa_bf16_train_fwd(const void* Q, const void* K, const void* V, void* O, void* Stats,
                                    int B, int H, int N_q, int N_kv, int D, float scale,
                                    const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                                    const int64_t* o_strides,
                                    int64_t q_offset_elems, int64_t k_offset_elems, int64_t v_offset_elems,
                                    int64_t o_offset_elems, int64_t stats_offset_elems, void* stream);

/* src/cuda/ffi.rs:682-716 (src/cuda/cudnn_sdpa_bwd.cpp:265-361).  The reference signature has no
 * workspace argument: this shim keeps one lazily grown scratch buffer per (device, stream), as the
 * reference's shim keeps a workspace per shape (src/cuda/cudnn_sdpa.cpp:204-212).  Calls on different
 * streams use different buffers and may overlap; host threads that share a stream are serialised while
 * they enqueue.  hipMalloc happens on the first call of a stream and on growth only; an outgrown buffer
 * is freed once its stream is idle.  Under a stream capture a call that would have to allocate returns
 * FLAME_ATTN_ERR_UNSUPPORTED and launches nothing (call once per shape before capturing, or use
 * flame_attn_bwd_bf16 / flame_attn_bwd_bf16_noalloc there).  The reference-named forward entry points
 * below take their scratch (head dims above 128 on a small grid only) from the same buffer. */
int flame_cudnn_sdpa_bwd_bf16(const void* Q, const void* K, const void* V, const void* O, const void* dO,
                              const void* Stats, void* dQ, void* dK, void* dV,
                              int B, int H, int N_q, int N_kv, int D, float scale,
                              const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                              const int64_t* o_strides, const int64_t* do_strides, const int64_t* dq_strides,
                              const int64_t* dk_strides, const int64_t* dv_strides,
                              int64_t q_offset_elems, int64_t k_offset_elems, int64_t v_offset_elems,
                              int64_t o_offset_elems, int64_t do_offset_elems, int64_t stats_offset_elems,
                              int64_t dq_offset_elems, int64_t dk_offset_elems, int64_t dv_offset_elems,
                              void* stream);

/* src/cuda/ffi.rs:584-595 (src/cuda/flash_attention_fwd.cu:352-366): contiguous [BH,N,HD],
 * scale = 1/sqrt(HD); LSE (may be null) is filled here, the reference left it unused. */
int flame_flash_attention_bf16(const void* Q, const void* K, const void* V, void* O, float* LSE,
                               int batch_heads, int seq_len_q, int seq_len_kv, int head_dim, void* stream);

/* src/ffi/cuda_ffi.h:98-115 (cuda/src/flame_sdpa_stub.cu:869-1379): contiguous tensors, optional bf16
 * keep-mask [B, mask_heads, Q, K] (< 0.5 excluded, flame_sdpa_stub.cu:793-802), read in place by the
 * kernel.  `workspace` is accepted and not used (the reference keeps its score chunks there,
 * flame_sdpa_stub.cu:973-976), so any size, including none, works.  V and out have head dim Dv, which
 * may differ from Dh (multiples of 8; Dh up to 128; Dv above 128 is served in column ranges of 128, the softmax being
 * independent of V: one forward per range). */
FlameAttnStatus flame_sdpa_chunked_bf16(const void* q, const void* k, const void* v, int B, int H, int Q, int K,
                                        int Dh, int Dv, float scale, int chunk, int causal, int mask_heads,
                                        const void* mask, void* out, void* workspace, uint64_t workspace_bytes,
                                        void* stream);

/* cuda/streaming_attn_bf16.h:7-17 (cuda/streaming_attn_bf16.cu:305-432): strided Q,K,V,O, causal,
 * key-padding mask uint8 [B,H,S] with 0 = excluded (streaming_attn_bf16.cu:164-170).  V and O have head
 * dim Dv, which may differ from Dh and exceed 128 (the reference's tests run Dh = 64 with Dv = 80 and 160,
 * tests/streaming_attn.rs:57-124, :298-411). */
int streaming_attn_bf16_fp32_launch(const void* Q, const void* K, const void* V, int B, int H, int S, int Dh, int Dv,
                                    long qB, long qH, long qS, long qD, long kB, long kH, long kS, long kD,
                                    long vB, long vH, long vS, long vD, void* O, long oB, long oH, long oS, long oD,
                                    float scale, int chunk_size, int causal, const uint8_t* k_pad_mask,
                                    void* stream);

/* src/cuda_ops_ffi.rs:199-221 (cuda/sdpa_stream_bf16.cu:180-413): contiguous Q, K, V, O.  attn_mask
 * (may be null) is bf16, addressed by the four element strides, 0 broadcasting heads or batches
 * (src/cuda_ops_bf16.rs:1848-1873); in this one entry point a value above 0.5 EXCLUDES the position
 * (cuda/sdpa_stream_bf16.cu:79-81, cuda/include/sdpa_stream_bf16.h:30-33).  What is not built is
 * reported as unsupported with a reason, which is the documented way for the caller to take its other
 * path (src/cuda_ops_bf16.rs:1955-2059). */
bool sdpa_stream_bf16_launch(const void* dQ, const void* dK, const void* dV, void* dO, int B, int H, int Q_len,
                             int K_len, int d, float scale, const void* attn_mask, int64_t mask_stride_ek,
                             int64_t mask_stride_eq, int64_t mask_stride_eh, int64_t mask_stride_eb, int head_tile,
                             int q_tile, int max_q_tile, void* stream, char* unsupported_reason, int reason_buflen);

/* ---- Launch-plan cache of flame_sdpa_chunked_bf16 (src/ffi/cuda_ffi.h:119-121, src/cuda_ops_ffi.rs:60-85 and
 * :308-310; implementation in the reference: cuda/src/flame_sdpa_stub.cu:38-650, :1080-1442).  The counters keep the
 * reference's names and order; "q chunk" is the query tile of a workgroup here (128 or 256 rows), "k chunk" the
 * key tile (64).  last_plan_source: 1 cache hit, 2 measured on this call, 3 taken from the rule, 4 forced by
 * FLAME_SDPA_QCHUNK.  Environment variables as in the reference (cuda/src/flame_sdpa_stub.cu:617-650). */
typedef struct FlameSdpaAutotuneStats {
    uint64_t env_forced, clamped, skipped, fallback, errors, cache_hits, cache_misses, tuned, last_q_chunk, last_k_chunk,
        cache_saved, cache_loads, cache_load_errors, cache_entries, last_candidate_count, last_best_time_ns,
        last_plan_source, last_shape_b, last_shape_h, last_shape_q, last_shape_k, last_shape_dh, last_shape_dv,
        last_shape_mask_heads, last_shape_causal;
} FlameSdpaAutotuneStats;
/* 0 on success, 1 (FLAME_ATTN_STATUS_ERR_INVALID, the reference's FLAME_CUDA_ERR_INVALID: cuda/src/flame_sdpa_stub.cu:1382-1385) for a null pointer. */
int flame_sdpa_autotune_get_stats(FlameSdpaAutotuneStats* out);
int flame_sdpa_autotune_reset_stats(void);
/* Writes the cache file now if persistence is on (FLAME_SDPA_AUTOTUNE_PERSIST=1) and the cache changed. */
int flame_sdpa_autotune_flush_cache(void);

/* ---- Element-wise primitives on score tiles, under the reference's names (src/cuda/ffi.rs:349-422, kernels in
 * src/kernels/sdpa_kernels.cu:34-403): what the reference's chunked host loops call between their GEMMs.  The
 * fused kernels above need none of them; they are for host code that keeps such a loop (the dropout path).
 * Tiles are contiguous [BH, q_t, k_t] (scores: [B, H, Q, K]).  Return 0 when the kernel was launched, 1 otherwise
 * (the reference's convention for these symbols); empty tiles return 0 without a launch. */

/* src/cuda/ffi.rs:349-358: scores[b,h,q,k] = -1e9 where k_offset + k > q_offset + q. */
int flame_apply_causal_mask_fp32(float* scores, int B, int H, int Q, int K, int q_offset, int k_offset, void* stream);
/* src/cuda/ffi.rs:360-368: scores = -1e9 where the uint8 mask of the same shape is 0. */
int flame_apply_attn_mask_fp32(float* scores, const uint8_t* mask, int B, int H, int Q, int K, void* stream);
/* src/cuda/ffi.rs:370-385: logits += user_add (+ -1e30 where user_bool excludes) (+ -1e30 where the absolute key
 * is past the absolute query), summed in that order.  Rank 3 operands have the tile's shape; rank 2 operands are
 * [BH, k_total] rows indexed by k_abs_start + kj; any other rank ignores the operand.  bool_zero_is_mask picks
 * which byte value excludes. */
int flame_sdpa_add_mask_tile_fp32(float* logits, const uint8_t* user_bool, const float* user_add, int BH, int q_t, int k_t,
                                  int q_abs_start, int k_abs_start, int user_bool_rank, int user_add_rank, int k_total,
                                  int bool_zero_is_mask, int causal_flag, void* stream);
/* src/cuda/ffi.rs:387-395: probs = bf16(exp(logits - lse_row[bh, qi])). */
int flame_sdpa_softmax_from_lse_tile(const float* logits, const float* lse_row, void* probs_bf16, int BH, int q_t, int k_t,
                                     void* stream);
/* src/cuda/ffi.rs:397-404: out_lse_row[bh, qi] = log sum_k exp(logits[bh, qi, k]); an empty row gives -inf. */
int flame_sdpa_lse_from_logits_tile(const float* logits, float* out_lse_row, int BH, int q_t, int k_t, void* stream);
/* src/cuda/ffi.rs:406-412: lse_row = log(exp(lse_row) + exp(tile_lse_row)), element-wise over BH * q_t rows.  Two
 * -inf give -inf (the reference's expression gives NaN there; its callers pass the finite -1e30). */
int flame_sdpa_lse_merge_rows(float* lse_row, const float* tile_lse_row, int BH, int q_t, void* stream);
/* src/cuda/ffi.rs:414-422: in place, probs = u < p ? 0 : bf16(float(probs) / (1 - p)), with the reference's
 * counter-based uniform u(seed, bh, qi, kj) of the coordinates inside the tile (sdpa_kernels.cu:18-33), so the
 * kept set is bit-identical to the reference's for the same seed and tile shape. */
int flame_sdpa_dropout_bf16_inplace(void* probs_bf16, float p, uint64_t seed, int BH, int q_t, int k_t, void* stream);

/* ------------------------------------------------------------------------------------------------
 * FP8 E4M3 form of saved activations (O, or Q / K / V) on their way to and from pinned host memory: the pair the
 * reference's activation offload pool runs on its transfer stream around the copies
 * (src/cuda/ffi.rs:545-562; src/cuda/fp8_quant.cu:74-92, src/cuda/fp8_dequant.cu:42-58; used by
 * src/activation_offload.rs:536-586, :678-700 with scale = 8 / 448).  Contiguous tensors of n_elements; any
 * alignment (16-byte aligned pointers take the vector path).  Return 0 or the HIP error code, like the reference.
 *   flame_bf16_to_fp8:  output[i] = fp8_e4m3(float(input[i]) * inv_scale)   (1 byte per element)
 *   flame_fp8_to_bf16:  output[i] = bf16(float(fp8(input[i])) * scale)
 * The codes are the reference's bit for bit, including its deviations from OCP E4M3: the mantissa is rounded half
 * up in magnitude; products of 256 and above all become 0x7F, which the decoder reads as 480 (no NaN code);
 * a product that would round up to the smallest normal stays at the largest subnormal; operands and products below
 * 2^-126 count as zero (the reference is built with flush-to-zero).  With the pool's fixed scale every |x| >= 32/7
 * therefore comes back as 60/7 = 8.57: callers whose activations reach that range should pass a larger scale.
 * ---------------------------------------------------------------------------------------------- */
int flame_bf16_to_fp8(const void* input, void* output, float inv_scale, size_t n_elements, void* stream);
int flame_fp8_to_bf16(const void* input, void* output, float scale, size_t n_elements, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Profiling aids (the counterpart of the reference's SdpaStats / SdpaHooks timing fields,
 * src/autograd_v4/ops/sdpa.rs:55-79).  No counterpart in the FFI of the reference.
 * ---------------------------------------------------------------------------------------------- */
enum { FLAME_ATTN_KERNEL_FWD = 0, FLAME_ATTN_KERNEL_UNUSED_1 = 1, FLAME_ATTN_KERNEL_BWD_DKDV = 2,
       FLAME_ATTN_KERNEL_BWD_DQ = 3, FLAME_ATTN_KERNEL_SAGE_KMEAN = 4, FLAME_ATTN_KERNEL_SAGE_QUANT = 5,
       FLAME_ATTN_KERNEL_SAGE_FWD = 6, FLAME_ATTN_KERNEL_INPUT_PREP = 7, FLAME_ATTN_KERNEL_BWD_MERGE = 8,
       FLAME_ATTN_KERNEL_BWD_JOINT = 9, FLAME_ATTN_KERNEL_BWD_ROWS = 10,
       FLAME_ATTN_N_KERNEL_KINDS = 12 };
typedef struct {
    double total_ms[FLAME_ATTN_N_KERNEL_KINDS];
    int launches[FLAME_ATTN_N_KERNEL_KINDS];
} FlameAttnKernelTimes;
/* When on, every kernel launch is bracketed by HIP events on the launch stream (events are created
 * on demand: this mode allocates).  Turning it on or off clears the samples. */
int flame_attn_profiling_enable(int on);
/* Waits for the recorded events and returns per-kernel sums since the last read. */
int flame_attn_profiling_read(FlameAttnKernelTimes* out);

/* ------------------------------------------------------------------------------------------------
 * Small conversions the host layer needs at the boundary.
 * ---------------------------------------------------------------------------------------------- */
enum { FLAME_ATTN_DTYPE_BF16 = 0, FLAME_ATTN_DTYPE_F32 = 1 };
/* Binary keep-mask in bf16 / fp32 (>= 0.5 attends; the public mask convention of the reference,
 * src/sdpa.rs:458-470) -> contiguous uint8 keep-mask of n elements. */
int flame_attn_convert_keep_mask(const void* src, int src_dtype, void* dst_u8, int64_t n, void* stream);
/* fp32 -> bf16, round to nearest even, n contiguous elements.  Lets the autograd shim hand an fp32
 * upstream gradient to the bf16 backward instead of falling back to the materialising recompute as
 * the reference does (src/autograd.rs:702-705). */
int flame_attn_cast_f32_to_bf16(const void* src_f32, void* dst_bf16, int64_t n, void* stream);
/* acc_f32[i] += float(grad[i]), grad bf16 or fp32, n contiguous elements: what Gradients::accumulate
 * of the reference's v4 engine does with tensor ops (src/autograd_v4/gradients.rs:20-32, gradients are
 * kept in fp32). */
int flame_attn_accumulate_f32(void* acc_f32, const void* grad, int grad_dtype, int64_t n, void* stream);
/* dst[i] = value (bf16 or fp32), n contiguous elements: the ones-seed of backward_v4
 * (src/autograd_v4/ops/mod.rs:37-38) and zero-initialised accumulators. */
int flame_attn_fill(void* dst, int dtype, float value, int64_t n, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Fused input preparation for joint attention: RMS normalisation over the head dim, interleaved-
 * pair rotary embedding and the [B,N,H,D] -> [B,H,N,D] layout change in one pass.  Replaces, run
 * back to back and with the same bf16 rounding between them,
 *   flame_fused_rms_norm_bf16   src/cuda/fused_rms_norm.cu:89-111  (src/norm.rs:686-732)
 *   rope_fused_bf16 / rope_fused_bf16_f32pe   src/bf16_ops.rs:361-394, :476-582 (tables [1,1,N,D/2])
 *   the permute that makes [B,H,N,D] contiguous   cuda/permute0213.cu
 * X is read through element strides given in (B,H,N,D) order (D stride must be 1, the others and the
 * offsets multiples of 8), so a [B,N,H,D] buffer is passed as strides (N*H*D, D, H*D, 1).
 * weight: [D] bf16 or null; eps as in the reference's RMSNorm; apply_norm = 0 skips the normalisation.
 * cos, sin: contiguous [N, D/2], bf16 (table_dtype = FLAME_ATTN_DTYPE_BF16) or fp32; null skips the
 * rotation.  D in {64, 128}.
 * ---------------------------------------------------------------------------------------------- */
int flame_attn_prep_rmsnorm_rope_bf16(const void* X, const void* weight, const void* cos, const void* sin,
                                      int table_dtype, void* Y, int B, int H, int N, int D, float eps,
                                      int apply_norm, const int64_t* x_strides, const int64_t* y_strides,
                                      int64_t x_off, int64_t y_off, void* stream);

/* "flame-attn-gfx950 <version> (hipcc <version of the compiler that built the library>)" */
const char* flame_attn_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FLAME_ATTN_H */
