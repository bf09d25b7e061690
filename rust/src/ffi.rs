//! Raw bindings to `libflame_attn_hip` (the gfx950 attention library), one declaration per function of
//! `include/flame_attn.h`, in the header's order.
//!
//! UNVERIFIED SOURCE: no Rust toolchain exists in the image this library is developed in, so this file has never been
//! compiled.  What is checked instead, without a compiler: `tests/test_rust_ffi_matches_header.py` parses every
//! declaration below and compares its name, argument count and every argument and return type with the C header.
//!
//! The three `flame_cudnn_sdpa_*` symbols, `flame_flash_attention_bf16`, `flame_sdpa_chunked_bf16`,
//! `sdpa_stream_bf16_launch`, `streaming_attn_bf16_fp32_launch`, the `flame_sdpa_autotune_*` trio, the seven tile
//! primitives and the FP8 pair keep the names and argument lists flame-core already declares
//! (`src/cuda/ffi.rs:349-422`, `:545-562`, `:584-716`; `src/cuda_ops_ffi.rs:60-85`, `:199-221`;
//! `src/ffi/cuda_ffi.h:98-121`; `cuda/streaming_attn_bf16.h:7-17`): with this library linked, those declarations need
//! no edit.  The `flame_attn_*` and `flame_sage_*` functions are what the reference's FFI cannot express (causal flag,
//! key lengths, keep-mask, bias, dropout, caller workspaces, int8 QK).
//!
//! Conventions (see the header for the full text): device pointers owned by the caller; `*_strides` point at four
//! element strides in (B, H, N, D) order with a D stride of 1; `stream` is a `hipStream_t` (null = default stream);
//! `c_int` results are 0 on success, -1 invalid argument, -2 unsupported, -3 too large for the allocation-free
//! backward, positive = `hipError_t`.
#![allow(non_camel_case_types, clippy::too_many_arguments)]

use core::ffi::{c_char, c_int, c_long, c_void};

pub const FLAME_ATTN_OK: c_int = 0;
pub const FLAME_ATTN_ERR_INVALID: c_int = -1;
pub const FLAME_ATTN_ERR_UNSUPPORTED: c_int = -2;
pub const FLAME_ATTN_ERR_TOO_LARGE: c_int = -3;
pub const FLAME_ATTN_NOALLOC_MAX_ROWS: c_int = 1 << 20;
pub const FLAME_ATTN_DTYPE_BF16: c_int = 0;
pub const FLAME_ATTN_DTYPE_F32: c_int = 1;
pub const FLAME_ATTN_N_KERNEL_KINDS: usize = 12;

/// Status of the `flame_*` / `fc_*` family (`cuda/include/flame_cuda_status.h:7-12`).
#[repr(C)]
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum FlameAttnStatus {
    Ok = 0,
    ErrInvalid = 1,
    ErrUnsupported = 2,
    ErrHip = 3,
}

/// The 25 counters of the launch-plan cache, names and order as `cuda/include/flame_cuda_common.cuh:72-98`.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct FlameSdpaAutotuneStats {
    pub env_forced: u64,
    pub clamped: u64,
    pub skipped: u64,
    pub fallback: u64,
    pub errors: u64,
    pub cache_hits: u64,
    pub cache_misses: u64,
    pub tuned: u64,
    pub last_q_chunk: u64,
    pub last_k_chunk: u64,
    pub cache_saved: u64,
    pub cache_loads: u64,
    pub cache_load_errors: u64,
    pub cache_entries: u64,
    pub last_candidate_count: u64,
    pub last_best_time_ns: u64,
    pub last_plan_source: u64,
    pub last_shape_b: u64,
    pub last_shape_h: u64,
    pub last_shape_q: u64,
    pub last_shape_k: u64,
    pub last_shape_dh: u64,
    pub last_shape_dv: u64,
    pub last_shape_mask_heads: u64,
    pub last_shape_causal: u64,
}

/// Per-kernel HIP-event sums of `flame_attn_profiling_read`.
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct FlameAttnKernelTimes {
    pub total_ms: [f64; FLAME_ATTN_N_KERNEL_KINDS],
    pub launches: [c_int; FLAME_ATTN_N_KERNEL_KINDS],
}

// linked by build.rs (static archive made from flame_attn.hip)
extern "C" {
    pub fn flame_attn_fwd_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *mut c_void, lse: *mut c_void, b: c_int,
        h: c_int, n_q: c_int, n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64,
        v_strides: *const i64, o_strides: *const i64, q_off: i64, k_off: i64, v_off: i64, o_off: i64,
        lse_off: i64, causal: c_int, kv_len: *const i32, keep_mask: *const u8, mask_strides: *const i64,
        stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_fwd_workspace_bytes(
        b: c_int, h: c_int, n_q: c_int, n_kv: c_int, d: c_int
    ) -> usize;
    pub fn flame_attn_fwd_ws_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *mut c_void, lse: *mut c_void, b: c_int,
        h: c_int, n_q: c_int, n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64,
        v_strides: *const i64, o_strides: *const i64, q_off: i64, k_off: i64, v_off: i64, o_off: i64,
        lse_off: i64, causal: c_int, kv_len: *const i32, keep_mask: *const u8, mask_strides: *const i64,
        workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_fwd_bias_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *mut c_void, lse: *mut c_void, b: c_int,
        h: c_int, n_q: c_int, n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64,
        v_strides: *const i64, o_strides: *const i64, q_off: i64, k_off: i64, v_off: i64, o_off: i64,
        lse_off: i64, bias: *const c_void, bias_dtype: c_int, bias_strides: *const i64, keep_mask: *const u8,
        mask_strides: *const i64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_fwd_dropout_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *mut c_void, lse: *mut c_void, b: c_int,
        h: c_int, n_q: c_int, n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64,
        v_strides: *const i64, o_strides: *const i64, q_off: i64, k_off: i64, v_off: i64, o_off: i64,
        lse_off: i64, causal: c_int, kv_len: *const i32, keep_mask: *const u8, mask_strides: *const i64,
        dropout_p: f32, dropout_seed: u64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_bwd_dropout_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *const c_void, d_o: *const c_void,
        lse: *const c_void, dq: *mut c_void, dk: *mut c_void, dv: *mut c_void, b: c_int, h: c_int, n_q: c_int,
        n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64, v_strides: *const i64,
        o_strides: *const i64, do_strides: *const i64, dq_strides: *const i64, dk_strides: *const i64,
        dv_strides: *const i64, q_off: i64, k_off: i64, v_off: i64, o_off: i64, do_off: i64, lse_off: i64,
        dq_off: i64, dk_off: i64, dv_off: i64, causal: c_int, kv_len: *const i32, keep_mask: *const u8,
        mask_strides: *const i64, dropout_p: f32, dropout_seed: u64, workspace: *mut c_void,
        workspace_bytes: usize, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_fwd_dropout_tiled_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *mut c_void, lse: *mut c_void, b: c_int,
        h: c_int, n_q: c_int, n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64,
        v_strides: *const i64, o_strides: *const i64, q_off: i64, k_off: i64, v_off: i64, o_off: i64,
        lse_off: i64, causal: c_int, kv_len: *const i32, keep_mask: *const u8, mask_strides: *const i64,
        dropout_p: f32, dropout_seed: u64, draw_chunk_q: c_int, draw_chunk_kv: c_int, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_bwd_dropout_tiled_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *const c_void, d_o: *const c_void,
        lse: *const c_void, dq: *mut c_void, dk: *mut c_void, dv: *mut c_void, b: c_int, h: c_int, n_q: c_int,
        n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64, v_strides: *const i64,
        o_strides: *const i64, do_strides: *const i64, dq_strides: *const i64, dk_strides: *const i64,
        dv_strides: *const i64, q_off: i64, k_off: i64, v_off: i64, o_off: i64, do_off: i64, lse_off: i64,
        dq_off: i64, dk_off: i64, dv_off: i64, causal: c_int, kv_len: *const i32, keep_mask: *const u8,
        mask_strides: *const i64, dropout_p: f32, dropout_seed: u64, draw_chunk_q: c_int, draw_chunk_kv: c_int,
        workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_bwd_workspace_bytes(
        b: c_int, h: c_int, n_q: c_int, d: c_int
    ) -> usize;
    pub fn flame_attn_bwd_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *const c_void, d_o: *const c_void,
        lse: *const c_void, dq: *mut c_void, dk: *mut c_void, dv: *mut c_void, b: c_int, h: c_int, n_q: c_int,
        n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64, v_strides: *const i64,
        o_strides: *const i64, do_strides: *const i64, dq_strides: *const i64, dk_strides: *const i64,
        dv_strides: *const i64, q_off: i64, k_off: i64, v_off: i64, o_off: i64, do_off: i64, lse_off: i64,
        dq_off: i64, dk_off: i64, dv_off: i64, causal: c_int, kv_len: *const i32, keep_mask: *const u8,
        mask_strides: *const i64, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_bwd_noalloc_max_rows(
    ) -> c_int;
    pub fn flame_attn_bwd_bf16_noalloc(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *const c_void, d_o: *const c_void,
        lse: *const c_void, dq: *mut c_void, dk: *mut c_void, dv: *mut c_void, b: c_int, h: c_int, n_q: c_int,
        n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64, v_strides: *const i64,
        o_strides: *const i64, do_strides: *const i64, dq_strides: *const i64, dk_strides: *const i64,
        dv_strides: *const i64, q_off: i64, k_off: i64, v_off: i64, o_off: i64, do_off: i64, lse_off: i64,
        dq_off: i64, dk_off: i64, dv_off: i64, causal: c_int, kv_len: *const i32, keep_mask: *const u8,
        mask_strides: *const i64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_materialised_workspace_bytes(
        b: c_int, h: c_int, n_q: c_int, n_kv: c_int, d: c_int, dv: c_int, backward: c_int
    ) -> usize;
    pub fn flame_attn_fwd_materialised_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *mut c_void, lse: *mut c_void, b: c_int,
        h: c_int, n_q: c_int, n_kv: c_int, d: c_int, dv: c_int, scale: f32, q_strides: *const i64,
        k_strides: *const i64, v_strides: *const i64, o_strides: *const i64, q_off: i64, k_off: i64, v_off: i64,
        o_off: i64, lse_off: i64, causal: c_int, kv_len: *const i32, keep_mask: *const u8,
        mask_strides: *const i64, bias: *const c_void, bias_dtype: c_int, bias_strides: *const i64,
        dropout_p: f32, dropout_seed: u64, draw_chunk_q: c_int, draw_chunk_kv: c_int,
        workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_bwd_materialised_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *const c_void, d_o: *const c_void,
        lse: *const c_void, dq: *mut c_void, dk: *mut c_void, dv_out: *mut c_void, b: c_int, h: c_int, n_q: c_int,
        n_kv: c_int, d: c_int, dv: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64,
        v_strides: *const i64, o_strides: *const i64, do_strides: *const i64, dq_strides: *const i64,
        dk_strides: *const i64, dv_strides: *const i64, q_off: i64, k_off: i64, v_off: i64, o_off: i64,
        do_off: i64, lse_off: i64, dq_off: i64, dk_off: i64, dv_off: i64, causal: c_int, kv_len: *const i32,
        keep_mask: *const u8, mask_strides: *const i64, dropout_p: f32, dropout_seed: u64, draw_chunk_q: c_int,
        draw_chunk_kv: c_int, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void
    ) -> c_int;
    pub fn flame_sage_quant_qk_int8(
        q: *const c_void, k: *const c_void, b: c_int, h: c_int, n_q: c_int, n_kv: c_int, d: c_int,
        q_strides: *const i64, k_strides: *const i64, q_off: i64, k_off: i64, smooth_k: c_int,
        qi8: *mut c_void, ki8: *mut c_void, q_scales: *mut c_void, k_scales: *mut c_void, k_mean: *mut c_void,
        stream: *mut c_void
    ) -> c_int;
    pub fn flame_sage_quant_qk_int8_ks(
        q: *const c_void, k: *const c_void, b: c_int, h: c_int, n_q: c_int, n_kv: c_int, d: c_int,
        q_strides: *const i64, k_strides: *const i64, q_off: i64, k_off: i64, smooth_k: c_int,
        qi8: *mut c_void, ki8: *mut c_void, q_scales: *mut c_void, k_scales: *mut c_void, k_mean: *mut c_void,
        k_smoothed: *mut c_void, stream: *mut c_void
    ) -> c_int;
    pub fn flame_sage_attn_fwd_int8(
        qi8: *const c_void, ki8: *const c_void, q_scales: *const c_void, k_scales: *const c_void,
        v: *const c_void, o: *mut c_void, lse: *mut c_void, b: c_int, h: c_int, n_q: c_int, n_kv: c_int,
        d: c_int, scale: f32, v_strides: *const i64, o_strides: *const i64, v_off: i64, o_off: i64,
        causal: c_int, kv_len: *const i32, stream: *mut c_void
    ) -> c_int;
    pub fn flame_sage_attn_fwd_bias_int8(
        qi8: *const c_void, ki8: *const c_void, q_scales: *const c_void, k_scales: *const c_void,
        v: *const c_void, o: *mut c_void, lse: *mut c_void, b: c_int, h: c_int, n_q: c_int, n_kv: c_int,
        d: c_int, scale: f32, v_strides: *const i64, o_strides: *const i64, v_off: i64, o_off: i64,
        causal: c_int, kv_len: *const i32, bias: *const c_void, bias_dtype: c_int, bias_strides: *const i64,
        stream: *mut c_void
    ) -> c_int;
    pub fn flame_cudnn_sdpa_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *mut c_void, b: c_int, h: c_int, n_q: c_int,
        n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64, v_strides: *const i64,
        o_strides: *const i64, q_offset_elems: i64, k_offset_elems: i64, v_offset_elems: i64,
        o_offset_elems: i64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_cudnn_sdpa_bf16_train_fwd(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *mut c_void, stats: *mut c_void, b: c_int,
        h: c_int, n_q: c_int, n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64,
        v_strides: *const i64, o_strides: *const i64, q_offset_elems: i64, k_offset_elems: i64,
        v_offset_elems: i64, o_offset_elems: i64, stats_offset_elems: i64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_cudnn_sdpa_bwd_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *const c_void, d_o: *const c_void,
        stats: *const c_void, dq: *mut c_void, dk: *mut c_void, dv: *mut c_void, b: c_int, h: c_int,
        n_q: c_int, n_kv: c_int, d: c_int, scale: f32, q_strides: *const i64, k_strides: *const i64,
        v_strides: *const i64, o_strides: *const i64, do_strides: *const i64, dq_strides: *const i64,
        dk_strides: *const i64, dv_strides: *const i64, q_offset_elems: i64, k_offset_elems: i64,
        v_offset_elems: i64, o_offset_elems: i64, do_offset_elems: i64, stats_offset_elems: i64,
        dq_offset_elems: i64, dk_offset_elems: i64, dv_offset_elems: i64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_flash_attention_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, o: *mut c_void, lse: *mut f32,
        batch_heads: c_int, seq_len_q: c_int, seq_len_kv: c_int, head_dim: c_int, stream: *mut c_void
    ) -> c_int;
    pub fn flame_sdpa_chunked_bf16(
        q: *const c_void, k: *const c_void, v: *const c_void, b: c_int, h: c_int, q_len: c_int, k_len: c_int,
        dh: c_int, dv: c_int, scale: f32, chunk: c_int, causal: c_int, mask_heads: c_int, mask: *const c_void,
        out: *mut c_void, workspace: *mut c_void, workspace_bytes: u64, stream: *mut c_void
    ) -> FlameAttnStatus;
    pub fn streaming_attn_bf16_fp32_launch(
        q: *const c_void, k: *const c_void, v: *const c_void, b: c_int, h: c_int, s: c_int, dh: c_int,
        dv: c_int, q_b: c_long, q_h: c_long, q_s: c_long, q_d: c_long, k_b: c_long, k_h: c_long, k_s: c_long,
        k_d: c_long, v_b: c_long, v_h: c_long, v_s: c_long, v_d: c_long, o: *mut c_void, o_b: c_long,
        o_h: c_long, o_s: c_long, o_d: c_long, scale: f32, chunk_size: c_int, causal: c_int,
        k_pad_mask: *const u8, stream: *mut c_void
    ) -> c_int;
    pub fn sdpa_stream_bf16_launch(
        dq: *const c_void, dk: *const c_void, dv: *const c_void, d_o: *mut c_void, b: c_int, h: c_int,
        q_len: c_int, k_len: c_int, d: c_int, scale: f32, attn_mask: *const c_void, mask_stride_ek: i64,
        mask_stride_eq: i64, mask_stride_eh: i64, mask_stride_eb: i64, head_tile: c_int, q_tile: c_int,
        max_q_tile: c_int, stream: *mut c_void, unsupported_reason: *mut c_char, reason_buflen: c_int
    ) -> bool;
    pub fn flame_sdpa_autotune_get_stats(
        out: *mut FlameSdpaAutotuneStats
    ) -> c_int;
    pub fn flame_sdpa_autotune_reset_stats(
    ) -> c_int;
    pub fn flame_sdpa_autotune_flush_cache(
    ) -> c_int;
    pub fn flame_apply_causal_mask_fp32(
        scores: *mut f32, b: c_int, h: c_int, q: c_int, k: c_int, q_offset: c_int, k_offset: c_int,
        stream: *mut c_void
    ) -> c_int;
    pub fn flame_apply_attn_mask_fp32(
        scores: *mut f32, mask: *const u8, b: c_int, h: c_int, q: c_int, k: c_int, stream: *mut c_void
    ) -> c_int;
    pub fn flame_sdpa_add_mask_tile_fp32(
        logits: *mut f32, user_bool: *const u8, user_add: *const f32, bh: c_int, q_t: c_int, k_t: c_int,
        q_abs_start: c_int, k_abs_start: c_int, user_bool_rank: c_int, user_add_rank: c_int, k_total: c_int,
        bool_zero_is_mask: c_int, causal_flag: c_int, stream: *mut c_void
    ) -> c_int;
    pub fn flame_sdpa_softmax_from_lse_tile(
        logits: *const f32, lse_row: *const f32, probs_bf16: *mut c_void, bh: c_int, q_t: c_int, k_t: c_int,
        stream: *mut c_void
    ) -> c_int;
    pub fn flame_sdpa_lse_from_logits_tile(
        logits: *const f32, out_lse_row: *mut f32, bh: c_int, q_t: c_int, k_t: c_int, stream: *mut c_void
    ) -> c_int;
    pub fn flame_sdpa_lse_merge_rows(
        lse_row: *mut f32, tile_lse_row: *const f32, bh: c_int, q_t: c_int, stream: *mut c_void
    ) -> c_int;
    pub fn flame_sdpa_dropout_bf16_inplace(
        probs_bf16: *mut c_void, p: f32, seed: u64, bh: c_int, q_t: c_int, k_t: c_int, stream: *mut c_void
    ) -> c_int;
    pub fn flame_bf16_to_fp8(
        input: *const c_void, output: *mut c_void, inv_scale: f32, n_elements: usize, stream: *mut c_void
    ) -> c_int;
    pub fn flame_fp8_to_bf16(
        input: *const c_void, output: *mut c_void, scale: f32, n_elements: usize, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_profiling_enable(
        on: c_int
    ) -> c_int;
    pub fn flame_attn_profiling_read(
        out: *mut FlameAttnKernelTimes
    ) -> c_int;
    pub fn flame_attn_convert_keep_mask(
        src: *const c_void, src_dtype: c_int, dst_u8: *mut c_void, n: i64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_cast_f32_to_bf16(
        src_f32: *const c_void, dst_bf16: *mut c_void, n: i64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_accumulate_f32(
        acc_f32: *mut c_void, grad: *const c_void, grad_dtype: c_int, n: i64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_fill(
        dst: *mut c_void, dtype: c_int, value: f32, n: i64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_prep_rmsnorm_rope_bf16(
        x: *const c_void, weight: *const c_void, cos: *const c_void, sin: *const c_void, table_dtype: c_int,
        y: *mut c_void, b: c_int, h: c_int, n: c_int, d: c_int, eps: f32, apply_norm: c_int,
        x_strides: *const i64, y_strides: *const i64, x_off: i64, y_off: i64, stream: *mut c_void
    ) -> c_int;
    pub fn flame_attn_version(
    ) -> *const c_char;
}
