//! The marshalling that flame-core's `sdpa.rs` does in front of its FFI, over a plain view type: what
//! `forward_cudnn_sdpa_bf16` / `forward_cudnn_sdpa_train_bf16` (src/sdpa.rs:595-770) and `try_cudnn_sdpa_backward`
//! (src/autograd.rs:672-772) become when the symbols behind them are this library's.  flame-core's own `Tensor`
//! supplies exactly these fields (`as_device_ptr_bf16`, `strides`, `offset`: src/tensor.rs:558, :2637, :2657).
//!
//! UNVERIFIED SOURCE: never compiled (no Rust toolchain in the image the library is developed in).
use core::ffi::c_void;

use crate::ffi;

/// A `[B, H, N, D]` bf16 tensor on the device: base pointer, shape, element strides (D stride 1), element offset.
#[derive(Clone, Copy, Debug)]
pub struct View4 {
    pub ptr: *mut c_void,
    pub shape: [i32; 4],
    pub strides: [i64; 4],
    pub offset: i64,
}

#[derive(Debug)]
pub enum Error {
    /// Shape or dtype disagreement found on the host, as `Error::InvalidInput` in flame-core (src/sdpa.rs:335-374).
    InvalidInput(String),
    /// A non-zero status from the library, as `Error::Cuda` in flame-core (src/sdpa.rs:680-682).
    Device(String),
}

pub type Result<T> = core::result::Result<T, Error>;

fn check(entry: &str, rc: i32) -> Result<()> {
    if rc == ffi::FLAME_ATTN_OK {
        Ok(())
    } else {
        Err(Error::Device(format!("{entry} HIP error: {rc}")))
    }
}

/// The checks of `forward_inner` (src/sdpa.rs:335-355): batch, heads and head dim agree, K and V agree in length.
fn validate(q: &View4, k: &View4, v: &View4) -> Result<(i32, i32, i32, i32, i32)> {
    let [b, h, n_q, d] = q.shape;
    let [kb, kh, n_kv, kd] = k.shape;
    if kb != b || kh != h || v.shape[0] != b || v.shape[1] != h {
        return Err(Error::InvalidInput("batch / head mismatch between q, k, v".into()));
    }
    if kd != d || v.shape[3] != d {
        return Err(Error::InvalidInput("head dim mismatch between q, k, v".into()));
    }
    if v.shape[2] != n_kv {
        return Err(Error::InvalidInput("k_len != v_len".into()));
    }
    Ok((b, h, n_q, n_kv, d))
}

/// Inference forward into a caller-allocated `o` (`sdpa::forward` without a mask, src/sdpa.rs:85-102, :595-684).
/// `stream`: a `hipStream_t`, null for the default stream (flame-core always passes null: src/cuda/device_lt.rs:18-21).
pub fn forward_into(q: &View4, k: &View4, v: &View4, o: &View4, stream: *mut c_void) -> Result<()> {
    let (b, h, n_q, n_kv, d) = validate(q, k, v)?;
    let scale = 1.0f32 / (d as f32).sqrt();
    let rc = unsafe {
        ffi::flame_cudnn_sdpa_bf16(
            q.ptr, k.ptr, v.ptr, o.ptr, b, h, n_q, n_kv, d, scale,
            q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
            q.offset, k.offset, v.offset, o.offset, stream,
        )
    };
    check("flame_cudnn_sdpa_bf16", rc)
}

/// Training forward: also fills `stats`, fp32 contiguous `[B*H, N_q]` (the saved log-sum-exp rows; src/sdpa.rs:691-770).
/// What the caller saves for the backward is {Q, K, V, O, stats} (src/sdpa.rs:170-201), never an `N_q x N_kv` tensor.
pub fn forward_train_into(q: &View4, k: &View4, v: &View4, o: &View4, stats: *mut c_void, stream: *mut c_void) -> Result<()> {
    let (b, h, n_q, n_kv, d) = validate(q, k, v)?;
    let scale = 1.0f32 / (d as f32).sqrt();
    let rc = unsafe {
        ffi::flame_cudnn_sdpa_bf16_train_fwd(
            q.ptr, k.ptr, v.ptr, o.ptr, stats, b, h, n_q, n_kv, d, scale,
            q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
            q.offset, k.offset, v.offset, o.offset, 0, stream,
        )
    };
    check("flame_cudnn_sdpa_bf16_train_fwd", rc)
}

/// Bytes of device scratch `backward_into` wants (two fp32 rows per query plus room for split dK/dV partial sums).
pub fn backward_workspace_bytes(q: &View4) -> usize {
    unsafe { ffi::flame_attn_bwd_workspace_bytes(q.shape[0], q.shape[1], q.shape[2], q.shape[3]) }
}

/// Backward of the `Op::FlashAttention` arm (src/autograd.rs:3824-3916) through the entry point that takes the
/// caller's workspace, so that nothing is allocated and the call can sit inside a captured backward
/// (src/autograd.rs:1298-1311).  `d_o` must be bf16: cast fp32 upstream gradients first
/// (`ffi::flame_attn_cast_f32_to_bf16`) instead of falling back to a materialising recompute (src/autograd.rs:702-705).
#[allow(clippy::too_many_arguments)]
pub fn backward_into(
    q: &View4, k: &View4, v: &View4, o: &View4, d_o: &View4, stats: *const c_void,
    dq: &View4, dk: &View4, dv: &View4, causal: bool,
    workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void,
) -> Result<()> {
    let (b, h, n_q, n_kv, d) = validate(q, k, v)?;
    let scale = 1.0f32 / (d as f32).sqrt();
    let rc = unsafe {
        ffi::flame_attn_bwd_bf16(
            q.ptr, k.ptr, v.ptr, o.ptr, d_o.ptr, stats, dq.ptr, dk.ptr, dv.ptr, b, h, n_q, n_kv, d, scale,
            q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
            d_o.strides.as_ptr(), dq.strides.as_ptr(), dk.strides.as_ptr(), dv.strides.as_ptr(),
            q.offset, k.offset, v.offset, o.offset, d_o.offset, 0, dq.offset, dk.offset, dv.offset,
            causal as i32, core::ptr::null(), core::ptr::null(), core::ptr::null(),
            workspace, workspace_bytes, stream,
        )
    };
    check("flame_attn_bwd_bf16", rc)
}
