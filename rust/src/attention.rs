//! The operator layer above `sdpa.rs`, as flame-core's `attention::{sdpa, attend, sdpa_with_bias, attention_impl}`
//! (src/attention/sdpa.rs:57-243, :411-458) and `sdpa::forward_with_bias` (src/sdpa.rs:221-326) would call this
//! library: a keep-mask in the caller's dtype is converted once to the uint8 mask the kernels read, the causal flag
//! is passed straight through instead of being turned into a mask tensor (`build_causal_mask`,
//! src/attention/sdpa.rs:460-483), and shapes the fused kernels refuse go through the materialised entry points,
//! which is where flame-core itself falls back (`forward_bf16_fallback`, src/sdpa.rs:788-961).
//!
//! UNVERIFIED SOURCE: never compiled (no Rust toolchain in the image the library is developed in).
use core::ffi::c_void;

use crate::ffi;
use crate::sdpa::{Error, Result, View4};

/// A keep-mask `[B|1, H|1, N_q, N_kv]` already in the kernels' form: uint8, non-zero attends; element strides, 0 for a
/// broadcast axis.  `convert_keep_mask` makes one from the bf16 / fp32 masks flame-core passes around (>= 0.5 attends,
/// src/sdpa.rs:458-470).
#[derive(Clone, Copy, Debug)]
pub struct KeepMask {
    pub ptr: *const u8,
    pub strides: [i64; 4],
}

/// An additive bias `[B|1, H|1, N_q, N_kv]` on the scaled logits, bf16 or fp32 (`-inf` excludes a position).
#[derive(Clone, Copy, Debug)]
pub struct Bias {
    pub ptr: *const c_void,
    pub is_f32: bool,
    pub strides: [i64; 4],
}

/// Device scratch a call may need; null / 0 where the caller has none (the call then fails with `Device` on a shape
/// that needs the materialised path).
#[derive(Clone, Copy, Debug)]
pub struct Workspace {
    pub ptr: *mut c_void,
    pub bytes: usize,
}

fn dims(q: &View4, k: &View4, v: &View4) -> Result<(i32, i32, i32, i32, i32, i32)> {
    let [b, h, n_q, d] = q.shape;
    if k.shape[0] != b || k.shape[1] != h || v.shape[0] != b || v.shape[1] != h {
        return Err(Error::InvalidInput("batch / head mismatch between q, k, v".into()));
    }
    if k.shape[3] != d {
        return Err(Error::InvalidInput("head dim mismatch between q and k".into()));
    }
    if v.shape[2] != k.shape[2] {
        return Err(Error::InvalidInput("k_len != v_len".into()));
    }
    Ok((b, h, n_q, k.shape[2], d, v.shape[3]))
}

fn status(entry: &str, rc: i32) -> Result<()> {
    if rc == ffi::FLAME_ATTN_OK {
        Ok(())
    } else {
        Err(Error::Device(format!("{entry} HIP error: {rc}")))
    }
}

/// bf16 (`is_f32 = false`) or fp32 binary mask of `n` contiguous elements -> uint8 keep-mask at `dst`.
pub fn convert_keep_mask(src: *const c_void, is_f32: bool, dst: *mut c_void, n: i64, stream: *mut c_void) -> Result<()> {
    let dt = if is_f32 { ffi::FLAME_ATTN_DTYPE_F32 } else { ffi::FLAME_ATTN_DTYPE_BF16 };
    status("flame_attn_convert_keep_mask", unsafe { ffi::flame_attn_convert_keep_mask(src, dt, dst, n, stream) })
}

/// Bytes of workspace with which `attend_into` can serve every shape (the materialised forward's need; the fused
/// kernels use none of it except the key-split forward for head dims above 128).
pub fn attend_workspace_bytes(q: &View4, k: &View4, v: &View4) -> usize {
    unsafe {
        ffi::flame_attn_materialised_workspace_bytes(q.shape[0], q.shape[1], q.shape[2], k.shape[2], q.shape[3], v.shape[3], 0)
    }
}

/// `attention_impl`: O (and, with `lse` non-null, the fp32 log-sum-exp rows `[B*H, N_q]`) for an optional keep-mask
/// and causal flag.  Fused kernels first; on "unsupported" (-2) the materialised path in the caller's workspace.
#[allow(clippy::too_many_arguments)]
pub fn attend_into(
    q: &View4, k: &View4, v: &View4, o: &View4, lse: *mut c_void, scale: Option<f32>, causal: bool,
    mask: Option<&KeepMask>, ws: Workspace, stream: *mut c_void,
) -> Result<()> {
    let (b, h, n_q, n_kv, d, dv) = dims(q, k, v)?;
    let scale = scale.unwrap_or(1.0f32 / (d as f32).sqrt());
    let (mptr, mst) = match mask {
        Some(m) => (m.ptr, m.strides.as_ptr()),
        None => (core::ptr::null(), core::ptr::null()),
    };
    let mut rc = ffi::FLAME_ATTN_ERR_UNSUPPORTED;
    if dv == d {
        rc = unsafe {
            ffi::flame_attn_fwd_ws_bf16(
                q.ptr, k.ptr, v.ptr, o.ptr, lse, b, h, n_q, n_kv, d, scale,
                q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
                q.offset, k.offset, v.offset, o.offset, 0, causal as i32, core::ptr::null(), mptr, mst,
                ws.ptr, ws.bytes, stream,
            )
        };
    }
    if rc == ffi::FLAME_ATTN_ERR_UNSUPPORTED {
        rc = unsafe {
            ffi::flame_attn_fwd_materialised_bf16(
                q.ptr, k.ptr, v.ptr, o.ptr, lse, b, h, n_q, n_kv, d, dv, scale,
                q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
                q.offset, k.offset, v.offset, o.offset, 0, causal as i32, core::ptr::null(), mptr, mst,
                core::ptr::null(), ffi::FLAME_ATTN_DTYPE_F32, core::ptr::null(), 0.0, 0, 0, 0,
                ws.ptr, ws.bytes, stream,
            )
        };
        return status("flame_attn_fwd_materialised_bf16", rc);
    }
    status("flame_attn_fwd_ws_bf16", rc)
}

/// `sdpa::forward_with_bias` (inference only, as in flame-core): an additive bias instead of a keep-mask.
#[allow(clippy::too_many_arguments)]
pub fn forward_with_bias_into(
    q: &View4, k: &View4, v: &View4, o: &View4, scale: Option<f32>, bias: &Bias, ws: Workspace, stream: *mut c_void,
) -> Result<()> {
    let (b, h, n_q, n_kv, d, dv) = dims(q, k, v)?;
    let scale = scale.unwrap_or(1.0f32 / (d as f32).sqrt());
    let dt = if bias.is_f32 { ffi::FLAME_ATTN_DTYPE_F32 } else { ffi::FLAME_ATTN_DTYPE_BF16 };
    let mut rc = ffi::FLAME_ATTN_ERR_UNSUPPORTED;
    if dv == d {
        rc = unsafe {
            ffi::flame_attn_fwd_bias_bf16(
                q.ptr, k.ptr, v.ptr, o.ptr, core::ptr::null_mut(), b, h, n_q, n_kv, d, scale,
                q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
                q.offset, k.offset, v.offset, o.offset, 0, bias.ptr, dt, bias.strides.as_ptr(),
                core::ptr::null(), core::ptr::null(), stream,
            )
        };
    }
    if rc == ffi::FLAME_ATTN_ERR_UNSUPPORTED {
        rc = unsafe {
            ffi::flame_attn_fwd_materialised_bf16(
                q.ptr, k.ptr, v.ptr, o.ptr, core::ptr::null_mut(), b, h, n_q, n_kv, d, dv, scale,
                q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
                q.offset, k.offset, v.offset, o.offset, 0, 0, core::ptr::null(), core::ptr::null(), core::ptr::null(),
                bias.ptr, dt, bias.strides.as_ptr(), 0.0, 0, 0, 0,
                ws.ptr, ws.bytes, stream,
            )
        };
        return status("flame_attn_fwd_materialised_bf16", rc);
    }
    status("flame_attn_fwd_bias_bf16", rc)
}
