//! SageAttention on this library: what `SageAttention::forward` (src/sage_attention.rs:59-171) and
//! `sage_attention_backward` (:470-505) of flame-core become.  The quantiser and the int8-QK forward are two calls
//! with caller-owned buffers between them; nothing of size `N_q x N_kv` exists at any point.
//!
//! UNVERIFIED SOURCE: never compiled (no Rust toolchain in the image the library is developed in).
use core::ffi::c_void;

use crate::attention::Bias;
use crate::ffi;
use crate::sdpa::{Error, Result, View4};

/// Row length of the tensors the quantiser writes for head dim `d`: 64 up to 64, else 128 (elements past `d` are
/// written as zero).
pub fn row_elems(d: i32) -> i32 {
    if d <= 64 { 64 } else { 128 }
}

/// Device buffers between the two calls, all caller-allocated and contiguous:
/// `qi8` int8 `[B,H,N_q,row_elems(D)]`, `ki8` int8 `[B,H,N_kv,row_elems(D)]`, `q_scales` fp32 `[B,H,ceil(N_q/128)]`,
/// `k_scales` fp32 `[B,H,ceil(N_kv/64)]`, `k_mean` fp32 `[B,H,row_elems(D)]`, and optionally `k_smoothed` bf16
/// `[B,H,N_kv,row_elems(D)]` (null unless a backward will follow).
#[derive(Clone, Copy, Debug)]
pub struct SageBuffers {
    pub qi8: *mut c_void,
    pub ki8: *mut c_void,
    pub q_scales: *mut c_void,
    pub k_scales: *mut c_void,
    pub k_mean: *mut c_void,
    pub k_smoothed: *mut c_void,
}

/// Builder-style options of the reference's operator (src/sage_attention.rs:21-57).
#[derive(Clone, Copy, Debug)]
pub struct SageAttention {
    pub scale: Option<f32>,
    pub causal: bool,
    pub smooth_k: bool,
}

impl Default for SageAttention {
    fn default() -> Self {
        SageAttention { scale: None, causal: false, smooth_k: true }
    }
}

fn status(entry: &str, rc: i32) -> Result<()> {
    if rc == ffi::FLAME_ATTN_OK {
        Ok(())
    } else {
        Err(Error::Device(format!("{entry} HIP error: {rc}")))
    }
}

impl SageAttention {
    /// Quantise Q and the mean-smoothed K, then O = softmax(dequantised int8 Q K^T * scale [+ bias]) V.
    /// `attention_mask`: the operator's additive mask (src/sage_attention.rs:126-131), or None.
    pub fn forward_into(
        &self, q: &View4, k: &View4, v: &View4, o: &View4, buf: &SageBuffers, attention_mask: Option<&Bias>,
        stream: *mut c_void,
    ) -> Result<()> {
        let [b, h, n_q, d] = q.shape;
        let n_kv = k.shape[2];
        if k.shape[0] != b || k.shape[1] != h || k.shape[3] != d || v.shape != k.shape {
            return Err(Error::InvalidInput("q, k, v shapes disagree".into()));
        }
        let rc = unsafe {
            ffi::flame_sage_quant_qk_int8_ks(
                q.ptr, k.ptr, b, h, n_q, n_kv, d, q.strides.as_ptr(), k.strides.as_ptr(), q.offset, k.offset,
                self.smooth_k as i32, buf.qi8, buf.ki8, buf.q_scales, buf.k_scales, buf.k_mean, buf.k_smoothed, stream,
            )
        };
        status("flame_sage_quant_qk_int8_ks", rc)?;
        let scale = self.scale.unwrap_or(1.0f32 / (d as f32).sqrt());
        let (bptr, bdt, bst) = match attention_mask {
            Some(m) => (m.ptr, if m.is_f32 { ffi::FLAME_ATTN_DTYPE_F32 } else { ffi::FLAME_ATTN_DTYPE_BF16 }, m.strides.as_ptr()),
            None => (core::ptr::null(), ffi::FLAME_ATTN_DTYPE_F32, core::ptr::null()),
        };
        let rc = unsafe {
            ffi::flame_sage_attn_fwd_bias_int8(
                buf.qi8, buf.ki8, buf.q_scales, buf.k_scales, v.ptr, o.ptr, core::ptr::null_mut(), b, h, n_q, n_kv, d,
                scale, v.strides.as_ptr(), o.strides.as_ptr(), v.offset, o.offset, self.causal as i32, core::ptr::null(),
                bptr, bdt, bst, stream,
            )
        };
        status("flame_sage_attn_fwd_bias_int8", rc)
    }
}

/// The smoothed K of `buf` as the `[B,H,N_kv,D]` view a backward reads (row stride `row_elems(D)`).
pub fn smoothed_k_view(k: &View4, buf: &SageBuffers) -> View4 {
    let [b, h, n_kv, d] = k.shape;
    let r = row_elems(d) as i64;
    View4 { ptr: buf.k_smoothed, shape: [b, h, n_kv, d], strides: [h as i64 * n_kv as i64 * r, n_kv as i64 * r, r, 1], offset: 0 }
}

/// `sage_attention_backward`: standard attention backward on (Q, smoothed K, V).  No attention weights are saved:
/// a bf16 forward on the same three tensors re-forms O and the log-sum-exp rows (`o_tmp`, `lse_tmp`: caller scratch of
/// O's size and of `B*H*N_q` floats), then the recompute backward runs.  The gradient with respect to the smoothed K
/// is the gradient with respect to K (the rows of dS sum to zero, so the mean subtraction's derivative drops out).
#[allow(clippy::too_many_arguments)]
pub fn backward_into(
    q: &View4, k_smoothed: &View4, v: &View4, d_o: &View4, dq: &View4, dk: &View4, dv: &View4, scale: f32, causal: bool,
    o_tmp: &View4, lse_tmp: *mut c_void, workspace: *mut c_void, workspace_bytes: usize, stream: *mut c_void,
) -> Result<()> {
    let [b, h, n_q, d] = q.shape;
    let n_kv = k_smoothed.shape[2];
    let rc = unsafe {
        ffi::flame_attn_fwd_bf16(
            q.ptr, k_smoothed.ptr, v.ptr, o_tmp.ptr, lse_tmp, b, h, n_q, n_kv, d, scale,
            q.strides.as_ptr(), k_smoothed.strides.as_ptr(), v.strides.as_ptr(), o_tmp.strides.as_ptr(),
            q.offset, k_smoothed.offset, v.offset, o_tmp.offset, 0, causal as i32, core::ptr::null(), core::ptr::null(),
            core::ptr::null(), stream,
        )
    };
    status("flame_attn_fwd_bf16", rc)?;
    let rc = unsafe {
        ffi::flame_attn_bwd_bf16(
            q.ptr, k_smoothed.ptr, v.ptr, o_tmp.ptr, d_o.ptr, lse_tmp, dq.ptr, dk.ptr, dv.ptr, b, h, n_q, n_kv, d, scale,
            q.strides.as_ptr(), k_smoothed.strides.as_ptr(), v.strides.as_ptr(), o_tmp.strides.as_ptr(),
            d_o.strides.as_ptr(), dq.strides.as_ptr(), dk.strides.as_ptr(), dv.strides.as_ptr(),
            q.offset, k_smoothed.offset, v.offset, o_tmp.offset, d_o.offset, 0, dq.offset, dk.offset, dv.offset,
            causal as i32, core::ptr::null(), core::ptr::null(), core::ptr::null(),
            workspace, workspace_bytes, stream,
        )
    };
    status("flame_attn_bwd_bf16", rc)
}
