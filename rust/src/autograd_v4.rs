//! The v4 SDPA operator on this library: `sdpa_forward` / `sdpa_backward` of flame-core
//! (src/autograd_v4/ops/sdpa.rs:98-326, :826-1009) with `SdpaSave::SaveLSE` semantics: the context keeps Q, K, V, O and
//! the log-sum-exp rows, never the probabilities (`SaveProbs`, :21-47, exists to keep the `[B,H,N_q,N_kv]` tensor this
//! path avoids and has no counterpart here).  Dropout draws the reference's kept set (one xorshift round of
//! seed ^ index, src/rng/mod.rs:14-24), over the whole tensor or, when the operator chunks, tile by tile.
//!
//! UNVERIFIED SOURCE: never compiled (no Rust toolchain in the image the library is developed in).
use core::ffi::c_void;

use crate::attention::{KeepMask, Workspace};
use crate::ffi;
use crate::sdpa::{Error, Result, View4};

/// The fields of `SdpaConfig` (src/autograd_v4/ops/sdpa.rs:60-96) that reach the kernels.
#[derive(Clone, Copy, Debug, Default)]
pub struct SdpaConfig {
    pub causal: bool,
    pub scale: Option<f32>,
    pub dropout_p: f32,
    /// Must be Some when `dropout_p > 0` (flame-core resolves a missing seed from its global generator, :120-124,
    /// and keeps it in the context; do the same before calling).
    pub dropout_seed: Option<u64>,
    /// Tiles of the chunked draw (`actual_chunk_q`, `actual_chunk_kv`, :182-191); 0 = one draw over the whole tensor.
    pub chunk_q: i32,
    pub chunk_kv: i32,
}

fn status(entry: &str, rc: i32) -> Result<()> {
    if rc == ffi::FLAME_ATTN_OK {
        Ok(())
    } else {
        Err(Error::Device(format!("{entry} HIP error: {rc}")))
    }
}

fn resolve(cfg: &SdpaConfig, d: i32) -> Result<(f32, u64)> {
    if !(cfg.dropout_p >= 0.0 && cfg.dropout_p < 1.0) {
        return Err(Error::InvalidInput(format!("sdpa_forward: dropout_p={} is out of range [0, 1)", cfg.dropout_p)));
    }
    if cfg.dropout_p > 0.0 && cfg.dropout_seed.is_none() {
        return Err(Error::InvalidInput("dropout seed required when dropout_p > 0".into()));
    }
    Ok((cfg.scale.unwrap_or(1.0f32 / (d as f32).sqrt()), cfg.dropout_seed.unwrap_or(0)))
}

/// Forward: O and the log-sum-exp rows `lse` (fp32 `[B*H, N_q]`, those of the undropped softmax).  Fused kernels
/// first; head dims they refuse go through the materialised entry point in `ws`.
#[allow(clippy::too_many_arguments)]
pub fn sdpa_forward_into(
    q: &View4, k: &View4, v: &View4, o: &View4, lse: *mut c_void, mask: Option<&KeepMask>, cfg: &SdpaConfig,
    ws: Workspace, stream: *mut c_void,
) -> Result<()> {
    let [b, h, n_q, d] = q.shape;
    let n_kv = k.shape[2];
    let (scale, seed) = resolve(cfg, d)?;
    let (mptr, mst) = match mask {
        Some(m) => (m.ptr, m.strides.as_ptr()),
        None => (core::ptr::null(), core::ptr::null()),
    };
    let rc = unsafe {
        ffi::flame_attn_fwd_dropout_tiled_bf16(
            q.ptr, k.ptr, v.ptr, o.ptr, lse, b, h, n_q, n_kv, d, scale,
            q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
            q.offset, k.offset, v.offset, o.offset, 0, cfg.causal as i32, core::ptr::null(), mptr, mst,
            cfg.dropout_p, seed, cfg.chunk_q, cfg.chunk_kv, stream,
        )
    };
    if rc != ffi::FLAME_ATTN_ERR_UNSUPPORTED {
        return status("flame_attn_fwd_dropout_tiled_bf16", rc);
    }
    let rc = unsafe {
        ffi::flame_attn_fwd_materialised_bf16(
            q.ptr, k.ptr, v.ptr, o.ptr, lse, b, h, n_q, n_kv, d, d, scale,
            q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
            q.offset, k.offset, v.offset, o.offset, 0, cfg.causal as i32, core::ptr::null(), mptr, mst,
            core::ptr::null(), ffi::FLAME_ATTN_DTYPE_F32, core::ptr::null(),
            cfg.dropout_p, seed, cfg.chunk_q, cfg.chunk_kv, ws.ptr, ws.bytes, stream,
        )
    };
    status("flame_attn_fwd_materialised_bf16", rc)
}

/// Backward from the saved {Q, K, V, O, lse} and the upstream gradient, with the forward's dropout values (the same
/// seed and tiles draw the same kept set).  `ws`: at least `flame_attn_bwd_workspace_bytes` bytes for the fused
/// kernels, `flame_attn_materialised_workspace_bytes(.., 1)` where the materialised path may be needed.
#[allow(clippy::too_many_arguments)]
pub fn sdpa_backward_into(
    q: &View4, k: &View4, v: &View4, o: &View4, lse: *const c_void, d_o: &View4, dq: &View4, dk: &View4, dv: &View4,
    mask: Option<&KeepMask>, cfg: &SdpaConfig, ws: Workspace, stream: *mut c_void,
) -> Result<()> {
    let [b, h, n_q, d] = q.shape;
    let n_kv = k.shape[2];
    let (scale, seed) = resolve(cfg, d)?;
    let (mptr, mst) = match mask {
        Some(m) => (m.ptr, m.strides.as_ptr()),
        None => (core::ptr::null(), core::ptr::null()),
    };
    let rc = unsafe {
        ffi::flame_attn_bwd_dropout_tiled_bf16(
            q.ptr, k.ptr, v.ptr, o.ptr, d_o.ptr, lse, dq.ptr, dk.ptr, dv.ptr, b, h, n_q, n_kv, d, scale,
            q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
            d_o.strides.as_ptr(), dq.strides.as_ptr(), dk.strides.as_ptr(), dv.strides.as_ptr(),
            q.offset, k.offset, v.offset, o.offset, d_o.offset, 0, dq.offset, dk.offset, dv.offset,
            cfg.causal as i32, core::ptr::null(), mptr, mst, cfg.dropout_p, seed, cfg.chunk_q, cfg.chunk_kv,
            ws.ptr, ws.bytes, stream,
        )
    };
    if rc != ffi::FLAME_ATTN_ERR_UNSUPPORTED {
        return status("flame_attn_bwd_dropout_tiled_bf16", rc);
    }
    let rc = unsafe {
        ffi::flame_attn_bwd_materialised_bf16(
            q.ptr, k.ptr, v.ptr, o.ptr, d_o.ptr, lse, dq.ptr, dk.ptr, dv.ptr, b, h, n_q, n_kv, d, d, scale,
            q.strides.as_ptr(), k.strides.as_ptr(), v.strides.as_ptr(), o.strides.as_ptr(),
            d_o.strides.as_ptr(), dq.strides.as_ptr(), dk.strides.as_ptr(), dv.strides.as_ptr(),
            q.offset, k.offset, v.offset, o.offset, d_o.offset, 0, dq.offset, dk.offset, dv.offset,
            cfg.causal as i32, core::ptr::null(), mptr, mst, cfg.dropout_p, seed, cfg.chunk_q, cfg.chunk_kv,
            ws.ptr, ws.bytes, stream,
        )
    };
    status("flame_attn_bwd_materialised_bf16", rc)
}
