//! Rust side of `libflame_attn_hip`: raw bindings and thin operator-level wrappers.
//!
//! UNVERIFIED SOURCE: never compiled (no Rust toolchain in the image the library is developed in).  The tested
//! boundary is the C ABI (`include/flame_attn.h`); `ffi.rs` is held to it by a declaration-by-declaration check.
pub mod attention;
pub mod autograd_v4;
pub mod ffi;
pub mod sage_attention;
pub mod sdpa;
