//! `extern "C"` view of include/moeflux_attn.h for the Rust host (the production
//! subset; the per-kernel hooks bind the same way).  Written against the header,
//! not compiled in this repository's image (no rustc).
#![allow(non_camel_case_types)]
use std::os::raw::{c_char, c_int, c_void};

#[repr(C)]
pub struct mfa_ctx { _private: [u8; 0] }

#[repr(C)]
#[derive(Clone, Copy)]
pub struct mfa_config {
    pub num_layers: i32, pub full_attn_interval: i32,
    pub num_attn_heads: i32, pub num_kv_heads: i32, pub head_dim: i32,
    pub kv_capacity: i32, pub kv_dtype: i32,
    pub linear_num_k_heads: i32, pub linear_num_v_heads: i32,
    pub linear_key_dim: i32, pub linear_value_dim: i32,
    pub conv_kernel_size: i32, pub rms_norm_eps: f32,
}

extern "C" {
    pub fn mfa_ctx_create(cfg: *const mfa_config) -> *mut mfa_ctx;
    pub fn mfa_ctx_destroy(ctx: *mut mfa_ctx);
    pub fn mfa_last_error_string() -> *const c_char;
    pub fn mfa_sync(ctx: *mut mfa_ctx) -> c_int;
    pub fn mfa_stream(ctx: *mut mfa_ctx) -> *mut c_void;
    pub fn mfa_set_linear_weights(ctx: *mut mfa_ctx, layer: i32, conv_w_bf16: *const u16,
        a_log: *const f32, dt_bias_bf16: *const u16, norm_w_bf16: *const u16) -> c_int;
    pub fn mfa_kv_append(ctx: *mut mfa_ctx, layer: i32, k: *const f32, v: *const f32) -> c_int;
    pub fn mfa_kv_len(ctx: *mut mfa_ctx, layer: i32) -> i32;
    pub fn mfa_sdpa_decode(ctx: *mut mfa_ctx, layer: i32, q: *const f32, q_gate: *const f32,
        out: *mut f32) -> c_int;
    pub fn mfa_gdn_step(ctx: *mut mfa_ctx, layer: i32, qkv_in: *const f32, z: *const f32,
        alpha: *const f32, beta: *const f32, out: *mut f32) -> c_int;
    pub fn mfa_prefill_attn(ctx: *mut mfa_ctx, layer: i32, t: i32, q: *const f32,
        q_gate: *const f32, k: *const f32, v: *const f32, out: *mut f32) -> c_int;
    pub fn mfa_prefill_gdn(ctx: *mut mfa_ctx, layer: i32, t: i32, qkv_in: *const f32,
        z: *const f32, alpha: *const f32, beta: *const f32, out: *mut f32) -> c_int;
    pub fn mfa_reset(ctx: *mut mfa_ctx) -> c_int;
    pub fn mfa_truncate(ctx: *mut mfa_ctx, p0: i32, p1: i32) -> c_int;
    pub fn mfa_pos_max(ctx: *mut mfa_ctx) -> i32;
    pub fn mfa_kv_export(ctx: *mut mfa_ctx, layer: i32, max_rows: i32, k: *mut f32, v: *mut f32) -> c_int;
    pub fn mfa_kv_import(ctx: *mut mfa_ctx, layer: i32, len: i32, k: *const f32, v: *const f32) -> c_int;
    pub fn mfa_linear_state_export(ctx: *mut mfa_ctx, layer: i32, conv: *mut f32, ssm: *mut f32) -> c_int;
    pub fn mfa_linear_state_import(ctx: *mut mfa_ctx, layer: i32, conv: *const f32, ssm: *const f32) -> c_int;
}
