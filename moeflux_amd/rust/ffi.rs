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

#[repr(C)]
#[derive(Clone, Copy)]
pub struct mfa_matvec_spec {
    pub w_packed: *const u32, pub scales: *const u16, pub biases: *const u16,
    pub x: *const f32, pub out: *mut f32, pub out_dim: i32, pub in_dim: i32,
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

    // device-pointer forms (no host round trip; asynchronous on mfa_stream)
    pub fn mfa_kv_append_dev(ctx: *mut mfa_ctx, layer: i32, k: *const f32, v: *const f32) -> c_int;
    pub fn mfa_sdpa_decode_dev(ctx: *mut mfa_ctx, layer: i32, q: *const f32, q_gate: *const f32,
        out: *mut f32) -> c_int;
    pub fn mfa_gdn_step_dev(ctx: *mut mfa_ctx, layer: i32, qkv_in: *const f32, z: *const f32,
        alpha: *const f32, beta: *const f32, out: *mut f32) -> c_int;
    pub fn mfa_token_sweep_dev(ctx: *mut mfa_ctx, full_q: *const f32, full_gate: *const f32,
        full_out: *mut f32, lin_qkv: *const f32, lin_z: *const f32, lin_alpha: *const f32,
        lin_beta: *const f32, lin_out: *mut f32) -> c_int;
    // what precedes the attention core in a full-attention layer
    pub fn mfa_set_full_weights(ctx: *mut mfa_ctx, layer: i32, q_norm_bf16: *const u16,
        k_norm_bf16: *const u16) -> c_int;
    pub fn mfa_set_rope(ctx: *mut mfa_ctx, theta: f32, rotary_dim: i32) -> c_int;
    pub fn mfa_attn_prologue_dev(ctx: *mut mfa_ctx, layer: i32, pos: i32, q_proj_out: *const f32,
        k: *const f32, v: *const f32, q_out: *mut f32, q_gate_out: *mut f32) -> c_int;
    pub fn mfa_full_attn_step_dev(ctx: *mut mfa_ctx, layer: i32, pos: i32, q_proj_out: *const f32,
        k: *const f32, v: *const f32, out: *mut f32) -> c_int;
    // projections either side of the core
    pub fn mfa_dequant_matvec_4bit_dev(ctx: *mut mfa_ctx, n: i32, specs: *const mfa_matvec_spec) -> c_int;
    pub fn mfa_dequant_matvec_4bit_tiled_dev(ctx: *mut mfa_ctx, n: i32, specs: *const mfa_matvec_spec) -> c_int;
    pub fn mfa_matvec_tiled_words(out_dim: i32, in_dim: i32) -> i64;
    pub fn mfa_matvec_tile_weights_dev(ctx: *mut mfa_ctx, out_dim: i32, in_dim: i32, w_packed: *const u32, w_tiled: *mut u32) -> c_int;
    // attention over a latent cache (MLA, folded form)
    pub fn mfa_mla_sdpa_folded_dev(ctx: *mut mfa_ctx, num_heads: i32, kv_lora_rank: i32,
        qk_rope_head_dim: i32, cache_len: i32, softmax_scale: f32, q_prime: *const f32,
        q_pe: *const f32, latent_cache: *const f32, rope_k_cache: *const f32,
        v_combine: *mut f32) -> c_int;
    // 'MFLX' snapshot
    pub fn mfa_state_size(ctx: *mut mfa_ctx) -> i64;
    pub fn mfa_state_save(ctx: *mut mfa_ctx, buf: *mut u8, buf_len: i64) -> i64;
    pub fn mfa_state_load(ctx: *mut mfa_ctx, buf: *const u8, buf_len: i64) -> c_int;
}
