//! `extern "C"` view of include/moeflux_attn.h for the Rust host: every entry point of the
//! header, the production path first, then the per-kernel hooks of the differential tests.
//! Written against the header, not compiled in this repository's image (no rustc); a test
//! checks names and parameter counts against the header.
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
    pub fn mfa_sdpa_decode_static_dev(ctx: *mut mfa_ctx, layer: i32, q_dev: *const f32, q_gate_dev: *const f32,
        out_dev: *mut f32) -> c_int;
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
    pub fn mfa_prefill_full_attn(ctx: *mut mfa_ctx, layer: i32, pos0: i32, t: i32, q_proj_out: *const f32,
        k: *const f32, v: *const f32, out: *mut f32) -> c_int;
    pub fn mfa_prefill_full_attn_dev(ctx: *mut mfa_ctx, layer: i32, pos0: i32, t: i32,
        q_proj_out_dev: *const f32, k_dev: *const f32, v_dev: *const f32, out_dev: *mut f32) -> c_int;
    // projections either side of the core
    pub fn mfa_dequant_matvec_4bit_dev(ctx: *mut mfa_ctx, n: i32, specs: *const mfa_matvec_spec) -> c_int;
    pub fn mfa_dequant_matvec_4bit_tiled_dev(ctx: *mut mfa_ctx, n: i32, specs: *const mfa_matvec_spec) -> c_int;
    pub fn mfa_matvec_tiled_words(out_dim: i32, in_dim: i32) -> i64;
    pub fn mfa_matvec_tile_weights_dev(ctx: *mut mfa_ctx, out_dim: i32, in_dim: i32, w_packed: *const u32, scales: *const u16, biases: *const u16, w_tiled: *mut u32) -> c_int;
    // attention over a latent cache (MLA, folded form)
    pub fn mfa_mla_sdpa_folded_dev(ctx: *mut mfa_ctx, num_heads: i32, kv_lora_rank: i32,
        qk_rope_head_dim: i32, cache_len: i32, softmax_scale: f32, q_prime: *const f32,
        q_pe: *const f32, latent_cache: *const f32, rope_k_cache: *const f32,
        v_combine: *mut f32) -> c_int;
    // 'MFLX' snapshot
    pub fn mfa_state_size(ctx: *mut mfa_ctx) -> i64;
    pub fn mfa_state_save(ctx: *mut mfa_ctx, buf: *mut u8, buf_len: i64) -> i64;
    pub fn mfa_state_load(ctx: *mut mfa_ctx, buf: *const u8, buf_len: i64) -> c_int;
    // checkpoints by sequence position, kept on the device
    pub fn mfa_checkpoint_pos(ctx: *mut mfa_ctx, pos: i32) -> c_int;
    pub fn mfa_restore_to(ctx: *mut mfa_ctx, pos: i32) -> c_int;
    pub fn mfa_set_max_checkpoints(ctx: *mut mfa_ctx, n: i32) -> c_int;
    pub fn mfa_checkpoint_count(ctx: *mut mfa_ctx) -> i32;

    // host-pointer forms of the layer step and the bulk bf16 import
    pub fn mfa_attn_prologue(ctx: *mut mfa_ctx, layer: i32, pos: i32, q_proj_out: *const f32,
        k: *const f32, v: *const f32, q_out: *mut f32, q_gate_out: *mut f32) -> c_int;
    pub fn mfa_full_attn_step(ctx: *mut mfa_ctx, layer: i32, pos: i32, q_proj_out: *const f32,
        k: *const f32, v: *const f32, out: *mut f32) -> c_int;
    pub fn mfa_kv_import_bf16(ctx: *mut mfa_ctx, layer: i32, len: i32, k: *const u16, v: *const u16) -> c_int;
    // prompt chunks on device pointers
    pub fn mfa_prefill_attn_dev(ctx: *mut mfa_ctx, layer: i32, t: i32, q_dev: *const f32,
        q_gate_dev: *const f32, k_dev: *const f32, v_dev: *const f32, out_dev: *mut f32) -> c_int;
    pub fn mfa_prefill_gdn_dev(ctx: *mut mfa_ctx, layer: i32, t: i32, qkv_in_dev: *const f32,
        z_dev: *const f32, alpha_dev: *const f32, beta_dev: *const f32, out_dev: *mut f32) -> c_int;
    // tuning and measurement
    pub fn mfa_set_num_splits(ctx: *mut mfa_ctx, num_splits: i32) -> c_int;
    pub fn mfa_set_partial_only(ctx: *mut mfa_ctx, on: i32) -> c_int;
    pub fn mfa_set_step_launches(ctx: *mut mfa_ctx, launches: i32) -> c_int;
    pub fn mfa_host_alloc(bytes: i64) -> *mut c_void;
    pub fn mfa_host_free(p: *mut c_void);
    pub fn mfa_set_sweep_per_layer(ctx: *mut mfa_ctx, on: i32) -> c_int;
    pub fn mfa_timer_start(ctx: *mut mfa_ctx) -> c_int;
    pub fn mfa_timer_stop(ctx: *mut mfa_ctx, elapsed_ms: *mut f32) -> c_int;

    // stateless per-kernel hooks (host pointers, synchronous): what tests/diff_oracle.rs drives
    pub fn mfa_sdpa(kv_len: i32, num_attn_heads: i32, num_kv_heads: i32, head_dim: i32, q: *const f32,
        q_gate: *const f32, k_cache: *const f32, v_cache: *const f32, out: *mut f32) -> c_int;
    pub fn mfa_sdpa_bf16kv(kv_len: i32, num_attn_heads: i32, num_kv_heads: i32, head_dim: i32,
        q: *const f32, q_gate: *const f32, k_cache: *const u16, v_cache: *const u16, out: *mut f32) -> c_int;
    pub fn mfa_attn_scores_batched(num_heads: i32, num_kv_heads: i32, head_dim: i32, seq_len: i32,
        q: *const f32, k_cache: *const f32, scale: f32, scores_out: *mut f32) -> c_int;
    pub fn mfa_attn_softmax_batched(num_heads: i32, seq_len: i32, scores_inout: *mut f32) -> c_int;
    pub fn mfa_attn_values_batched(num_heads: i32, num_kv_heads: i32, head_dim: i32, seq_len: i32,
        scores: *const f32, v_cache: *const f32, out: *mut f32) -> c_int;
    pub fn mfa_sigmoid_gate(dim: i32, gate: *const f32, x_inout: *mut f32) -> c_int;
    pub fn mfa_conv1d_step(channels: i32, kernel_size: i32, conv_state_inout: *mut f32,
        new_input: *const f32, weight_bf16: *const u16, out: *mut f32) -> c_int;
    pub fn mfa_rms_norm_qk(num_k_heads: i32, key_dim: i32, q_inout: *mut f32, k_inout: *mut f32) -> c_int;
    pub fn mfa_rms_norm_bare(dim: i32, eps: f32, x: *const f32, out: *mut f32) -> c_int;
    pub fn mfa_compute_decay_beta(num_v_heads: i32, alpha: *const f32, beta: *const f32,
        a_log: *const f32, dt_bias_bf16: *const u16, g_decay_out: *mut f32, beta_gate_out: *mut f32) -> c_int;
    pub fn mfa_gated_delta_net_step(v_heads: i32, k_heads: i32, key_dim: i32, value_dim: i32,
        g_decay: *const f32, beta_gate: *const f32, q: *const f32, k: *const f32, v: *const f32,
        ssm_state_inout: *mut f32, out_values: *mut f32) -> c_int;
    pub fn mfa_gated_delta_recurrence(a_log: *const f32, dt_bias_bf16: *const u16, alpha: *const f32,
        beta: *const f32, q: *const f32, k: *const f32, v: *const f32, v_heads: i32, k_heads: i32,
        key_dim: i32, value_dim: i32, ssm_state_inout: *mut f32, out_values: *mut f32) -> c_int;
    pub fn mfa_gated_rms_norm(num_heads: i32, dim: i32, eps: f32, x: *const f32, z: *const f32,
        weight_bf16: *const u16, out: *mut f32) -> c_int;
    pub fn mfa_dequant_matvec_4bit(out_dim: i32, in_dim: i32, group_size: i32, w_packed: *const u32,
        scales: *const u16, biases: *const u16, x: *const f32, out: *mut f32) -> c_int;
    pub fn mfa_mla_sdpa_folded(num_heads: i32, kv_lora_rank: i32, qk_rope_head_dim: i32, cache_len: i32,
        softmax_scale: f32, q_prime: *const f32, q_pe: *const f32, latent_cache: *const f32,
        rope_k_cache: *const f32, v_combine: *mut f32) -> c_int;

    // diagnostics of the cache layout, the split planning and the copy used to calibrate counters
    pub fn mfa_debug_kv_offset(kv_dtype: i32, is_v: i32, pos: i64, x: i32, head_dim: i32) -> i64;
    pub fn mfa_debug_num_splits(kv_dtype: i32, num_attn_heads: i32, num_kv_heads: i32, head_dim: i32,
        kv_len: i64, num_cus: i32, forced_splits: i32) -> i32;
    pub fn mfa_debug_max_splits(kv_dtype: i32, num_attn_heads: i32, num_kv_heads: i32, head_dim: i32,
        max_len: i64, num_cus: i32, forced_splits: i32) -> i32;
    pub fn mfa_debug_copy_dev(ctx: *mut mfa_ctx, dst_dev: *mut c_void, src_dev: *const c_void,
        nbytes: usize) -> c_int;
    pub fn mfa_debug_read_dev(ctx: *mut mfa_ctx, src_dev: *const c_void, nbytes: usize, workgroups: i32) -> c_int;
    pub fn mfa_debug_fill_workspace(ctx: *mut mfa_ctx, pattern: u32) -> c_int;
}
