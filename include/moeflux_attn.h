/*
 * moeflux_attn.h — C ABI of the MI355X (gfx950) attention path for moeflux.
 *
 * The library replaces, for the attention core of each layer, what the Rust
 * host of mdegans/moeflux hands to metal-rs: the four full-attention kernels
 * and the five Gated-DeltaNet kernels, together with the per-layer state they
 * read and write (KV cache, conv state, recurrent state).  Each declaration
 * cites the reference interface it stands in for.  Conventions are those of
 * the reference's own C API (crates/moeflux-sys/metal_infer/moeflux.h:9-11,
 * 38, 52-64, 177-182): an opaque context first, int32_t shapes, caller-owned
 * buffers, 0 on success and a negative code on error, NULL from create on
 * failure, destroy(NULL) is a no-op.  A context is single-threaded
 * (crates/moeflux/src/lib.rs:22-27); two contexts may be used concurrently.
 *
 * Host-pointer entry points are synchronous at return.  `_dev` entry points
 * take device pointers, enqueue on the context's HIP stream and return; pair
 * them with mfa_sync().
 */
#ifndef MOEFLUX_ATTN_H
#define MOEFLUX_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Every declaration below is an exported symbol of libmoeflux_attn_hip.so. */
#pragma GCC visibility push(default)

typedef struct mfa_ctx mfa_ctx;

/* Error codes.  The reference collapses every failure to -1
 * (moeflux.h:177-178, 473-474); this library keeps "negative means failure"
 * and distinguishes the classes the Rust side maps to typed errors
 * (SdpaError sdpa.rs:41-55, LinearAttnError linear_attn.rs:29-54,
 * GpuAttnError gpu_attn.rs:46-63). */
#define MFA_OK 0
#define MFA_ERR_INVALID (-1)  /* NULL pointer, non-positive shape, kv_len <= 0, divisibility */
#define MFA_ERR_SHAPE (-2)    /* valid but unsupported by the kernels (head_dim, key_dim ...) */
#define MFA_ERR_OVERFLOW (-3) /* KV append past capacity (full_attn_forward.rs:283-288) */
#define MFA_ERR_LAYER (-4)    /* layer index out of range or of the other kind */
#define MFA_ERR_HIP (-5)      /* a HIP runtime call failed; see mfa_last_error_string() */
#define MFA_ERR_STATE (-6)    /* snapshot does not match this context (state_snapshot.rs preflight) */
#define MFA_ERR_NO_CHECKPOINT (-7) /* mfa_restore_to: nothing stored at that position (CheckpointError::NoCheckpoint, riir/mod.rs:111-124) */

#define MFA_KV_F32 0
#define MFA_KV_BF16 1

/* Shapes are run-time values, as the reference's kernel arguments are
 * (NOTES.md:92-103); they mirror the fields of `Variant`
 * (crates/moeflux/src/riir/variants.rs:383-465). */
typedef struct mfa_config {
    int32_t num_layers;
    int32_t full_attn_interval;  /* layer i is full attention iff (i+1) % interval == 0 (variants.rs:258-264) */
    int32_t num_attn_heads;
    int32_t num_kv_heads;
    int32_t head_dim;            /* 64, 128 or 256 */
    int32_t kv_capacity;         /* positions per full-attention layer (reference: GPU_KV_SEQ / MAX_SEQ_LEN, variants.rs:377-379) */
    int32_t kv_dtype;            /* MFA_KV_F32 or MFA_KV_BF16 */
    int32_t linear_num_k_heads;
    int32_t linear_num_v_heads;
    int32_t linear_key_dim;      /* 128 (variants.rs:219-223) */
    int32_t linear_value_dim;    /* 128 */
    int32_t conv_kernel_size;    /* 4 */
    float rms_norm_eps;          /* 1e-6 (variants.rs:358) */
} mfa_config;

/* ---- lifecycle ----------------------------------------------------------- */

/* Replaces RsCtx::open's state allocation (riir/mod.rs:270-318,
 * state.rs:400-413) and LayerForwardBuffers::new (linear_attn_forward.rs:
 * 180-244) for the attention state: allocates, zero-filled, one KV cache per
 * full-attention layer and one conv + recurrent state per linear layer, plus
 * the split-K workspace and one HIP stream.  NULL on failure. */
mfa_ctx *mfa_ctx_create(const mfa_config *cfg);
/* moeflux.h:62-64 (mf_free_model).  No-op on NULL. */
void mfa_ctx_destroy(mfa_ctx *ctx);
/* Text of the last error on the calling thread ("" if none). */
const char *mfa_last_error_string(void);
/* Block until everything enqueued on the context's stream has finished. */
int mfa_sync(mfa_ctx *ctx);
/* The context's hipStream_t, for callers that enqueue their own work around
 * the `_dev` calls. */
void *mfa_stream(mfa_ctx *ctx);

/* Per-layer constants of a linear-attention layer, read by the reference from
 * the weight file inside each call (linear_attn_forward.rs:607-664 passes
 * conv1d.weight, A_log, dt_bias, norm.weight offsets).  Host pointers, copied.
 *   conv_w_bf16 [C*K] channel-major, a_log f32 [Hv], dt_bias_bf16 [Hv],
 *   norm_w_bf16 [dv]. */
int mfa_set_linear_weights(mfa_ctx *ctx, int32_t layer, const uint16_t *conv_w_bf16,
                           const float *a_log, const uint16_t *dt_bias_bf16,
                           const uint16_t *norm_w_bf16);

/* Override the split-K partition count of the decode kernel and of
 * mfa_mla_sdpa_folded_dev (0 = automatic).
 * The result must not depend on it; tests use it to check exactly that, as
 * the reference checks tiled against single-shot MLA (tests/mla_sdpa_tiled.rs:
 * 176-216). */
int mfa_set_num_splits(mfa_ctx *ctx, int32_t num_splits);
/* Measurement aid with no reference counterpart: when `on` is non-zero the
 * decode entry points launch only the split-K partial kernel (no merge, `out`
 * is not written), so that a timed loop isolates the kernel that streams the
 * cache.  Default off. */
int mfa_set_partial_only(mfa_ctx *ctx, int32_t on);

/* ---- full attention: production path -------------------------------------- */

/* Replaces the KV append of full_attn_forward.rs:282-323 (host cache row +
 * GPU mirror row).  k, v: [num_kv_heads*head_dim] f32 host rows (K post-norm
 * post-RoPE, V raw).  MFA_ERR_OVERFLOW when the layer is full. */
int mfa_kv_append(mfa_ctx *ctx, int32_t layer, const float *k, const float *v);
int mfa_kv_append_dev(mfa_ctx *ctx, int32_t layer, const float *k_dev, const float *v_dev);
/* KvCache::len (state.rs:37-41). */
int32_t mfa_kv_len(mfa_ctx *ctx, int32_t layer);

/* Replaces both branches of full_attn_forward.rs:331-389: the four-kernel GPU
 * chain attn_scores_batched / attn_softmax_batched / attn_values_batched /
 * sigmoid_gate (linear_attn_forward.rs:850-902) and the sdpa_cpu fallback
 * (sdpa.rs:63-172), at every kv_len >= 1.  q, q_gate, out: [Hq*head_dim] f32. */
int mfa_sdpa_decode(mfa_ctx *ctx, int32_t layer, const float *q, const float *q_gate,
                    float *out);
int mfa_sdpa_decode_dev(mfa_ctx *ctx, int32_t layer, const float *q_dev,
                        const float *q_gate_dev, float *out_dev);

/* mfa_sdpa_decode_dev for callers that cannot allocate.  It has no counterpart in the
 * reference: it is for code under HIP graph capture, tight serving loops and harnesses that
 * forbid hipMalloc.  Same arguments, same kernels, same results bit for bit; the split-K
 * partials go into a file-scope device array of the library (8.25 MiB per GPU, held until the
 * process ends; its address is looked up when the first context on a device is created)
 * instead of the context's workspace, and the call makes no hipMalloc, hipFree or other
 * allocating call whatever the cache length.  MFA_ERR_INVALID, with nothing launched, when the
 * split plan's partials exceed the array (more than 2 Mi f32 of partial rows: for instance
 * more than 128 splits of 2 kv-head groups at head_dim 256).  All calls on one GPU share the
 * array: calls that overlap on one GPU (two contexts, two streams) race; calls on one context
 * are ordered by its stream.  Nothing in the array has to be cleared between calls. */
int mfa_sdpa_decode_static_dev(mfa_ctx *ctx, int32_t layer, const float *q_dev,
                               const float *q_gate_dev, float *out_dev);

/* ---- the projections either side of the attention core ------------------------ */

/* One 4-bit group-64 affine dequantising matrix-vector product, all pointers on
 * the device: w_packed [out_dim, in_dim/8] u32 (nibble n of a word is input
 * 8*word+n), scales, biases [out_dim, in_dim/64] bf16, x [in_dim], out [out_dim]. */
typedef struct mfa_matvec_spec {
    const uint32_t *w_packed;
    const uint16_t *scales;
    const uint16_t *biases;
    const float *x;
    float *out;
    int32_t out_dim;
    int32_t in_dim;
} mfa_matvec_spec;

/* Replaces the batched dequant_matvec_4bit_v3 dispatches that feed and drain the
 * attention core (shaders.metal:251-340; encoders gpu_matvec.rs; call sites
 * full_attn_forward.rs:193-227 for q/k/v_proj, linear_attn_forward.rs:560-605 for
 * in_proj_qkv/z/a/b, and o_proj / out_proj): n (1..8) products in one launch on
 * the context's stream.  in_dim a multiple of 64, at most 16384.  w and x must be
 * 16-byte aligned (MFA_ERR_INVALID otherwise); scales and biases may start anywhere,
 * rows of them on 16-byte boundaries are read faster. */
int mfa_dequant_matvec_4bit_dev(mfa_ctx *ctx, int32_t n, const mfa_matvec_spec *specs);
/* The same products over a matrix re-ordered once at load time (the reference uploads its weight
 * file once, weights.rs / WeightFile; on a discrete GPU that upload is the place to re-order):
 * for every 16 rows and every 1024 inputs the bytes a wave requests, in request order - the
 * scales and biases it multiplies with, then its weights - so that a wave's requests are nine
 * contiguous KiB.  mfa_matvec_tiled_words gives the size of the re-ordered copy in 32-bit words
 * (rows padded to 16, inputs to 1024; negative on a bad shape), mfa_matvec_tile_weights_dev
 * writes it from the file's three arrays (device to device, on the context's stream), and
 * mfa_dequant_matvec_4bit_tiled_dev takes specs whose w_packed point at such copies and whose
 * scales and biases are not read (they may be NULL); x, out and the results, bit for bit, are
 * those of mfa_dequant_matvec_4bit_dev. */
int64_t mfa_matvec_tiled_words(int32_t out_dim, int32_t in_dim);
int mfa_matvec_tile_weights_dev(mfa_ctx *ctx, int32_t out_dim, int32_t in_dim, const uint32_t *w_packed,
                                const uint16_t *scales, const uint16_t *biases, uint32_t *w_tiled);
int mfa_dequant_matvec_4bit_tiled_dev(mfa_ctx *ctx, int32_t n, const mfa_matvec_spec *specs);
/* Stateless host-pointer twin of dequant_matvec_4bit_cpu (cpu_matvec.rs:83-160;
 * cpu_dequant_matvec, infer.m:671).  group_size must be 64. */
int mfa_dequant_matvec_4bit(int32_t out_dim, int32_t in_dim, int32_t group_size,
                            const uint32_t *w_packed, const uint16_t *scales,
                            const uint16_t *biases, const float *x, float *out);

/* ---- attention over a latent cache (multi-head latent attention, folded) ------ */

/* Replaces mla_sdpa_folded and its tiled form mla_sdpa_tile_accumulate /
 * mla_sdpa_tile_finalize (shaders.metal:1688-1987; encoders
 * gpu_mla.rs:146-200 encode_mla_sdpa_folded and :202 encode_mla_sdpa_folded_tiled;
 * call site mla_attn_forward.rs:462-476) at every cache_len >= 1, one launch pair whatever the
 * length: per head h, scores (q_prime[h] . latent[t] + q_pe[h] . rope_k[t]) *
 * softmax_scale over t in [0, cache_len), softmax, v_combine[h] = sum_t w[t]
 * latent[t].  All f32, all on the device, on the context's stream:
 *   q_prime, v_combine [num_heads, kv_lora_rank]; q_pe [num_heads, qk_rope_head_dim];
 *   latent_cache [cache_len, kv_lora_rank]; rope_k_cache [cache_len, qk_rope_head_dim].
 * Built for kv_lora_rank 512, qk_rope_head_dim 64 (variants.rs, the MLA variants);
 * other widths return MFA_ERR_SHAPE.  The context supplies the stream and the
 * split workspace; its own layers and caches are not touched. */
int mfa_mla_sdpa_folded_dev(mfa_ctx *ctx, int32_t num_heads, int32_t kv_lora_rank,
                            int32_t qk_rope_head_dim, int32_t cache_len, float softmax_scale,
                            const float *q_prime_dev, const float *q_pe_dev,
                            const float *latent_cache_dev, const float *rope_k_cache_dev,
                            float *v_combine_dev);
/* Stateless host-pointer twin (the shape of the reference's test harness,
 * tests/mla_sdpa_tiled.rs:84-140): uploads, runs the same kernels, downloads. */
int mfa_mla_sdpa_folded(int32_t num_heads, int32_t kv_lora_rank, int32_t qk_rope_head_dim,
                        int32_t cache_len, float softmax_scale, const float *q_prime,
                        const float *q_pe, const float *latent_cache, const float *rope_k_cache,
                        float *v_combine);

/* ---- what precedes the attention core in a full-attention layer -------------- */

/* Per-layer constants of the prologue: the bf16 weights of the per-head RMS
 * norms of q and k (model.layers.N.self_attn.{q,k}_norm.weight,
 * full_attn_forward.rs:256-277), head_dim values each. */
int mfa_set_full_weights(mfa_ctx *ctx, int32_t layer, const uint16_t *q_norm_bf16,
                         const uint16_t *k_norm_bf16);
/* The rotation of q and k: base frequency and number of rotated channels per
 * head.  Defaults at create: theta = 1e7, rotary_dim = head_dim / 4
 * (variants.rs:245-250, 369). */
int mfa_set_rope(mfa_ctx *ctx, float theta, int32_t rotary_dim);

/* Replaces the host round trip of full_attn_forward.rs:234-323 for one token:
 * the q projection's output [Hq][q_h | gate_h] is split (238-254), q and k get
 * the per-head RMS norm (rms_norm.rs:104-156), the first rotary_dim channels of
 * every q and k head are rotated at position `pos` (rope.rs:65-131), and k
 * (normed, rotated) and v (as is) are appended to the layer's cache
 * (282-323).  q_out, q_gate_out: [Hq*head_dim], what mfa_sdpa_decode takes.
 * MFA_ERR_OVERFLOW when the layer is full. */
int mfa_attn_prologue(mfa_ctx *ctx, int32_t layer, int32_t pos, const float *q_proj_out,
                      const float *k, const float *v, float *q_out, float *q_gate_out);
int mfa_attn_prologue_dev(mfa_ctx *ctx, int32_t layer, int32_t pos, const float *q_proj_out_dev,
                          const float *k_dev, const float *v_dev, float *q_out_dev,
                          float *q_gate_out_dev);
/* The prologue followed by the attention core on the appended cache: everything
 * of full_attn_layer_forward between the projections and o_proj
 * (full_attn_forward.rs:234-389).  out: [Hq*head_dim]. */
int mfa_full_attn_step(mfa_ctx *ctx, int32_t layer, int32_t pos, const float *q_proj_out,
                       const float *k, const float *v, float *out);
int mfa_full_attn_step_dev(mfa_ctx *ctx, int32_t layer, int32_t pos, const float *q_proj_out_dev,
                           const float *k_dev, const float *v_dev, float *out_dev);
/* How many launches mfa_full_attn_step makes; no counterpart in the reference and no result
 * depends on it beyond rounding.  2 (default, where rotary_dim / 2 is a multiple of 8 channels
 * for a bf16 cache, 4 for f32): the attention launch norms and rotates its own query heads from
 * q_proj_out, attends to the positions the cache already holds, and scores and appends the new
 * token; the merge launch takes the token as one more split.  3: prologue, attention, merge. */
int mfa_set_step_launches(mfa_ctx *ctx, int32_t launches);
/* The same for a chunk of T prompt tokens at positions pos0 .. pos0+T-1 (the token
 * loop of eval_prompt, riir/mod.rs:1196-1214, over full_attn_layer_forward): every
 * token's q and k are normed and rotated at its own position, the T rows are
 * appended, and row t attends to the cache up to and including itself.  Same
 * results as T calls of mfa_full_attn_step.  q_proj_out: [T][Hq][2*head_dim],
 * k, v: [T][num_kv_heads*head_dim], out: [T][Hq*head_dim].  Nothing is appended
 * when the call fails (MFA_ERR_OVERFLOW when the chunk does not fit). */
int mfa_prefill_full_attn(mfa_ctx *ctx, int32_t layer, int32_t pos0, int32_t T,
                          const float *q_proj_out, const float *k, const float *v, float *out);
int mfa_prefill_full_attn_dev(mfa_ctx *ctx, int32_t layer, int32_t pos0, int32_t T,
                              const float *q_proj_out_dev, const float *k_dev,
                              const float *v_dev, float *out_dev);

/* A chunk of T prompt tokens on one full-attention layer.  The reference has
 * no batched prefill: eval_prompt is a token loop (riir/mod.rs:1196-1214); the
 * result equals T successive mfa_kv_append + mfa_sdpa_decode calls.
 *   q, q_gate, out: [T, Hq*head_dim]; k, v: [T, num_kv_heads*head_dim]. */
int mfa_prefill_attn(mfa_ctx *ctx, int32_t layer, int32_t T, const float *q,
                     const float *q_gate, const float *k, const float *v, float *out);
int mfa_prefill_attn_dev(mfa_ctx *ctx, int32_t layer, int32_t T, const float *q_dev,
                         const float *q_gate_dev, const float *k_dev, const float *v_dev,
                         float *out_dev);

/* ---- Gated DeltaNet: production path -------------------------------------- */

/* Replaces the five-kernel chain conv1d_step, rms_norm_qk, compute_decay_beta,
 * gated_delta_net_step, gated_rms_norm encoded at linear_attn_forward.rs:
 * 607-664 (encoders gpu_linear_attn.rs:54-202).  qkv_in [C] = [q|k|v] f32 with
 * C = 2*Hk*dk + Hv*dv; z, out [Hv*dv]; alpha, beta [Hv].  Advances the
 * layer's conv state and recurrent state. */
int mfa_gdn_step(mfa_ctx *ctx, int32_t layer, const float *qkv_in, const float *z,
                 const float *alpha, const float *beta, float *out);
int mfa_gdn_step_dev(mfa_ctx *ctx, int32_t layer, const float *qkv_in_dev,
                     const float *z_dev, const float *alpha_dev, const float *beta_dev,
                     float *out_dev);

/* T prompt tokens on one linear layer; equals T successive mfa_gdn_step calls
 * (riir/mod.rs:1196-1214).  Inputs are [T, ...] row-major. */
int mfa_prefill_gdn(mfa_ctx *ctx, int32_t layer, int32_t T, const float *qkv_in,
                    const float *z, const float *alpha, const float *beta, float *out);
int mfa_prefill_gdn_dev(mfa_ctx *ctx, int32_t layer, int32_t T, const float *qkv_in_dev,
                        const float *z_dev, const float *alpha_dev, const float *beta_dev,
                        float *out_dev);

/* ---- one token's attention launches over the whole stack ------------------ */

/* The attention work of one step_internal layer loop (riir/mod.rs:1769-1888):
 * for each layer in order, mfa_sdpa_decode_dev or mfa_gdn_step_dev on that
 * layer's slice of the inputs.  Inputs are packed per kind, in layer order:
 *   full_q, full_gate, full_out: [n_full, Hq*head_dim];
 *   lin_qkv [n_lin, C]; lin_z, lin_out [n_lin, Hv*dv]; lin_alpha, lin_beta [n_lin, Hv].
 * The KV caches are used as they stand (append first).
 *
 * Because all of a token's inputs are handed over at once, the layers of a kind
 * that stand at the same position (equal kv length; equal conv ring slot) are
 * computed by one launch over all of them; results equal the per-layer loop.
 * A caller whose layers depend on each other (the model itself: layer i+1's
 * projections read layer i's output) calls mfa_sdpa_decode_dev / mfa_gdn_step_dev
 * layer by layer instead; a caller that batches independent sequences or layers
 * uses this. */
int mfa_token_sweep_dev(mfa_ctx *ctx, const float *full_q, const float *full_gate,
                        float *full_out, const float *lin_qkv, const float *lin_z,
                        const float *lin_alpha, const float *lin_beta, float *lin_out);

/* Measurement control for mfa_token_sweep_dev: on != 0 forces one launch chain per
 * layer (the cost a data-dependent caller sees); 0 (default) lets it launch once per
 * kind.  No counterpart in the reference. */
int mfa_set_sweep_per_layer(mfa_ctx *ctx, int32_t on);

/* ---- state operations ------------------------------------------------------ */

/* memory_clear (riir/mod.rs:1950-1969; state.rs clear_all): KV lengths to 0,
 * caches zeroed, conv and recurrent state zeroed, checkpoints dropped. */
int mfa_reset(mfa_ctx *ctx);
/* memory_seq_rm (state.rs:431-455): every KV cache keeps positions
 * [0, min(max(p0,0), p1<0 ? len : min(p1,len))) and the dropped rows are
 * zero-filled; every linear layer is reset (lossy, as in the reference). */
int mfa_truncate(mfa_ctx *ctx, int32_t p0, int32_t p1);
/* memory_seq_pos_max (state.rs:457-473): largest KV length, -1 if the stack
 * has no full-attention layer. */
int32_t mfa_pos_max(mfa_ctx *ctx);

/* Per-layer state in the reference's host layouts (the buffers
 * state_snapshot.rs:16-27 serialises).  KV rows are [len, num_kv_heads*head_dim]
 * f32 (a bf16 cache widens exactly on export and rounds to nearest-even on
 * import); conv state is [K-1, C] time-major with the newest input last;
 * recurrent state is [Hv, dv, dk]. */
int mfa_kv_export(mfa_ctx *ctx, int32_t layer, int32_t max_rows, float *k_out, float *v_out);
int mfa_kv_import(mfa_ctx *ctx, int32_t layer, int32_t len, const float *k, const float *v);
/* Same as mfa_kv_import with rows already in bf16 bits (context must be MFA_KV_BF16). */
int mfa_kv_import_bf16(mfa_ctx *ctx, int32_t layer, int32_t len, const uint16_t *k,
                       const uint16_t *v);
int mfa_linear_state_export(mfa_ctx *ctx, int32_t layer, float *conv_state_out,
                            float *ssm_state_out);
int mfa_linear_state_import(mfa_ctx *ctx, int32_t layer, const float *conv_state,
                            const float *ssm_state);

/* The whole context's state in the reference's snapshot wire format ('MFLX',
 * state_snapshot.rs:1-73; state_size :184-216, state_save :218-360, state_load
 * :362-640): header of 10 little-endian u32, then per layer `i32 len` + K rows + V
 * rows ([len, num_kv_heads*head_dim] f32) or conv state + recurrent state.  Saved
 * as version 2 with both MLA fields 0; versions 1 and 2 load.  Call at token
 * boundaries only (moeflux.h:614-617).  mfa_state_size / mfa_state_save return a
 * byte count or a negative code; mfa_state_load checks the whole buffer before
 * it restores anything (MFA_ERR_STATE for magic, version, shape, truncation,
 * negative length; MFA_ERR_OVERFLOW for a length beyond kv_capacity). */
/* Page-locked host memory for buffers that cross PCIe whole: a snapshot saved into or loaded
 * from such a buffer moves at the link's rate, one from malloc'd memory at the rate of the
 * runtime's staging copies (about a third).  No counterpart in the reference, whose state lives
 * in host memory.  NULL on failure; mfa_host_free(NULL) is a no-op. */
void *mfa_host_alloc(int64_t bytes);
void mfa_host_free(void *p);
int64_t mfa_state_size(mfa_ctx *ctx);
int64_t mfa_state_save(mfa_ctx *ctx, uint8_t *buf, int64_t buf_len);
int mfa_state_load(mfa_ctx *ctx, const uint8_t *buf, int64_t buf_len);

/* Checkpoints keyed by sequence position, for rewinding to a prompt-cache
 * breakpoint without prefilling again (RsCtx::checkpoint_pos riir/mod.rs:2015-2061,
 * restore_to :2072-2087, set_max_checkpoints :2094-2096, checkpoint_count :2098-2100;
 * tests/checkpoint_restore.rs).  The reference keeps state_save buffers on the host;
 * here a checkpoint is a device-resident copy of the same state (every KV cache up to
 * its length, every conv state and recurrent state) and costs device memory of about
 * mfa_state_size bytes (half that for the KV part of a bf16 cache).
 * mfa_checkpoint_pos stores the current state under `pos`; a checkpoint already at
 * `pos` is replaced and becomes the newest.  Beyond the cap (default 4) the oldest is
 * dropped, never position 0 nor the one just stored.
 * mfa_restore_to brings back exactly the stored state, then drops every checkpoint
 * at a position > pos; MFA_ERR_NO_CHECKPOINT, with nothing changed, when there is none
 * at `pos`.  mfa_set_max_checkpoints takes effect at the next store.  mfa_reset drops
 * all checkpoints (memory_clear, riir/mod.rs:1965-1968); mfa_truncate and
 * mfa_state_load leave them, as in the reference.  Call at token boundaries only. */
int mfa_checkpoint_pos(mfa_ctx *ctx, int32_t pos);
int mfa_restore_to(mfa_ctx *ctx, int32_t pos);
int mfa_set_max_checkpoints(mfa_ctx *ctx, int32_t n);
int32_t mfa_checkpoint_count(mfa_ctx *ctx);

/* ---- timing ---------------------------------------------------------------- */

/* hipEvent pair on the context's stream (the reference's counterpart is the
 * wall-clock LayerTimingAccum, infer.m:96-114). */
int mfa_timer_start(mfa_ctx *ctx);
int mfa_timer_stop(mfa_ctx *ctx, float *elapsed_ms);

/* ---- stateless per-kernel hooks (host pointers, synchronous) --------------- */
/* Twins of the reference's per-kernel test hooks: each uploads its operands,
 * runs ONE kernel, waits and copies back (gpu_attn.rs:247-416). */

/* mf_sdpa_cpu (moeflux.h:179-182; RsCtx::sdpa_cpu riir/mod.rs:444) with the
 * shape passed explicitly. */
int mfa_sdpa(int32_t kv_len, int32_t num_attn_heads, int32_t num_kv_heads, int32_t head_dim,
             const float *q, const float *q_gate, const float *k_cache, const float *v_cache,
             float *out);
/* The same over a bf16 K/V cache (rows of uint16 bf16 bits). */
int mfa_sdpa_bf16kv(int32_t kv_len, int32_t num_attn_heads, int32_t num_kv_heads,
                    int32_t head_dim, const float *q, const float *q_gate,
                    const uint16_t *k_cache, const uint16_t *v_cache, float *out);
/* mf_attn_scores_batched (moeflux.h:475-483; shaders.metal:976-1019). */
int mfa_attn_scores_batched(int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                            int32_t seq_len, const float *q, const float *k_cache, float scale,
                            float *scores_out);
/* mf_attn_softmax_batched (moeflux.h:494-497; shaders.metal:1026-1084). */
int mfa_attn_softmax_batched(int32_t num_heads, int32_t seq_len, float *scores_inout);
/* mf_attn_values_batched (moeflux.h:508-515; shaders.metal:1095-1117). */
int mfa_attn_values_batched(int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                            int32_t seq_len, const float *scores, const float *v_cache,
                            float *out);
/* mf_sigmoid_gate (moeflux.h:524-527; shaders.metal:1125-1134). */
int mfa_sigmoid_gate(int32_t dim, const float *gate, float *x_inout);

/* conv1d_step kernel (shaders.metal:1213-1244; encoder gpu_linear_attn.rs:54-77):
 * out = silu(conv) AND the state is rolled in place, as the GPU kernel does.
 * (mf_conv1d_step_cpu, moeflux.h:224-228, leaves the roll to its caller.) */
int mfa_conv1d_step(int32_t channels, int32_t kernel_size, float *conv_state_inout,
                    const float *new_input, const uint16_t *weight_bf16, float *out);
/* rms_norm_qk kernel (shaders.metal:1254-1303; gpu_linear_attn.rs:82-103). In place. */
int mfa_rms_norm_qk(int32_t num_k_heads, int32_t key_dim, float *q_inout, float *k_inout);
/* mf_rms_norm_bare_cpu (moeflux.h:234-235; linear_attn.rs:160-184). */
int mfa_rms_norm_bare(int32_t dim, float eps, const float *x, float *out);
/* compute_decay_beta kernel (shaders.metal:1312-1327; gpu_linear_attn.rs:108-133). */
int mfa_compute_decay_beta(int32_t num_v_heads, const float *alpha, const float *beta,
                           const float *a_log, const uint16_t *dt_bias_bf16, float *g_decay_out,
                           float *beta_gate_out);
/* gated_delta_net_step kernel (shaders.metal:1154-1194; gpu_linear_attn.rs:140-172). */
int mfa_gated_delta_net_step(int32_t v_heads, int32_t k_heads, int32_t key_dim,
                             int32_t value_dim, const float *g_decay, const float *beta_gate,
                             const float *q, const float *k, const float *v,
                             float *ssm_state_inout, float *out_values);
/* mf_gated_delta_recurrence_cpu (moeflux.h:266-272; linear_attn.rs:288-414) with
 * A_log / dt_bias passed instead of looked up by layer. */
int mfa_gated_delta_recurrence(const float *a_log, const uint16_t *dt_bias_bf16,
                               const float *alpha, const float *beta, const float *q,
                               const float *k, const float *v, int32_t v_heads, int32_t k_heads,
                               int32_t key_dim, int32_t value_dim, float *ssm_state_inout,
                               float *out_values);
/* gated_rms_norm kernel (shaders.metal:1337-1370; gpu_linear_attn.rs:177-202;
 * mf_rms_norm_gated_cpu moeflux.h:245-249 is the one-head case num_heads = 1).
 * x, z, out: [num_heads*dim]; weight_bf16 [dim] shared by all heads. */
int mfa_gated_rms_norm(int32_t num_heads, int32_t dim, float eps, const float *x,
                       const float *z, const uint16_t *weight_bf16, float *out);

/* ---- diagnostics (host only, no GPU needed) --------------------------------- */
/* No counterpart in the reference.  The device KV cache is not row-major (it is
 * stored in the order the decode kernel's matrix-instruction operands consume
 * it); these two functions expose the host-side arithmetic so that it can be
 * tested without a GPU.
 * Element offset, inside one kv head's plane, of channel x of position pos
 * (is_v selects the V plane's order); -1 on a bad argument. */
int64_t mfa_debug_kv_offset(int32_t kv_dtype, int32_t is_v, int64_t pos, int32_t x,
                            int32_t head_dim);
/* Number of split-K partitions the decode launcher uses for this shape. */
int32_t mfa_debug_num_splits(int32_t kv_dtype, int32_t num_attn_heads, int32_t num_kv_heads,
                             int32_t head_dim, int64_t kv_len, int32_t num_cus,
                             int32_t forced_splits);
/* The most partitions it uses at any cache length from 1 to max_len, which is what a context's
 * split-K workspace is sized for: the count is not monotonic in the length (every workgroup
 * gets whole passes), so the count at the capacity is not the bound. */
int32_t mfa_debug_max_splits(int32_t kv_dtype, int32_t num_attn_heads, int32_t num_kv_heads,
                             int32_t head_dim, int64_t max_len, int32_t num_cus,
                             int32_t forced_splits);

/* A plain device-to-device copy kernel on the context's stream (nbytes read, nbytes
 * written, nbytes a multiple of 16): a launch of known memory traffic, used to scale
 * hardware memory counters when profiling.  No counterpart in the reference. */
int mfa_debug_copy_dev(mfa_ctx *ctx, void *dst_dev, const void *src_dev, size_t nbytes);
/* A launch on the context's stream that only reads nbytes (a multiple of 16) with the
 * decode kernel's access pattern - `workgroups` workgroups of 256 threads, each reading
 * one contiguous share with eight 1 KiB wave loads in flight, non-temporal - and computes
 * nothing: the time the memory system allows a launch of that size, against which the
 * decode kernel's own time is read.  No counterpart in the reference. */
int mfa_debug_read_dev(mfa_ctx *ctx, const void *src_dev, size_t nbytes, int32_t workgroups);
/* Fills the split-K workspace (partial outputs and their (max, sum) pairs) with a 32-bit
 * pattern and waits.  Tests use it to show that no result depends on what the workspace
 * held before a call (for instance NaN bit patterns).  No counterpart in the reference. */
int mfa_debug_fill_workspace(mfa_ctx *ctx, uint32_t pattern);

#pragma GCC visibility pop

#ifdef __cplusplus
}
#endif
#endif /* MOEFLUX_ATTN_H */
