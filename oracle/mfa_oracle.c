/*
 * CPU oracle for the per-token attention path (gated GQA SDPA decode and the
 * Gated-DeltaNet step).
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against and the code timed as the CPU baseline.  Nothing in the
 * shipped library links, loads or calls it.
 *
 * Every function is a plain scalar fp32 restatement, written from the text of
 * the reference (no reference source is compiled or copied); the citation
 * above each function names the lines it follows.  Built with
 * -ffp-contract=off so that a*b+c is two roundings exactly where the Rust
 * reference writes `a * b + c`, and fmaf() is used exactly where the Rust
 * reference writes `mul_add`.
 *
 * Pinning status (which independent check holds each function in place is
 * listed in tests/test_oracle_pinning.py):
 *   orc_sdpa, orc_sdpa_bf16kv, orc_attn_scores, orc_attn_softmax,
 *   orc_attn_values, orc_sigmoid_gate, orc_conv1d_step, orc_conv_state_shift,
 *   orc_rms_norm_bare, orc_rms_norm_qk, orc_rms_norm_gated, orc_decay_beta,
 *   orc_gated_delta_recurrence, orc_gdn_step, orc_prefill_attn,
 *   orc_prefill_gdn, orc_rms_norm_per_head, orc_apply_rotary_emb,
 *   orc_attn_prologue, orc_dequant_matvec_4bit, orc_mla_sdpa_folded : pinned by float64 brute force on small shapes, closed
 *   forms and invariants (the reference holds no numeric vectors for them).
 *   The Accelerate-BLAS variant of the recurrence (infer.m:4954-4993) is not
 *   restated: parity unpinned at that boundary (mathematically identical to
 *   orc_gated_delta_recurrence).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* crates/moeflux/src/riir/embedding.rs:153-155 — bf16 is the top half of an f32. */
static inline float orc_bf16_to_f32(uint16_t bits) {
    uint32_t u = ((uint32_t)bits) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* Round-to-nearest-even f32 -> bf16.  Used only to make test inputs; both the
 * oracle and the HIP path are fed the identical bits, so the rounding mode
 * never enters a parity comparison. */
ORC_API uint16_t orc_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

ORC_API void orc_f32_to_bf16_array(const float *x, uint16_t *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = orc_f32_to_bf16(x[i]);
}

ORC_API void orc_bf16_to_f32_array(const uint16_t *x, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = orc_bf16_to_f32(x[i]);
}

/* ------------------------------------------------------------------------ */
/* Full attention                                                           */
/* ------------------------------------------------------------------------ */

/* crates/moeflux/src/riir/sdpa.rs:63-172 (C twin infer.m:762-804, softmax
 * infer.m:821-835).  Per head: s[p] = (q_h . K[p,kv_h]) * scale, softmax with
 * the max taken from s[0], expf, multiply by 1/sum; o_h = sum_p w[p] V[p,kv_h];
 * then out *= 1/(1+expf(-gate)).  Returns -1 on the argument errors the
 * reference rejects (sdpa.rs:71, moeflux.h:177-178). */
ORC_API int orc_sdpa(int32_t kv_len, int32_t num_attn_heads, int32_t num_kv_heads,
                     int32_t head_dim, const float *q, const float *q_gate,
                     const float *k_cache, const float *v_cache, float *out) {
    if (!q || !q_gate || !k_cache || !v_cache || !out) return -1;
    if (kv_len <= 0 || num_attn_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0) return -1;
    if (num_attn_heads % num_kv_heads != 0) return -1;
    const int q_dim = num_attn_heads * head_dim;
    const int64_t kv_dim = (int64_t)num_kv_heads * head_dim;
    const int heads_per_kv = num_attn_heads / num_kv_heads;
    const float scale = 1.0f / sqrtf((float)head_dim);

    for (int i = 0; i < q_dim; i++) out[i] = 0.0f;
    float *scores = (float *)malloc((size_t)kv_len * sizeof(float));
    if (!scores) return -1;
    for (int h = 0; h < num_attn_heads; h++) {
        const int kv_h = h / heads_per_kv;
        const float *qh = q + (int64_t)h * head_dim;
        for (int p = 0; p < kv_len; p++) {
            const float *kp = k_cache + (int64_t)p * kv_dim + (int64_t)kv_h * head_dim;
            float dot = 0.0f;
            for (int d = 0; d < head_dim; d++) dot += qh[d] * kp[d];
            scores[p] = dot * scale;
        }
        float max_val = scores[0];
        for (int p = 1; p < kv_len; p++)
            if (scores[p] > max_val) max_val = scores[p];
        float sum = 0.0f;
        for (int p = 0; p < kv_len; p++) {
            scores[p] = expf(scores[p] - max_val);
            sum += scores[p];
        }
        const float inv_sum = 1.0f / sum;
        for (int p = 0; p < kv_len; p++) scores[p] *= inv_sum;

        float *oh = out + (int64_t)h * head_dim;
        for (int p = 0; p < kv_len; p++) {
            const float *vp = v_cache + (int64_t)p * kv_dim + (int64_t)kv_h * head_dim;
            const float w = scores[p];
            for (int d = 0; d < head_dim; d++) oh[d] += w * vp[d];
        }
    }
    free(scores);
    for (int i = 0; i < q_dim; i++) {
        const float g = 1.0f / (1.0f + expf(-q_gate[i]));
        out[i] *= g;
    }
    return 0;
}

/* The same function over a bf16 K/V cache: the stored bits are widened exactly
 * (embedding.rs:153-155) and everything else is orc_sdpa.  The reference has no
 * bf16 cache; its semantics are defined as sdpa.rs:63-172 on the widened
 * values. */
ORC_API int orc_sdpa_bf16kv(int32_t kv_len, int32_t num_attn_heads, int32_t num_kv_heads,
                            int32_t head_dim, const float *q, const float *q_gate,
                            const uint16_t *k_cache, const uint16_t *v_cache, float *out) {
    if (!k_cache || !v_cache) return -1;
    if (kv_len <= 0 || num_kv_heads <= 0 || head_dim <= 0) return -1;
    const int64_t n = (int64_t)kv_len * num_kv_heads * head_dim;
    float *kf = (float *)malloc((size_t)n * sizeof(float));
    float *vf = (float *)malloc((size_t)n * sizeof(float));
    if (!kf || !vf) { free(kf); free(vf); return -1; }
    for (int64_t i = 0; i < n; i++) { kf[i] = orc_bf16_to_f32(k_cache[i]); vf[i] = orc_bf16_to_f32(v_cache[i]); }
    int rc = orc_sdpa(kv_len, num_attn_heads, num_kv_heads, head_dim, q, q_gate, kf, vf, out);
    free(kf); free(vf);
    return rc;
}

/* crates/moeflux/shaders/shaders.metal:976-1019 (host contract moeflux.h:475-483):
 * scores[h*seq_stride + p] = (Q[h] . K[p, h/heads_per_kv]) * scale. */
ORC_API int orc_attn_scores(int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                            int32_t seq_len, int32_t seq_stride, const float *q,
                            const float *k_cache, float scale, float *scores_out) {
    if (!q || !k_cache || !scores_out) return -1;
    if (num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || seq_len <= 0) return -1;
    if (num_heads % num_kv_heads != 0 || seq_stride < seq_len) return -1;
    const int hpk = num_heads / num_kv_heads;
    const int64_t kv_dim = (int64_t)num_kv_heads * head_dim;
    for (int h = 0; h < num_heads; h++) {
        const float *qh = q + (int64_t)h * head_dim;
        for (int p = 0; p < seq_len; p++) {
            const float *kp = k_cache + (int64_t)p * kv_dim + (int64_t)(h / hpk) * head_dim;
            float acc = 0.0f;
            for (int d = 0; d < head_dim; d++) acc += qh[d] * kp[d];
            scores_out[(int64_t)h * seq_stride + p] = acc * scale;
        }
    }
    return 0;
}

/* crates/moeflux/shaders/shaders.metal:1026-1084: per-head softmax in place;
 * running max starts at -1e30f, exp, multiply by 1/sum. */
ORC_API int orc_attn_softmax(int32_t num_heads, int32_t seq_len, int32_t seq_stride,
                             float *scores) {
    if (!scores || num_heads <= 0 || seq_len <= 0 || seq_stride < seq_len) return -1;
    for (int h = 0; h < num_heads; h++) {
        float *s = scores + (int64_t)h * seq_stride;
        float m = -1e30f;
        for (int i = 0; i < seq_len; i++) m = s[i] > m ? s[i] : m;
        float sum = 0.0f;
        for (int i = 0; i < seq_len; i++) { s[i] = expf(s[i] - m); sum += s[i]; }
        const float inv = 1.0f / sum;
        for (int i = 0; i < seq_len; i++) s[i] *= inv;
    }
    return 0;
}

/* crates/moeflux/shaders/shaders.metal:1095-1117:
 * out[h,d] = sum_p scores[h*seq_stride+p] * V[p, kv_h*head_dim + d], p ascending. */
ORC_API int orc_attn_values(int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                            int32_t seq_len, int32_t seq_stride, const float *scores,
                            const float *v_cache, float *out) {
    if (!scores || !v_cache || !out) return -1;
    if (num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || seq_len <= 0) return -1;
    if (num_heads % num_kv_heads != 0 || seq_stride < seq_len) return -1;
    const int hpk = num_heads / num_kv_heads;
    const int64_t kv_dim = (int64_t)num_kv_heads * head_dim;
    for (int h = 0; h < num_heads; h++) {
        const float *s = scores + (int64_t)h * seq_stride;
        for (int d = 0; d < head_dim; d++) {
            float acc = 0.0f;
            for (int p = 0; p < seq_len; p++)
                acc += s[p] * v_cache[(int64_t)p * kv_dim + (int64_t)(h / hpk) * head_dim + d];
            out[(int64_t)h * head_dim + d] = acc;
        }
    }
    return 0;
}

/* crates/moeflux/shaders/shaders.metal:1125-1134: x[i] *= 1/(1+exp(-gate[i])). */
ORC_API int orc_sigmoid_gate(int32_t dim, const float *gate, float *x_inout) {
    if (!gate || !x_inout || dim <= 0) return -1;
    for (int i = 0; i < dim; i++) {
        const float g = 1.0f / (1.0f + expf(-gate[i]));
        x_inout[i] = x_inout[i] * g;
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Gated DeltaNet                                                           */
/* ------------------------------------------------------------------------ */

/* crates/moeflux/src/riir/linear_attn.rs:89-156 (C twin infer.m:922-945):
 * acc = fma(state[k,c], w[c,k], acc) for k < K-1, then fma(in[c], w[c,K-1], acc);
 * out = acc / (1 + exp(-acc)).  conv_state is [(K-1), channels] time-major, the
 * weight is bf16 [channels, K] channel-major.  Does not advance the state. */
ORC_API int orc_conv1d_step(const float *conv_state, const float *new_input,
                            const uint16_t *weight_bf16, int32_t channels,
                            int32_t kernel_size, float *out) {
    if (!conv_state || !new_input || !weight_bf16 || !out) return -1;
    if (channels <= 0 || kernel_size <= 0) return -1;
    for (int c = 0; c < channels; c++) {
        float acc = 0.0f;
        for (int k = 0; k < kernel_size - 1; k++) {
            const float w = orc_bf16_to_f32(weight_bf16[(int64_t)c * kernel_size + k]);
            acc = fmaf(conv_state[(int64_t)k * channels + c], w, acc);
        }
        const float w = orc_bf16_to_f32(weight_bf16[(int64_t)c * kernel_size + (kernel_size - 1)]);
        acc = fmaf(new_input[c], w, acc);
        out[c] = acc;
    }
    for (int c = 0; c < channels; c++) out[c] = out[c] / (1.0f + expf(-out[c]));
    return 0;
}

/* crates/moeflux-sys/metal_infer/infer.m:2636-2639 (= shaders.metal:1241-1243):
 * drop the oldest slot, append the new input as the newest. */
ORC_API int orc_conv_state_shift(float *conv_state, const float *new_input,
                                 int32_t channels, int32_t kernel_size) {
    if (!conv_state || !new_input || channels <= 0 || kernel_size < 2) return -1;
    memmove(conv_state, conv_state + channels,
            (size_t)(kernel_size - 2) * channels * sizeof(float));
    memcpy(conv_state + (size_t)(kernel_size - 2) * channels, new_input,
           (size_t)channels * sizeof(float));
    return 0;
}

/* crates/moeflux/src/riir/linear_attn.rs:160-184: out = x / sqrt(mean(x^2)+eps). */
ORC_API int orc_rms_norm_bare(int32_t dim, float eps, const float *x, float *out) {
    if (!x || !out || dim <= 0) return -1;
    float sum_sq = 0.0f;
    for (int i = 0; i < dim; i++) sum_sq += x[i] * x[i];
    const float inv_rms = 1.0f / sqrtf(sum_sq / (float)dim + eps);
    for (int i = 0; i < dim; i++) out[i] = x[i] * inv_rms;
    return 0;
}

/* crates/moeflux-sys/metal_infer/infer.m:2655-2667 (= shaders.metal:1254-1303):
 * per k-head bare RMS norm with eps 1e-6, then q *= (1/sqrt(dk))^2 and
 * k *= 1/sqrt(dk).  In place. */
ORC_API int orc_rms_norm_qk(int32_t num_k_heads, int32_t key_dim, float *q, float *k) {
    if (!q || !k || num_k_heads <= 0 || key_dim <= 0) return -1;
    const float inv_scale = 1.0f / sqrtf((float)key_dim);
    for (int h = 0; h < num_k_heads; h++) {
        float *qh = q + (int64_t)h * key_dim;
        orc_rms_norm_bare(key_dim, 1e-6f, qh, qh);
        const float q_scale = inv_scale * inv_scale;
        for (int d = 0; d < key_dim; d++) qh[d] *= q_scale;
    }
    for (int h = 0; h < num_k_heads; h++) {
        float *kh = k + (int64_t)h * key_dim;
        orc_rms_norm_bare(key_dim, 1e-6f, kh, kh);
        for (int d = 0; d < key_dim; d++) kh[d] *= inv_scale;
    }
    return 0;
}

/* crates/moeflux/src/riir/linear_attn.rs:190-242 (C twin infer.m:2529-2539):
 * out = x * inv_rms(x) * w * silu(z), left-to-right products. */
ORC_API int orc_rms_norm_gated(int32_t dim, float eps, const float *x, const float *z,
                               const uint16_t *w_bf16, float *out) {
    if (!x || !z || !w_bf16 || !out || dim <= 0) return -1;
    float sum_sq = 0.0f;
    for (int i = 0; i < dim; i++) sum_sq += x[i] * x[i];
    const float inv_rms = 1.0f / sqrtf(sum_sq / (float)dim + eps);
    for (int i = 0; i < dim; i++) {
        const float w = orc_bf16_to_f32(w_bf16[i]);
        const float silu_z = z[i] / (1.0f + expf(-z[i]));
        out[i] = x[i] * inv_rms * w * silu_z;
    }
    return 0;
}

/* crates/moeflux/src/riir/linear_attn.rs:357-370 (= shaders.metal:1312-1327):
 * g = exp(-exp(A_log) * log(1 + exp(alpha + dt_bias))), beta_gate = sigmoid(beta).
 * The softplus is the naive form and overflows to +inf (g = 0) for large
 * arguments, as the reference's does. */
ORC_API int orc_decay_beta(int32_t v_heads, const float *alpha, const float *beta,
                           const float *a_log, const uint16_t *dt_bias_bf16,
                           float *g_decay, float *beta_gate) {
    if (!alpha || !beta || !a_log || !dt_bias_bf16 || !g_decay || !beta_gate) return -1;
    if (v_heads <= 0) return -1;
    for (int vh = 0; vh < v_heads; vh++) {
        const float dt_b = orc_bf16_to_f32(dt_bias_bf16[vh]);
        const float a_capital = expf(a_log[vh]);
        const float softplus_val = logf(1.0f + expf(alpha[vh] + dt_b));
        g_decay[vh] = expf(-a_capital * softplus_val);
        beta_gate[vh] = 1.0f / (1.0f + expf(-beta[vh]));
    }
    return 0;
}

/* crates/moeflux/shaders/shaders.metal:1154-1194 — the recurrence proper with
 * g and beta_gate already computed.  Loops follow linear_attn.rs:373-411: decay
 * the whole head state; per row kv_mem via fma, delta = (v - kv_mem) * beta,
 * S[vi,:] = fma(k, delta, S[vi,:]); then out[vi] = S[vi,:] . q via fma. */
ORC_API int orc_delta_net_step(int32_t v_heads, int32_t k_heads, int32_t key_dim,
                               int32_t value_dim, const float *g_decay,
                               const float *beta_gate, const float *q, const float *k,
                               const float *v, float *ssm_state, float *out_values) {
    if (!g_decay || !beta_gate || !q || !k || !v || !ssm_state || !out_values) return -1;
    if (v_heads <= 0 || k_heads <= 0 || key_dim <= 0 || value_dim <= 0) return -1;
    if (v_heads % k_heads != 0) return -1;
    const int k_heads_per_v = v_heads / k_heads;
    const int64_t head_stride = (int64_t)value_dim * key_dim;
    for (int vh = 0; vh < v_heads; vh++) {
        const int kh = vh / k_heads_per_v;
        const float g = g_decay[vh];
        const float b_gate = beta_gate[vh];
        float *S = ssm_state + (int64_t)vh * head_stride;
        const float *kk = k + (int64_t)kh * key_dim;
        const float *qq = q + (int64_t)kh * key_dim;
        const float *vv = v + (int64_t)vh * value_dim;
        float *oo = out_values + (int64_t)vh * value_dim;
        for (int64_t i = 0; i < head_stride; i++) S[i] *= g;
        for (int vi = 0; vi < value_dim; vi++) {
            float *row = S + (int64_t)vi * key_dim;
            float kv_mem = 0.0f;
            for (int ki = 0; ki < key_dim; ki++) kv_mem = fmaf(row[ki], kk[ki], kv_mem);
            const float delta = (vv[vi] - kv_mem) * b_gate;
            for (int ki = 0; ki < key_dim; ki++) row[ki] = fmaf(kk[ki], delta, row[ki]);
        }
        for (int vi = 0; vi < value_dim; vi++) {
            const float *row = S + (int64_t)vi * key_dim;
            float sum = 0.0f;
            for (int ki = 0; ki < key_dim; ki++) sum = fmaf(row[ki], qq[ki], sum);
            oo[vi] = sum;
        }
    }
    return 0;
}

/* crates/moeflux/src/riir/linear_attn.rs:288-414 (C twin infer.m:7931-7988):
 * decay/beta precomputation followed by the recurrence. */
ORC_API int orc_gated_delta_recurrence(const float *a_log, const uint16_t *dt_bias_bf16,
                                       const float *alpha, const float *beta,
                                       const float *q, const float *k, const float *v,
                                       int32_t v_heads, int32_t k_heads, int32_t key_dim,
                                       int32_t value_dim, float *ssm_state,
                                       float *out_values) {
    if (v_heads <= 0) return -1;
    float *g = (float *)malloc((size_t)v_heads * sizeof(float));
    float *b = (float *)malloc((size_t)v_heads * sizeof(float));
    if (!g || !b) { free(g); free(b); return -1; }
    int rc = orc_decay_beta(v_heads, alpha, beta, a_log, dt_bias_bf16, g, b);
    if (rc == 0)
        rc = orc_delta_net_step(v_heads, k_heads, key_dim, value_dim, g, b, q, k, v,
                                ssm_state, out_values);
    free(g); free(b);
    return rc;
}

/* One whole Gated-DeltaNet layer step between the projections and o_proj, in
 * the order of crates/moeflux-sys/metal_infer/infer.m:2625-2760 and of the GPU
 * chain at crates/moeflux/src/riir/linear_attn_forward.rs:607-664:
 * conv1d+SiLU over [q|k|v] channels, roll the conv state, per-head q/k norm,
 * recurrence, gated RMS norm (weight shared by all v-heads).
 *   qkv_in [C], C = 2*k_heads*key_dim + v_heads*value_dim; z [v_heads*value_dim];
 *   conv_state [(K-1), C] and ssm_state [v_heads, value_dim, key_dim] mutated. */
ORC_API int orc_gdn_step(int32_t k_heads, int32_t v_heads, int32_t key_dim,
                         int32_t value_dim, int32_t kernel_size, float eps,
                         const uint16_t *conv_w_bf16, const float *a_log,
                         const uint16_t *dt_bias_bf16, const uint16_t *norm_w_bf16,
                         const float *qkv_in, const float *z, const float *alpha,
                         const float *beta, float *conv_state, float *ssm_state,
                         float *out) {
    if (!conv_w_bf16 || !a_log || !dt_bias_bf16 || !norm_w_bf16 || !qkv_in || !z ||
        !alpha || !beta || !conv_state || !ssm_state || !out)
        return -1;
    if (k_heads <= 0 || v_heads <= 0 || key_dim <= 0 || value_dim <= 0 || kernel_size < 2)
        return -1;
    if (v_heads % k_heads != 0) return -1;
    const int total_key = k_heads * key_dim;
    const int total_value = v_heads * value_dim;
    const int C = 2 * total_key + total_value;
    float *conv_out = (float *)malloc((size_t)C * sizeof(float));
    float *vals = (float *)malloc((size_t)total_value * sizeof(float));
    if (!conv_out || !vals) { free(conv_out); free(vals); return -1; }
    int rc = orc_conv1d_step(conv_state, qkv_in, conv_w_bf16, C, kernel_size, conv_out);
    if (rc == 0) rc = orc_conv_state_shift(conv_state, qkv_in, C, kernel_size);
    float *lin_q = conv_out, *lin_k = conv_out + total_key, *lin_v = conv_out + 2 * total_key;
    if (rc == 0) rc = orc_rms_norm_qk(k_heads, key_dim, lin_q, lin_k);
    if (rc == 0)
        rc = orc_gated_delta_recurrence(a_log, dt_bias_bf16, alpha, beta, lin_q, lin_k, lin_v,
                                        v_heads, k_heads, key_dim, value_dim, ssm_state, vals);
    for (int vh = 0; rc == 0 && vh < v_heads; vh++)
        rc = orc_rms_norm_gated(value_dim, eps, vals + (int64_t)vh * value_dim,
                                z + (int64_t)vh * value_dim, norm_w_bf16,
                                out + (int64_t)vh * value_dim);
    free(conv_out); free(vals);
    return rc;
}

/* ------------------------------------------------------------------------ */
/* Prompt chunks: the reference has no batched prefill; eval_prompt is a      */
/* token loop (crates/moeflux/src/riir/mod.rs:1196-1214), so a chunk is        */
/* defined as that loop.                                                       */
/* ------------------------------------------------------------------------ */

/* Causal attention over a chunk of T new tokens appended after `kv_len0`
 * cached positions: token t runs orc_sdpa with kv_len = kv_len0 + t + 1 (the
 * current token attends to itself, full_attn_forward.rs:293,331).
 *   q, q_gate, out: [T, Hq*d];  k_cache, v_cache: [kv_len0 + T, Hkv*d] already
 *   holding the chunk's rows at positions kv_len0.. . */
ORC_API int orc_prefill_attn(int32_t T, int32_t kv_len0, int32_t num_attn_heads,
                             int32_t num_kv_heads, int32_t head_dim, const float *q,
                             const float *q_gate, const float *k_cache,
                             const float *v_cache, float *out) {
    if (T <= 0 || kv_len0 < 0) return -1;
    const int64_t q_dim = (int64_t)num_attn_heads * head_dim;
    for (int t = 0; t < T; t++) {
        int rc = orc_sdpa(kv_len0 + t + 1, num_attn_heads, num_kv_heads, head_dim,
                          q + t * q_dim, q_gate + t * q_dim, k_cache, v_cache,
                          out + t * q_dim);
        if (rc) return rc;
    }
    return 0;
}

/* T sequential orc_gdn_step calls; inputs are [T, ...] row-major. */
ORC_API int orc_prefill_gdn(int32_t T, int32_t k_heads, int32_t v_heads, int32_t key_dim,
                            int32_t value_dim, int32_t kernel_size, float eps,
                            const uint16_t *conv_w_bf16, const float *a_log,
                            const uint16_t *dt_bias_bf16, const uint16_t *norm_w_bf16,
                            const float *qkv_in, const float *z, const float *alpha,
                            const float *beta, float *conv_state, float *ssm_state,
                            float *out) {
    if (T <= 0) return -1;
    const int64_t C = 2 * (int64_t)k_heads * key_dim + (int64_t)v_heads * value_dim;
    const int64_t tv = (int64_t)v_heads * value_dim;
    for (int t = 0; t < T; t++) {
        int rc = orc_gdn_step(k_heads, v_heads, key_dim, value_dim, kernel_size, eps,
                              conv_w_bf16, a_log, dt_bias_bf16, norm_w_bf16,
                              qkv_in + t * C, z + t * tv, alpha + (int64_t)t * v_heads,
                              beta + (int64_t)t * v_heads, conv_state, ssm_state,
                              out + t * tv);
        if (rc) return rc;
    }
    return 0;
}

/* ---- what precedes the attention core in a full-attention layer -------------- */

/* crates/moeflux/src/riir/rms_norm.rs:104-156 (rms_norm_per_head_cpu): each
 * head's head_dim-long slice is normalised on its own and scaled by one shared
 * bf16 weight vector; x * inv_rms * weight, in that order. */
ORC_API int orc_rms_norm_per_head(int32_t num_heads, int32_t head_dim, float eps,
                                  const uint16_t *weight_bf16, float *x_inout) {
    if (num_heads <= 0 || head_dim <= 0 || !weight_bf16 || !x_inout) return -1;
    const float head_dim_f = (float)head_dim;
    for (int h = 0; h < num_heads; h++) {
        float *xh = x_inout + (int64_t)h * head_dim;
        float sum_sq = 0.0f;
        for (int i = 0; i < head_dim; i++) sum_sq += xh[i] * xh[i];
        const float inv_rms = 1.0f / sqrtf(sum_sq / head_dim_f + eps);
        for (int i = 0; i < head_dim; i++) xh[i] = xh[i] * inv_rms * orc_bf16_to_f32(weight_bf16[i]);
    }
    return 0;
}

/* The frequency table of crates/moeflux/src/riir/rope.rs:99-103:
 * inv_freq[i] = 1 / powf(theta, 2 i / rotary_dim), i < rotary_dim / 2.  The
 * library computes the same table with the host's powf when the rotation is
 * configured, so that no second powf implementation enters the angle. */
ORC_API int orc_rope_inv_freq(float theta, int32_t rotary_dim, float *inv_freq) {
    if (rotary_dim <= 0 || (rotary_dim & 1) || !inv_freq) return -1;
    const float rdim_f = (float)rotary_dim;
    for (int i = 0; i < rotary_dim / 2; i++) inv_freq[i] = 1.0f / powf(theta, (float)(2 * i) / rdim_f);
    return 0;
}

/* crates/moeflux/src/riir/rope.rs:65-131 (apply_rotary_emb): the first
 * rotary_dim channels of every q and k head are rotated, channel i paired with
 * channel i + rotary_dim/2; angle = pos * inv_freq[i]. */
ORC_API int orc_apply_rotary_emb(int32_t pos, int32_t num_heads, int32_t num_kv_heads,
                                 int32_t head_dim, int32_t rotary_dim, float theta, float *q,
                                 float *k) {
    if (pos < 0 || !q || !k || rotary_dim <= 0 || rotary_dim > head_dim || (rotary_dim & 1)) return -1;
    const int half = rotary_dim / 2;
    const float pos_f = (float)pos, rdim_f = (float)rotary_dim;
    for (int pass = 0; pass < 2; pass++) {
        float *x = pass ? k : q;
        const int nh = pass ? num_kv_heads : num_heads;
        for (int h = 0; h < nh; h++) {
            float *xh = x + (int64_t)h * head_dim;
            for (int i = 0; i < half; i++) {
                const float freq = 1.0f / powf(theta, (float)(2 * i) / rdim_f);
                const float angle = pos_f * freq;
                const float cos_a = cosf(angle), sin_a = sinf(angle);
                const float x0 = xh[i], x1 = xh[i + half];
                xh[i] = x0 * cos_a - x1 * sin_a;
                xh[i + half] = x0 * sin_a + x1 * cos_a;
            }
        }
    }
    return 0;
}

/* crates/moeflux/src/riir/full_attn_forward.rs:238-293: the q projection's
 * output is [q_h | gate_h] per head with stride 2*head_dim; q and k get the
 * per-head norm and the rotation; v is untouched.  k_row / v_row are what is
 * appended to the cache; q / q_gate what the attention core receives. */
ORC_API int orc_attn_prologue(int32_t pos, int32_t num_heads, int32_t num_kv_heads,
                              int32_t head_dim, int32_t rotary_dim, float theta, float eps,
                              const uint16_t *q_norm_bf16, const uint16_t *k_norm_bf16,
                              const float *q_proj_out, const float *k_in, const float *v_in,
                              float *q, float *q_gate, float *k_row, float *v_row) {
    if (!q_proj_out || !k_in || !v_in || !q || !q_gate || !k_row || !v_row) return -1;
    for (int h = 0; h < num_heads; h++) {
        memcpy(q + (int64_t)h * head_dim, q_proj_out + (int64_t)h * 2 * head_dim, sizeof(float) * head_dim);
        memcpy(q_gate + (int64_t)h * head_dim, q_proj_out + (int64_t)h * 2 * head_dim + head_dim,
               sizeof(float) * head_dim);
    }
    memcpy(k_row, k_in, sizeof(float) * (size_t)num_kv_heads * head_dim);
    memcpy(v_row, v_in, sizeof(float) * (size_t)num_kv_heads * head_dim);
    int rc = orc_rms_norm_per_head(num_heads, head_dim, eps, q_norm_bf16, q);
    if (rc) return rc;
    rc = orc_rms_norm_per_head(num_kv_heads, head_dim, eps, k_norm_bf16, k_row);
    if (rc) return rc;
    return orc_apply_rotary_emb(pos, num_heads, num_kv_heads, head_dim, rotary_dim, theta, q, k_row);
}

/* ---- the projections either side of the attention core ------------------------ */

/* crates/moeflux/src/riir/cpu_matvec.rs:83-160 (dequant_matvec_4bit_cpu; C twin
 * cpu_dequant_matvec, infer.m:671): out[r] = sum_c (nibble(r,c) * scale + bias) * x[c],
 * weights packed 8 nibbles per u32 (nibble n of a word at bits 4n..4n+3), one bf16
 * scale and one bf16 bias per group of 64 inputs; both steps are mul_add. */
ORC_API int orc_dequant_matvec_4bit(const uint32_t *packed, const uint16_t *scales,
                                    const uint16_t *biases, int32_t in_dim, int32_t out_dim,
                                    const float *x, float *out) {
    if (!packed || !scales || !biases || !x || !out || in_dim <= 0 || out_dim <= 0) return -1;
    if (in_dim % 64 != 0) return -1;
    const int in_packed = in_dim / 8, in_groups = in_dim / 64;
    for (int r = 0; r < out_dim; r++) {
        const uint32_t *row = packed + (int64_t)r * in_packed;
        float acc = 0.0f;
        for (int g = 0; g < in_groups; g++) {
            const float scale = orc_bf16_to_f32(scales[(int64_t)r * in_groups + g]);
            const float bias = orc_bf16_to_f32(biases[(int64_t)r * in_groups + g]);
            for (int p = 0; p < 8; p++) {
                const uint32_t word = row[g * 8 + p];
                for (int n = 0; n < 8; n++) {
                    const float nibble = (float)((word >> (n * 4)) & 0xFu);
                    const float w = fmaf(nibble, scale, bias);
                    acc = fmaf(w, x[g * 64 + p * 8 + n], acc);
                }
            }
        }
        out[r] = acc;
    }
    return 0;
}

/* ---- attention over a compressed (latent) cache --------------------------------- */

/* crates/moeflux/shaders/shaders.metal:1688-1816 (mla_sdpa_folded; the tiled form
 * :1818-1987 computes the same function): per head h
 *   s[t] = (q'[h] . latent[t] + q_pe[h] . rope_k[t]) * softmax_scale   (fma accumulation,
 *          the latent part first), softmax over t (max, exp, sum, times 1/sum),
 *   out[h, c] = sum_t s[t] latent[t, c]                                  (fma accumulation).
 * q_prime, out: [H, R]; q_pe: [H, P]; latent: [L, R]; rope_k: [L, P]. */
ORC_API int orc_mla_sdpa_folded(int32_t num_heads, int32_t kv_lora_rank, int32_t qk_rope_head_dim,
                                int32_t cache_len, float softmax_scale, const float *q_prime,
                                const float *q_pe, const float *latent, const float *rope_k, float *out) {
    if (!q_prime || !q_pe || !latent || !rope_k || !out) return -1;
    if (num_heads <= 0 || kv_lora_rank <= 0 || qk_rope_head_dim <= 0 || cache_len <= 0) return -1;
    const int R = kv_lora_rank, P = qk_rope_head_dim;
    float *scores = (float *)malloc((size_t)cache_len * sizeof(float));
    if (!scores) return -1;
    for (int h = 0; h < num_heads; h++) {
        const float *qh = q_prime + (int64_t)h * R, *qp = q_pe + (int64_t)h * P;
        for (int t = 0; t < cache_len; t++) {
            const float *lt = latent + (int64_t)t * R, *rt = rope_k + (int64_t)t * P;
            float s = 0.0f;
            for (int c = 0; c < R; c++) s = fmaf(qh[c], lt[c], s);
            for (int r = 0; r < P; r++) s = fmaf(qp[r], rt[r], s);
            scores[t] = s * softmax_scale;
        }
        float maxv = -INFINITY;
        for (int t = 0; t < cache_len; t++) maxv = fmaxf(maxv, scores[t]);
        float sum = 0.0f;
        for (int t = 0; t < cache_len; t++) {
            scores[t] = expf(scores[t] - maxv);
            sum += scores[t];
        }
        const float inv_sum = 1.0f / sum;
        for (int t = 0; t < cache_len; t++) scores[t] *= inv_sum;
        for (int c = 0; c < R; c++) {
            float acc = 0.0f;
            for (int t = 0; t < cache_len; t++) acc = fmaf(scores[t], latent[(int64_t)t * R + c], acc);
            out[(int64_t)h * R + c] = acc;
        }
    }
    free(scores);
    return 0;
}
