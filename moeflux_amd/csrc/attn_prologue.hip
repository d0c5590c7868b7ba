// What a full-attention layer does between its q/k/v projections and the attention
// core, as one launch on the device.
//
// The reference reads the three projection outputs back to the host and, per token,
// splits the q projection into q and its output gate, applies the per-head RMS norm to
// q and k, rotates the first rotary_dim channels of every q and k head, appends k and v
// to the layer's cache and mirrors the row to the GPU
// (crates/moeflux/src/riir/full_attn_forward.rs:238-323; rms_norm.rs:104-156;
// rope.rs:65-131).  Here the projection outputs stay on the device: one workgroup per
// q head, k head and v head does the same arithmetic and writes q, the gate and the
// cache row (in the cache's tiled layout) directly.  Two forms: a group of lanes per head
// (attn_prologue.h; the arithmetic the attention launch of a single decode step repeats, so
// both leave the same bits in the cache) wherever half the rotated channels are whole operand
// slots, one thread per channel otherwise.
#include "attn_prologue.h"

namespace mfa {

// The lane-group form (attn_prologue.h): LPH = D / EPS lanes per head, lane j its channels
// [EPS j, EPS j + EPS).  Heads are numbered per token as below ([0, Hq) q, then Hkv k, then Hkv
// v); a workgroup of 256 threads takes 256 / LPH consecutive heads, grid (ceil, n_tok).
template <typename KV, int D>
__global__ __launch_bounds__(256) void attn_prologue_lanes_kernel(
    int Hq, int Hkv, int rotary_dim, float eps, int32_t pos, int64_t cache_pos, size_t plane_elems,
    const uint16_t *__restrict__ q_norm, const uint16_t *__restrict__ k_norm, const float *__restrict__ inv_freq,
    const float *__restrict__ q_proj, const float *__restrict__ k_in, const float *__restrict__ v_in,
    float *__restrict__ q_out, float *__restrict__ gate_out, KV *__restrict__ k_tiled, KV *__restrict__ v_tiled) {
    constexpr int EPS = sizeof(KV) == 2 ? 8 : 4;
    constexpr int LPH = D / EPS;
    {
        const size_t t = blockIdx.y;
        pos += (int32_t)t;
        cache_pos += (int64_t)t;
        q_proj += t * Hq * 2 * D;
        k_in += t * Hkv * D;
        v_in += t * Hkv * D;
        q_out += t * Hq * D;
        gate_out += t * Hq * D;
    }
    const int nheads = Hq + 2 * Hkv;
    int b = (blockIdx.x * 256 + threadIdx.x) / LPH;
    const bool live = b < nheads;   // whole lane groups; dead ones follow the exchanges with head 0's data
    if (!live) b = 0;
    const int j = threadIdx.x % LPH, c0 = EPS * j;
    const bool is_q = b < Hq, is_v = b >= Hq + Hkv;
    const int h = is_q ? b : (is_v ? b - Hq - Hkv : b - Hq);
    const float *src = is_q ? q_proj + (size_t)h * 2 * D : (is_v ? v_in : k_in) + (size_t)h * D;
    __shared__ float2 s_tab[128];
    float x[EPS], w[EPS], gt[EPS];
#pragma unroll
    for (int e = 0; e < EPS; e += 4) {
        const float4 a = load_f4(src + c0 + e);
        x[e] = a.x; x[e + 1] = a.y; x[e + 2] = a.z; x[e + 3] = a.w;
        const float4 g = load_f4(q_proj + (size_t)(is_q ? h : 0) * 2 * D + D + c0 + e);
        gt[e] = g.x; gt[e + 1] = g.y; gt[e + 2] = g.z; gt[e + 3] = g.w;
    }
#pragma unroll
    for (int e = 0; e < EPS; e++) w[e] = bf16_bits_to_f32((is_q ? q_norm : k_norm)[c0 + e]);
    HeadRotor<EPS, D>::table(HeadRotor<EPS, D>::table_request(inv_freq, rotary_dim), pos, rotary_dim, s_tab);
    __syncthreads();
    HeadRotor<EPS, D> hr;
    hr.init(j, rotary_dim, s_tab);
    float y[EPS];
#pragma unroll
    for (int e = 0; e < EPS; e++) y[e] = x[e];
    hr.apply(y, w, eps);
    if (!live) return;
    if (is_q) {
#pragma unroll
        for (int e = 0; e < EPS; e++) {
            q_out[(size_t)h * D + c0 + e] = y[e];
            gate_out[(size_t)h * D + c0 + e] = gt[e];
        }
    } else if (is_v) {   // v is cached as it comes
#pragma unroll
        for (int e = 0; e < EPS; e++)
            v_tiled[(size_t)h * plane_elems + KvTile<KV>::v_off(cache_pos, c0 + e, D)] = to_kv<KV>(x[e]);
    } else {
#pragma unroll
        for (int e = 0; e < EPS; e++)
            k_tiled[(size_t)h * plane_elems + KvTile<KV>::k_off(cache_pos, c0 + e, D)] = to_kv<KV>(y[e]);
    }
}

// grid (Hq + 2*Hkv, n_tok) workgroups of D threads (D = 64, 128 or 256); along x:
//   [0, Hq)           q head: split off the gate, norm, rotate
//   [Hq, Hq+Hkv)      k head: norm, rotate, store at cache position `cache_pos`
//   [Hq+Hkv, Hq+2Hkv) v head: store at cache position `cache_pos`
// q_proj: [Hq][2][D] (q_h then gate_h, full_attn_forward.rs:240-254).  inv_freq: the table
// 1 / theta^(2i/rotary_dim), i < rotary_dim/2, computed on the host.
// Token t of a chunk (blockIdx.y) has its inputs and outputs t rows further on, is rotated at
// position pos + t and goes to cache position cache_pos + t.
template <typename KV>
__global__ void attn_prologue_kernel(int Hq, int Hkv, int D, int rotary_dim, float eps, int32_t pos,
                                     int64_t cache_pos, size_t plane_elems,
                                     const uint16_t *__restrict__ q_norm, const uint16_t *__restrict__ k_norm,
                                     const float *__restrict__ inv_freq, const float *__restrict__ q_proj,
                                     const float *__restrict__ k_in, const float *__restrict__ v_in,
                                     float *__restrict__ q_out, float *__restrict__ gate_out,
                                     KV *__restrict__ k_tiled, KV *__restrict__ v_tiled) {
    __shared__ float s_y[256];
    __shared__ float s_part[4];
    const int b = blockIdx.x, x = threadIdx.x;
    {
        const size_t t = blockIdx.y;
        pos += (int32_t)t;
        cache_pos += (int64_t)t;
        q_proj += t * Hq * 2 * D;
        k_in += t * Hkv * D;
        v_in += t * Hkv * D;
        q_out += t * Hq * D;
        gate_out += t * Hq * D;
    }
    if (b >= Hq + Hkv) {  // v is cached as it comes
        const int kvh = b - Hq - Hkv;
        v_tiled[(size_t)kvh * plane_elems + KvTile<KV>::v_off(cache_pos, x, D)] = to_kv<KV>(v_in[(size_t)kvh * D + x]);
        return;
    }
    const bool is_q = b < Hq;
    const int h = is_q ? b : b - Hq;
    const float v = is_q ? q_proj[(size_t)h * 2 * D + x] : k_in[(size_t)h * D + x];
    if (is_q) gate_out[(size_t)h * D + x] = q_proj[(size_t)h * 2 * D + D + x];
    // per-head RMS norm: x * inv_rms * weight (rms_norm.rs:138-151)
    const float ws = group_sum<64>(v * v);
    if ((x & 63) == 0) s_part[x >> 6] = ws;
    __syncthreads();
    float sum = 0.f;
    for (int w = 0; w < D / 64; w++) sum += s_part[w];
    const float inv_rms = 1.0f / sqrtf(sum / (float)D + eps);
    const float y = v * inv_rms * bf16_bits_to_f32((is_q ? q_norm : k_norm)[x]);
    s_y[x] = y;
    __syncthreads();
    // rotation of the pairs (i, i + half), i < half = rotary_dim / 2 (rope.rs:96-112)
    const int half = rotary_dim >> 1;
    float r = y;
    if (x < rotary_dim) {
        const int i = x < half ? x : x - half;
        const float angle = (float)pos * inv_freq[i];
        const float cos_a = cosf(angle), sin_a = sinf(angle);
        const float x0 = s_y[i], x1 = s_y[i + half];
        r = x < half ? x0 * cos_a - x1 * sin_a : x0 * sin_a + x1 * cos_a;
    }
    if (is_q) q_out[(size_t)h * D + x] = r;
    else k_tiled[(size_t)h * plane_elems + KvTile<KV>::k_off(cache_pos, x, D)] = to_kv<KV>(r);
}

int launch_attn_prologue(hipStream_t s, int kv_dtype, int Hq, int Hkv, int D, int rotary_dim, float eps, int n_tok,
                         int32_t pos, int64_t cache_pos, size_t plane_elems, const uint16_t *q_norm,
                         const uint16_t *k_norm, const float *inv_freq, const float *q_proj, const float *k_in,
                         const float *v_in, float *q_out, float *gate_out, void *k_tiled, void *v_tiled) {
    if (D != 64 && D != 128 && D != 256) return fail(MFA_ERR_SHAPE, "attention prologue: head_dim %d not supported", D);
    if (rotary_dim <= 0 || rotary_dim > D || (rotary_dim & 1))
        return fail(MFA_ERR_INVALID, "attention prologue: rotary_dim %d must be even and in (0, head_dim]", rotary_dim);
    if (pos < 0) return fail(MFA_ERR_INVALID, "attention prologue: pos %d < 0", pos);
    if (n_tok <= 0 || n_tok > 65535) return fail(MFA_ERR_INVALID, "attention prologue: %d tokens (1..65535 per launch)", n_tok);
    if ((int64_t)pos + n_tok - 1 > INT32_MAX) return fail(MFA_ERR_INVALID, "attention prologue: position overflow");
    if (head_rotor_applies(kv_dtype, D, rotary_dim)) {
        const int eps_ = kv_dtype == MFA_KV_BF16 ? 8 : 4, per_wg = 256 / (D / eps_);
        const dim3 grid((Hq + 2 * Hkv + per_wg - 1) / per_wg, n_tok);
#define MFA_PRO(KV, DD)                                                                                          \
    hipLaunchKernelGGL((attn_prologue_lanes_kernel<KV, DD>), grid, dim3(256), 0, s, Hq, Hkv, rotary_dim, eps, pos, \
                       cache_pos, plane_elems, q_norm, k_norm, inv_freq, q_proj, k_in, v_in, q_out, gate_out,     \
                       (KV *)k_tiled, (KV *)v_tiled)
        if (kv_dtype == MFA_KV_BF16) {
            if (D == 64) MFA_PRO(uint16_t, 64);
            else if (D == 128) MFA_PRO(uint16_t, 128);
            else MFA_PRO(uint16_t, 256);
        } else {
            if (D == 64) MFA_PRO(float, 64);
            else if (D == 128) MFA_PRO(float, 128);
            else MFA_PRO(float, 256);
        }
#undef MFA_PRO
    } else if (kv_dtype == MFA_KV_BF16)
        hipLaunchKernelGGL((attn_prologue_kernel<uint16_t>), dim3(Hq + 2 * Hkv, n_tok), dim3(D), 0, s, Hq, Hkv, D, rotary_dim,
                           eps, pos, cache_pos, plane_elems, q_norm, k_norm, inv_freq, q_proj, k_in, v_in, q_out,
                           gate_out, (uint16_t *)k_tiled, (uint16_t *)v_tiled);
    else
        hipLaunchKernelGGL((attn_prologue_kernel<float>), dim3(Hq + 2 * Hkv, n_tok), dim3(D), 0, s, Hq, Hkv, D, rotary_dim,
                           eps, pos, cache_pos, plane_elems, q_norm, k_norm, inv_freq, q_proj, k_in, v_in, q_out,
                           gate_out, (float *)k_tiled, (float *)v_tiled);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
