// Gated-DeltaNet linear-attention step for gfx950.
//
// gdn_step_kernel fuses the reference's five launches
//   conv1d_step, rms_norm_qk, compute_decay_beta, gated_delta_net_step,
//   gated_rms_norm   (crates/moeflux/shaders/shaders.metal:1154-1370, encoded
//   at crates/moeflux/src/riir/linear_attn_forward.rs:607-664)
// into one: one workgroup per value head, 8 lanes per state row, each lane
// holding dk/8 floats of its row in registers, so the [dv, dk] f32 state is
// read once and written once with 128-byte-per-row coalesced accesses.  The
// conv history is a ring of K slots (slot = step % K) instead of a shifted
// [K-1, C] array, which removes the reference kernel's read-modify-write of
// the whole history; export/import convert to the reference's time-major
// order.
//
// The remaining kernels in this file are one-launch twins of the five
// reference kernels for per-kernel parity tests.
#include "gdn_device.h"
#include "sdpa_merge.h"

namespace mfa {

// grid (Hv, layers): one workgroup of DV*8 threads per value head.  With more than one
// layer every per-layer array is a layer-major slab and the packed inputs and outputs
// are [layers, ...]: the kernel offsets each pointer by blockIdx.y strides.  KC is the conv width when it is the usual 4
// (the taps are then requested up front, ahead of the state rows), 0 for any other width.
template <int DK, int DV, int KC>
__device__ __forceinline__ void gdn_step_body(
    const size_t ly, int Hk, int Hv, int K, float eps, const uint16_t *__restrict__ conv_w,
    const float *__restrict__ a_log, const uint16_t *__restrict__ dt_bias,
    const uint16_t *__restrict__ norm_w, float *__restrict__ conv_ring, int slot_new,
    float *__restrict__ ssm, const float *__restrict__ qkv_in, const float *__restrict__ z,
    const float *__restrict__ alpha, const float *__restrict__ beta, float *__restrict__ out) {
    constexpr int NI = DK / 32;
    constexpr int NT = DV * 8;
    constexpr int KT = KC > 0 ? KC : 1;
    constexpr int NCONV = 2 * DK + DV;   // conv channels of a head: whole waves
    static_assert(NCONV % 64 == 0 && DV % 64 == 0 && NCONV < NT, "conv channels and outputs fill whole waves");
    __shared__ float s_q[DK], s_k[DK], s_v[DV], s_o[DV];
    __shared__ float s_gb[2];

    const int tid = threadIdx.x;
    const int vh = blockIdx.x;
    const int rep = Hv / Hk;
    const int kh = vh / rep;
    const int C = 2 * Hk * DK + Hv * DV;
    const int r = tid >> 3, j = tid & 7;
    {
        conv_w += ly * C * K;
        a_log += ly * Hv;
        dt_bias += ly * Hv;
        norm_w += ly * DV;
        conv_ring += ly * K * C;
        ssm += ly * Hv * DV * DK;
        qkv_in += ly * C;
        z += ly * Hv * DV;
        alpha += ly * Hv;
        beta += ly * Hv;
        out += ly * Hv * DV;
    }

    // Which conv channel this thread serves: the head's q, k and v channels are the first
    // NCONV threads (whole waves); the other waves only hold state rows.
    const bool conv_thread = tid < NCONV;
    int ch = 0;
    bool owner = true;  // q/k channels are shared by `rep` value heads; one of them rolls the ring
    if (tid < DK) { ch = kh * DK + tid; owner = (vh % rep) == 0; }
    else if (tid < 2 * DK) { ch = Hk * DK + kh * DK + (tid - DK); owner = (vh % rep) == 0; }
    else if (conv_thread) ch = 2 * Hk * DK + vh * DV + (tid - 2 * DK);

    // 1. Requests.  A CU takes a wave's request for 16 bytes per lane in 16 clocks and returns
    //    data in request order, so the few small operands the whole workgroup waits for (conv
    //    inputs and taps; z and the norm weight) are requested by the waves that use them and
    //    nobody else, and the barrier keeps every wave's state rows (1024 clocks of requests
    //    at dk = dv = 128) behind them.
    float x_in = 0.f, tap[KT], wt[KT];
    float z_in = 0.f, nw_in = 0.f;
    if (conv_thread) {
        if (KC > 0) {
            x_in = qkv_in[ch];
            const uint2 wbits = *(const uint2 *)(conv_w + (size_t)ch * 4);  // four bf16 taps
            wt[0] = bf16_bits_to_f32((uint16_t)(wbits.x & 0xffffu));
            if (KC > 1) wt[1 % KT] = bf16_bits_to_f32((uint16_t)(wbits.x >> 16));
            if (KC > 2) wt[2 % KT] = bf16_bits_to_f32((uint16_t)(wbits.y & 0xffffu));
            if (KC > 3) wt[3 % KT] = bf16_bits_to_f32((uint16_t)(wbits.y >> 16));
#pragma unroll
            for (int k = 0; k < KT - 1; k++) {
                int sl = slot_new + 1 + k;
                if (sl >= KC) sl -= KC;
                tap[k] = conv_ring[(size_t)sl * C + ch];
            }
        }
        if (tid < DV) {
            z_in = z[(size_t)vh * DV + tid];
            nw_in = bf16_bits_to_f32(norm_w[tid]);
        }
    }
    const float a_log_in = a_log[vh], alpha_in = alpha[vh], beta_in = beta[vh];
    const float dt_in = bf16_bits_to_f32(dt_bias[vh]);
    __builtin_amdgcn_s_barrier();
    float *srow = ssm + ((size_t)vh * DV + r) * DK + 4 * j;
    float4 s[NI];
#pragma unroll
    for (int i = 0; i < NI; i++) s[i] = load_f4(srow + 32 * i);

    // 2. depthwise conv + SiLU on this head's q, k and v channels
    //    (linear_attn.rs:132-154; taps oldest first, the new input is tap K-1).
    if (conv_thread) {
        float acc = 0.f;
        if (KC > 0) {
#pragma unroll
            for (int k = 0; k < KT - 1; k++) acc = fmaf(tap[k], wt[k], acc);
            acc = fmaf(x_in, wt[KT - 1], acc);
        } else {
            x_in = qkv_in[ch];
            for (int k = 0; k < K - 1; k++) {
                int sl = slot_new + 1 + k;
                if (sl >= K) sl -= K;
                acc = fmaf(conv_ring[(size_t)sl * C + ch], bf16_bits_to_f32(conv_w[(size_t)ch * K + k]), acc);
            }
            acc = fmaf(x_in, bf16_bits_to_f32(conv_w[(size_t)ch * K + (K - 1)]), acc);
        }
        const float cval = silu_f(acc);
        if (owner) conv_ring[(size_t)slot_new * C + ch] = x_in;
        if (tid < DK) s_q[tid] = cval;
        else if (tid < 2 * DK) s_k[tid - DK] = cval;
        else s_v[tid - 2 * DK] = cval;
    }
    // 3. decay and beta gate (shaders.metal:1321-1326)
    if (tid == NT - 1) {
        // One lane, and every wave waits for it: the hardware exp2 / log2 / reciprocal (1 ulp each)
        // instead of the library routines, about 100 clocks instead of 1000.
        const float a_cap = __expf(a_log_in);
        const float sp = __logf(1.0f + __expf(alpha_in + dt_in));   // the reference's plain softplus
        s_gb[0] = __expf(-a_cap * sp);
        s_gb[1] = __builtin_amdgcn_rcpf(1.0f + __expf(-beta_in));
    }
    const float og = nw_in * silu_f(z_in);   // the output's gate and weight, ready before the read-out
    __syncthreads();

    // 4. q and k as this thread's row slice needs them, normed on the way: the 8 lanes of a row
    //    hold all dk channels between them, so each row forms both sums of squares itself
    //    (infer.m:2655-2667: x * inv_rms, then q *= (1/sqrt(dk))^2, k *= 1/sqrt(dk)).
    float4 kk[NI], qq[NI];
    {
        float sq = 0.f, sk = 0.f;
#pragma unroll
        for (int i = 0; i < NI; i++) {
            kk[i] = *(const float4 *)(s_k + 32 * i + 4 * j);
            qq[i] = *(const float4 *)(s_q + 32 * i + 4 * j);
            sq += qq[i].x * qq[i].x + qq[i].y * qq[i].y + qq[i].z * qq[i].z + qq[i].w * qq[i].w;
            sk += kk[i].x * kk[i].x + kk[i].y * kk[i].y + kk[i].z * kk[i].z + kk[i].w * kk[i].w;
        }
        sq = group_sum<8>(sq);
        sk = group_sum<8>(sk);
        const float inv_scale = 1.0f / sqrtf((float)DK);
        const float iq = __builtin_amdgcn_rsqf(sq / (float)DK + 1e-6f);
        const float ik = __builtin_amdgcn_rsqf(sk / (float)DK + 1e-6f);
        const float q2 = inv_scale * inv_scale;
#pragma unroll
        for (int i = 0; i < NI; i++) {
            qq[i].x = qq[i].x * iq * q2; qq[i].y = qq[i].y * iq * q2;
            qq[i].z = qq[i].z * iq * q2; qq[i].w = qq[i].w * iq * q2;
            kk[i].x = kk[i].x * ik * inv_scale; kk[i].y = kk[i].y * ik * inv_scale;
            kk[i].z = kk[i].z * ik * inv_scale; kk[i].w = kk[i].w * ik * inv_scale;
        }
    }

    // 5. recurrence on this thread's row slice
    const float o = delta_row<DK>(s, kk, qq, s_gb[0], s_gb[1], s_v[r]);
    if (j == 0) s_o[r] = o;
#pragma unroll
    for (int i = 0; i < NI; i++) *(float4 *)(srow + 32 * i) = s[i];
    __syncthreads();

    // 6. gated RMS norm over the head's dv outputs (linear_attn.rs:230-240): each of the first
    //    dv/64 waves forms the whole sum of squares itself (hardware reciprocal square root, 1 ulp).
    if (tid < DV) {
        float ss = 0.f;
#pragma unroll
        for (int w = 0; w < DV / 64; w++) {
            const float y = s_o[(tid & 63) + 64 * w];
            ss += y * y;
        }
        const float sum = group_sum<64>(ss);
        const float inv_rms = __builtin_amdgcn_rsqf(sum / (float)DV + eps);
        out[(size_t)vh * DV + tid] = s_o[tid] * inv_rms * og;
    }
}

// grid (Hv, layers): workgroup (vh, ly) steps value head vh of layer ly.
template <int DK, int DV, int KC>
__global__ __launch_bounds__(DV * 8) void gdn_step_kernel(
    int Hk, int Hv, int K, float eps, const uint16_t *__restrict__ conv_w,
    const float *__restrict__ a_log, const uint16_t *__restrict__ dt_bias,
    const uint16_t *__restrict__ norm_w, float *__restrict__ conv_ring, int slot_new,
    float *__restrict__ ssm, const float *__restrict__ qkv_in, const float *__restrict__ z,
    const float *__restrict__ alpha, const float *__restrict__ beta, float *__restrict__ out) {
    gdn_step_body<DK, DV, KC>(blockIdx.y, Hk, Hv, K, eps, conv_w, a_log, dt_bias, norm_w, conv_ring, slot_new, ssm, qkv_in,
                              z, alpha, beta, out);
}

// The same with a merge of split-K partials in its first rows of workgroups (grid (Hv, merge_rows +
// layers)): the attention layers' launch of a token sweep leaves its partials to this launch, which
// follows it on the stream, so the sweep is two launches and the merge's round trip to memory
// passes while the first DeltaNet workgroups wait for their operands.  A wave merges one 64-output
// unit.
template <int DK, int DV, int KC>
__global__ __launch_bounds__(DV * 8) void gdn_step_merge_kernel(
    int Hk, int Hv, int K, float eps, const uint16_t *__restrict__ conv_w,
    const float *__restrict__ a_log, const uint16_t *__restrict__ dt_bias,
    const uint16_t *__restrict__ norm_w, float *__restrict__ conv_ring, int slot_new,
    float *__restrict__ ssm, const float *__restrict__ qkv_in, const float *__restrict__ z,
    const float *__restrict__ alpha, const float *__restrict__ beta, float *__restrict__ out,
    SdpaMergeTask merge, int merge_rows) {
    if ((int)blockIdx.y < merge_rows) {
        const int unit = ((int)blockIdx.y * (int)gridDim.x + (int)blockIdx.x) * (DV * 8 / 64) + (int)(threadIdx.x >> 6);
        if (unit < merge.n_units) sdpa_merge_unit(merge, unit, threadIdx.x & 63);   // whole waves, no barrier
        return;
    }
    gdn_step_body<DK, DV, KC>(blockIdx.y - merge_rows, Hk, Hv, K, eps, conv_w, a_log, dt_bias, norm_w, conv_ring, slot_new,
                              ssm, qkv_in, z, alpha, beta, out);
}

// ---- one-launch twins of the reference kernels ------------------------------

// shaders.metal:1213-1244: conv + SiLU, then the state is rolled in place.
__global__ void conv1d_step_kernel(float *__restrict__ state, const float *__restrict__ in,
                                   const uint16_t *__restrict__ w, float *__restrict__ out, int C,
                                   int K) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    float acc = 0.f;
    for (int k = 0; k < K - 1; k++)
        acc = fmaf(state[(size_t)k * C + c], bf16_bits_to_f32(w[(size_t)c * K + k]), acc);
    const float x = in[c];
    acc = fmaf(x, bf16_bits_to_f32(w[(size_t)c * K + (K - 1)]), acc);
    out[c] = silu_f(acc);
    for (int k = 0; k + 1 < K - 1; k++) state[(size_t)k * C + c] = state[(size_t)(k + 1) * C + c];
    state[(size_t)(K - 2) * C + c] = x;
}

// Block-wide sum for blocks of up to 1024 threads.
__device__ inline float block_sum(float v, float *scratch) {
    v = group_sum<64>(v);
    const int nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < nw; w++) t += scratch[w];
    return t;
}

// shaders.metal:1254-1303.  grid Hk, any block size; strided over dk.
__global__ void rms_norm_qk_kernel(float *__restrict__ q, float *__restrict__ k, int dk) {
    __shared__ float scratch[16];
    const int base = blockIdx.x * dk;
    const float inv_scale = 1.0f / sqrtf((float)dk);
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < dk; i += blockDim.x) {
        sq += q[base + i] * q[base + i];
        sk += k[base + i] * k[base + i];
    }
    const float tq = block_sum(sq, scratch);
    const float tk = block_sum(sk, scratch);
    const float iq = 1.0f / sqrtf(tq / (float)dk + 1e-6f);
    const float ik = 1.0f / sqrtf(tk / (float)dk + 1e-6f);
    for (int i = threadIdx.x; i < dk; i += blockDim.x) {
        float a = q[base + i] * iq;
        a *= inv_scale * inv_scale;
        q[base + i] = a;
        float b = k[base + i] * ik;
        b *= inv_scale;
        k[base + i] = b;
    }
}

// linear_attn.rs:160-184.  One block.
__global__ void rms_norm_bare_kernel(const float *__restrict__ x, float *__restrict__ out, int dim,
                                     float eps) {
    __shared__ float scratch[16];
    float s = 0.f;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) s += x[i] * x[i];
    const float t = block_sum(s, scratch);
    const float inv = 1.0f / sqrtf(t / (float)dim + eps);
    for (int i = threadIdx.x; i < dim; i += blockDim.x) out[i] = x[i] * inv;
}

// shaders.metal:1312-1327.
__global__ void decay_beta_kernel(const float *__restrict__ alpha, const float *__restrict__ beta,
                                  const float *__restrict__ a_log,
                                  const uint16_t *__restrict__ dt_bias, float *__restrict__ g,
                                  float *__restrict__ b, int Hv) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= Hv) return;
    const float a_cap = expf(a_log[i]);
    const float sp = logf(1.0f + expf(alpha[i] + bf16_bits_to_f32(dt_bias[i])));
    g[i] = expf(-a_cap * sp);
    b[i] = 1.0f / (1.0f + expf(-beta[i]));
}

// shaders.metal:1154-1194 with the row layout of gdn_step_kernel.
template <int DK, int DV>
__global__ __launch_bounds__(DV * 8) void delta_net_step_kernel(
    int Hk, int Hv, const float *__restrict__ g, const float *__restrict__ b,
    const float *__restrict__ q, const float *__restrict__ k, const float *__restrict__ v,
    float *__restrict__ ssm, float *__restrict__ out) {
    constexpr int NI = DK / 32;
    const int vh = blockIdx.x, kh = vh / (Hv / Hk);
    const int r = threadIdx.x >> 3, j = threadIdx.x & 7;
    float *srow = ssm + ((size_t)vh * DV + r) * DK + 4 * j;
    float4 s[NI], kk[NI], qq[NI];
#pragma unroll
    for (int i = 0; i < NI; i++) {
        s[i] = *(const float4 *)(srow + 32 * i);
        kk[i] = *(const float4 *)(k + (size_t)kh * DK + 32 * i + 4 * j);
        qq[i] = *(const float4 *)(q + (size_t)kh * DK + 32 * i + 4 * j);
    }
    const float o = delta_row<DK>(s, kk, qq, g[vh], b[vh], v[(size_t)vh * DV + r]);
#pragma unroll
    for (int i = 0; i < NI; i++) *(float4 *)(srow + 32 * i) = s[i];
    if (j == 0) out[(size_t)vh * DV + r] = o;
}

// shaders.metal:1337-1370.  grid H heads; strided over dim.
__global__ void gated_rms_norm_kernel(const float *__restrict__ x, const float *__restrict__ z,
                                      const uint16_t *__restrict__ w, float *__restrict__ out,
                                      int dim, float eps) {
    __shared__ float scratch[16];
    const size_t base = (size_t)blockIdx.x * dim;
    float s = 0.f;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) s += x[base + i] * x[base + i];
    const float t = block_sum(s, scratch);
    const float inv = 1.0f / sqrtf(t / (float)dim + eps);
    for (int i = threadIdx.x; i < dim; i += blockDim.x)
        out[base + i] = x[base + i] * inv * bf16_bits_to_f32(w[i]) * silu_f(z[base + i]);
}

// ring slot of history row jrow (0 = oldest) when `step` inputs have been consumed
__host__ __device__ inline int ring_slot(int64_t step, int jrow, int K) {
    return (int)((step + 1 + jrow) % K);
}

__global__ void conv_ring_export_kernel(const float *__restrict__ ring, float *__restrict__ state,
                                        int C, int K, int64_t step) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)(K - 1) * C) return;
    const int jrow = (int)(i / C), c = (int)(i % C);
    state[i] = ring[(size_t)ring_slot(step, jrow, K) * C + c];
}

// import resets the step counter to 0: history row j goes to slot j+1, slot 0 is cleared.
__global__ void conv_ring_import_kernel(const float *__restrict__ state, float *__restrict__ ring,
                                        int C, int K) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)K * C) return;
    const int sl = (int)(i / C), c = (int)(i % C);
    ring[i] = sl == 0 ? 0.f : state[(size_t)(sl - 1) * C + c];
}

// ---- launchers ----------------------------------------------------------------

bool gdn_shape_supported(int Hk, int Hv, int dk, int dv, int K) {
    if (Hk <= 0 || Hv <= 0 || Hv % Hk != 0) return false;
    if (K < 2 || K > 8) return false;
    return (dk == 128 && dv == 128) || (dk == 64 && dv == 64);
}

int launch_gdn_step(hipStream_t s, int Hk, int Hv, int dk, int dv, int K, float eps,
                    const LinearWeights &w, float *conv_ring, int64_t step, float *ssm,
                    const float *qkv_in, const float *z, const float *alpha, const float *beta,
                    float *out, int n_layers, const SdpaMergeTask *merge) {
    if (n_layers < 1 || n_layers > 65535) return fail(MFA_ERR_INVALID, "gdn_step: bad layer count %d", n_layers);
    if (!gdn_shape_supported(Hk, Hv, dk, dv, K))
        return fail(MFA_ERR_SHAPE, "gdn_step: shape Hk=%d Hv=%d dk=%d dv=%d K=%d not supported", Hk,
                    Hv, dk, dv, K);
    const int slot_new = (int)(step % K);
#define MFA_GDN(DKK, KCC)                                                                       \
    hipLaunchKernelGGL((gdn_step_kernel<DKK, DKK, KCC>), dim3(Hv, n_layers), dim3(DKK * 8), 0, s, Hk, Hv, K, eps, \
                       w.conv_w, w.a_log, w.dt_bias, w.norm_w, conv_ring, slot_new, ssm, qkv_in, z,  \
                       alpha, beta, out)
    if (merge && merge->n_units > 0) {
        // a wave per unit, dv / 8 waves per workgroup, Hv workgroups per row
        const int per_row = Hv * (dv / 8);
        const int merge_rows = (merge->n_units + per_row - 1) / per_row;
        if (n_layers + merge_rows > 65535) return fail(MFA_ERR_INVALID, "gdn_step: bad layer count %d", n_layers);
#define MFA_GDN_M(DKK, KCC)                                                                                       \
    hipLaunchKernelGGL((gdn_step_merge_kernel<DKK, DKK, KCC>), dim3(Hv, merge_rows + n_layers), dim3(DKK * 8), 0, s, Hk, \
                       Hv, K, eps, w.conv_w, w.a_log, w.dt_bias, w.norm_w, conv_ring, slot_new, ssm, qkv_in, z,   \
                       alpha, beta, out, *merge, merge_rows)
        if (dk == 128 && K == 4) MFA_GDN_M(128, 4);
        else if (dk == 128) MFA_GDN_M(128, 0);
        else if (K == 4) MFA_GDN_M(64, 4);
        else MFA_GDN_M(64, 0);
#undef MFA_GDN_M
        MFA_HIP(hipGetLastError());
        return MFA_OK;
    }
    if (dk == 128 && K == 4) MFA_GDN(128, 4);
    else if (dk == 128) MFA_GDN(128, 0);
    else if (K == 4) MFA_GDN(64, 4);
    else MFA_GDN(64, 0);
#undef MFA_GDN
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_conv1d_step(hipStream_t s, int C, int K, float *conv_state, const float *in,
                       const uint16_t *w, float *out) {
    hipLaunchKernelGGL(conv1d_step_kernel, dim3((C + 255) / 256), dim3(256), 0, s, conv_state, in, w,
                       out, C, K);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_rms_norm_qk(hipStream_t s, int Hk, int dk, float *q, float *k) {
    hipLaunchKernelGGL(rms_norm_qk_kernel, dim3(Hk), dim3(128), 0, s, q, k, dk);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_rms_norm_bare(hipStream_t s, int dim, float eps, const float *x, float *out) {
    hipLaunchKernelGGL(rms_norm_bare_kernel, dim3(1), dim3(256), 0, s, x, out, dim, eps);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_decay_beta(hipStream_t s, int Hv, const float *alpha, const float *beta,
                      const float *a_log, const uint16_t *dt_bias, float *g, float *b) {
    hipLaunchKernelGGL(decay_beta_kernel, dim3((Hv + 63) / 64), dim3(64), 0, s, alpha, beta, a_log,
                       dt_bias, g, b, Hv);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_delta_net_step(hipStream_t s, int Hv, int Hk, int dk, int dv, const float *g,
                          const float *b, const float *q, const float *k, const float *v,
                          float *ssm, float *out) {
    if (!gdn_shape_supported(Hk, Hv, dk, dv, 4))
        return fail(MFA_ERR_SHAPE, "delta_net_step: shape Hk=%d Hv=%d dk=%d dv=%d not supported", Hk,
                    Hv, dk, dv);
    if (dk == 128)
        hipLaunchKernelGGL((delta_net_step_kernel<128, 128>), dim3(Hv), dim3(1024), 0, s, Hk, Hv, g,
                           b, q, k, v, ssm, out);
    else
        hipLaunchKernelGGL((delta_net_step_kernel<64, 64>), dim3(Hv), dim3(512), 0, s, Hk, Hv, g, b,
                           q, k, v, ssm, out);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_gated_rms_norm(hipStream_t s, int H, int dim, float eps, const float *x,
                          const float *z, const uint16_t *w, float *out) {
    hipLaunchKernelGGL(gated_rms_norm_kernel, dim3(H), dim3(128), 0, s, x, z, w, out, dim, eps);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_conv_ring_export(hipStream_t s, int C, int K, int64_t step, const float *ring,
                            float *state_out) {
    const int64_t n = (int64_t)(K - 1) * C;
    hipLaunchKernelGGL(conv_ring_export_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                       ring, state_out, C, K, step);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_conv_ring_import(hipStream_t s, int C, int K, const float *state, float *ring) {
    const int64_t n = (int64_t)K * C;
    hipLaunchKernelGGL(conv_ring_import_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                       state, ring, C, K);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
