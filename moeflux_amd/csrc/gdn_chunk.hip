// A chunk of T prompt tokens through one Gated-DeltaNet layer.
//
// The reference has no batched prefill: eval_prompt is a token loop
// (crates/moeflux/src/riir/mod.rs:1196-1214), every token running the
// five-kernel chain of crates/moeflux/src/riir/linear_attn_forward.rs:607-664
// and re-reading and re-writing the [dv, dk] state.  Here the chunk is three
// launches whose results are those of the loop, token for token:
//
//   gdn_chunk_pre_kernel    everything that does not depend on the state, for all T
//                           tokens at once: conv + SiLU, per-head q/k norm, decay, beta.
//   gdn_chunk_recur_kernel  a workgroup keeps 16 rows of one value head's state in registers
//                           (16 lanes per row) across the whole chunk; the state is read
//                           once and written once per chunk instead of once per token.
//                           k^, q^, v, g, beta of a slab of tokens are staged in LDS.
//   gdn_chunk_post_kernel   gated RMS norm for all (token, head) pairs, and the conv
//                           history ring advanced by T inputs.
#include "gdn_device.h"

namespace mfa {

static constexpr int kSlab = 32;  // tokens staged in LDS at a time

static constexpr int kPreTok = 8;  // tokens per workgroup of the first kernel

// grid (ceil(T / 8), Hk + ceil(Hv*DV / 256) + 1), 256 threads; a workgroup serves 8 tokens.
//   y <  Hk            : q and k channels of k-head y (conv, SiLU, norm, scaling, k^ . q^)
//   Hk <= y < Hk + nvb : 256 v channels each (conv, SiLU)
//   y == Hk + nvb      : decay and beta of every value head
template <int DK>
__global__ __launch_bounds__(256) void gdn_chunk_pre_kernel(
    int Hk, int Hv, int DV, int K, int T, int step_mod, const uint16_t *__restrict__ conv_w,
    const float *__restrict__ a_log, const uint16_t *__restrict__ dt_bias,
    const float *__restrict__ ring, const float *__restrict__ qkv, const float *__restrict__ alpha,
    const float *__restrict__ beta, float *__restrict__ qn, float *__restrict__ kn,
    float *__restrict__ vv, float *__restrict__ gd, float *__restrict__ bg, float *__restrict__ kq,
    float *__restrict__ lg) {
    static_assert(2 * DK <= 256, "one workgroup covers a k-head's q and k channels");
    constexpr int TT = kPreTok;
    __shared__ float s_part[TT][4];
    __shared__ float s_qk[TT][2 * DK];
    const int t0 = blockIdx.x * TT, y = blockIdx.y, tid = threadIdx.x;
    const int nt = T - t0 < TT ? T - t0 : TT;
    const int C = 2 * Hk * DK + Hv * DV;
    const int nvb = (Hv * DV + 255) / 256;
    if (y < Hk) {
        // threads [0, DK) are q channels, [DK, 2DK) are k channels of this head
        const bool act = tid < 2 * DK, is_q = tid < DK;
        const int ch = is_q ? y * DK + tid : Hk * DK + y * DK + (tid - DK);
        float c[TT];
#pragma unroll
        for (int i = 0; i < TT; i++) c[i] = 0.f;
        if (act) {
            if (K == 4) {
                conv_silu_run<TT, 4>(ring, qkv, conv_w, C, step_mod, t0, nt, ch, c);
            } else {
#pragma unroll
                for (int i = 0; i < TT; i++)
                    if (i < nt) c[i] = conv_silu(ring, qkv, conv_w, C, K, step_mod, t0 + i, ch);
            }
        }
#pragma unroll
        for (int i = 0; i < TT; i++) {
            const float ws = group_sum<64>(c[i] * c[i]);
            if ((tid & 63) == 0) s_part[i][tid >> 6] = ws;
        }
        __syncthreads();
        if (act) {
            // infer.m:2655-2667: x * inv_rms, then q *= (1/sqrt(dk))^2, k *= 1/sqrt(dk)
            const float inv_scale = 1.0f / sqrtf((float)DK);
#pragma unroll
            for (int i = 0; i < TT; i++) {
                float sum = 0.f;
#pragma unroll
                for (int w = 0; w < DK / 64; w++) sum += s_part[i][(is_q ? 0 : DK / 64) + w];
                const float inv_rms = 1.0f / sqrtf(sum / (float)DK + 1e-6f);
                float v = c[i] * inv_rms;
                v *= is_q ? inv_scale * inv_scale : inv_scale;
                s_qk[i][tid] = v;
                if (i < nt) {
                    if (is_q) qn[((size_t)(t0 + i) * Hk + y) * DK + tid] = v;
                    else kn[((size_t)(t0 + i) * Hk + y) * DK + (tid - DK)] = v;
                }
            }
        }
        // k^ . q^ of each token, for the read-out of the token-by-token recurrence
        __syncthreads();
        for (int i = tid >> 6; i < nt; i += 4) {
            const int l = tid & 63;
            float d = 0.f;
#pragma unroll
            for (int u = 0; u < DK / 64; u++) d = fmaf(s_qk[i][l + 64 * u], s_qk[i][DK + l + 64 * u], d);
            d = group_sum<64>(d);
            if (l == 0) kq[(size_t)(t0 + i) * Hk + y] = d;
        }
    } else if (y < Hk + nvb) {
        const int i = (y - Hk) * 256 + tid;
        if (i < Hv * DV) {
            float c[TT];
            if (K == 4) {
                conv_silu_run<TT, 4>(ring, qkv, conv_w, C, step_mod, t0, nt, 2 * Hk * DK + i, c);
            } else {
#pragma unroll
                for (int u = 0; u < TT; u++)
                    c[u] = u < nt ? conv_silu(ring, qkv, conv_w, C, K, step_mod, t0 + u, 2 * Hk * DK + i) : 0.f;
            }
#pragma unroll
            for (int u = 0; u < TT; u++)
                if (u < nt) vv[(size_t)(t0 + u) * Hv * DV + i] = c[u];
        }
    } else {
        for (int p = tid; p < nt * Hv; p += 256) {
            const int t = t0 + p / Hv, h = p % Hv;
            // shaders.metal:1321-1326
            const float a_cap = expf(a_log[h]);
            const float sp = logf(1.0f + expf(alpha[(size_t)t * Hv + h] + bf16_bits_to_f32(dt_bias[h])));
            gd[(size_t)t * Hv + h] = expf(-a_cap * sp);
            lg[(size_t)t * Hv + h] = -a_cap * sp;  // log of the decay, for the blocked form
            bg[(size_t)t * Hv + h] = 1.0f / (1.0f + expf(-beta[(size_t)t * Hv + h]));
        }
    }
}

// grid (Hv, DV/16), 256 threads: a workgroup keeps 16 rows of one head's state in registers
// across the chunk, 16 lanes per row (rows are independent, so a head's rows are spread
// over DV/16 workgroups and every CU gets one).  o_raw [T, Hv*DV] receives the
// un-normalised read-outs.
template <int DK, int DV>
__global__ __launch_bounds__(256) void gdn_chunk_recur_kernel(
    int Hk, int Hv, int T, const float *__restrict__ qn, const float *__restrict__ kn,
    const float *__restrict__ vv, const float *__restrict__ gd, const float *__restrict__ bg,
    const float *__restrict__ kq, float *__restrict__ ssm, float *__restrict__ o_raw) {
    constexpr int NI = DK / 64;
    constexpr int NT = 256, ROWS = 16;
    __shared__ __align__(16) float s_k[kSlab][DK];
    __shared__ __align__(16) float s_q[kSlab][DK];
    __shared__ float s_v[kSlab][ROWS];
    __shared__ float4 s_sc[kSlab];  // decay, beta gate, k . q
    const int tid = threadIdx.x, vh = blockIdx.x, kh = vh / (Hv / Hk);
    const int row0 = blockIdx.y * ROWS;
    const int r = tid >> 4, j = tid & 15;
    float *srow = ssm + ((size_t)vh * DV + row0 + r) * DK + 4 * j;
    float4 s[NI];
#pragma unroll
    for (int i = 0; i < NI; i++) s[i] = *(const float4 *)(srow + 64 * i);

    // A slab's operands travel global -> registers -> LDS; the registers are loaded one slab
    // ahead, while the previous slab is being computed on.  Tokens past the end of the chunk
    // re-read its last token (never used).
    constexpr int KQ_T = kSlab * (DK / 4) / NT;  // float4 of k^ (and of q^) per thread
    constexpr int V_T = kSlab * ROWS / NT;       // floats of v per thread
    static_assert(kSlab * (DK / 4) % NT == 0 && kSlab * ROWS % NT == 0 && kSlab <= NT, "slab staging");
    float4 pk[KQ_T], pq[KQ_T], psc;
    float pv[V_T];
    auto prefetch = [&](int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < KQ_T; u++) {
            const int i = tid + u * NT;
            int t = t0 + i / (DK / 4);
            if (t > T - 1) t = T - 1;
            const size_t src = ((size_t)t * Hk + kh) * DK + (i % (DK / 4)) * 4;
            pk[u] = load_f4(kn + src);
            pq[u] = load_f4(qn + src);
        }
#pragma unroll
        for (int u = 0; u < V_T; u++) {
            const int i = tid + u * NT;
            int t = t0 + i / ROWS;
            if (t > T - 1) t = T - 1;
            pv[u] = vv[((size_t)t * Hv + vh) * DV + row0 + i % ROWS];
        }
        {
            int t = t0 + (tid < kSlab ? tid : 0);
            if (t > T - 1) t = T - 1;
            psc = float4{gd[(size_t)t * Hv + vh], bg[(size_t)t * Hv + vh], kq[(size_t)t * Hk + kh], 0.f};
        }
    };
    prefetch(0);
    for (int t0 = 0; t0 < T; t0 += kSlab) {
        const int nt = (T - t0 < kSlab) ? T - t0 : kSlab;
        __syncthreads();  // the previous slab has been consumed
#pragma unroll
        for (int u = 0; u < KQ_T; u++) {
            const int i = tid + u * NT;
            *(float4 *)&s_k[i / (DK / 4)][(i % (DK / 4)) * 4] = pk[u];
            *(float4 *)&s_q[i / (DK / 4)][(i % (DK / 4)) * 4] = pq[u];
        }
#pragma unroll
        for (int u = 0; u < V_T; u++) {
            const int i = tid + u * NT;
            s_v[i / ROWS][i % ROWS] = pv[u];
        }
        if (tid < kSlab) s_sc[tid] = psc;
        __syncthreads();
        prefetch(t0 + kSlab);
        // One instruction stream per SIMD: what counts is the instruction count per token.
        // Groups of 4 tokens are written out so that their LDS reads go out together, with
        // immediate offsets, and nothing is copied between registers.
        auto token = [&](int tt) __attribute__((always_inline)) {
            float4 kk[NI], qq[NI];
#pragma unroll
            for (int i = 0; i < NI; i++) {
                kk[i] = *(const float4 *)(&s_k[tt][64 * i + 4 * j]);
                qq[i] = *(const float4 *)(&s_q[tt][64 * i + 4 * j]);
            }
            const float4 sc = s_sc[tt];
            const float o = delta_row16<DK>(s, kk, qq, sc.x, sc.y, s_v[tt][r], sc.z);
            if (j == 0) o_raw[((size_t)(t0 + tt) * Hv + vh) * DV + row0 + r] = o;
        };
        int tt = 0;
        for (; tt + 4 <= nt; tt += 4) {
            token(tt);
            token(tt + 1);
            token(tt + 2);
            token(tt + 3);
        }
        for (; tt < nt; tt++) token(tt);
    }
#pragma unroll
    for (int i = 0; i < NI; i++) *(float4 *)(srow + 64 * i) = s[i];
}

// The gated norm (shaders.metal:1337-1370): DV / 4 lanes per (token, head) pair, four channels per
// lane (16-byte loads and stores), 1024 / DV pairs per workgroup, in blocks [0, npb); blocks
// [npb, npb + 32) advance the conv ring: input number s lives in slot s % K, so the last min(T, K)
// inputs of the chunk overwrite their slots.
__global__ __launch_bounds__(256) void gdn_chunk_post_kernel(
    int Hv, int DV, int T, int C, int K, int64_t step, float eps, int npb, const float *__restrict__ o_raw,
    const float *__restrict__ z, const uint16_t *__restrict__ norm_w, const float *__restrict__ qkv,
    float *__restrict__ ring, float *__restrict__ out) {
    const int tid = threadIdx.x;
    if ((int)blockIdx.x >= npb) {
        const int first = T > K ? T - K : 0, nb = gridDim.x - npb;
        for (int t = first; t < T; t++) {
            const int slot = (int)((step + t) % K);
            for (int ch = (blockIdx.x - npb) * 256 + tid; ch < C; ch += nb * 256)
                ring[(size_t)slot * C + ch] = qkv[(size_t)t * C + ch];
        }
        return;
    }
    const int lpr = DV >> 2;                       // lanes per pair: 16 or 32
    const int64_t pair = (int64_t)blockIdx.x * (256 / lpr) + tid / lpr;
    const bool ok = pair < (int64_t)T * Hv;
    const int ch = (tid % lpr) * 4;
    const size_t base = (size_t)(ok ? pair : 0) * DV + ch;
    const float4 x = load_f4(o_raw + base), zz = load_f4(z + base);
    const uint2 wb = *reinterpret_cast<const uint2 *>(norm_w + ch);
    float sum = group_sum<16>((x.x * x.x + x.y * x.y) + (x.z * x.z + x.w * x.w));
    if (lpr == 32) sum += __shfl_xor(sum, 16, 64);
    const float inv = 1.0f / sqrtf(sum / (float)DV + eps);
    if (!ok) return;
    float4 y;
    y.x = x.x * inv * bf16_bits_to_f32((uint16_t)(wb.x & 0xffffu)) * silu_f(zz.x);
    y.y = x.y * inv * bf16_bits_to_f32((uint16_t)(wb.x >> 16)) * silu_f(zz.y);
    y.z = x.z * inv * bf16_bits_to_f32((uint16_t)(wb.y & 0xffffu)) * silu_f(zz.z);
    y.w = x.w * inv * bf16_bits_to_f32((uint16_t)(wb.y >> 16)) * silu_f(zz.w);
    *reinterpret_cast<float4 *>(out + base) = y;
}

// Chunks of at least this many tokens take the blocked form on the matrix cores; shorter
// ones step the recurrence token by token.
static constexpr int kWyMinTokens = 48;

static size_t chunk_common_elems(int Hk, int Hv, int dk, int dv, int T) {
    // (a multiple of 4 floats: the blocked form's arrays behind it are read and written 16 bytes at a time)
    return ((size_t)T * (2 * (size_t)Hk * dk + 2 * (size_t)Hv * dv + 3 * (size_t)Hv + (size_t)Hk) + 3) / 4 * 4;
}

size_t gdn_chunk_scratch_elems(int Hk, int Hv, int dk, int dv, int T) {
    return chunk_common_elems(Hk, Hv, dk, dv, T) + (T >= kWyMinTokens ? gdn_wy_scratch_elems(Hv, dk, dv, T) : 0);
}

int launch_gdn_chunk(hipStream_t s, int Hk, int Hv, int dk, int dv, int K, float eps, int T,
                     const LinearWeights &w, float *conv_ring, int64_t step, float *ssm,
                     const float *qkv_in, const float *z, const float *alpha, const float *beta,
                     float *scratch, float *out) {
    if (!gdn_shape_supported(Hk, Hv, dk, dv, K))
        return fail(MFA_ERR_SHAPE, "gdn chunk: shape Hk=%d Hv=%d dk=%d dv=%d K=%d not supported", Hk, Hv,
                    dk, dv, K);
    if (T <= 0) return fail(MFA_ERR_INVALID, "gdn chunk: T must be > 0");
    if (T > 65535) return fail(MFA_ERR_SHAPE, "gdn chunk: at most 65535 tokens per call");
    const int C = 2 * Hk * dk + Hv * dv;
    float *qn = scratch;
    float *kn = qn + (size_t)T * Hk * dk;
    float *vv = kn + (size_t)T * Hk * dk;
    float *o_raw = vv + (size_t)T * Hv * dv;
    float *gd = o_raw + (size_t)T * Hv * dv;
    float *bg = gd + (size_t)T * Hv;
    float *lg = bg + (size_t)T * Hv;
    float *kq = lg + (size_t)T * Hv;
    float *wy = scratch + chunk_common_elems(Hk, Hv, dk, dv, T);
    const int nvb = (Hv * dv + 255) / 256;
    const bool blocked = T >= kWyMinTokens;
    if (blocked && K == 4) {
        // the blocks of the blocked form compute conv, norms and gates themselves
        const WyInputs in{qkv_in, conv_ring, w.conv_w, w.a_log, w.dt_bias, alpha, beta, K, (int)(step % K)};
        MFA_TRY(launch_gdn_wy(s, Hk, Hv, dk, dv, T, nullptr, nullptr, nullptr, nullptr, nullptr, wy, ssm, o_raw, &in));
    } else {
        if (dk == 128)
            hipLaunchKernelGGL((gdn_chunk_pre_kernel<128>), dim3((T + kPreTok - 1) / kPreTok, Hk + nvb + 1), dim3(256), 0, s,
                               Hk, Hv, dv, K, T, (int)(step % K), w.conv_w, w.a_log, w.dt_bias, conv_ring, qkv_in, alpha, beta, qn, kn,
                               vv, gd, bg, kq, lg);
        else
            hipLaunchKernelGGL((gdn_chunk_pre_kernel<64>), dim3((T + kPreTok - 1) / kPreTok, Hk + nvb + 1), dim3(256), 0, s,
                               Hk, Hv, dv, K, T, (int)(step % K), w.conv_w, w.a_log, w.dt_bias, conv_ring, qkv_in, alpha, beta, qn, kn,
                               vv, gd, bg, kq, lg);
        MFA_HIP(hipGetLastError());
        if (blocked)
            MFA_TRY(launch_gdn_wy(s, Hk, Hv, dk, dv, T, qn, kn, vv, lg, bg, wy, ssm, o_raw));
        else if (dk == 128)
            hipLaunchKernelGGL((gdn_chunk_recur_kernel<128, 128>), dim3(Hv, 128 / 16), dim3(256), 0, s, Hk, Hv, T, qn,
                               kn, vv, gd, bg, kq, ssm, o_raw);
        else
            hipLaunchKernelGGL((gdn_chunk_recur_kernel<64, 64>), dim3(Hv, 64 / 16), dim3(256), 0, s, Hk, Hv, T, qn, kn,
                               vv, gd, bg, kq, ssm, o_raw);
    }
    MFA_HIP(hipGetLastError());
    const int ppb = 1024 / dv;   // pairs per workgroup of the gated norm
    const int npb = (int)(((int64_t)T * Hv + ppb - 1) / ppb);
    hipLaunchKernelGGL(gdn_chunk_post_kernel, dim3(npb + 32), dim3(256), 0, s, Hv, dv, T, C, K, step, eps, npb,
                       o_raw, z, w.norm_w, qkv_in, conv_ring, out);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
