// One-launch twins of the reference's four full-attention kernels
// (crates/moeflux/shaders/shaders.metal:976-1134), over row-major f32 K/V
// [seq_len, kv_dim] exactly as the reference's per-kernel hooks take them
// (crates/moeflux/src/riir/gpu_attn.rs:247-416).  They exist for per-kernel
// parity tests; the production decode path is sdpa_decode.hip.
#include "mfa_internal.h"

namespace mfa {

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) v += __shfl_xor(v, m, 64);
    return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return v;
}

// shaders.metal:976-1019.  grid (ceil(L/4), Hq), 4 waves; one wave per (head, position),
// each lane reading 16 contiguous bytes of the K row slice per pass.
__global__ __launch_bounds__(256) void attn_scores_kernel(
    const float *__restrict__ q, const float *__restrict__ k, float *__restrict__ scores, int D,
    int kv_dim, int L, int stride, float scale, int hpk) {
    const int lane = threadIdx.x & 63;
    const int p = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int h = blockIdx.y;
    if (p >= L) return;
    const float *qh = q + (size_t)h * D;
    const float *kp = k + (size_t)p * kv_dim + (size_t)(h / hpk) * D;
    float acc = 0.f;
    for (int d = lane * 4; d < D; d += 256) {
        const float4 a = *(const float4 *)(qh + d);
        const float4 b = *(const float4 *)(kp + d);
        acc += a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
    }
    acc = wave_sum(acc);
    if (lane == 0) scores[(size_t)h * stride + p] = acc * scale;
}

// shaders.metal:1026-1084.  One block per head; max seeded with -1e30f as the reference does.
__global__ __launch_bounds__(256) void attn_softmax_kernel(float *__restrict__ scores, int L,
                                                           int stride) {
    __shared__ float sh[4];
    float *s = scores + (size_t)blockIdx.x * stride;
    const int tid = threadIdx.x;
    float m = -1e30f;
    for (int i = tid; i < L; i += 256) m = fmaxf(m, s[i]);
    m = wave_max(m);
    if ((tid & 63) == 0) sh[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
    __syncthreads();
    float sum = 0.f;
    for (int i = tid; i < L; i += 256) {
        const float e = expf(s[i] - m);
        s[i] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    if ((tid & 63) == 0) sh[tid >> 6] = sum;
    __syncthreads();
    sum = sh[0] + sh[1] + sh[2] + sh[3];
    const float inv = 1.0f / sum;
    for (int i = tid; i < L; i += 256) s[i] *= inv;
}

// shaders.metal:1095-1117.  grid (D/64, Hq), 256 threads = 64 output channels x 4 position
// lanes; the four partial sums are combined through LDS.
__global__ __launch_bounds__(256) void attn_values_kernel(
    const float *__restrict__ scores, const float *__restrict__ v, float *__restrict__ out, int D,
    int kv_dim, int L, int stride, int hpk) {
    __shared__ float sh[256];
    const int dl = threadIdx.x & 63, pg = threadIdx.x >> 6;
    const int d = blockIdx.x * 64 + dl;
    const int h = blockIdx.y;
    const float *s = scores + (size_t)h * stride;
    const float *vp = v + (size_t)(h / hpk) * D + d;
    float acc = 0.f;
    if (d < D)
        for (int p = pg; p < L; p += 4) acc += s[p] * vp[(size_t)p * kv_dim];
    sh[threadIdx.x] = acc;
    __syncthreads();
    if (pg == 0 && d < D) out[(size_t)h * D + d] = sh[dl] + sh[64 + dl] + sh[128 + dl] + sh[192 + dl];
}

// shaders.metal:1125-1134.
__global__ void sigmoid_gate_kernel(float *__restrict__ x, const float *__restrict__ gate, int dim) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= dim) return;
    const float g = 1.0f / (1.0f + expf(-gate[i]));
    x[i] = x[i] * g;
}

int launch_attn_scores(hipStream_t s, int Hq, int Hkv, int D, int L, int stride, const float *q,
                       const float *k, float scale, float *scores) {
    if (D % 4 != 0) return fail(MFA_ERR_SHAPE, "attn_scores: head_dim %d must be a multiple of 4", D);
    hipLaunchKernelGGL(attn_scores_kernel, dim3((L + 3) / 4, Hq), dim3(256), 0, s, q, k, scores, D,
                       Hkv * D, L, stride, scale, Hq / Hkv);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_attn_softmax(hipStream_t s, int Hq, int L, int stride, float *scores) {
    hipLaunchKernelGGL(attn_softmax_kernel, dim3(Hq), dim3(256), 0, s, scores, L, stride);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_attn_values(hipStream_t s, int Hq, int Hkv, int D, int L, int stride,
                       const float *scores, const float *v, float *out) {
    hipLaunchKernelGGL(attn_values_kernel, dim3((D + 63) / 64, Hq), dim3(256), 0, s, scores, v, out,
                       D, Hkv * D, L, stride, Hq / Hkv);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_sigmoid_gate(hipStream_t s, int dim, const float *gate, float *x) {
    hipLaunchKernelGGL(sigmoid_gate_kernel, dim3((dim + 255) / 256), dim3(256), 0, s, x, gate, dim);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
