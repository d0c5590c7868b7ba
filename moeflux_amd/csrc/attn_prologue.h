// Per-head RMS norm and rotation of q and k ahead of the attention core, as a group of lanes
// computes them: the arithmetic shared by the stand-alone prologue kernel (attn_prologue.hip)
// and the prologue inside the split-K attention launch (sdpa_decode.hip), so that both leave
// bit-identical key rows in the cache.
//
// A head of D channels is served by LPH = D / EPS neighbouring lanes, lane j holding channels
// [EPS j, EPS j + EPS) (EPS = 8 for a bf16 cache, 4 for f32: one operand slot of the attention
// kernel).  x * inv_rms * weight (crates/moeflux/src/riir/rms_norm.rs:138-151), then the rotation
// of the pairs (i, i + rotary_dim / 2) (crates/moeflux/src/riir/rope.rs:96-112); rotary_dim / 2
// must be a multiple of EPS so that a lane's partner channels are one other lane's.
#pragma once
#include "gdn_device.h"

namespace mfa {

// f32 <-> cache element
template <typename KV> __device__ inline KV to_kv(float x);
template <> __device__ inline float to_kv<float>(float x) { return x; }
template <> __device__ inline uint16_t to_kv<uint16_t>(float x) { return f32_to_bf16_bits(x); }
__device__ inline float from_kv(float x) { return x; }
__device__ inline float from_kv(uint16_t x) { return bf16_bits_to_f32(x); }

// (cos, sin) with the device library's full-range routines; one copy of their code instead of
// one per channel.
static __device__ __noinline__ float2 head_cos_sin(float angle) { return float2{cosf(angle), sinf(angle)}; }

// Sum over aligned groups of LPH lanes (8, 16, 32 or 64), the same value in every lane: data-parallel
// primitives within a row of 16 lanes (no LDS round trip), one lane exchange for 32.
template <int LPH> __device__ inline float lanes_sum(float v) {
    static_assert(LPH == 8 || LPH == 16 || LPH == 32 || LPH == 64, "lanes per head");
    if constexpr (LPH == 32) {
        v = group_sum<16>(v);
        return v + __shfl_xor(v, 16, 64);
    } else {
        return group_sum<LPH>(v);
    }
}

template <int EPS, int D> struct HeadRotor {
    static constexpr int LPH = D / EPS;
    static_assert(LPH == 8 || LPH == 16 || LPH == 32 || LPH == 64, "a head's lanes fit a wave");
    float cs[EPS], sn[EPS];   // cos, and sin with the sign of the lane's half: out = y cos + partner's y * sn
    int partner;

    // The workgroup's table of (cos, sin)(pos * inv_freq[i]), i < rotary_dim / 2, in LDS: thread i
    // requests frequency i (table_request, to be placed among a kernel's first requests: data
    // comes back in request order) and later computes entry i (table), so whole waves without
    // such a thread skip the routine.  A workgroup barrier must separate table() from init().
    __device__ static inline float table_request(const float *__restrict__ inv_freq, int rotary_dim) {
        return (int)threadIdx.x < (rotary_dim >> 1) ? inv_freq[threadIdx.x] : 0.f;
    }
    __device__ static inline void table(float freq, int pos, int rotary_dim, float2 *tab) {
        if ((int)threadIdx.x < (rotary_dim >> 1)) tab[threadIdx.x] = head_cos_sin((float)pos * freq);
    }
    // j: the lane's index within its head.  The pair (x0, x1) = (channel c, channel c + half)
    // becomes (x0 cos - x1 sin, x0 sin + x1 cos): the lane of the low channel holds y = x0 and gets
    // x1 from its partner, the lane of the high channel holds y = x1 and gets x0, so both are
    // y cos + other * (-sin | +sin); channels past rotary_dim have cos = 1, sin = 0 and themselves
    // as partner.  No branch, and the lane exchanges of a slot are all issued before the first use.
    __device__ inline void init(int j, int rotary_dim, const float2 *tab) {
        const int c0 = EPS * j, half = rotary_dim >> 1;
        const bool rot = c0 < rotary_dim, low = c0 < half;
#pragma unroll
        for (int e = 0; e < EPS; e++) {
            const int c = c0 + e;
            const float2 t = tab[rot ? (c < half ? c : c - half) : 0];
            cs[e] = rot ? t.x : 1.f;
            sn[e] = rot ? (low ? -t.y : t.y) : 0.f;
        }
        const int lane = threadIdx.x & 63, dj = half / EPS;
        partner = rot ? (low ? lane + dj : lane - dj) : lane;
    }
    // every lane of the wave calls this together
    __device__ inline void apply(float (&x)[EPS], const float (&w)[EPS], float eps) const {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < EPS; e++) ss += x[e] * x[e];
        ss = lanes_sum<LPH>(ss);
        const float inv_rms = 1.0f / sqrtf(ss / (float)D + eps);
        float y[EPS], o[EPS];
#pragma unroll
        for (int e = 0; e < EPS; e++) y[e] = x[e] * inv_rms * w[e];
#pragma unroll
        for (int e = 0; e < EPS; e++) o[e] = __shfl(y[e], partner, 64);
#pragma unroll
        for (int e = 0; e < EPS; e++) x[e] = y[e] * cs[e] + o[e] * sn[e];
    }
};

// Whether the lane-group form applies: otherwise attn_prologue.hip falls back to one thread per channel.
inline bool head_rotor_applies(int kv_dtype, int D, int rotary_dim) {
    const int eps = kv_dtype == MFA_KV_BF16 ? 8 : 4;
    return rotary_dim > 0 && rotary_dim <= D && rotary_dim % 2 == 0 && (rotary_dim / 2) % eps == 0 && rotary_dim / 2 <= 128;
}

}  // namespace mfa
