// Device helpers shared by the Gated-DeltaNet kernels (gdn.hip, gdn_chunk.hip).
#pragma once

#include <type_traits>

#include "mfa_internal.h"

namespace mfa {

// A 16-byte load as a register value (assigning through a float4 pointer is a struct copy,
// which the compiler may leave as a memcpy into a stack slot when the target is an array).
typedef float gdn_f32x4 __attribute__((ext_vector_type(4)));
__device__ inline float4 load_f4(const float *p) {
    const gdn_f32x4 v = *reinterpret_cast<const gdn_f32x4 *>(p);
    return float4{v.x, v.y, v.z, v.w};
}

// x / (1 + e^-x) from the hardware exp2 and reciprocal (1 ulp each): 5 instructions where expf and a
// full division are about 40; conv + SiLU and the gated norm apply it to every element of a prompt
// chunk, where it was the largest part of both kernels' instruction count.
__device__ inline float silu_f(float x) {
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// v + (v of the lane selected by a DPP control word); no LDS round trip.
template <int CTRL> __device__ inline float dpp_add(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false);
    return v + __builtin_bit_cast(float, t);
}

// Sum over aligned groups of W lanes, result in every lane of the group.
// 8: quad_perm(1,0,3,2), quad_perm(2,3,0,1), row_half_mirror; 16: + row_mirror;
// 64: the four row sums are combined through v_readlane.
template <int W> __device__ inline float group_sum(float v) {
    static_assert(W == 8 || W == 16 || W == 64, "group width");
    v = dpp_add<0xB1>(v);
    v = dpp_add<0x4E>(v);
    v = dpp_add<0x141>(v);
    if (W >= 16) v = dpp_add<0x140>(v);
    if (W == 64) {
        const int b = __builtin_bit_cast(int, v);
        v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) +
            __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16)) +
            __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) +
            __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    }
    return v;
}

// Maximum over the 64 lanes of a wave, in every lane (same data movement as group_sum<64>).
__device__ inline float wave_max(float v) {
    auto step = [](float x, auto ctrl) {
        const int t = __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x),
                                                  decltype(ctrl)::value, 0xF, 0xF, false);
        return fmaxf(x, __builtin_bit_cast(float, t));
    };
    v = step(v, std::integral_constant<int, 0xB1>{});
    v = step(v, std::integral_constant<int, 0x4E>{});
    v = step(v, std::integral_constant<int, 0x141>{});
    v = step(v, std::integral_constant<int, 0x140>{});
    const int b = __builtin_bit_cast(int, v);
    return fmaxf(fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)),
                       __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16))),
                 fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)),
                       __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48))));
}

// Delta-rule update of one state row held by 8 lanes (lane j owns floats
// 32*i + 4*j .. +3 for i < DK/32).  Follows the operation order of
// crates/moeflux/src/riir/linear_attn.rs:383-410: decay, kv_mem, delta,
// rank-1 update, read-out from the updated row.
template <int DK>
__device__ inline float delta_row(float4 (&s)[DK / 32], const float4 (&kk)[DK / 32],
                                  const float4 (&qq)[DK / 32], float g, float beta, float v) {
    constexpr int NI = DK / 32;
    float kv = 0.f;
#pragma unroll
    for (int i = 0; i < NI; i++) {
        s[i].x *= g; s[i].y *= g; s[i].z *= g; s[i].w *= g;
        kv = fmaf(s[i].x, kk[i].x, kv);
        kv = fmaf(s[i].y, kk[i].y, kv);
        kv = fmaf(s[i].z, kk[i].z, kv);
        kv = fmaf(s[i].w, kk[i].w, kv);
    }
    kv = group_sum<8>(kv);
    const float delta = (v - kv) * beta;
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < NI; i++) {
        s[i].x = fmaf(kk[i].x, delta, s[i].x);
        s[i].y = fmaf(kk[i].y, delta, s[i].y);
        s[i].z = fmaf(kk[i].z, delta, s[i].z);
        s[i].w = fmaf(kk[i].w, delta, s[i].w);
        o = fmaf(s[i].x, qq[i].x, o);
        o = fmaf(s[i].y, qq[i].y, o);
        o = fmaf(s[i].z, qq[i].z, o);
        o = fmaf(s[i].w, qq[i].w, o);
    }
    return group_sum<8>(o);
}

// The same update for a wave that walks a whole chunk, with a row spread over 16 lanes
// (lane j owns floats 64*i + 4*j .. +3 for i < DK/64) and the dependent chain per token
// kept short: both dot products are taken on the row before this token's update,
//   kv = g (S k),  delta = beta (v - kv),  out = g (S q) + delta (k . q),  S <- g S + delta k^T,
// which equals decay / kv_mem / delta / rank-1 update / read-out of the updated row
// (crates/moeflux/src/riir/linear_attn.rs:383-410) up to rounding.  kq = k . q of the token.
template <int DK>
__device__ inline float delta_row16(float4 (&s)[DK / 64], const float4 (&kk)[DK / 64],
                                    const float4 (&qq)[DK / 64], float g, float beta, float v, float kq) {
    constexpr int NI = DK / 64;
    float a0 = 0.f, a1 = 0.f, c0 = 0.f, c1 = 0.f;
#pragma unroll
    for (int i = 0; i < NI; i++) {
        a0 = fmaf(s[i].x, kk[i].x, a0);
        a1 = fmaf(s[i].y, kk[i].y, a1);
        c0 = fmaf(s[i].x, qq[i].x, c0);
        c1 = fmaf(s[i].y, qq[i].y, c1);
        a0 = fmaf(s[i].z, kk[i].z, a0);
        a1 = fmaf(s[i].w, kk[i].w, a1);
        c0 = fmaf(s[i].z, qq[i].z, c0);
        c1 = fmaf(s[i].w, qq[i].w, c1);
    }
    const float sk = group_sum<16>(a0 + a1);
    const float sq = group_sum<16>(c0 + c1);
    const float delta = (v - g * sk) * beta;
#pragma unroll
    for (int i = 0; i < NI; i++) {
        s[i].x = fmaf(kk[i].x, delta, g * s[i].x);
        s[i].y = fmaf(kk[i].y, delta, g * s[i].y);
        s[i].z = fmaf(kk[i].z, delta, g * s[i].z);
        s[i].w = fmaf(kk[i].w, delta, g * s[i].w);
    }
    return fmaf(delta, kq, g * sq);
}

// Depthwise conv + SiLU of channel ch for TT consecutive inputs of the layer, the first
// of them input number `step + t0` (crates/moeflux/src/riir/linear_attn.rs:132-154): tap
// k < K-1 of token t multiplies input step+t-(K-1)+k, which is row t-(K-1)+k of `chunk`
// when that is >= 0 and the ring slot (input number mod K) of the history otherwise; tap
// K-1 multiplies the new input.  Tokens at or past nt give 0.  step_mod = step % K.
// Each input is loaded once and the taps stay in registers.
template <int TT, int KC>
__device__ inline void conv_silu_run(const float *__restrict__ ring, const float *__restrict__ chunk,
                                     const uint16_t *__restrict__ w, int C, int step_mod, int t0, int nt,
                                     int ch, float (&out)[TT]) {
    float wt[KC], xs[TT + KC - 1];
#pragma unroll
    for (int k = 0; k < KC; k++) wt[k] = bf16_bits_to_f32(w[(size_t)ch * KC + k]);
#pragma unroll
    for (int j = 0; j < TT + KC - 1; j++) {
        const int idx = t0 - (KC - 1) + j;  // row of the chunk, negative: history
        float x = 0.f;
        if (idx >= 0) {
            if (idx < t0 + nt) x = chunk[(size_t)idx * C + ch];
        } else {
            x = ring[(size_t)(((step_mod + idx) % KC + KC) % KC) * C + ch];
        }
        xs[j] = x;
    }
#pragma unroll
    for (int i = 0; i < TT; i++) {
        float acc = 0.f;
#pragma unroll
        for (int k = 0; k < KC; k++) acc = fmaf(xs[i + k], wt[k], acc);
        out[i] = i < nt ? silu_f(acc) : 0.f;
    }
}

// The same for a conv width known only at run time, one token at a time.
__device__ inline float conv_silu(const float *__restrict__ ring, const float *__restrict__ chunk,
                                  const uint16_t *__restrict__ w, int C, int K, int step_mod, int t,
                                  int ch) {
    float acc = 0.f;
    for (int k = 0; k < K - 1; k++) {
        const int idx = t - (K - 1) + k;
        float x;
        if (idx >= 0) x = chunk[(size_t)idx * C + ch];
        else x = ring[(size_t)(((step_mod + idx) % K + K) % K) * C + ch];
        acc = fmaf(x, bf16_bits_to_f32(w[(size_t)ch * K + k]), acc);
    }
    acc = fmaf(chunk[(size_t)t * C + ch], bf16_bits_to_f32(w[(size_t)ch * K + (K - 1)]), acc);
    return silu_f(acc);
}

}  // namespace mfa
