// Split-K flash-decode GQA attention with the sigmoid output gate, for gfx950.
//
// Replaces the reference's four-kernel chain attn_scores_batched /
// attn_softmax_batched / attn_values_batched / sigmoid_gate
// (crates/moeflux/shaders/shaders.metal:976-1134, encoded at
// crates/moeflux/src/riir/linear_attn_forward.rs:850-902) and its CPU fallback
// sdpa_cpu (crates/moeflux/src/riir/sdpa.rs:63-172) with two launches:
//
//   sdpa_partial_kernel  grid (splits, head groups, kv heads), 4 or 8 waves each.
//     A wave streams whole position blocks of its kv head's K and V planes
//     exactly once, each wave-level load being a contiguous 1 KiB run that
//     lands directly in MFMA operand registers (see KvTile in mfa_internal.h).
//     The up to 16 query heads that share the kv head are the N dimension of
//     the matrix instruction:   S^T[pos, head] = K[pos, :] . Q[head, :]
//                               O^T[d, head]  += V^T[d, pos] . P^T[pos, head]
//     so lane%16 is the head index in both products and the online-softmax
//     state (running max, running sum) lives in that lane with no transposes.
//     bf16 caches use v_mfma_f32_16x16x32_bf16 with the f32 query and the f32
//     probabilities each split into a bf16 high and low part (two
//     instructions), which keeps the products exact to ~2^-17; f32 caches use
//     v_mfma_f32_16x16x4_f32.  The query (pre-multiplied by scale*log2 e, so
//     that probabilities are single v_exp_f32) is converted once per
//     workgroup into LDS in operand order.  A block's K and V are a stream of
//     groups of up to eight 1 KiB loads; two register buffers alternate, the
//     one just consumed being refilled with the group after next.  The waves
//     are merged through LDS and one (max, sum, O[16, D]) partial per
//     workgroup is written.
//   sdpa_merge_kernel    log-sum-exp merge of the partials, normalisation and
//     the sigmoid gate.
#include "mfa_internal.h"

namespace mfa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;

static constexpr int kMaxSplits = 1024;
static constexpr float kLog2e = 1.4426950408889634f;

__device__ inline float neg_inf() { return -__builtin_huge_valf(); }
__device__ inline float lane_xor(float v, int mask) { return __shfl_xor(v, mask, 64); }
__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// (a, b) -> packed bf16 pair, round to nearest even (v_cvt_pk_bf16_f32)
__device__ inline uint32_t pack_bf16(float a, float b) {
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
// x = hi + lo + O(2^-17 x): hi = bf16(x), lo = bf16(x - hi); x - hi is exact in f32.
__device__ inline void split_pair(float a, float b, uint32_t &hi, uint32_t &lo) {
    hi = pack_bf16(a, b);
    const float ah = __builtin_bit_cast(float, hi << 16);
    const float bh = __builtin_bit_cast(float, hi & 0xffff0000u);
    lo = pack_bf16(a - ah, b - bh);
}
__device__ inline bf16x8 as_bf16x8(uint4 u) { return __builtin_bit_cast(bf16x8, u); }

template <typename KV, int D> struct Wave;

// ---------------------------------------------------------------------------
// bf16 cache: blocks of 32 positions (64*D bytes of K and of V each)
// ---------------------------------------------------------------------------
template <int D> struct Wave<uint16_t, D> {
    static constexpr int BLK = 32;
    static constexpr int KSTEPS = D / 32;          // MFMA k-steps per 16-position sub-tile
    static constexpr int NACC = D / 16;            // 16-wide output tiles of O^T
    static constexpr int NLOAD = D / 16;           // 1 KiB loads per block, for K and for V alike
    static constexpr int G = NLOAD < 8 ? NLOAD : 8;  // loads per register group
    static constexpr int NG = NLOAD / G;           // groups per block for K, same for V
    static constexpr int QLDS_U4 = KSTEPS * 2 * 64;

    // Query operands in LDS: [k-step][hi|lo][lane] of 16 bytes.
    __device__ static void prep_q(uint4 *qlds, const float *q, int kvh, int hg, int hpk, float qscale) {
        for (int slot = threadIdx.x; slot < KSTEPS * 64; slot += blockDim.x) {
            const int s = slot >> 6, lane = slot & 63, n = lane & 15, g = lane >> 4;
            const int hin = hg * 16 + n;
            uint4 hi = {0, 0, 0, 0}, lo = {0, 0, 0, 0};
            if (hin < hpk) {
                const float *p = q + (size_t)(kvh * hpk + hin) * D + 8 * (4 * s + g);
                const float4 a = *(const float4 *)p, b = *(const float4 *)(p + 4);
                split_pair(a.x * qscale, a.y * qscale, hi.x, lo.x);
                split_pair(a.z * qscale, a.w * qscale, hi.y, lo.y);
                split_pair(b.x * qscale, b.y * qscale, hi.z, lo.z);
                split_pair(b.z * qscale, b.w * qscale, hi.w, lo.w);
            }
            qlds[(s * 2 + 0) * 64 + lane] = hi;
            qlds[(s * 2 + 1) * 64 + lane] = lo;
        }
    }

    struct Scores {
        f32x4 s[2];
    };
    struct Probs {
        uint4 hi, lo;
    };

    // group `grp` of a block: loads grp*G .. grp*G+G-1 of the block's contiguous run
    __device__ static void load_group(uint4 (&dst)[G], const uint16_t *plane, int64_t blk, int grp, int lane) {
        const uint4 *b = (const uint4 *)(plane + blk * (int64_t)(BLK * D)) + lane + grp * G * 64;
#pragma unroll
        for (int i = 0; i < G; i++) dst[i] = b[i * 64];
    }

    __device__ static void zero_scores(Scores &sc) {
        sc.s[0] = f32x4{0.f, 0.f, 0.f, 0.f};
        sc.s[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // load index li = 2*s + sub: both sub-tiles of a k-step share one read of the query operands
    __device__ static void consume_k(const uint4 (&src)[G], int grp, const uint4 *qlds, int lane, Scores &sc) {
#pragma unroll
        for (int i = 0; i < G; i++) {
            const int li = grp * G + i, s = li / 2, sub = li % 2;
            const bf16x8 a = as_bf16x8(src[i]);
            const bf16x8 qh = as_bf16x8(qlds[(s * 2 + 0) * 64 + lane]);
            const bf16x8 ql = as_bf16x8(qlds[(s * 2 + 1) * 64 + lane]);
            sc.s[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qh, sc.s[sub], 0, 0, 0);
            sc.s[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, ql, sc.s[sub], 0, 0, 0);
        }
    }

    // Row 4g+i of sub-tile `sub` is position blk*32 + 16*sub + 4g + i; scores are in
    // log2 units.  Returns the rescale factor of the running state (1 if unchanged).
    __device__ static float softmax(Scores &sc, int64_t blk, int64_t kv_len, int g, float &m_run,
                                    float &l_run, Probs &p) {
        float x[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            x[i] = sc.s[0][i];
            x[4 + i] = sc.s[1][i];
        }
        if ((blk + 1) * BLK > kv_len) {  // only the last block of the cache is ragged
            const int64_t base = blk * BLK + 4 * g;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (base + i >= kv_len) x[i] = neg_inf();
                if (base + 16 + i >= kv_len) x[4 + i] = neg_inf();
            }
        }
        float tmax = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])),
                           fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
        tmax = fmaxf(tmax, lane_xor(tmax, 16));
        tmax = fmaxf(tmax, lane_xor(tmax, 32));
        const float m_new = fmaxf(m_run, tmax);  // finite: position blk*32 is always valid
        const float alpha = fast_exp2(m_run - m_new);
        float e[8];
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            e[i] = fast_exp2(x[i] - m_new);
            psum += e[i];
        }
        split_pair(e[0], e[1], p.hi.x, p.lo.x);
        split_pair(e[2], e[3], p.hi.y, p.lo.y);
        split_pair(e[4], e[5], p.hi.z, p.lo.z);
        split_pair(e[6], e[7], p.hi.w, p.lo.w);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        return alpha;
    }

    __device__ static void consume_v(const uint4 (&src)[G], int grp, const Probs &p, f32x4 (&o)[NACC]) {
        const bf16x8 ph = as_bf16x8(p.hi), pl = as_bf16x8(p.lo);
#pragma unroll
        for (int i = 0; i < G; i++) {
            const int dt = grp * G + i;
            const bf16x8 a = as_bf16x8(src[i]);
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, ph, o[dt], 0, 0, 0);
            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pl, o[dt], 0, 0, 0);
        }
    }

    // accumulator a, lane group g, holds d = 16a + 4g + {0,1,2,3}
    __device__ static void store_o(float *row, int g, const f32x4 (&o)[NACC]) {
#pragma unroll
        for (int a = 0; a < NACC; a++) {
            float4 v = {o[a][0], o[a][1], o[a][2], o[a][3]};
            *(float4 *)(row + 16 * a + 4 * g) = v;
        }
    }
};

// ---------------------------------------------------------------------------
// f32 cache: blocks of 16 positions (64*D bytes of K and of V each)
// ---------------------------------------------------------------------------
template <int D> struct Wave<float, D> {
    static constexpr int BLK = 16;
    static constexpr int KSTEPS = D / 16;  // 1 KiB loads of K per block (4 MFMAs each)
    static constexpr int NC = D / 64;
    static constexpr int NACC = D / 16;    // = NC * 4
    static constexpr int NLOAD = D / 16;   // loads per block, for K and for V alike
    static constexpr int G = NLOAD < 8 ? NLOAD : 8;
    static constexpr int NG = NLOAD / G;
    static constexpr int QLDS_U4 = KSTEPS * 64;

    // Query operands in LDS: [k-step][lane] float4; lane (n, g) holds q[n][4(4s+g) .. +3].
    __device__ static void prep_q(uint4 *qlds, const float *q, int kvh, int hg, int hpk, float qscale) {
        for (int slot = threadIdx.x; slot < KSTEPS * 64; slot += blockDim.x) {
            const int s = slot >> 6, lane = slot & 63, n = lane & 15, g = lane >> 4;
            const int hin = hg * 16 + n;
            float4 v = {0.f, 0.f, 0.f, 0.f};
            if (hin < hpk) {
                v = *(const float4 *)(q + (size_t)(kvh * hpk + hin) * D + 4 * (4 * s + g));
                v.x *= qscale; v.y *= qscale; v.z *= qscale; v.w *= qscale;
            }
            qlds[slot] = __builtin_bit_cast(uint4, v);
        }
    }

    struct Scores {
        f32x4 s;
    };
    struct Probs {
        float p[4];
    };

    __device__ static void load_group(uint4 (&dst)[G], const float *plane, int64_t blk, int grp, int lane) {
        const uint4 *b = (const uint4 *)(plane + blk * (int64_t)(BLK * D)) + lane + grp * G * 64;
#pragma unroll
        for (int i = 0; i < G; i++) dst[i] = b[i * 64];
    }

    __device__ static void zero_scores(Scores &sc) { sc.s = f32x4{0.f, 0.f, 0.f, 0.f}; }

    __device__ static void consume_k(const uint4 (&src)[G], int grp, const uint4 *qlds, int lane, Scores &sc) {
#pragma unroll
        for (int i = 0; i < G; i++) {
            const int s = grp * G + i;
            const float4 a = __builtin_bit_cast(float4, src[i]);
            const float4 b = __builtin_bit_cast(float4, qlds[s * 64 + lane]);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, sc.s, 0, 0, 0);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, sc.s, 0, 0, 0);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, sc.s, 0, 0, 0);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, sc.s, 0, 0, 0);
        }
    }

    __device__ static float softmax(Scores &sc, int64_t blk, int64_t kv_len, int g, float &m_run,
                                    float &l_run, Probs &p) {
        float x[4] = {sc.s[0], sc.s[1], sc.s[2], sc.s[3]};
        if ((blk + 1) * BLK > kv_len) {
            const int64_t base = blk * BLK + 4 * g;
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (base + i >= kv_len) x[i] = neg_inf();
        }
        float tmax = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
        tmax = fmaxf(tmax, lane_xor(tmax, 16));
        tmax = fmaxf(tmax, lane_xor(tmax, 32));
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = fast_exp2(m_run - m_new);
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            p.p[i] = fast_exp2(x[i] - m_new);
            psum += p.p[i];
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
        return alpha;
    }

    // load index li = i*NC + c: MFMA set i contracts positions 4g+i; accumulator 4c+j
    // collects d = 64c + 4m + j.
    __device__ static void consume_v(const uint4 (&src)[G], int grp, const Probs &p, f32x4 (&o)[NACC]) {
#pragma unroll
        for (int x = 0; x < G; x++) {
            const int li = grp * G + x, i = li / NC, c = li % NC;
            const float4 a = __builtin_bit_cast(float4, src[x]);
            o[4 * c + 0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, p.p[i], o[4 * c + 0], 0, 0, 0);
            o[4 * c + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, p.p[i], o[4 * c + 1], 0, 0, 0);
            o[4 * c + 2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, p.p[i], o[4 * c + 2], 0, 0, 0);
            o[4 * c + 3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, p.p[i], o[4 * c + 3], 0, 0, 0);
        }
    }

    // accumulator 4c+j, lane group g, element i holds d = 64c + 16g + 4i + j
    __device__ static void store_o(float *row, int g, const f32x4 (&o)[NACC]) {
#pragma unroll
        for (int c = 0; c < NC; c++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float4 v = {o[4 * c + 0][i], o[4 * c + 1][i], o[4 * c + 2][i], o[4 * c + 3][i]};
                *(float4 *)(row + 64 * c + 16 * g + 4 * i) = v;
            }
    }
};

// Dynamic LDS of the partial kernel: the query operands, later overlaid by WAVES/2
// reduction slots of one wave's O accumulators each, then per-wave (max, sum) rows.
template <typename KV, int D, int WAVES> struct PartialLds {
    using W = Wave<KV, D>;
    static constexpr size_t kSlotBytes = (size_t)W::NACC * 64 * 16;
    static constexpr size_t kQBytes = (size_t)W::QLDS_U4 * 16;
    static constexpr size_t kRedBytes = kSlotBytes * (WAVES / 2);
    static constexpr size_t kRegion0 = kRedBytes > kQBytes ? kRedBytes : kQBytes;
    static constexpr size_t kBytes = kRegion0 + 2 * WAVES * 16 * sizeof(float);
};

// part_o:  [kv head][head group][split][16 heads][D]
// part_ml: [kv head][head group][split][2][16]   (max in log2 units, then sum)
template <typename KV, int D, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void sdpa_partial_kernel(
    const KV *__restrict__ k_tiled, const KV *__restrict__ v_tiled, size_t plane_elems,
    const float *__restrict__ q, int hpk, int64_t kv_len, int blocks_per_split, float qscale,
    float *__restrict__ part_o, float *__restrict__ part_ml) {
    using W = Wave<KV, D>;
    using L = PartialLds<KV, D, WAVES>;
    constexpr int NACC = W::NACC;
    constexpr int NG = W::NG;
    constexpr int G = W::G;
    constexpr int NITEM = 2 * NG;  // a block's stream: NG groups of K, then NG groups of V
    extern __shared__ __align__(16) unsigned char lds_raw[];
    uint4 *qlds = reinterpret_cast<uint4 *>(lds_raw);
    f32x4 *red = reinterpret_cast<f32x4 *>(lds_raw);  // [WAVES/2][NACC][64], after the main loop
    float *sm = reinterpret_cast<float *>(lds_raw + L::kRegion0);  // [WAVES][16]
    float *sl = sm + WAVES * 16;                                   // [WAVES][16]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int split = blockIdx.x, hg = blockIdx.y, kvh = blockIdx.z;
    const int nsplit = gridDim.x, nhg = gridDim.y;

    const KV *kplane = k_tiled + (size_t)kvh * plane_elems;
    const KV *vplane = v_tiled + (size_t)kvh * plane_elems;
    const int64_t nblk = (kv_len + W::BLK - 1) / W::BLK;
    const int64_t b0 = (int64_t)split * blocks_per_split;
    int64_t b1 = b0 + blocks_per_split;
    if (b1 > nblk) b1 = nblk;

    // Stream item t of a block is K group t (t < NG) or V group t-NG; item t lives in
    // buf[t & 1].  The first two items go out before anything else; the query
    // conversion below overlaps their latency.
    uint4 buf[2][G];
    int64_t b = b0 + wave;
    if (b < b1) {
        W::load_group(buf[0], kplane, b, 0, lane);
        if (NG > 1) W::load_group(buf[1], kplane, b, 1, lane);
        else W::load_group(buf[1], vplane, b, 0, lane);
    }
    W::prep_q(qlds, q, kvh, hg, hpk, qscale);
    __syncthreads();

    f32x4 o[NACC];
#pragma unroll
    for (int a = 0; a < NACC; a++) o[a] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = neg_inf(), l_run = 0.f;

    for (; b < b1; b += WAVES) {
        const int64_t bn = b + WAVES;
        const bool more = bn < b1;
        typename W::Scores sc;
        typename W::Probs p;
        W::zero_scores(sc);
#pragma unroll
        for (int t = 0; t < NITEM; t++) {
            if (t == NG) {
                const float alpha = W::softmax(sc, b, kv_len, g, m_run, l_run, p);
                if (__any(alpha != 1.0f)) {  // the running max moved: rescale what has been accumulated
#pragma unroll
                    for (int a = 0; a < NACC; a++) {
                        o[a][0] *= alpha; o[a][1] *= alpha; o[a][2] *= alpha; o[a][3] *= alpha;
                    }
                }
            }
            if (t < NG) W::consume_k(buf[t & 1], t, qlds, lane, sc);
            else W::consume_v(buf[t & 1], t - NG, p, o);
            // refill the buffer just consumed with the item two ahead in the stream
            const int t2 = t + 2;
            if (t2 < NITEM) {
                if (t2 < NG) W::load_group(buf[t & 1], kplane, b, t2, lane);
                else W::load_group(buf[t & 1], vplane, b, t2 - NG, lane);
            } else if (more) {
                const int t3 = t2 - NITEM;
                if (t3 < NG) W::load_group(buf[t & 1], kplane, bn, t3, lane);
                else W::load_group(buf[t & 1], vplane, bn, t3 - NG, lane);
            }
        }
    }
    l_run += lane_xor(l_run, 16);
    l_run += lane_xor(l_run, 32);

    // ---- merge the waves ---------------------------------------------------------
    if (g == 0) sm[wave * 16 + n] = m_run;
    __syncthreads();  // also: every wave is done reading the query operands
    float M = sm[n];
#pragma unroll
    for (int x = 1; x < WAVES; x++) M = fmaxf(M, sm[x * 16 + n]);
    const float f = (m_run == neg_inf()) ? 0.f : fast_exp2(m_run - M);
    l_run *= f;
#pragma unroll
    for (int a = 0; a < NACC; a++) {
        o[a][0] *= f; o[a][1] *= f; o[a][2] *= f; o[a][3] *= f;
    }
    if (g == 0) sl[wave * 16 + n] = l_run;
#pragma unroll
    for (int half = WAVES / 2; half >= 1; half >>= 1) {
        if (wave >= half && wave < 2 * half) {
#pragma unroll
            for (int a = 0; a < NACC; a++) red[((wave - half) * NACC + a) * 64 + lane] = o[a];
        }
        __syncthreads();
        if (wave < half) {
#pragma unroll
            for (int a = 0; a < NACC; a++) {
                const f32x4 t = red[(wave * NACC + a) * 64 + lane];
                o[a][0] += t[0]; o[a][1] += t[1]; o[a][2] += t[2]; o[a][3] += t[3];
            }
        }
        __syncthreads();
    }
    if (wave == 0) {
        const size_t pid = ((size_t)kvh * nhg + hg) * nsplit + split;
        W::store_o(part_o + (pid * 16 + n) * D, g, o);
        if (g == 0) {
            float lsum = 0.f;
#pragma unroll
            for (int x = 0; x < WAVES; x++) lsum += sl[x * 16 + n];
            part_ml[pid * 32 + n] = M;
            part_ml[pid * 32 + 16 + n] = lsum;
        }
    }
}

// grid (Hq, D/64), 256 threads: 16 lanes x float4 cover 64 outputs of one split's row,
// 16 such rows per pass.  Each thread's partial rows are requested before the weights
// are known, so the kernel pays one memory round trip.
static constexpr int kMergeRows = 8;  // partial rows a thread keeps in flight
__global__ __launch_bounds__(256) void sdpa_merge_kernel(
    const float *__restrict__ part_o, const float *__restrict__ part_ml, int nsplit, int hpk,
    int nhg, int D, const float *__restrict__ gate, float *__restrict__ out) {
    __shared__ float wsh[kMaxSplits];
    __shared__ float redf[4];
    __shared__ float4 acc4[16][16];
    const int h = blockIdx.x;
    const int kvh = h / hpk, hin = h % hpk, hg = hin / 16, n = hin % 16;
    const size_t pid0 = ((size_t)kvh * nhg + hg) * nsplit;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int dl = tid & 15, sg = tid >> 4;  // 16 float4 lanes x 16 split lanes
    const int d0 = blockIdx.y * 64 + dl * 4;

    float4 rows[kMergeRows];
#pragma unroll
    for (int r = 0; r < kMergeRows; r++) {
        const int s = sg + 16 * r;
        rows[r] = (s < nsplit) ? *(const float4 *)(part_o + ((pid0 + s) * 16 + n) * D + d0)
                               : float4{0.f, 0.f, 0.f, 0.f};
    }
    const float gt_in = (tid < 64) ? gate[(size_t)h * D + blockIdx.y * 64 + tid] : 0.f;

    // every thread sees (max, sum) of up to 4 splits; nsplit <= kMaxSplits = 4 * 256
    float ms[4], ls[4];
    float m = neg_inf();
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int s = tid + 256 * r;
        ms[r] = (s < nsplit) ? part_ml[(pid0 + s) * 32 + n] : neg_inf();
        ls[r] = (s < nsplit) ? part_ml[(pid0 + s) * 32 + 16 + n] : 0.f;
        m = fmaxf(m, ms[r]);
    }
#pragma unroll
    for (int x = 1; x < 64; x <<= 1) m = fmaxf(m, __shfl_xor(m, x, 64));
    if (lane == 0) redf[wave] = m;
    __syncthreads();
    const float M = fmaxf(fmaxf(redf[0], redf[1]), fmaxf(redf[2], redf[3]));
    __syncthreads();
    float den = 0.f;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int s = tid + 256 * r;
        const float ws = (ms[r] == neg_inf()) ? 0.f : fast_exp2(ms[r] - M);
        if (s < nsplit) wsh[s] = ws;
        den += ws * ls[r];
    }
#pragma unroll
    for (int x = 1; x < 64; x <<= 1) den += __shfl_xor(den, x, 64);
    if (lane == 0) redf[wave] = den;
    __syncthreads();
    den = redf[0] + redf[1] + redf[2] + redf[3];

    float4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < kMergeRows; r++) {
        const int s = sg + 16 * r;
        const float w = (s < nsplit) ? wsh[s] : 0.f;
        acc.x += w * rows[r].x; acc.y += w * rows[r].y; acc.z += w * rows[r].z; acc.w += w * rows[r].w;
    }
    for (int s = sg + 16 * kMergeRows; s < nsplit; s += 16) {
        const float w = wsh[s];
        const float4 v = *(const float4 *)(part_o + ((pid0 + s) * 16 + n) * D + d0);
        acc.x += w * v.x; acc.y += w * v.y; acc.z += w * v.z; acc.w += w * v.w;
    }
    acc4[sg][dl] = acc;
    __syncthreads();
    if (tid < 64) {
        // thread -> one scalar output: float4 lane tid/4, component tid%4
        const int ql = tid >> 2, qc = tid & 3;
        float t = 0.f;
#pragma unroll
        for (int x = 0; x < 16; x++) t += ((const float *)&acc4[x][ql])[qc];
        const int d = blockIdx.y * 64 + tid;
        const float gt = 1.0f / (1.0f + expf(-gt_in));
        out[(size_t)h * D + d] = (t / den) * gt;
    }
}

// ---------------------------------------------------------------------------
// cache maintenance
// ---------------------------------------------------------------------------
template <typename KV, typename SRC> __device__ inline KV convert_kv(SRC x);
template <> __device__ inline float convert_kv<float, float>(float x) { return x; }
template <> __device__ inline uint16_t convert_kv<uint16_t, float>(float x) { return f32_to_bf16_bits(x); }
template <> __device__ inline uint16_t convert_kv<uint16_t, uint16_t>(uint16_t x) { return x; }
template <> __device__ inline float convert_kv<float, uint16_t>(uint16_t x) { return bf16_bits_to_f32(x); }

template <typename KV, typename SRC>
__global__ void kv_scatter_kernel(const SRC *__restrict__ k_rows, const SRC *__restrict__ v_rows,
                                  KV *__restrict__ k_tiled, KV *__restrict__ v_tiled,
                                  size_t plane_elems, int Hkv, int D, int64_t pos0,
                                  int64_t n_rows) {
    const int64_t kv_dim = (int64_t)Hkv * D;
    const int64_t total = n_rows * kv_dim;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / kv_dim;
        const int c = (int)(i % kv_dim);
        const int kvh = c / D, x = c % D;
        const int64_t pos = pos0 + r;
        k_tiled[(size_t)kvh * plane_elems + KvTile<KV>::k_off(pos, x, D)] = convert_kv<KV, SRC>(k_rows[i]);
        v_tiled[(size_t)kvh * plane_elems + KvTile<KV>::v_off(pos, x, D)] = convert_kv<KV, SRC>(v_rows[i]);
    }
}

template <typename KV>
__global__ void kv_gather_kernel(const KV *__restrict__ k_tiled, const KV *__restrict__ v_tiled,
                                 float *__restrict__ k_rows, float *__restrict__ v_rows,
                                 size_t plane_elems, int Hkv, int D, int64_t n_rows) {
    const int64_t kv_dim = (int64_t)Hkv * D;
    const int64_t total = n_rows * kv_dim;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / kv_dim;
        const int c = (int)(i % kv_dim);
        const int kvh = c / D, x = c % D;
        k_rows[i] = convert_kv<float, KV>(k_tiled[(size_t)kvh * plane_elems + KvTile<KV>::k_off(r, x, D)]);
        v_rows[i] = convert_kv<float, KV>(v_tiled[(size_t)kvh * plane_elems + KvTile<KV>::v_off(r, x, D)]);
    }
}

template <typename KV>
__global__ void kv_zero_kernel(KV *__restrict__ k_tiled, KV *__restrict__ v_tiled,
                               size_t plane_elems, int Hkv, int D, int64_t pos0, int64_t pos1) {
    const int64_t kv_dim = (int64_t)Hkv * D;
    const int64_t total = (pos1 - pos0) * kv_dim;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t pos = pos0 + i / kv_dim;
        const int c = (int)(i % kv_dim);
        const int kvh = c / D, x = c % D;
        k_tiled[(size_t)kvh * plane_elems + KvTile<KV>::k_off(pos, x, D)] = (KV)0;
        v_tiled[(size_t)kvh * plane_elems + KvTile<KV>::v_off(pos, x, D)] = (KV)0;
    }
}

static int grid_for(int64_t total, int block) {
    int64_t gsz = (total + block - 1) / block;
    if (gsz > 65536) gsz = 65536;
    if (gsz < 1) gsz = 1;
    return (int)gsz;
}

bool sdpa_shape_supported(int kv_dtype, int head_dim) {
    if (kv_dtype != MFA_KV_F32 && kv_dtype != MFA_KV_BF16) return false;
    return head_dim == 64 || head_dim == 128 || head_dim == 256;
}

static int blk_of(int kv_dtype) { return kv_dtype == MFA_KV_BF16 ? 32 : 16; }

// Partition of the cache's position blocks over workgroups.  Workgroups have 8 waves
// (one block in flight per wave) when that still leaves one workgroup per CU, else 4.
struct SplitPlan {
    int splits;
    int waves;
    int64_t bps;  // blocks per split
};

static SplitPlan plan_splits(int kv_dtype, int Hq, int Hkv, int64_t kv_len, int num_cus, int forced) {
    const int hpk = Hq / Hkv;
    const int nhg = (hpk + 15) / 16;
    const int64_t nblk = (kv_len + blk_of(kv_dtype) - 1) / blk_of(kv_dtype);
    int64_t target = forced > 0 ? forced : (num_cus / (Hkv * nhg));
    if (target < 1) target = 1;
    if (target > kMaxSplits) target = kMaxSplits;
    SplitPlan p;
    p.bps = (nblk + target - 1) / target;
    if (p.bps < 1) p.bps = 1;
    p.waves = p.bps >= 8 ? 8 : 4;
    if (forced <= 0 && p.bps < p.waves) p.bps = p.waves;  // at least one block per wave
    p.splits = (int)((nblk + p.bps - 1) / p.bps);
    if (p.splits < 1) p.splits = 1;
    return p;
}

int sdpa_pick_splits(int kv_dtype, int Hq, int Hkv, int D, int64_t kv_len, int num_cus, int forced) {
    (void)D;
    return plan_splits(kv_dtype, Hq, Hkv, kv_len, num_cus, forced).splits;
}

size_t sdpa_workspace_o_elems(int Hq, int Hkv, int D, int splits) {
    const int nhg = (Hq / Hkv + 15) / 16;
    return (size_t)Hkv * nhg * splits * 16 * D;
}
size_t sdpa_workspace_ml_elems(int Hq, int Hkv, int splits) {
    const int nhg = (Hq / Hkv + 15) / 16;
    return (size_t)Hkv * nhg * splits * 32;
}

template <typename KV, int D, int WAVES>
static int launch_partial(hipStream_t stream, dim3 grid, const void *k, const void *v,
                          size_t plane_elems, const float *q, int hpk, int64_t kv_len, int bps,
                          float qscale, float *po, float *pml) {
    constexpr size_t lds = PartialLds<KV, D, WAVES>::kBytes;
    static bool attr_set = false;  // more than 64 KiB of dynamic LDS has to be allowed once per kernel
    if (lds > 48 * 1024 && !attr_set) {
        MFA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&sdpa_partial_kernel<KV, D, WAVES>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set = true;
    }
    hipLaunchKernelGGL((sdpa_partial_kernel<KV, D, WAVES>), grid, dim3(WAVES * 64), lds, stream,
                       (const KV *)k, (const KV *)v, plane_elems, q, hpk, kv_len, bps, qscale, po,
                       pml);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

template <typename KV, int D>
static int launch_partial_w(int waves, hipStream_t stream, dim3 grid, const void *k, const void *v,
                            size_t plane_elems, const float *q, int hpk, int64_t kv_len, int bps,
                            float qscale, float *po, float *pml) {
    if (waves == 8)
        return launch_partial<KV, D, 8>(stream, grid, k, v, plane_elems, q, hpk, kv_len, bps, qscale, po, pml);
    return launch_partial<KV, D, 4>(stream, grid, k, v, plane_elems, q, hpk, kv_len, bps, qscale, po, pml);
}

int launch_sdpa_decode(hipStream_t stream, int kv_dtype, int Hq, int Hkv, int D, int64_t kv_len,
                       size_t plane_elems, const void *k_tiled, const void *v_tiled,
                       const float *q, const float *gate, float *out, const SdpaWorkspace &ws,
                       int num_cus, int forced_splits, int partial_only) {
    if (!sdpa_shape_supported(kv_dtype, D))
        return fail(MFA_ERR_SHAPE, "sdpa: head_dim %d / kv dtype %d not supported", D, kv_dtype);
    if (kv_len <= 0) return fail(MFA_ERR_INVALID, "sdpa: kv_len must be > 0 (got %lld)", (long long)kv_len);
    const int hpk = Hq / Hkv;
    const int nhg = (hpk + 15) / 16;
    SplitPlan plan = plan_splits(kv_dtype, Hq, Hkv, kv_len, num_cus, forced_splits);
    // never exceed the workspace
    while (plan.splits > 1 && (sdpa_workspace_o_elems(Hq, Hkv, D, plan.splits) > ws.part_o_elems ||
                               sdpa_workspace_ml_elems(Hq, Hkv, plan.splits) > ws.part_ml_elems))
        plan = plan_splits(kv_dtype, Hq, Hkv, kv_len, num_cus, (plan.splits + 1) / 2);
    if (sdpa_workspace_o_elems(Hq, Hkv, D, plan.splits) > ws.part_o_elems)
        return fail(MFA_ERR_INVALID, "sdpa: split-K workspace too small");
    // scores are produced in log2 units: q is pre-multiplied by (1/sqrt(D)) * log2(e)
    const float qscale = (1.0f / sqrtf((float)D)) * kLog2e;
    dim3 grid(plan.splits, nhg, Hkv);
    int rc;
#define MFA_LAUNCH(KV, DD)                                                                        \
    rc = launch_partial_w<KV, DD>(plan.waves, stream, grid, k_tiled, v_tiled, plane_elems, q, hpk, \
                                  kv_len, (int)plan.bps, qscale, ws.part_o, ws.part_ml)
    if (kv_dtype == MFA_KV_BF16) {
        if (D == 64) MFA_LAUNCH(uint16_t, 64);
        else if (D == 128) MFA_LAUNCH(uint16_t, 128);
        else MFA_LAUNCH(uint16_t, 256);
    } else {
        if (D == 64) MFA_LAUNCH(float, 64);
        else if (D == 128) MFA_LAUNCH(float, 128);
        else MFA_LAUNCH(float, 256);
    }
#undef MFA_LAUNCH
    MFA_TRY(rc);
    if (partial_only) return MFA_OK;
    hipLaunchKernelGGL(sdpa_merge_kernel, dim3(Hq, D / 64), dim3(256), 0, stream, ws.part_o,
                       ws.part_ml, plan.splits, hpk, nhg, D, gate, out);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_kv_scatter(hipStream_t stream, int kv_dtype, int src_is_bf16, int Hkv, int D,
                      size_t plane_elems, int64_t pos0, int64_t n_rows, const void *k_rows,
                      const void *v_rows, void *k_tiled, void *v_tiled) {
    if (n_rows <= 0) return MFA_OK;
    const int64_t total = n_rows * Hkv * D;
    const int grid = grid_for(total, 256);
    if (kv_dtype == MFA_KV_BF16 && src_is_bf16)
        hipLaunchKernelGGL((kv_scatter_kernel<uint16_t, uint16_t>), dim3(grid), dim3(256), 0, stream,
                           (const uint16_t *)k_rows, (const uint16_t *)v_rows, (uint16_t *)k_tiled,
                           (uint16_t *)v_tiled, plane_elems, Hkv, D, pos0, n_rows);
    else if (kv_dtype == MFA_KV_BF16)
        hipLaunchKernelGGL((kv_scatter_kernel<uint16_t, float>), dim3(grid), dim3(256), 0, stream,
                           (const float *)k_rows, (const float *)v_rows, (uint16_t *)k_tiled,
                           (uint16_t *)v_tiled, plane_elems, Hkv, D, pos0, n_rows);
    else if (src_is_bf16)
        hipLaunchKernelGGL((kv_scatter_kernel<float, uint16_t>), dim3(grid), dim3(256), 0, stream,
                           (const uint16_t *)k_rows, (const uint16_t *)v_rows, (float *)k_tiled,
                           (float *)v_tiled, plane_elems, Hkv, D, pos0, n_rows);
    else
        hipLaunchKernelGGL((kv_scatter_kernel<float, float>), dim3(grid), dim3(256), 0, stream,
                           (const float *)k_rows, (const float *)v_rows, (float *)k_tiled,
                           (float *)v_tiled, plane_elems, Hkv, D, pos0, n_rows);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_kv_gather(hipStream_t stream, int kv_dtype, int Hkv, int D, size_t plane_elems,
                     int64_t n_rows, const void *k_tiled, const void *v_tiled, float *k_rows,
                     float *v_rows) {
    if (n_rows <= 0) return MFA_OK;
    const int grid = grid_for(n_rows * Hkv * D, 256);
    if (kv_dtype == MFA_KV_BF16)
        hipLaunchKernelGGL((kv_gather_kernel<uint16_t>), dim3(grid), dim3(256), 0, stream,
                           (const uint16_t *)k_tiled, (const uint16_t *)v_tiled, k_rows, v_rows,
                           plane_elems, Hkv, D, n_rows);
    else
        hipLaunchKernelGGL((kv_gather_kernel<float>), dim3(grid), dim3(256), 0, stream,
                           (const float *)k_tiled, (const float *)v_tiled, k_rows, v_rows,
                           plane_elems, Hkv, D, n_rows);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_kv_zero(hipStream_t stream, int kv_dtype, int Hkv, int D, size_t plane_elems,
                   int64_t pos0, int64_t pos1, void *k_tiled, void *v_tiled) {
    if (pos1 <= pos0) return MFA_OK;
    const int grid = grid_for((pos1 - pos0) * Hkv * D, 256);
    if (kv_dtype == MFA_KV_BF16)
        hipLaunchKernelGGL((kv_zero_kernel<uint16_t>), dim3(grid), dim3(256), 0, stream,
                           (uint16_t *)k_tiled, (uint16_t *)v_tiled, plane_elems, Hkv, D, pos0, pos1);
    else
        hipLaunchKernelGGL((kv_zero_kernel<float>), dim3(grid), dim3(256), 0, stream,
                           (float *)k_tiled, (float *)v_tiled, plane_elems, Hkv, D, pos0, pos1);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
