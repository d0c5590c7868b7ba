// Split-K flash-decode GQA attention with the sigmoid output gate, for gfx950.
//
// Replaces the reference's four-kernel chain attn_scores_batched /
// attn_softmax_batched / attn_values_batched / sigmoid_gate
// (crates/moeflux/shaders/shaders.metal:976-1134, encoded at
// crates/moeflux/src/riir/linear_attn_forward.rs:850-902) and its CPU fallback
// sdpa_cpu (crates/moeflux/src/riir/sdpa.rs:63-172) with two launches:
//
//   sdpa_partial_kernel  grid (splits, head groups, kv heads), 4 waves each.
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
//     v_mfma_f32_16x16x4_f32.  The four waves are merged through LDS and one
//     (max, sum, O[16, D]) partial per workgroup is written.
//   sdpa_merge_kernel    log-sum-exp merge of the partials, normalisation and
//     the sigmoid gate.
#include "mfa_internal.h"

namespace mfa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

static constexpr int kWaves = 4;
static constexpr int kMaxSplits = 1024;

__device__ inline float neg_inf() { return -__builtin_huge_valf(); }

__device__ inline float lane_xor(float v, int mask) { return __shfl_xor(v, mask, 64); }

// x -> (hi, lo) with hi = bf16(x), lo = bf16(x - hi); x - hi is exact in f32.
__device__ inline void split_bf16(float x, uint16_t &hi, uint16_t &lo) {
    hi = f32_to_bf16_bits(x);
    lo = f32_to_bf16_bits(x - bf16_bits_to_f32(hi));
}

union Pack8 {
    uint16_t h[8];
    uint4 u;
    bf16x8 v;
};

template <typename KV, int D> struct Wave;

// ---------------------------------------------------------------------------
// bf16 cache
// ---------------------------------------------------------------------------
template <int D> struct Wave<uint16_t, D> {
    static constexpr int BLK = 32;
    static constexpr int KSTEPS = D / 32;  // MFMA steps per 16-position sub-tile
    static constexpr int NACC = D / 16;

    bf16x8 qhi[KSTEPS], qlo[KSTEPS];

    __device__ void load_q(const float *qrow, bool ok, int g) {
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            Pack8 hi, lo;
            float x[8];
            if (ok) {
                const float4 a = *(const float4 *)(qrow + 8 * (4 * s + g));
                const float4 b = *(const float4 *)(qrow + 8 * (4 * s + g) + 4);
                x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
                x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) x[e] = 0.f;
            }
#pragma unroll
            for (int e = 0; e < 8; e++) split_bf16(x[e], hi.h[e], lo.h[e]);
            qhi[s] = hi.v;
            qlo[s] = lo.v;
        }
    }

    struct Tile {
        uint4 k[2][KSTEPS];
        uint4 v[NACC];
    };

    __device__ static void load_tile(Tile &t, const uint16_t *kplane, const uint16_t *vplane,
                                     int64_t blk, int lane) {
        const uint4 *kb = (const uint4 *)(kplane + blk * (int64_t)(BLK * D)) + lane;
        const uint4 *vb = (const uint4 *)(vplane + blk * (int64_t)(BLK * D)) + lane;
#pragma unroll
        for (int sub = 0; sub < 2; sub++)
#pragma unroll
            for (int s = 0; s < KSTEPS; s++) t.k[sub][s] = kb[(sub * KSTEPS + s) * 64];
#pragma unroll
        for (int dt = 0; dt < NACC; dt++) t.v[dt] = vb[dt * 64];
    }

    // One block of 32 positions.  lane = 16*g + n, n = head within the group.
    __device__ void step(const Tile &t, int64_t blk, int64_t kv_len, float scale, int g,
                         float &m_run, float &l_run, f32x4 (&o)[NACC]) {
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            Pack8 a0, a1;
            a0.u = t.k[0][s];
            a1.u = t.k[1][s];
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0.v, qhi[s], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1.v, qhi[s], s1, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0.v, qlo[s], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1.v, qlo[s], s1, 0, 0, 0);
        }
        // Row 4g+i of sub-tile `sub` is position blk*32 + 16*sub + 4g + i.
        float sc[8];
        const int64_t base = blk * BLK + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            sc[i] = (base + i < kv_len) ? s0[i] * scale : neg_inf();
            sc[4 + i] = (base + 16 + i < kv_len) ? s1[i] * scale : neg_inf();
        }
        float tmax = sc[0];
#pragma unroll
        for (int e = 1; e < 8; e++) tmax = fmaxf(tmax, sc[e]);
        tmax = fmaxf(tmax, lane_xor(tmax, 16));
        tmax = fmaxf(tmax, lane_xor(tmax, 32));
        const float m_new = fmaxf(m_run, tmax);  // finite: position blk*32 is always valid
        const float alpha = expf(m_run - m_new);
        Pack8 phi, plo;
        float psum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float p = expf(sc[e] - m_new);
            psum += p;
            split_bf16(p, phi.h[e], plo.h[e]);
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int dt = 0; dt < NACC; dt++) {
            Pack8 a;
            a.u = t.v[dt];
            f32x4 acc = o[dt];
            acc[0] *= alpha; acc[1] *= alpha; acc[2] *= alpha; acc[3] *= alpha;
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, phi.v, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, plo.v, acc, 0, 0, 0);
            o[dt] = acc;
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
// f32 cache
// ---------------------------------------------------------------------------
template <int D> struct Wave<float, D> {
    static constexpr int BLK = 16;
    static constexpr int KSTEPS = D / 16;  // 16-byte chunks per lane per block
    static constexpr int NC = D / 64;
    static constexpr int NACC = D / 16;    // = NC * 4

    float4 qv[KSTEPS];

    __device__ void load_q(const float *qrow, bool ok, int g) {
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            float4 z = {0.f, 0.f, 0.f, 0.f};
            qv[s] = ok ? *(const float4 *)(qrow + 4 * (4 * s + g)) : z;
        }
    }

    struct Tile {
        float4 k[KSTEPS];
        float4 v[4][NC];
    };

    __device__ static void load_tile(Tile &t, const float *kplane, const float *vplane,
                                     int64_t blk, int lane) {
        const float4 *kb = (const float4 *)(kplane + blk * (int64_t)(BLK * D)) + lane;
        const float4 *vb = (const float4 *)(vplane + blk * (int64_t)(BLK * D)) + lane;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) t.k[s] = kb[s * 64];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int c = 0; c < NC; c++) t.v[i][c] = vb[(i * NC + c) * 64];
    }

    __device__ void step(const Tile &t, int64_t blk, int64_t kv_len, float scale, int g,
                         float &m_run, float &l_run, f32x4 (&o)[NACC]) {
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(t.k[s].x, qv[s].x, s0, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(t.k[s].y, qv[s].y, s0, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(t.k[s].z, qv[s].z, s0, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(t.k[s].w, qv[s].w, s0, 0, 0, 0);
        }
        float sc[4];
        const int64_t base = blk * BLK + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) sc[i] = (base + i < kv_len) ? s0[i] * scale : neg_inf();
        float tmax = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        tmax = fmaxf(tmax, lane_xor(tmax, 16));
        tmax = fmaxf(tmax, lane_xor(tmax, 32));
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = expf(m_run - m_new);
        float p[4];
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            p[i] = expf(sc[i] - m_new);
            psum += p[i];
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int a = 0; a < NACC; a++) {
            o[a][0] *= alpha; o[a][1] *= alpha; o[a][2] *= alpha; o[a][3] *= alpha;
        }
        // accumulator 4c+j collects d = 64c + 4m + j; MFMA set i contracts positions 4g+i.
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int c = 0; c < NC; c++) {
                o[4 * c + 0] = __builtin_amdgcn_mfma_f32_16x16x4f32(t.v[i][c].x, p[i], o[4 * c + 0], 0, 0, 0);
                o[4 * c + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(t.v[i][c].y, p[i], o[4 * c + 1], 0, 0, 0);
                o[4 * c + 2] = __builtin_amdgcn_mfma_f32_16x16x4f32(t.v[i][c].z, p[i], o[4 * c + 2], 0, 0, 0);
                o[4 * c + 3] = __builtin_amdgcn_mfma_f32_16x16x4f32(t.v[i][c].w, p[i], o[4 * c + 3], 0, 0, 0);
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

// part_o:  [kv head][head group][split][16 heads][D]
// part_ml: [kv head][head group][split][2][16]   (max, then sum)
template <typename KV, int D>
__global__ __launch_bounds__(kWaves * 64) void sdpa_partial_kernel(
    const KV *__restrict__ k_tiled, const KV *__restrict__ v_tiled, size_t plane_elems,
    const float *__restrict__ q, int hpk, int64_t kv_len, int blocks_per_split, float scale,
    float *__restrict__ part_o, float *__restrict__ part_ml) {
    using W = Wave<KV, D>;
    constexpr int NACC = W::NACC;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int split = blockIdx.x, hg = blockIdx.y, kvh = blockIdx.z;
    const int nsplit = gridDim.x, nhg = gridDim.y;

    const int head_in_kv = hg * 16 + n;
    const bool head_ok = head_in_kv < hpk;
    W w;
    w.load_q(q + (int64_t)(kvh * hpk + (head_ok ? head_in_kv : 0)) * D, head_ok, g);

    const KV *kplane = k_tiled + (size_t)kvh * plane_elems;
    const KV *vplane = v_tiled + (size_t)kvh * plane_elems;
    const int64_t nblk = (kv_len + W::BLK - 1) / W::BLK;
    const int64_t b0 = (int64_t)split * blocks_per_split;
    int64_t b1 = b0 + blocks_per_split;
    if (b1 > nblk) b1 = nblk;

    f32x4 o[NACC];
#pragma unroll
    for (int a = 0; a < NACC; a++) o[a] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = neg_inf(), l_run = 0.f;

    // Two tiles in flight: the loads of block b+4 are issued before block b is consumed.
    typename W::Tile t0, t1;
    int64_t b = b0 + wave;
    if (b < b1) W::load_tile(t0, kplane, vplane, b, lane);
    while (b < b1) {
        const int64_t bn = b + kWaves;
        if (bn < b1) W::load_tile(t1, kplane, vplane, bn, lane);
        w.step(t0, b, kv_len, scale, g, m_run, l_run, o);
        if (bn >= b1) break;
        const int64_t bnn = bn + kWaves;
        if (bnn < b1) W::load_tile(t0, kplane, vplane, bnn, lane);
        w.step(t1, bn, kv_len, scale, g, m_run, l_run, o);
        b = bnn;
    }
    l_run += lane_xor(l_run, 16);
    l_run += lane_xor(l_run, 32);

    // ---- merge the four waves ------------------------------------------------
    __shared__ float sm[kWaves][16];
    __shared__ float sl[kWaves][16];
    __shared__ f32x4 red[2][NACC][64];
    if (g == 0) sm[wave][n] = m_run;
    __syncthreads();
    float M = sm[0][n];
#pragma unroll
    for (int x = 1; x < kWaves; x++) M = fmaxf(M, sm[x][n]);
    const float f = (m_run == neg_inf()) ? 0.f : expf(m_run - M);
    l_run *= f;
#pragma unroll
    for (int a = 0; a < NACC; a++) {
        o[a][0] *= f; o[a][1] *= f; o[a][2] *= f; o[a][3] *= f;
    }
    if (g == 0) sl[wave][n] = l_run;
    if (wave >= 2) {
#pragma unroll
        for (int a = 0; a < NACC; a++) red[wave - 2][a][lane] = o[a];
    }
    __syncthreads();
    if (wave < 2) {
#pragma unroll
        for (int a = 0; a < NACC; a++) {
            const f32x4 r = red[wave][a][lane];
            o[a][0] += r[0]; o[a][1] += r[1]; o[a][2] += r[2]; o[a][3] += r[3];
        }
    }
    __syncthreads();
    if (wave == 1) {
#pragma unroll
        for (int a = 0; a < NACC; a++) red[0][a][lane] = o[a];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int a = 0; a < NACC; a++) {
            const f32x4 r = red[0][a][lane];
            o[a][0] += r[0]; o[a][1] += r[1]; o[a][2] += r[2]; o[a][3] += r[3];
        }
        const size_t pid = ((size_t)kvh * nhg + hg) * nsplit + split;
        W::store_o(part_o + (pid * 16 + n) * D, g, o);
        if (g == 0) {
            part_ml[pid * 32 + n] = M;
            part_ml[pid * 32 + 16 + n] = sl[0][n] + sl[1][n] + sl[2][n] + sl[3][n];
        }
    }
}

// grid (Hq, D/32), 256 threads: 32 output elements x 8 split lanes.
__global__ __launch_bounds__(256) void sdpa_merge_kernel(
    const float *__restrict__ part_o, const float *__restrict__ part_ml, int nsplit, int hpk,
    int nhg, int D, const float *__restrict__ gate, float *__restrict__ out) {
    __shared__ float wsh[kMaxSplits];
    __shared__ float redf[256];
    const int h = blockIdx.x;
    const int kvh = h / hpk, hin = h % hpk, hg = hin / 16, n = hin % 16;
    const size_t pid0 = ((size_t)kvh * nhg + hg) * nsplit;
    const int tid = threadIdx.x;

    float m = neg_inf();
    for (int s = tid; s < nsplit; s += 256) m = fmaxf(m, part_ml[(pid0 + s) * 32 + n]);
    redf[tid] = m;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if (tid < w) redf[tid] = fmaxf(redf[tid], redf[tid + w]);
        __syncthreads();
    }
    const float M = redf[0];
    __syncthreads();
    float den = 0.f;
    for (int s = tid; s < nsplit; s += 256) {
        const float ms = part_ml[(pid0 + s) * 32 + n];
        const float ws = (ms == neg_inf()) ? 0.f : expf(ms - M);
        wsh[s] = ws;
        den += ws * part_ml[(pid0 + s) * 32 + 16 + n];
    }
    redf[tid] = den;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if (tid < w) redf[tid] += redf[tid + w];
        __syncthreads();
    }
    den = redf[0];
    __syncthreads();

    const int dl = tid & 31, sl = tid >> 5;
    const int d = blockIdx.y * 32 + dl;
    float acc = 0.f;
    for (int s = sl; s < nsplit; s += 8)
        acc += wsh[s] * part_o[((pid0 + s) * 16 + n) * D + d];
    redf[tid] = acc;
    __syncthreads();
    if (sl == 0) {
        float t = 0.f;
#pragma unroll
        for (int x = 0; x < 8; x++) t += redf[x * 32 + dl];
        const float gt = 1.0f / (1.0f + expf(-gate[(size_t)h * D + d]));
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

// Returns blocks-per-split through *bps.
int sdpa_pick_splits(int kv_dtype, int Hq, int Hkv, int D, int64_t kv_len, int num_cus, int forced) {
    (void)D;
    const int hpk = Hq / Hkv;
    const int nhg = (hpk + 15) / 16;
    const int64_t nblk = (kv_len + blk_of(kv_dtype) - 1) / blk_of(kv_dtype);
    int64_t target = forced > 0 ? forced : (num_cus / (Hkv * nhg));
    if (target < 1) target = 1;
    if (target > kMaxSplits) target = kMaxSplits;
    int64_t bps = (nblk + target - 1) / target;
    if (forced <= 0 && bps < kWaves) bps = kWaves;  // at least one block per wave
    if (bps < 1) bps = 1;
    int64_t ns = (nblk + bps - 1) / bps;
    if (ns < 1) ns = 1;
    return (int)ns;
}

static int64_t bps_for(int kv_dtype, int64_t kv_len, int splits) {
    const int64_t nblk = (kv_len + blk_of(kv_dtype) - 1) / blk_of(kv_dtype);
    int64_t bps = (nblk + splits - 1) / splits;
    return bps < 1 ? 1 : bps;
}

size_t sdpa_workspace_o_elems(int Hq, int Hkv, int D, int splits) {
    const int nhg = (Hq / Hkv + 15) / 16;
    return (size_t)Hkv * nhg * splits * 16 * D;
}
size_t sdpa_workspace_ml_elems(int Hq, int Hkv, int splits) {
    const int nhg = (Hq / Hkv + 15) / 16;
    return (size_t)Hkv * nhg * splits * 32;
}

template <typename KV, int D>
static void launch_partial(hipStream_t stream, dim3 grid, const void *k, const void *v,
                           size_t plane_elems, const float *q, int hpk, int64_t kv_len, int bps,
                           float scale, float *po, float *pml) {
    hipLaunchKernelGGL((sdpa_partial_kernel<KV, D>), grid, dim3(kWaves * 64), 0, stream,
                       (const KV *)k, (const KV *)v, plane_elems, q, hpk, kv_len, bps, scale, po,
                       pml);
}

int launch_sdpa_decode(hipStream_t stream, int kv_dtype, int Hq, int Hkv, int D, int64_t kv_len,
                       size_t plane_elems, const void *k_tiled, const void *v_tiled,
                       const float *q, const float *gate, float *out, const SdpaWorkspace &ws,
                       int num_cus, int forced_splits) {
    if (!sdpa_shape_supported(kv_dtype, D))
        return fail(MFA_ERR_SHAPE, "sdpa: head_dim %d / kv dtype %d not supported", D, kv_dtype);
    if (kv_len <= 0) return fail(MFA_ERR_INVALID, "sdpa: kv_len must be > 0 (got %lld)", (long long)kv_len);
    const int hpk = Hq / Hkv;
    const int nhg = (hpk + 15) / 16;
    int splits = sdpa_pick_splits(kv_dtype, Hq, Hkv, D, kv_len, num_cus, forced_splits);
    // never exceed the workspace
    while (splits > 1 && (sdpa_workspace_o_elems(Hq, Hkv, D, splits) > ws.part_o_elems ||
                          sdpa_workspace_ml_elems(Hq, Hkv, splits) > ws.part_ml_elems))
        splits = (splits + 1) / 2;
    if (sdpa_workspace_o_elems(Hq, Hkv, D, splits) > ws.part_o_elems)
        return fail(MFA_ERR_INVALID, "sdpa: split-K workspace too small");
    const int64_t bps = bps_for(kv_dtype, kv_len, splits);
    const int64_t nblk = (kv_len + blk_of(kv_dtype) - 1) / blk_of(kv_dtype);
    splits = (int)((nblk + bps - 1) / bps);
    const float scale = 1.0f / sqrtf((float)D);
    dim3 grid(splits, nhg, Hkv);
#define MFA_LAUNCH(KV, DD)                                                                      \
    launch_partial<KV, DD>(stream, grid, k_tiled, v_tiled, plane_elems, q, hpk, kv_len, (int)bps, \
                           scale, ws.part_o, ws.part_ml)
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
    MFA_HIP(hipGetLastError());
    hipLaunchKernelGGL(sdpa_merge_kernel, dim3(Hq, D / 32), dim3(256), 0, stream, ws.part_o,
                       ws.part_ml, splits, hpk, nhg, D, gate, out);
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
