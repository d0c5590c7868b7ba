// Attention over a compressed (latent) cache for gfx950: the folded form of multi-head
// latent attention, one query token.
//
// Per head h:  s[t] = (q'[h] . latent[t] + q_pe[h] . rope_k[t]) * scale,  w = softmax(s),
//              out[h] = sum_t w[t] latent[t].
// Every head reads the same keys ([latent | rope_k], R + P wide) and the same values
// (latent): the heads are the free dimension of both products, so they form the N side
// of f32 MFMA tiles and the cache is read H/64 times instead of H times.
//
//   mla_partial_kernel   grid (splits, ceil(H/64)); 4 waves, each owning 16 heads.  The
//     workgroup walks its range of 16-position blocks; the 256 threads stage a block
//     (16 rows of R + P floats) global -> registers -> LDS, double buffered, one barrier
//     per block, and every wave then runs both products from that one copy:
//       scores  S[pos][head] = sum_c X[pos][c] q[head][c]      (R+P)/4 instructions
//       online softmax over the positions, per head
//       values  O[c][head]  += sum_pos X[pos][c] P[pos][head]   R/4 instructions
//     The score tile comes out in the layout the second product wants for P.
//     Partials (unnormalised O, running max and sum per head) go to the workspace in the
//     layout of the decode kernel's partials, and sdpa_merge_kernel combines them.
//
// The arithmetic is f32 throughout (v_mfma_f32_16x16x4_f32), so the result matches a
// scalar f32 evaluation to rounding-order differences.
#include "mfa_internal.h"

namespace mfa {

typedef float mla_f32x4 __attribute__((ext_vector_type(4)));

__device__ inline mla_f32x4 mla_mfma4(mla_f32x4 a, mla_f32x4 b, mla_f32x4 acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], acc, 0, 0, 0);
    return acc;
}

__device__ inline mla_f32x4 mla_load4(const float *p) { return *reinterpret_cast<const mla_f32x4 *>(p); }

__device__ inline float mla_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

static constexpr int kMlaBlk = 16;    // positions per block
static constexpr int kMlaWaves = 4;   // waves per workgroup = 16-head groups per workgroup

template <int R, int P>
__global__ __launch_bounds__(kMlaWaves * 64) void mla_partial_kernel(
    const float *__restrict__ q_prime, const float *__restrict__ q_pe, const float *__restrict__ latent,
    const float *__restrict__ rope_k, int H, int L, int blocks_per_split, float qscale,
    float *__restrict__ part_o, float *__restrict__ part_ml) {
    constexpr int DK = R + P;
    constexpr int LD = DK + 4;          // row stride in LDS: 4 floats of padding spread the rows over the banks
    constexpr int NS = DK / 16;         // 16-wide steps of the score contraction
    constexpr int NSR = R / 16;         // of which the latent part
    constexpr int NT = R / 16;          // output tiles (16 channels each)
    constexpr int F4_ROW = DK / 4;      // float4 per staged row
    constexpr int NLD = kMlaBlk * F4_ROW / (kMlaWaves * 64);  // float4 per thread per block
    static_assert(R % 16 == 0 && P % 16 == 0, "widths must be multiples of 16");
    static_assert((kMlaBlk * F4_ROW) % (kMlaWaves * 64) == 0, "a block must divide over the threads");
    __shared__ float blk[2][kMlaBlk][LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int split = blockIdx.x, nsplit = gridDim.x;
    const int nhg = (H + 15) / 16;
    const int hg = blockIdx.y * kMlaWaves + wave;
    const bool active = hg < nhg;  // a wave past the last head group only helps with the staging

    const int nblk = (L + kMlaBlk - 1) / kMlaBlk;
    const int b0 = split * blocks_per_split;
    const int b1 = min(b0 + blocks_per_split, nblk);
    const size_t pid = (size_t)hg * nsplit + split;
    if (b0 >= b1) {
        if (active && g == 0) {
            part_ml[pid * 32 + n] = -__builtin_huge_valf();
            part_ml[pid * 32 + 16 + n] = 0.f;
        }
        return;
    }

    // ---- staging: thread -> NLD float4 of the block, row-major over [latent | rope_k] ----
    mla_f32x4 stage[NLD];
    auto fetch =[&](int b) {
#pragma unroll
        for (int u = 0; u < NLD; u++) {
            const int idx = tid + u * kMlaWaves * 64;
            const int row = idx / F4_ROW, c4 = idx % F4_ROW;
            const int pos = min(b * kMlaBlk + row, L - 1);  // rows past the end repeat the last one; their weight is 0
            const float *src = (c4 < R / 4) ? latent + (size_t)pos * R + 4 * c4
                                            : rope_k + (size_t)pos * P + 4 * (c4 - R / 4);
            stage[u] = mla_load4(src);
        }
    };
    auto commit =[&](int buf) {
#pragma unroll
        for (int u = 0; u < NLD; u++) {
            const int idx = tid + u * kMlaWaves * 64;
            const int row = idx / F4_ROW, c4 = idx % F4_ROW;
            *reinterpret_cast<mla_f32x4 *>(&blk[buf][row][4 * c4]) = stage[u];
        }
    };
    fetch(b0);

    // ---- this wave's 16 queries as B operands: lane (n, g) holds head n, columns 16s + 4g .. +3 ----
    mla_f32x4 qreg[NS];
    {
        const int head = min(hg * 16 + n, H - 1);
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const float *src = (s < NSR) ? q_prime + (size_t)head * R + 16 * s + 4 * g
                                         : q_pe + (size_t)head * P + 16 * (s - NSR) + 4 * g;
            qreg[s] = mla_load4(src) * qscale;
        }
    }
    mla_f32x4 o[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) o[t] = mla_f32x4{0.f, 0.f, 0.f, 0.f};
    float m_ref = -__builtin_huge_valf(), l_sum = 0.f;

    commit(0);
    __syncthreads();

    for (int b = b0; b < b1; b++) {
        const int buf = (b - b0) & 1;
        fetch(min(b + 1, b1 - 1));
        if (active) {
            // scores: rows = positions 4g + i of the block, column = head n (log2 units)
            mla_f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NS; s++) sc = mla_mfma4(mla_load4(&blk[buf][n][16 * s + 4 * g]), qreg[s], sc);
            const int pos0 = b * kMlaBlk + 4 * g;
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (pos0 + i >= L) sc[i] = -__builtin_huge_valf();
            float mb = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
            mb = fmaxf(mb, __shfl_xor(mb, 16, 64));
            mb = fmaxf(mb, __shfl_xor(mb, 32, 64));
            if (__any(mb > m_ref)) {  // some head's maximum moved: rescale what has been accumulated
                const float m_new = fmaxf(m_ref, mb);
                const float alpha = mla_exp2(m_ref - m_new);
                m_ref = m_new;
                l_sum *= alpha;
#pragma unroll
                for (int t = 0; t < NT; t++) o[t] *= alpha;
            }
            mla_f32x4 p;
#pragma unroll
            for (int i = 0; i < 4; i++) p[i] = mla_exp2(sc[i] - m_ref);
            l_sum += (p[0] + p[1]) + (p[2] + p[3]);
            // values: O[c][head] += sum_pos X[pos][c] p[pos][head]; lane (m, g) supplies X[4g + i][16t + m]
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const mla_f32x4 a = {blk[buf][4 * g + 0][16 * t + n], blk[buf][4 * g + 1][16 * t + n],
                                     blk[buf][4 * g + 2][16 * t + n], blk[buf][4 * g + 3][16 * t + n]};
                o[t] = mla_mfma4(a, p, o[t]);
            }
        }
        commit(buf ^ 1);
        __syncthreads();
    }

    if (!active) return;
    l_sum += __shfl_xor(l_sum, 16, 64);
    l_sum += __shfl_xor(l_sum, 32, 64);
    // o[t][i] is channel 16t + 4g + i of head n
    float *po = part_o + (pid * 16 + n) * R + 4 * g;
#pragma unroll
    for (int t = 0; t < NT; t++) *reinterpret_cast<mla_f32x4 *>(po + 16 * t) = o[t];
    if (g == 0) {
        part_ml[pid * 32 + n] = m_ref;
        part_ml[pid * 32 + 16 + n] = l_sum;
    }
}

bool mla_shape_supported(int kv_lora_rank, int qk_rope_head_dim) {
    return kv_lora_rank == 512 && qk_rope_head_dim == 64;
}

// Partition of the cache's blocks over workgroups: enough splits that every CU has a
// workgroup, never more than there are blocks.
MlaPlan mla_plan(int H, int L, int num_cus) {
    MlaPlan p;
    p.nhg = (H + 15) / 16;
    p.nwg_heads = (p.nhg + kMlaWaves - 1) / kMlaWaves;
    const int nblk = (L + kMlaBlk - 1) / kMlaBlk;
    int splits = (num_cus + p.nwg_heads - 1) / p.nwg_heads;
    if (splits > nblk) splits = nblk;
    if (splits > 1024) splits = 1024;
    if (splits < 1) splits = 1;
    p.bps = (nblk + splits - 1) / splits;
    p.splits = (nblk + p.bps - 1) / p.bps;
    return p;
}

size_t mla_workspace_o_elems(const MlaPlan &p, int R) { return (size_t)p.nhg * p.splits * 16 * R; }
size_t mla_workspace_ml_elems(const MlaPlan &p) { return (size_t)p.nhg * p.splits * 32; }

int launch_mla_sdpa_folded(hipStream_t stream, int H, int R, int P, int L, float softmax_scale,
                           const float *q_prime, const float *q_pe, const float *latent, const float *rope_k,
                           float *out, const SdpaWorkspace &ws, const MlaPlan &plan) {
    if (!mla_shape_supported(R, P))
        return fail(MFA_ERR_SHAPE, "latent attention: kv_lora_rank %d / qk_rope_head_dim %d not built (512 / 64)", R, P);
    if (H <= 0 || L <= 0) return fail(MFA_ERR_INVALID, "latent attention: num_heads %d, cache_len %d", H, L);
    if (ws.part_o_elems < mla_workspace_o_elems(plan, R) || ws.part_ml_elems < mla_workspace_ml_elems(plan))
        return fail(MFA_ERR_INVALID, "latent attention: workspace too small for %d splits", plan.splits);
    const float qscale = softmax_scale * 1.4426950408889634f;  // scores in log2 units
    hipLaunchKernelGGL((mla_partial_kernel<512, 64>), dim3(plan.splits, plan.nwg_heads), dim3(kMlaWaves * 64), 0,
                       stream, q_prime, q_pe, latent, rope_k, H, L, plan.bps, qscale, ws.part_o, ws.part_ml);
    MFA_HIP(hipGetLastError());
    return launch_sdpa_merge(stream, ws, plan.splits, /*hpk=*/H, /*Hq=*/H, plan.nhg, R, /*n_tok=*/1,
                             /*gate=*/nullptr, out);
}

}  // namespace mfa
