// Attention over a compressed (latent) cache for gfx950: the folded form of multi-head
// latent attention, one query token.
//
// Per head h:  s[t] = (q'[h] . latent[t] + q_pe[h] . rope_k[t]) * scale,  w = softmax(s),
//              out[h] = sum_t w[t] latent[t].
// Every head reads the same keys ([latent | rope_k], R + P wide) and the same values
// (latent): the heads are the free dimension of both products, so they form the N side
// of MFMA tiles and the cache is read once per 16*HG heads instead of once per head.
//
// Both products run on the bf16 matrix pipeline at f32-like accuracy: every f32 operand x
// is split into bf16 parts hi = bf16(x), lo = bf16(x - hi)  (x = hi + lo to 2^-18 x), and a
// product a b is evaluated as a_hi b_hi + a_hi b_lo + a_lo b_hi with f32 accumulation.
//
//   mla_partial_kernel<R, P, HG>   grid (splits, ceil(H / 16 HG)); 2 HG waves: wave
//     (hg, half) serves 16 heads.  The workgroup walks its range of 32-position blocks.
//     All threads fetch a block into registers while the previous one is computed, split
//     it and store it to LDS twice:
//       krow[hi|lo][position][channel]            A operand of the scores (contraction over channels)
//       vt  [hi|lo][channel row][position slot]   A operand of the values (contraction over positions)
//     and the two waves of a head group share the work on it:
//       scores  S[pos][head] = sum_c X[pos][c] q[head][c]   each wave one half of the channels;
//               the halves are exchanged through LDS and added (so each wave keeps only
//               half of the queries in registers)
//       online softmax over the 32 positions, per head      (both waves, identically)
//       values  O[row][head] += sum_pos X[pos][row] P[pos][head]   each wave one half of the rows
//     The score tiles come out in the layout the second product wants for P: position
//     slot 8g + j of the block is position 4g + j (j < 4) or 16 + 4g + j - 4, which is the
//     order vt is stored in.  Channel c = 4 c4 + e of the latent lives in vt row
//     e * R/4 + c4, so that the staging threads (consecutive c4) write consecutive rows.
//     Partials (unnormalised O, running max and sum per head) go to the workspace in the
//     layout of the decode kernel's partials, and sdpa_merge_kernel combines them.
#include "sdpa_wave.h"

namespace mfa {

__device__ inline f32x4 mla_load4(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }
__device__ inline bf16x8 mla_lds8(const void *p) { return *reinterpret_cast<const bf16x8 *>(p); }

static constexpr int kMlaBlk = 32;    // positions per block
static constexpr int kMlaHG = 4;      // 16-head groups per workgroup
static constexpr float kMlaLazy = 8.f;

template <int R, int P, int HG>
__global__ __launch_bounds__(HG * 128) void mla_partial_kernel(
    const float *__restrict__ q_prime, const float *__restrict__ q_pe, const float *__restrict__ latent,
    const float *__restrict__ rope_k, int H, int L, int blocks_per_split, float qscale,
    float *__restrict__ part_o, float *__restrict__ part_ml) {
    constexpr int WAVES = 2 * HG;
    constexpr int NTHR = WAVES * 64;
    constexpr int DK = R + P;
    constexpr int KROW = DK + 8;          // krow row stride (bf16): 16 B of padding spread the rows over the banks
    constexpr int NS = DK / 32;           // 32-wide steps of the score contraction
    constexpr int NSH = NS / 2;           // per wave
    constexpr int NT = R / 16;            // output tiles (16 vt rows each)
    constexpr int NTH = NT / 2;           // per wave
    constexpr int NJOB = R / NTHR;        // latent jobs per thread: (4 channels) x (8 position slots)
    constexpr int NROPE = kMlaBlk * (P / 4) / NTHR;  // float4 of the rotary keys per thread
    static_assert(NS % 2 == 0 && NT % 2 == 0, "the two waves of a head group take equal halves");
    static_assert(R % NTHR == 0 && R % 32 == 0 && P % 32 == 0, "widths");
    static_assert((kMlaBlk * (P / 4)) % NTHR == 0, "rotary keys must divide over the threads");
    constexpr int KROW_BYTES = 2 * kMlaBlk * KROW * 2, VT_BYTES = 2 * R * (kMlaBlk / 8) * 16;
    constexpr int OS = R + 1;             // row stride of the output tile in LDS (floats): odd, so that a wave's
                                          // 16 heads x 4 row groups fall into 64 different banks
    static_assert(HG * 16 * OS * 4 <= KROW_BYTES + VT_BYTES, "the output tile reuses the block's LDS");
    __shared__ __attribute__((aligned(16))) unsigned char smem[KROW_BYTES + VT_BYTES];
    __shared__ f32x4 xch[WAVES][2][64];   // partial scores of a wave, for its partner
    uint16_t (*krow)[kMlaBlk][KROW] = reinterpret_cast<uint16_t (*)[kMlaBlk][KROW]>(smem);
    uint4 (*vt)[R][kMlaBlk / 8] = reinterpret_cast<uint4 (*)[R][kMlaBlk / 8]>(smem + KROW_BYTES);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int hgl = wave % HG, half = wave / HG;
    const int split = blockIdx.x, nsplit = gridDim.x;
    const int nhg = (H + 15) / 16;
    const int hg = blockIdx.y * HG + hgl;
    const bool active = hg < nhg;  // a wave past the last head group repeats the last head and stores nothing

    const int nblk = (L + kMlaBlk - 1) / kMlaBlk;
    const int b0 = split * blocks_per_split;
    const int b1 = min(b0 + blocks_per_split, nblk);
    const size_t pid = (size_t)hg * nsplit + split;
    if (b0 >= b1) {
        if (active && half == 0 && g == 0) {
            part_ml[pid * 32 + n] = neg_inf();
            part_ml[pid * 32 + 16 + n] = 0.f;
        }
        return;
    }

    // ---- staging.  Latent job: channels 4 c4 .. 4 c4 + 3 at the 8 positions of slot octet go ----
    const int go = tid & 3, c4lo = tid >> 2;
    f32x4 raw[NJOB][8];
    f32x4 rraw[NROPE];
    auto fetch =[&](int b) {
#pragma unroll
        for (int job = 0; job < NJOB; job++)
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
                const int pb = (jj < 4) ? 4 * go + jj : 16 + 4 * go + (jj - 4);
                const int pos = min(b * kMlaBlk + pb, L - 1);  // positions past the end repeat the last one; weight 0
                raw[job][jj] = mla_load4(latent + (size_t)pos * R + 4 * (c4lo + (NTHR / 4) * job));
            }
#pragma unroll
        for (int u = 0; u < NROPE; u++) {
            const int idx = tid + u * NTHR;
            const int pos = min(b * kMlaBlk + idx / (P / 4), L - 1);
            rraw[u] = mla_load4(rope_k + (size_t)pos * P + 4 * (idx % (P / 4)));
        }
    };
    auto commit =[&]() {
#pragma unroll
        for (int job = 0; job < NJOB; job++) {
            const int c4 = c4lo + (NTHR / 4) * job;
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {  // row-major copy: 4 channels of one position
                const int pb = (jj < 4) ? 4 * go + jj : 16 + 4 * go + (jj - 4);
                uint2 hi, lo;
                split_pair(raw[job][jj][0], raw[job][jj][1], hi.x, lo.x);
                split_pair(raw[job][jj][2], raw[job][jj][3], hi.y, lo.y);
                *reinterpret_cast<uint2 *>(&krow[0][pb][4 * c4]) = hi;
                *reinterpret_cast<uint2 *>(&krow[1][pb][4 * c4]) = lo;
            }
#pragma unroll
            for (int e = 0; e < 4; e++) {  // transposed copy: 8 position slots of one channel
                uint4 hi, lo;
                split_pair(raw[job][0][e], raw[job][1][e], hi.x, lo.x);
                split_pair(raw[job][2][e], raw[job][3][e], hi.y, lo.y);
                split_pair(raw[job][4][e], raw[job][5][e], hi.z, lo.z);
                split_pair(raw[job][6][e], raw[job][7][e], hi.w, lo.w);
                vt[0][e * (R / 4) + c4][go] = hi;
                vt[1][e * (R / 4) + c4][go] = lo;
            }
        }
#pragma unroll
        for (int u = 0; u < NROPE; u++) {
            const int idx = tid + u * NTHR;
            uint2 hi, lo;
            split_pair(rraw[u][0], rraw[u][1], hi.x, lo.x);
            split_pair(rraw[u][2], rraw[u][3], hi.y, lo.y);
            *reinterpret_cast<uint2 *>(&krow[0][idx / (P / 4)][R + 4 * (idx % (P / 4))]) = hi;
            *reinterpret_cast<uint2 *>(&krow[1][idx / (P / 4)][R + 4 * (idx % (P / 4))]) = lo;
        }
    };
    fetch(b0);

    // ---- this wave's half of its 16 queries as B operands: lane (n, g) holds head n,
    //      channels 32 (NSH half + s) + 8 g .. + 7 of [q' | q_pe]
    bf16x8 qh[NSH], ql[NSH];
    {
        const int head = min(hg * 16 + n, H - 1);
#pragma unroll
        for (int s = 0; s < NSH; s++) {
            const int c0 = 32 * (NSH * half + s) + 8 * g;
            const float *src = (c0 < R) ? q_prime + (size_t)head * R + c0 : q_pe + (size_t)head * P + (c0 - R);
            const f32x4 a = mla_load4(src) * qscale, b = mla_load4(src + 4) * qscale;
            uint4 hi, lo;
            split_pair(a[0], a[1], hi.x, lo.x);
            split_pair(a[2], a[3], hi.y, lo.y);
            split_pair(b[0], b[1], hi.z, lo.z);
            split_pair(b[2], b[3], hi.w, lo.w);
            qh[s] = as_bf16x8(hi);
            ql[s] = as_bf16x8(lo);
        }
    }
    f32x4 o[NTH];
#pragma unroll
    for (int t = 0; t < NTH; t++) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_ref = neg_inf(), l_sum = 0.f;
    const uint16_t *kr_hi = &krow[0][n][32 * NSH * half + 8 * g];
    const uint16_t *kr_lo = &krow[1][n][32 * NSH * half + 8 * g];

    for (int b = b0; b < b1; b++) {
        if (b > b0) __syncthreads();  // every wave is done with the previous block
        commit();
        fetch(min(b + 1, b1 - 1));
        __syncthreads();
        // scores over this wave's half of the channels: tile `sub` holds positions
        // 16 sub + 4g + i of the block, column = head n (log2 units)
        f32x4 sc[2];
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
            sc[sub] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < NSH; s++) {
                const bf16x8 ah = mla_lds8(kr_hi + 16 * sub * KROW + 32 * s);
                const bf16x8 al = mla_lds8(kr_lo + 16 * sub * KROW + 32 * s);
                sc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al, qh[s], sc[sub], 0, 0, 0);
                sc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, ql[s], sc[sub], 0, 0, 0);
                sc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, qh[s], sc[sub], 0, 0, 0);
            }
        }
        xch[wave][0][lane] = sc[0];
        xch[wave][1][lane] = sc[1];
        __syncthreads();
        const int partner = hgl + HG * (1 - half);
        sc[0] += xch[partner][0][lane];
        sc[1] += xch[partner][1][lane];
        const int pos0 = b * kMlaBlk + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (pos0 + i >= L) sc[0][i] = neg_inf();
            if (pos0 + 16 + i >= L) sc[1][i] = neg_inf();
        }
        float mb = fmaxf(fmaxf(fmaxf(sc[0][0], sc[0][1]), fmaxf(sc[0][2], sc[0][3])),
                         fmaxf(fmaxf(sc[1][0], sc[1][1]), fmaxf(sc[1][2], sc[1][3])));
        mb = fmaxf(mb, lane_xor(mb, 16));
        mb = fmaxf(mb, lane_xor(mb, 32));
        // Rescale what has been accumulated only when some head's maximum has moved far:
        // weights stay below 2^kMlaLazy, and the reference point cancels in the merge.
        if (__any(mb > m_ref + kMlaLazy)) {
            const float m_new = fmaxf(m_ref, mb);
            const float alpha = fast_exp2(m_ref - m_new);
            m_ref = m_new;
            l_sum *= alpha;
#pragma unroll
            for (int t = 0; t < NTH; t++) o[t] *= alpha;
        }
        float p[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            p[i] = fast_exp2(sc[0][i] - m_ref);
            p[4 + i] = fast_exp2(sc[1][i] - m_ref);
        }
        l_sum += ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
        uint4 phu, plu;
        split_pair(p[0], p[1], phu.x, plu.x);
        split_pair(p[2], p[3], phu.y, plu.y);
        split_pair(p[4], p[5], phu.z, plu.z);
        split_pair(p[6], p[7], phu.w, plu.w);
        const bf16x8 ph = as_bf16x8(phu), pl = as_bf16x8(plu);
        // values: O[row][head] += sum_slot vt[row][slot] p[slot][head], this wave's half of the rows
#pragma unroll
        for (int t = 0; t < NTH; t++) {
            const bf16x8 ah = as_bf16x8(vt[0][16 * (NTH * half + t) + n][g]);
            const bf16x8 al = as_bf16x8(vt[1][16 * (NTH * half + t) + n][g]);
            o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al, ph, o[t], 0, 0, 0);
            o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, pl, o[t], 0, 0, 0);
            o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, ph, o[t], 0, 0, 0);
        }
    }

    l_sum += lane_xor(l_sum, 16);
    l_sum += lane_xor(l_sum, 32);
    if (active && half == 0 && g == 0) {
        part_ml[pid * 32 + n] = m_ref;
        part_ml[pid * 32 + 16 + n] = l_sum;
    }
    // o[t][i] is vt row r = 16 (NTH half + t) + 4g + i of head n, i.e. channel 4 (r % (R/4)) + r / (R/4):
    // through LDS into [head][channel] order, then out in whole rows.
    __syncthreads();
    float *obuf = reinterpret_cast<float *>(smem);
#pragma unroll
    for (int t = 0; t < NTH; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int r = 16 * (NTH * half + t) + 4 * g + i;
            obuf[(hgl * 16 + n) * OS + 4 * (r % (R / 4)) + r / (R / 4)] = o[t][i];
        }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < HG * 16 * (R / 4) / NTHR; u++) {
        const int idx = tid + u * NTHR;
        const int row = idx / (R / 4), c4 = idx % (R / 4);
        const int rhg = blockIdx.y * HG + row / 16;
        if (rhg >= nhg) continue;
        const float *src = obuf + row * OS + 4 * c4;
        const f32x4 v = {src[0], src[1], src[2], src[3]};
        *reinterpret_cast<f32x4 *>(part_o + (((size_t)rhg * nsplit + split) * 16 + row % 16) * R + 4 * c4) = v;
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
    p.nwg_heads = (p.nhg + kMlaHG - 1) / kMlaHG;
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
    hipLaunchKernelGGL((mla_partial_kernel<512, 64, kMlaHG>), dim3(plan.splits, plan.nwg_heads), dim3(kMlaHG * 128), 0,
                       stream, q_prime, q_pe, latent, rope_k, H, L, plan.bps, qscale, ws.part_o, ws.part_ml);
    MFA_HIP(hipGetLastError());
    return launch_sdpa_merge(stream, ws, plan.splits, /*hpk=*/H, /*Hq=*/H, plan.nhg, R, /*n_tok=*/1,
                             /*gate=*/nullptr, out);
}

}  // namespace mfa
