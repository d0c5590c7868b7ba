// Attention over a compressed (latent) cache for gfx950: the folded form of multi-head
// latent attention, one query token.
//
// Per head h:  s[t] = (q'[h] . latent[t] + q_pe[h] . rope_k[t]) * scale,  w = softmax(s),
//              out[h] = sum_t w[t] latent[t].
// Every head reads the same keys ([latent | rope_k], R + P wide) and the same values
// (latent): the heads are the free dimension of both products, so they form the N side
// of MFMA tiles and the cache is read once per 64 heads instead of once per head.
//
// Both products run on the bf16 matrix pipeline at f32-like accuracy: every f32 operand x
// is split into bf16 parts hi = bf16(x), lo = bf16(x - hi)  (x = hi + lo to 2^-18 x), and a
// product a b is evaluated as a_hi b_hi + a_hi b_lo + a_lo b_hi with f32 accumulation.
//
//   mla_partial_kernel<R, P>   grid (splits, ceil(H / 64)); 8 waves in two roles.  Wave hg
//     (0..3) computes the scores and the softmax of head group hg, wave 4 + hg accumulates
//     that group's values; the two share a SIMD and run one block apart, so that one of
//     them always has matrix work while the other converts, exponentiates or stores:
//       iteration it:   score waves   S(it + 1): 16 positions x 16 heads over R + P channels,
//                                     online softmax, weights to LDS as bf16 hi/lo operands
//                       value waves   V(it):  O[channel][head] += X[slot][channel] P[slot][head]
//       and both stage block it + 2 (one barrier per iteration).
//     A block of 16 positions lives in LDS once, split but not transposed:
//       krow[hi|lo][position][channel], three buffers (scored, accumulated, being written);
//     rows are 1184 bytes apart, the stride at which both kinds of read below run without
//     bank conflicts.  The scores read it as an A operand directly (a lane's 8 channels of
//     one position are contiguous).  The values need 8 positions of one channel per lane:
//     ds_read_b64_tr_b16 delivers exactly that from the row-major block (within 16 lanes,
//     lane j receives element j % 4 of the 8 bytes addressed by lanes j/4, j/4 + 4, j/4 + 8,
//     j/4 + 12; with lane L pointing at position L/4, channels 4 (L % 4) .. + 3, lane j
//     ends up with channel j at four positions).  The value product's 32 slots are the hi
//     parts of the 16 positions followed by their lo parts, so that with P = [p_hi | p_hi]
//     one instruction adds x_hi p_hi + x_lo p_hi and a second with [p_lo | p_lo] adds x_hi p_lo
//     (and x_lo p_lo, which comes for free).
//     The value waves fetch and split 6 of a block's 16 latent rows (two channels per
//     thread), the score waves the other 10 and the rotary keys: the split at which the call is
//     fastest (12 / 4, which evens out the clocks the two roles spend per block, is 4 % slower).
//     Partials (unnormalised O, running max and sum per head) go to the workspace in the
//     layout of the decode kernel's partials, and sdpa_merge_kernel combines them.
#include "sdpa_wave.h"

namespace mfa {

__device__ inline f32x4 mla_load4(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }
__device__ inline f32x2 mla_load2(const float *p) { return *reinterpret_cast<const f32x2 *>(p); }
__device__ inline bf16x8 mla_lds8(const void *p) { return *reinterpret_cast<const bf16x8 *>(p); }

typedef short mla_i16x4 __attribute__((ext_vector_type(4)));
typedef short mla_i16x8 __attribute__((ext_vector_type(8)));
// Transposing 8-byte LDS read (see the layout note above).
__device__ inline mla_i16x4 mla_lds_tr(const unsigned char *p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (mla_i16x4 __attribute__((address_space(3))) *)(__attribute__((address_space(3))) unsigned char *)p);
}

static constexpr int kMlaBlk = 16;    // positions per block
static constexpr int kMlaHG = 4;      // 16-head groups per workgroup
static constexpr float kMlaLazy = 8.f;

template <int R, int P>
__global__ __launch_bounds__(kMlaHG * 128) void mla_partial_kernel(
    const float *__restrict__ q_prime, const float *__restrict__ q_pe, const float *__restrict__ latent,
    const float *__restrict__ rope_k, int H, int L, int blocks_per_split, float qscale,
    float *__restrict__ part_o, float *__restrict__ part_ml) {
    constexpr int HG = kMlaHG, NROLE = HG * 64;
    constexpr int DK = R + P;
    constexpr int KROW = DK + 16;         // row stride (bf16): 1184 bytes
    constexpr int NS = DK / 32;           // 32-wide steps of the score contraction
    constexpr int NT = R / 16;            // output tiles (16 channels each)
    static_assert(NROLE == 256 && R == 512 && P == 64, "the staging maps 256 threads per role onto a 16 x (512 + 64) block");
    constexpr int KPLANE = kMlaBlk * KROW * 2;           // bytes of one plane (hi or lo) of a block
    constexpr int KBUF = 2 * KPLANE;                     // one buffer
    constexpr int VPOS = 6;              // positions of a block whose latent rows the value waves stage; the score waves take the rest
    __shared__ __attribute__((aligned(16))) unsigned char smem[3 * KBUF];
    __shared__ __attribute__((aligned(16))) uint16_t pbuf[2][HG][2][16][kMlaBlk];  // weights [buffer][group][hi|lo][head][position]
    __shared__ float abuf[2][HG][16];                                             // rescale factor of a block, per head

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const bool score_role = wave < HG;
    const int hgl = wave % HG, rtid = tid % NROLE;
    const int split = blockIdx.x, nsplit = gridDim.x;
    const int nhg = (H + 15) / 16;
    const int hg = blockIdx.y * HG + hgl;
    const bool active = hg < nhg;  // a wave past the last head group repeats the last head and stores nothing

    const int nblk = (L + kMlaBlk - 1) / kMlaBlk;
    const int b0 = split * blocks_per_split;
    const int b1 = min(b0 + blocks_per_split, nblk);
    const size_t pid = (size_t)hg * nsplit + split;
    if (b0 >= b1) {
        if (active && score_role && g == 0) {
            part_ml[pid * 32 + n] = neg_inf();
            part_ml[pid * 32 + 16 + n] = 0.f;
        }
        return;
    }
    auto clampb =[&](int b) { return min(b, b1 - 1); };  // requests past the range repeat its last block; nobody reads them
    // block b lives in buffer (b - b0) % 3
    auto bufof =[&](int b) { return smem + ((b - b0) % 3) * KBUF; };

    if (score_role) {
        // ================= scores and softmax of head group hgl =================
        // staging: the rotary keys, two channels at positions rp and rp + 8, and the latent rows the value waves leave
        const int rp = rtid >> 5, rc2 = rtid & 31;
        f32x2 rraw[2], lraw[kMlaBlk - VPOS];
        auto fetch =[&](int b) {
#pragma unroll
            for (int k = 0; k < 2; k++)
                rraw[k] = mla_load2(rope_k + (size_t)min(clampb(b) * kMlaBlk + rp + 8 * k, L - 1) * P + 2 * rc2);
#pragma unroll
            for (int j = VPOS; j < kMlaBlk; j++)
                lraw[j - VPOS] = mla_load2(latent + (size_t)min(clampb(b) * kMlaBlk + j, L - 1) * R + 2 * rtid);
        };
        const int kr_off = (rp * KROW + R + 2 * rc2) * 2;
        auto commit =[&](int b) {
            unsigned char *base = bufof(b);
#pragma unroll
            for (int k = 0; k < 2; k++) {
                uint32_t rh, rl;
                split_pair(rraw[k][0], rraw[k][1], rh, rl);
                *reinterpret_cast<uint32_t *>(base + kr_off + 8 * k * KROW * 2) = rh;
                *reinterpret_cast<uint32_t *>(base + kr_off + 8 * k * KROW * 2 + KPLANE) = rl;
            }
#pragma unroll
            for (int j = VPOS; j < kMlaBlk; j++) {   // the last latent rows of the block, channels 2 rtid, 2 rtid + 1
                uint32_t hi, lo;
                split_pair(lraw[j - VPOS][0], lraw[j - VPOS][1], hi, lo);
                *reinterpret_cast<uint32_t *>(base + 4 * rtid + j * KROW * 2) = hi;
                *reinterpret_cast<uint32_t *>(base + 4 * rtid + j * KROW * 2 + KPLANE) = lo;
            }
        };
        fetch(b0);
        // the 16 queries as B operands: lane (n, g) holds head n, channels 32 s + 8 g .. + 7 of [q' | q_pe]
        bf16x8 qh[NS], ql[NS];
        {
            const int head = min(hg * 16 + n, H - 1);
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const int c0 = 32 * s + 8 * g;
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
        float m_ref = neg_inf(), l_sum = 0.f;
        const int kr_rd = (n * KROW + 8 * g) * 2;   // [hi][position n][8 g]; lo at + KPLANE; step s at + 64 s
        commit(b0);
        fetch(b0 + 1);
        __syncthreads();
        // iteration b0 - 1: block b0 is scored, nothing is accumulated yet; then one iteration per block
        for (int it = b0 - 1; it < b1 - 1; it++) {
            const int b = it + 1;   // the block scored in this iteration
            const unsigned char *base = bufof(b);
            f32x4 sc = {0.f, 0.f, 0.f, 0.f};  // rows = positions 4g + i, column = head n (log2 units)
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const bf16x8 ah = mla_lds8(base + kr_rd + 64 * s);
                const bf16x8 al = mla_lds8(base + kr_rd + 64 * s + KPLANE);
                sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al, qh[s], sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, ql[s], sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah, qh[s], sc, 0, 0, 0);
            }
            // the rotary keys of block it + 2 (its buffer was accumulated from in the previous
            // iteration); block it + 3 is requested
            commit(it + 2);
            fetch(it + 3);
            {
                const int pos0 = b * kMlaBlk + 4 * g;
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (pos0 + i >= L) sc[i] = neg_inf();
                float mb = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
                mb = rows_max(mb);
                // Move the reference point only when some head's maximum has moved far: weights stay
                // below 2^kMlaLazy, and the reference point cancels in the merge.
                float alpha = 1.f;
                if (__any(mb > m_ref + kMlaLazy)) {
                    const float m_new = fmaxf(m_ref, mb);
                    alpha = fast_exp2(m_ref - m_new);
                    m_ref = m_new;
                    l_sum *= alpha;
                }
                float p[4];
#pragma unroll
                for (int i = 0; i < 4; i++) p[i] = fast_exp2(sc[i] - m_ref);
                l_sum += (p[0] + p[1]) + (p[2] + p[3]);
                uint2 ph, pl;
                split_pair(p[0], p[1], ph.x, pl.x);
                split_pair(p[2], p[3], ph.y, pl.y);
                *reinterpret_cast<uint2 *>(&pbuf[b & 1][hgl][0][n][4 * g]) = ph;
                *reinterpret_cast<uint2 *>(&pbuf[b & 1][hgl][1][n][4 * g]) = pl;
                if (g == 0) abuf[b & 1][hgl][n] = alpha;
            }
            __syncthreads();
        }
        l_sum = rows_sum(l_sum);
        if (active && g == 0) {
            part_ml[pid * 32 + n] = m_ref;
            part_ml[pid * 32 + 16 + n] = l_sum;
        }
        __syncthreads();  // iteration b1 - 1: the value waves accumulate the last block
    } else {
        // ================= values of head group hgl =================
        // staging: the latent rows, channels 2 c2, 2 c2 + 1 at the block's first VPOS positions
        const int c2 = rtid;
        f32x2 raw[VPOS];
        auto fetch =[&](int b) {
#pragma unroll
            for (int j = 0; j < VPOS; j++)
                raw[j] = mla_load2(latent + (size_t)min(clampb(b) * kMlaBlk + j, L - 1) * R + 2 * c2);
        };
        auto commit =[&](int b) {
            unsigned char *base = bufof(b) + 4 * c2;
#pragma unroll
            for (int j = 0; j < VPOS; j++) {
                uint32_t hi, lo;
                split_pair(raw[j][0], raw[j][1], hi, lo);
                *reinterpret_cast<uint32_t *>(base + j * KROW * 2) = hi;
                *reinterpret_cast<uint32_t *>(base + j * KROW * 2 + KPLANE) = lo;
            }
        };
        f32x4 o[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        // A operand of tile t: lane (j, g) points at position 8 (g & 1) + j/4 [+ 4], channels 16 t + 4 (j % 4) .. + 3,
        // in the hi plane for g < 2 and the lo plane otherwise; the transposing read hands lane j channel 16 t + j
        // at positions 8 (g & 1) .. + 3 [+ 4]
        const bool hi_slots = g < 2;
        const int tr_rd = (hi_slots ? 0 : KPLANE) + ((8 * (g & 1) + (n >> 2)) * KROW + 4 * (n & 3)) * 2;
        fetch(b0);
        commit(b0);
        fetch(b0 + 1);
        __syncthreads();
        // iteration b0 - 1: no weights yet
        commit(b0 + 1);
        fetch(b0 + 2);
        __syncthreads();
        for (int it = b0; it < b1; it++) {
            commit(it + 2);    // its buffer held block it - 1
            fetch(it + 3);
            const unsigned char *base = bufof(it) + tr_rd;
            // lane (n, g): weights of head n at positions 8 (g & 1) .. + 7
            const bf16x8 pb_h = mla_lds8(&pbuf[it & 1][hgl][0][n][8 * (g & 1)]);
            const bf16x8 pb_l = mla_lds8(&pbuf[it & 1][hgl][1][n][8 * (g & 1)]);
            const float alpha = abuf[it & 1][hgl][n];
            if (__any(alpha != 1.f)) {
#pragma unroll
                for (int t = 0; t < NT; t++) o[t] *= alpha;
            }
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const mla_i16x4 a0 = mla_lds_tr(base + 32 * t);
                const mla_i16x4 a1 = mla_lds_tr(base + 32 * t + 4 * KROW * 2);
                const mla_i16x8 a8 = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
                const bf16x8 a = __builtin_bit_cast(bf16x8, a8);
                o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb_l, o[t], 0, 0, 0);
                o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb_h, o[t], 0, 0, 0);
            }
            __syncthreads();
        }
        // o[t][i] is channel 16 t + 4g + i of head n
        if (active) {
            float *po = part_o + (pid * 16 + n) * R + 4 * g;
#pragma unroll
            for (int t = 0; t < NT; t++) *reinterpret_cast<f32x4 *>(po + 16 * t) = o[t];
        }
    }
}

bool mla_shape_supported(int kv_lora_rank, int qk_rope_head_dim) {
    return kv_lora_rank == 512 && qk_rope_head_dim == 64;
}

// Partition of the cache's blocks over workgroups: enough splits that every CU has a
// workgroup, never more than there are blocks.
MlaPlan mla_plan(int H, int L, int num_cus, int forced_splits) {
    MlaPlan p;
    p.nhg = (H + 15) / 16;
    p.nwg_heads = (p.nhg + kMlaHG - 1) / kMlaHG;
    const int nblk = (L + kMlaBlk - 1) / kMlaBlk;
    int splits = forced_splits > 0 ? forced_splits : (num_cus + p.nwg_heads - 1) / p.nwg_heads;
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
    hipLaunchKernelGGL((mla_partial_kernel<512, 64>), dim3(plan.splits, plan.nwg_heads), dim3(kMlaHG * 128), 0,
                       stream, q_prime, q_pe, latent, rope_k, H, L, plan.bps, qscale, ws.part_o, ws.part_ml);
    MFA_HIP(hipGetLastError());
    return launch_sdpa_merge(stream, ws, plan.splits, /*hpk=*/H, /*Hq=*/H, plan.nhg, R, /*n_tok=*/1,
                             /*gate=*/nullptr, out);
}

}  // namespace mfa
