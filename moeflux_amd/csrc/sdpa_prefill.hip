// Causal attention of a prompt chunk over the tiled KV cache, for chunks large enough
// that the query rows alone fill the machine.
//
// The reference has no batched prefill: eval_prompt is a token loop
// (crates/moeflux/src/riir/mod.rs:1196-1214) whose every token runs the decode chain of
// crates/moeflux/src/riir/sdpa.rs:63-172.  Row t of the chunk equals that decode at
// kv_len = kv_len0 + t + 1.
//
// A workgroup is 4 waves; every wave owns RG groups of 16 query rows (rows of one kv
// head: token-major, then the hpk query heads that share it) from start to end: its
// query operands and its output tiles stay in registers and its soft-max needs no other
// wave.  The workgroup walks the cache blocks (of V: 32 or 16 positions) that its rows may see; each
// block's K and V (already in MFMA operand order in memory) is copied into LDS once by all 256 threads,
// double buffered, and every wave takes its operands from there.  With RG = 2 an operand
// read from LDS feeds two row groups.  Nothing is split along the cache, so the gated,
// normalised output is written directly.
#include "sdpa_wave.h"

namespace mfa {

// 1 / (1 + e^-x) from the hardware exp2 and reciprocal (each good to 1 ulp)
__device__ inline float fast_sigmoid(float x) {
    return __builtin_amdgcn_rcpf(1.0f + fast_exp2(-x * kLog2e));
}

// How far (in log2 units) a row's running maximum may rise above the reference its
// exponentials are taken against before the accumulators are rescaled: probabilities
// stay below 2^8, which costs nothing in f32 and spares most rescaling passes.
static constexpr float kLazyRescale = 8.0f;

// grid (workgroups of RW*RG row groups, Hkv), 64*RW*KS threads.  Waves RW*ks .. RW*ks+RW-1
// form set ks: all sets serve the same RW*RG row groups, set ks taking blocks ks, ks + KS, ...
// (more waves per SIMD when the rows alone cannot provide them); sets are merged
// through LDS at the end.
template <typename KV, int D, int RG, int DEPTH, int KS, int RW>
__global__ __launch_bounds__(64 * RW * KS) void sdpa_prefill_kernel(
    const KV *__restrict__ k_tiled, const KV *__restrict__ v_tiled, size_t plane_elems,
    const float *__restrict__ q, const float *__restrict__ gate, int hpk, int Hq, int n_tok,
    int64_t kv_len0, float qscale, float *__restrict__ out) {
    using W = Wave<KV, D>;
    constexpr int NLOAD = W::NLOAD, NACC = W::NACC, NX = W::NX;
    constexpr int BLK_U4 = (NLOAD + NACC) * 64;  // 16-byte words of one block's K and V
    constexpr int SET = 64 * RW;                 // threads of a wave set
    constexpr int PER_T = BLK_U4 / SET;
    constexpr int K_T = NLOAD * 64 / SET;        // of which K
    static_assert(NLOAD % RW == 0 && NACC % RW == 0, "a set's threads copy whole rounds of a block's K and of its V");
    static_assert(DEPTH == 2 || DEPTH == 4, "the pipeline is written out for two or four stages");
    static_assert(KS == 1 || (KS - 1) * RW * RG * NACC * 64 <= 2 * KS * BLK_U4, "the merge reuses the staging buffers");
    // LAG: the scores of a block are issued one iteration ahead of its soft-max and value
    // product (three LDS buffers); measured 5-8 % faster at head_dim 256 and 4 % slower at 128.
    constexpr bool LAG = D == 256;
    constexpr int NBUF = LAG ? 3 : 2;
    __shared__ uint4 kv[NBUF][KS][BLK_U4];
    __shared__ float s_m[KS][RW][RG][16], s_l[KS][RW][RG][16];

    // The query operands of the first wave set pass to the others (same rows; requested from memory
    // once) through the last staging buffer, which the walk first writes in its second iteration.
    static_assert(KS == 1 || RW * RG * W::QREGS * 64 <= KS * BLK_U4, "the query operands fit a staging buffer");
    uint4 (*s_q)[64] = reinterpret_cast<uint4 (*)[64]>(&kv[NBUF - 1][0][0]);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rw = wave % RW, ks = wave / RW, tid = threadIdx.x % SET;
    const int n = lane & 15, g = lane >> 4;
    const int kvh = blockIdx.y, wg = blockIdx.x;
    const int hg0 = (wg * RW + rw) * RG;  // this wave's first row group
    const int64_t blk_elems = (int64_t)W::BLK * D;
    const KV *kplane = k_tiled + (size_t)kvh * plane_elems;
    const KV *vplane = v_tiled + (size_t)kvh * plane_elems;

    // blocks the workgroup walks: up to the last position its last row sees
    const RowGroup wg_last{kvh, wg * RW * RG + RW * RG - 1, hpk, Hq, n_tok, kv_len0};
    const int64_t nblk = (wg_last.limit_max() + W::BLK - 1) / W::BLK;
    const int64_t nit = (nblk + KS - 1) / KS;  // iterations: set ks computes block it * KS + ks

    // Each set stages its own blocks.  The block of iteration it + DEPTH is requested when
    // the block of iteration it leaves its staging registers, so DEPTH blocks are in flight
    // while one is computed on.  Requests past the last block re-read it (unconditional
    // loads keep the outstanding-load count exact).
    uint4 stage[DEPTH * PER_T];
    auto fetch = [&](auto st, int64_t it) __attribute__((always_inline)) {
        constexpr int s0 = st.value * PER_T;
        int64_t blk = it * KS + ks;
        if (blk > nblk - 1) blk = nblk - 1;
        // K lies in chunks of 64 positions, a k-step's four 16-position sub-tiles side by side
        // (KvTile): piece li of the block (SUBS sub-tiles per k-step) is piece
        // (li / SUBS) * 4 + first sub-tile + li % SUBS of its chunk.
        constexpr int VB = KvTile<KV>::KCH / W::BLK, SUBS = 4 / VB;
        const uint4 *kc = (const uint4 *)(kplane + (blk / VB) * (int64_t)(KvTile<KV>::KCH * D)) + (tid & 63);
        const int sub0 = (int)(blk % VB) * SUBS;
        const uint4 *vp = (const uint4 *)(vplane + blk * blk_elems) + tid;
#pragma unroll
        for (int i = 0; i < PER_T; i++) {
            const int li = (i * SET + tid) >> 6;   // i < K_T: the piece of K this thread copies
            stage[s0 + i] = vec_load(i < K_T ? kc + (((li / SUBS) * 4 + sub0 + li % SUBS) << 6) : vp + (i - K_T) * SET);
        }
    };
    auto commit = [&](int buf, auto st) __attribute__((always_inline)) {
        constexpr int s0 = st.value * PER_T;
#pragma unroll
        for (int i = 0; i < PER_T; i++) kv[buf][ks][i * SET + tid] = stage[s0 + i];
    };

    fetch(std::integral_constant<int, 0>{}, 0);
    fetch(std::integral_constant<int, 1>{}, 1);
    if constexpr (DEPTH > 2) {
        fetch(std::integral_constant<int, 2>{}, 2);
        fetch(std::integral_constant<int, 3>{}, 3);
    }
    // A bf16 cache's scores are products of the raw query, split into a bf16 high and low part, and are
    // scaled as they leave the matrix core: a query that is exact in bf16 (what a bf16 model hands
    // over) then has no low parts, and a wave all of whose rows are such leaves their products out.
    uint4 qr[RG][W::QREGS];
    bool q_exact = true;
    int64_t limit[RG], limit_min[RG], limit_max[RG];
    bool full[RG];
#pragma unroll
    for (int r = 0; r < RG; r++) {
        const RowGroup rows{kvh, hg0 + r, hpk, Hq, n_tok, kv_len0};
        if (KS == 1 || ks == 0) {   // uniform over the wave
            W::load_q_regs(qr[r], q, lane, rows, W::kScaleAfter ? 1.0f : qscale);
            if constexpr (KS > 1) {
#pragma unroll
                for (int i = 0; i < W::QREGS; i++) s_q[(rw * RG + r) * W::QREGS + i][lane] = qr[r][i];
            }
        }
        limit[r] = rows.limit(n);
        limit_min[r] = rows.limit_min();
        // a group wholly past the chunk's rows sees nothing
        limit_max[r] = rows.valid(0) ? rows.limit_max() : 0;
        full[r] = rows.full();
    }
    if constexpr (KS > 1) {
        __syncthreads();
        if (ks > 0) {
#pragma unroll
            for (int r = 0; r < RG; r++)
#pragma unroll
                for (int i = 0; i < W::QREGS; i++) qr[r][i] = s_q[(rw * RG + r) * W::QREGS + i][lane];
        }
    }
#pragma unroll
    for (int r = 0; r < RG; r++) q_exact = q_exact && W::q_low_parts_zero(qr[r]);
    q_exact = __all(q_exact);
    int64_t wave_max = limit_max[0];
#pragma unroll
    for (int r = 1; r < RG; r++) wave_max = limit_max[r] > wave_max ? limit_max[r] : wave_max;

    // m_ref: the value the row's exponentials are taken against (-inf until the row has
    // seen a position); it follows the running maximum lazily.
    f32x4 o[RG][NACC];
    float m_ref[RG], l_run[RG];
#pragma unroll
    for (int r = 0; r < RG; r++) {
        m_ref[r] = neg_inf();
        l_run[r] = 0.f;
#pragma unroll
        for (int t = 0; t < NACC; t++) o[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // A block's work in two halves: its scores (matrix pipeline), then the soft-max (vector
    // pipeline) and the value product.
    auto qk = [&](const uint4 *cur, typename W::Scores (&sc)[RG]) __attribute__((always_inline)) {
        uint4 kreg[NLOAD];
#pragma unroll
        for (int i = 0; i < NLOAD; i++) kreg[i] = cur[i * 64 + lane];
        if (q_exact) {
#pragma unroll
            for (int r = 0; r < RG; r++) W::template scores_reg<true>(kreg, qr[r], sc[r]);
        } else {
#pragma unroll
            for (int r = 0; r < RG; r++) W::template scores_reg<false>(kreg, qr[r], sc[r]);
        }
    };
    auto finish = [&](int64_t b, const uint4 *cur, const typename W::Scores (&sc)[RG]) __attribute__((always_inline)) {
        uint4 p[RG][W::P_U4];
#pragma unroll
        for (int r = 0; r < RG; r++) {
            float x[NX];
            W::unpack(sc[r], x);
            // kScaleAfter: x is unscaled; the scale (positive) enters the row maximum once and the
            // exponentials' arguments as a fused multiply-add
            const float xs = W::kScaleAfter ? qscale : 1.0f;
            if (!full[r] || (b + 1) * W::BLK > limit_min[r]) {  // a block some row must not see in full
#pragma unroll
                for (int e = 0; e < NX; e++)
                    if (W::pos_of(b, g, e) >= limit[r]) x[e] = neg_inf();
            }
            float m_loc = x[0];
#pragma unroll
            for (int e = 1; e < NX; e++) m_loc = fmaxf(m_loc, x[e]);
            m_loc = rows_max(m_loc);
            if constexpr (W::kScaleAfter) m_loc *= xs;
            // m_loc > -inf + 8 is false while the row has seen nothing, so m_ref stays
            // -inf; the exponent's reference is then 0 and every probability is 0.
            const bool move = m_loc > m_ref[r] + kLazyRescale;
            float alpha = 1.0f;
            if (move) {
                alpha = fast_exp2(m_ref[r] - m_loc);  // 0 on the row's first block
                m_ref[r] = m_loc;
            }
            const float ref = (m_ref[r] == neg_inf()) ? 0.f : m_ref[r];
            float e[NX], psum = 0.f;
#pragma unroll
            for (int i = 0; i < NX; i++) {
                e[i] = fast_exp2(W::kScaleAfter ? fmaf(x[i], xs, -ref) : x[i] - ref);  // 0 for masked positions
                psum += e[i];
            }
            l_run[r] = l_run[r] * alpha + psum;
            W::pack_probs(e, p[r]);
            if (__any(move)) {
#pragma unroll
                for (int t = 0; t < NACC; t++) {
                    o[r][t][0] *= alpha; o[r][t][1] *= alpha; o[r][t][2] *= alpha; o[r][t][3] *= alpha;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < NACC; t++) {
            const uint4 vreg = cur[(NLOAD + t) * 64 + lane];
#pragma unroll
            for (int r = 0; r < RG; r++) o[r][t] = W::pv(vreg, p[r], o[r][t]);
        }
    };
    // LAG state: the block whose second half is still to come
    typename W::Scores sc_prev[RG];
    bool prev_live = false;
    int64_t b_prev = 0;
    const uint4 *kv_prev = kv[0][ks];
    auto compute = [&](int64_t b, const uint4 *cur) __attribute__((always_inline)) {
        const bool live = b * W::BLK < wave_max;  // some row of this wave sees the block
        if constexpr (!LAG) {
            if (!live) return;
            typename W::Scores sc[RG];
            qk(cur, sc);
            finish(b, cur, sc);
        } else {
            // the scores of block b do not depend on the soft-max of the block before, so the two
            // pipelines overlap inside the wave (a wave's blocks come in increasing order: once a
            // block lies past its rows, all later ones do)
            if (live && prev_live) {
                typename W::Scores sc_new[RG];
                qk(cur, sc_new);
                finish(b_prev, kv_prev, sc_prev);
#pragma unroll
                for (int r = 0; r < RG; r++) sc_prev[r] = sc_new[r];
            } else if (live) {
                qk(cur, sc_prev);
            } else if (prev_live) {
                finish(b_prev, kv_prev, sc_prev);
            }
            prev_live = live;
            b_prev = b;
            kv_prev = cur;
        }
    };

    // Iteration it: its block leaves the registers for LDS buffer it % NBUF, the registers take
    // the request for iteration it + DEPTH, barrier, compute.  Without LAG buffer it % 2 was last
    // read in iteration it - 2; with it, iteration it reads buffers it % 3 (scores) and
    // (it - 1) % 3 (the rest of block it - 1), and buffer it % 3 was last read in iteration
    // it - 2.  Either way every wave finished that iteration before the barrier of iteration it - 1.
    int buf = 0;
    for (int64_t i0 = 0; i0 < nit; i0 += DEPTH) {
#define MFA_STEP(S)                                                   \
    if constexpr (S < DEPTH) {                                        \
        if (i0 + S < nit) { /* uniform over the workgroup */          \
            commit(buf, std::integral_constant<int, S>{});            \
            fetch(std::integral_constant<int, S>{}, i0 + S + DEPTH);  \
            __syncthreads();                                          \
            compute((i0 + S) * KS + ks, kv[buf][ks]);                 \
            buf = buf == NBUF - 1 ? 0 : buf + 1;                      \
        }                                                             \
    }
        MFA_STEP(0) MFA_STEP(1) MFA_STEP(2) MFA_STEP(3)
#undef MFA_STEP
    }
    if constexpr (LAG) {
        if (prev_live) finish(b_prev, kv_prev, sc_prev);   // the last block's second half
    }

    // ---- merge the sets: set 0 takes in the others ----------------------------------
    if constexpr (KS > 1) {
        __syncthreads();  // every wave is done with the staging buffers
        float4 *xo = reinterpret_cast<float4 *>(&kv[0][0][0]);  // [set - 1][row wave][group][tile][lane]
#pragma unroll
        for (int r = 0; r < RG; r++) {
            float l = l_run[r];
            l = rows_sum(l);
            l_run[r] = l;
            if (ks > 0) {
                if (g == 0) {
                    s_m[ks][rw][r][n] = m_ref[r];
                    s_l[ks][rw][r][n] = l;
                }
#pragma unroll
                for (int t = 0; t < NACC; t++)
                    xo[((((ks - 1) * RW + rw) * RG + r) * NACC + t) * 64 + lane] =
                        float4{o[r][t][0], o[r][t][1], o[r][t][2], o[r][t][3]};
            }
        }
        __syncthreads();
        if (ks > 0) return;
#pragma unroll
        for (int r = 0; r < RG; r++) {
            float m_all = m_ref[r];
#pragma unroll
            for (int j = 1; j < KS; j++) m_all = fmaxf(m_all, s_m[j][rw][r][n]);
            const float ref = (m_all == neg_inf()) ? 0.f : m_all;
            const float a0 = fast_exp2(m_ref[r] - ref);
            float l = l_run[r] * a0;
#pragma unroll
            for (int t = 0; t < NACC; t++) {
                o[r][t][0] *= a0; o[r][t][1] *= a0; o[r][t][2] *= a0; o[r][t][3] *= a0;
            }
#pragma unroll
            for (int j = 1; j < KS; j++) {
                const float aj = fast_exp2(s_m[j][rw][r][n] - ref);
                l += aj * s_l[j][rw][r][n];
#pragma unroll
                for (int t = 0; t < NACC; t++) {
                    const float4 v = xo[((((j - 1) * RW + rw) * RG + r) * NACC + t) * 64 + lane];
                    o[r][t][0] += aj * v.x; o[r][t][1] += aj * v.y; o[r][t][2] += aj * v.z; o[r][t][3] += aj * v.w;
                }
            }
            l_run[r] = l;
        }
    } else {
#pragma unroll
        for (int r = 0; r < RG; r++) {
            float l = l_run[r];
            l = rows_sum(l);
            l_run[r] = l;
        }
    }

    // ---- normalise, gate, store (all of the gate is requested before the first use) ----
#pragma unroll
    for (int r = 0; r < RG; r++) {
        const RowGroup rows{kvh, hg0 + r, hpk, Hq, n_tok, kv_len0};
        const bool ok = rows.valid(n);
        const size_t base = (ok ? rows.q_row(n) : 0) * D + 4 * g;
        uint4 gt[NACC];
#pragma unroll
        for (int t = 0; t < NACC; t++) gt[t] = vec_load((const uint4 *)(gate + base + 16 * t));
        if (!ok) continue;
        const float inv = 1.0f / l_run[r];
#pragma unroll
        for (int t = 0; t < NACC; t++) {
            // tile t, lane group g, element i is channel 16 t + 4 g + i of row n
            const float4 gv = __builtin_bit_cast(float4, gt[t]);
            float4 y;
            y.x = o[r][t][0] * inv * fast_sigmoid(gv.x);
            y.y = o[r][t][1] * inv * fast_sigmoid(gv.y);
            y.z = o[r][t][2] * inv * fast_sigmoid(gv.z);
            y.w = o[r][t][3] * inv * fast_sigmoid(gv.w);
            *(float4 *)(out + base + 16 * t) = y;
        }
    }
}

// Whether a chunk of n_tok tokens is better served by this kernel than by the split-K
// row-group path: either the cache is short (nothing to gain from splitting it) or the
// rows alone give at least half the CUs a workgroup.
bool sdpa_prefill_applies(int kv_dtype, int Hq, int Hkv, int n_tok, int64_t kv_len, int num_cus) {
    if (n_tok < 2) return false;
    const int blk = kv_dtype == MFA_KV_BF16 ? 32 : 16;
    const int64_t nblk = (kv_len + blk - 1) / blk;
    const int64_t nhg = ((int64_t)n_tok * (Hq / Hkv) + 15) / 16;
    const int64_t nwg = (nhg + 3) / 4 * Hkv;
    return nblk <= 64 || nwg >= num_cus / 2;
}

int launch_sdpa_prefill(hipStream_t stream, int kv_dtype, int Hq, int Hkv, int D, int n_tok, int64_t kv_len,
                        size_t plane_elems, const void *k_tiled, const void *v_tiled, const float *q,
                        const float *gate, float *out, int num_cus) {
    if (!sdpa_shape_supported(kv_dtype, D))
        return fail(MFA_ERR_SHAPE, "sdpa: head_dim %d / kv dtype %d not supported", D, kv_dtype);
    if (n_tok <= 0 || kv_len < n_tok)
        return fail(MFA_ERR_INVALID, "sdpa: kv_len must be > 0 (got %lld for %d tokens)", (long long)kv_len, n_tok);
    const int hpk = Hq / Hkv;
    const int64_t nhg = ((int64_t)n_tok * hpk + 15) / 16;
    // Shapes of a workgroup (row waves RW x row groups per wave RG x wave sets KS):
    //   large chunks  4 x 2 x 1: two row groups per wave share each operand read from LDS;
    //   medium        4 x 1 x 1 (every CU still gets two workgroups);
    //   small (the rows alone would leave a wave alone on its SIMD)  4 x 1 x 2: the blocks are
    //   split over two wave sets.  (2 x 2 x 2, four waves with two row groups each, was
    //   measured 35 % slower at 512 tokens: the two groups' instructions do not interleave;
    //   2 x 1 x 2, two small workgroups per CU, 15 % slower.)
    const bool big = (nhg + 7) / 8 * Hkv >= 2 * (int64_t)num_cus && D <= 128;
    const bool small = !big && D <= 128 && (nhg + 3) / 4 * Hkv < 2 * (int64_t)num_cus;
    const int rw = 4, rg = big ? 2 : 1;
    const int64_t nwg = (nhg + rw * rg - 1) / (rw * rg);
    if (nwg > 0x7fffffff || Hkv > 65535) return fail(MFA_ERR_SHAPE, "sdpa: too many query rows in one call");
    const float qscale = (1.0f / sqrtf((float)D)) * kLog2e;
    const int64_t kv_len0 = kv_len - n_tok;
    const dim3 grid((unsigned)nwg, Hkv);
#define MFA_LAUNCH(KV, DD, RGG, DEP, KSS, RWW)                                                                 \
    hipLaunchKernelGGL((sdpa_prefill_kernel<KV, DD, RGG, DEP, KSS, RWW>), grid, dim3(64 * RWW * KSS), 0, stream, \
                       (const KV *)k_tiled, (const KV *)v_tiled, plane_elems, q, gate, hpk, Hq, n_tok, kv_len0,   \
                       qscale, out)
#define MFA_LAUNCH_D(KV)                                         \
    if (D == 256) MFA_LAUNCH(KV, 256, 1, 2, 1, 4);               \
    else if (D == 128) {                                         \
        if (big) MFA_LAUNCH(KV, 128, 2, 2, 1, 4);                \
        else if (small) MFA_LAUNCH(KV, 128, 1, 4, 2, 4);         \
        else MFA_LAUNCH(KV, 128, 1, 4, 1, 4);                    \
    } else {                                                     \
        if (big) MFA_LAUNCH(KV, 64, 2, 2, 1, 4);                 \
        else if (small) MFA_LAUNCH(KV, 64, 1, 4, 2, 4);          \
        else MFA_LAUNCH(KV, 64, 1, 4, 1, 4);                     \
    }
    if (kv_dtype == MFA_KV_BF16) { MFA_LAUNCH_D(uint16_t) } else { MFA_LAUNCH_D(float) }
#undef MFA_LAUNCH_D
#undef MFA_LAUNCH
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
