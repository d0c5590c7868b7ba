// Split-K flash-decode GQA attention with the sigmoid output gate, for gfx950.
//
// Replaces the reference's four-kernel chain attn_scores_batched /
// attn_softmax_batched / attn_values_batched / sigmoid_gate
// (crates/moeflux/shaders/shaders.metal:976-1134, encoded at
// crates/moeflux/src/riir/linear_attn_forward.rs:850-902) and its CPU fallback
// sdpa_cpu (crates/moeflux/src/riir/sdpa.rs:63-172) with two launches:
//
//   sdpa_partial_kernel  grid (splits, head groups, kv heads), W = 4 or 8 waves.
//     The cache is consumed in super-blocks of W position blocks.  The up to 16
//     query heads that share the kv head are the N dimension of the matrix
//     instruction, so lane%16 is the head index throughout:
//       phase 1  wave w:  S^T[pos, head] = K[pos, :] . Q[head, :] for its own
//                block (the block's K is one contiguous run, read as 1 KiB
//                wave loads straight into MFMA operand registers); the tile
//                maxima meet in LDS, every wave forms the same running max,
//                and the probabilities go to LDS already in operand order.
//       phase 2  wave w:  O^T[d, head] += V^T[d, pos] . P^T[pos, head] for ALL W
//                blocks of the super-block but only its own D/(16 W) output
//                tiles, so no wave ever holds more than its slice of O and
//                nothing has to be summed across waves at the end.
//     Each byte of K and V is read exactly once.  All loads of a super-block
//     are issued before its first use (the query's first of all, because
//     loads return in order); the next super-block's K is requested when the
//     K registers free up after phase 1, its V after phase 2.
//     bf16 caches use v_mfma_f32_16x16x32_bf16 with the f32 query and the f32
//     probabilities each split into a bf16 high and low part (two
//     instructions, products exact to ~2^-17); f32 caches use
//     v_mfma_f32_16x16x4_f32.  The query is pre-multiplied by scale*log2 e so a
//     probability is one v_exp_f32.  One (max, sum, O[16, D]) partial per
//     workgroup is written.
//   The log-sum-exp merge of the partials, the normalisation and the sigmoid gate
//   run in the same launch: every workgroup takes a ticket of its row group when its
//   partial is visible device-wide, and the one that draws the last ticket (helped,
//   when the group has many splits, by workgroups that arrived a moment earlier and
//   looked on for a bounded time) combines the group's partials.  No workgroup ever
//   depends on another one making progress.  sdpa_merge_kernel / sdpa_merge_few_kernel
//   are the same merge as a launch of its own (the latent-cache attention uses them).
#include "attn_prologue.h"
#include "sdpa_merge.h"

namespace mfa {

static constexpr int kMaxSplits = 1024;

// part_o:  [kv head][head group][split][16 heads][D]
// part_ml: [kv head][head group][split][2][16]   (max in log2 units, then sum)
// The merge inside the split-K launch.  A row group's record is one 64-bit word, zero when the
// launch starts: arrivals in the high half, claimed chunks of the group's output in the low half.
//   * A workgroup makes its partial visible device-wide (release fence), then adds 1 to the
//     arrivals with one device-scope atomic; the value that comes back is its ticket.  The one
//     that draws the last ticket knows every partial of the group is complete.
//   * Few splits (<= 16): that workgroup merges the whole group, all requests in flight at once.
//   * Many splits: the group's output is cut into chunks and the workgroups of the first splits
//     are helpers: a helper claims chunk `split` in the same atomic that takes its ticket, then
//     reads the record a bounded number of times; when it sees the last arrival it merges its
//     chunk.  A helper that gives up hands the chunk back (one atomic; should the last arrival
//     have come in between, it merges the chunk after all).  The last arrival merges every chunk
//     nobody held when it arrived.  Each chunk has exactly one owner, who only starts once all
//     partials are visible, and no workgroup waits without a bound: progress never depends on
//     which workgroups are resident.
//   * Records are never reset by the launch that uses them: launches alternate between two sets
//     of records, and each launch zeroes the records the previous user of the other set touched.
struct FusedMerge {
    unsigned long long *rec;    // this launch's records [kv head][row group]; null: no merge in this launch
    unsigned long long *zero;   // records of the other set to clear, [0, n_zero)
    int n_zero;
    int wait;                   // polls a helper makes before it gives up
    const float *gate;
    float *out;
};

// The attention prologue of one decode token inside the split-K launch
// (full_attn_forward.rs:238-323: q/gate split, per-head RMS norms of q and k, rotation of the
// first rotary_dim channels, cache append).  The launch attends to the positions the cache held
// before the token; the token's own score and value enter in the merge as one more split.
struct StepPrologue {
    const float *q_proj;       // [Hq][2][D]: q_h then gate_h
    const float *k_in, *v_in;  // [Hkv * D] projections of the new token
    const uint16_t *q_norm, *k_norm;
    const float *inv_freq;     // 1 / theta^(2i/rotary_dim), i < rotary_dim / 2
    int rotary_dim;
    float eps;
    int pos;                   // rotation position of the token
    int64_t cache_pos;         // where its row goes: the cache length before the call
    float *new_score;          // [kv head][row group][16]: q . k_new in log2 units
    void *k_tiled, *v_tiled;   // the planes, to append to
    int token_split;           // the split whose workgroup also scores and appends the token
};

// The query operands of the workgroup's 16 rows from the raw q projection: a group of
// LPH = D / EPS lanes serves one head, lane j its channels [EPS j, EPS j + EPS), which is exactly
// operand slot (k-step j / 4, lane group j % 4, row n).  Norm and rotation stay inside the
// group (sums and partners by lane exchange); the arithmetic is that of attn_prologue_kernel.
// request() only asks for the operands (all loads unconditional, so the cache requests that
// follow can be counted apart from them); finish() does the arithmetic.  With `with_new` every
// group also forms the new token's normed, rotated key (each the same one) and its score
// against the group's head, and group 0 of row group 0 appends the token's key and value row.
template <typename KV, int D, int NT> struct StepQuery {
    using W = Wave<KV, D>;
    static constexpr int EPS = sizeof(KV) == 2 ? 8 : 4;
    static constexpr int LPH = D / EPS;
    static constexpr int NQ = (W::QSLOTS + NT - 1) / NT;
    static_assert(LPH <= 64 && W::QSLOTS == 16 * LPH, "a head's lanes fit a wave");
    float qraw[NQ][EPS], kraw[EPS], vraw[EPS], wq[EPS], wk[EPS], freq;

    __device__ inline void request(const StepPrologue &sp, const RowGroup &rows) {
        const int j = threadIdx.x % LPH, c0 = EPS * j;
        freq = HeadRotor<EPS, D>::table_request(sp.inv_freq, sp.rotary_dim);
#pragma unroll
        for (int i = 0; i < NQ; i++) {
            int v = threadIdx.x + i * NT;
            if (v >= W::QSLOTS) v = W::QSLOTS - 1;
            const int n = v / LPH;
            const float *p = sp.q_proj + (rows.valid(n) ? rows.q_row(n) : 0) * 2 * D + c0;
#pragma unroll
            for (int e = 0; e < EPS; e += 4) {
                const float4 t = load_f4(p + e);
                qraw[i][e] = t.x; qraw[i][e + 1] = t.y; qraw[i][e + 2] = t.z; qraw[i][e + 3] = t.w;
            }
        }
        const float *pk = sp.k_in + (size_t)rows.kvh * D + c0, *pv = sp.v_in + (size_t)rows.kvh * D + c0;
#pragma unroll
        for (int e = 0; e < EPS; e += 4) {
            const float4 a = load_f4(pk + e), b = load_f4(pv + e);
            kraw[e] = a.x; kraw[e + 1] = a.y; kraw[e + 2] = a.z; kraw[e + 3] = a.w;
            vraw[e] = b.x; vraw[e + 1] = b.y; vraw[e + 2] = b.z; vraw[e + 3] = b.w;
        }
        {   // EPS bf16 weights each: one 8- or 16-byte request per array
            typedef unsigned short __attribute__((ext_vector_type(EPS))) wvec;
            const wvec a = *reinterpret_cast<const wvec *>(sp.q_norm + c0), b = *reinterpret_cast<const wvec *>(sp.k_norm + c0);
#pragma unroll
            for (int e = 0; e < EPS; e++) {
                wq[e] = bf16_bits_to_f32(a[e]);
                wk[e] = bf16_bits_to_f32(b[e]);
            }
        }
    }

    // `tab`: the workgroup's (cos, sin) table (HeadRotor::table), complete before this call
    __device__ inline void finish(const StepPrologue &sp, const RowGroup &rows, float qscale, size_t plane_elems,
                                  bool with_new, uint4 *qlds, int nhg, const float2 *tab) {
        const int j = threadIdx.x % LPH, c0 = EPS * j;
        HeadRotor<EPS, D> hr;
        hr.init(j, sp.rotary_dim, tab);
        auto norm_rotate = [&](float (&x)[EPS], const float (&w)[EPS]) { hr.apply(x, w, sp.eps); };
        float knew[EPS];
        if (with_new) {   // uniform over the workgroup
            norm_rotate(kraw, wk);
#pragma unroll
            for (int e = 0; e < EPS; e++) knew[e] = from_kv(to_kv<KV>(kraw[e]));   // as the cache will hold it
        }
#pragma unroll
        for (int i = 0; i < NQ; i++) {
            const int v = threadIdx.x + i * NT;
            const bool in = v < W::QSLOTS;
            const int n = (in ? v : W::QSLOTS - 1) / LPH;
            const bool ok = in && rows.valid(n);
            norm_rotate(qraw[i], wq);
            if (with_new) {
                float d = 0.f;
#pragma unroll
                for (int e = 0; e < EPS; e++) d = fmaf(qraw[i][e], knew[e], d);
                d = lanes_sum<LPH>(d);
                if (ok && j == 0) sp.new_score[((size_t)rows.kvh * nhg + rows.hg) * 16 + n] = d * qscale;
            }
            if (in) {
                float4 raw[W::QRAW_F4];
#pragma unroll
                for (int e = 0; e < EPS; e += 4)
                    raw[e / 4] = ok ? float4{qraw[i][e], qraw[i][e + 1], qraw[i][e + 2], qraw[i][e + 3]}
                                    : float4{0.f, 0.f, 0.f, 0.f};
                W::store_q_slot(qlds, raw, (j / 4) * 64 + (j % 4) * 16 + n, qscale);
            }
        }
        if (with_new && rows.hg == 0 && threadIdx.x < LPH) {   // the token's row: key normed and rotated, value as it comes
            KV *kp = (KV *)sp.k_tiled + (size_t)rows.kvh * plane_elems, *vp = (KV *)sp.v_tiled + (size_t)rows.kvh * plane_elems;
#pragma unroll
            for (int e = 0; e < EPS; e++) {
                kp[KvTile<KV>::k_off(sp.cache_pos, c0 + e, D)] = to_kv<KV>(kraw[e]);
                vp[KvTile<KV>::v_off(sp.cache_pos, c0 + e, D)] = to_kv<KV>(vraw[e]);
            }
        }
    }
};

static constexpr int kFewSplits = 16;        // at most this many: merged by one workgroup in one go
static constexpr int kMaxMergeChunks = 32;   // claim bits of a record

template <typename KV, int D, int WAVES, bool STEP>
__global__ __launch_bounds__(WAVES * 64) void sdpa_partial_kernel(
    const KV *__restrict__ k_tiled, const KV *__restrict__ v_tiled, size_t plane_elems,
    const float *__restrict__ q, int hpk, int Hq, int n_tok, int64_t kv_len0,
    int blocks_per_split, float qscale, float *__restrict__ part_o, float *__restrict__ part_ml,
    FusedMerge fm, StepPrologue sp) {
    using W = Wave<KV, D>;
    constexpr int NACC = W::NACC;
    constexpr int TPW = NACC / WAVES;  // output tiles owned by one wave
    constexpr int NLOAD = W::NLOAD;
    constexpr int NX = W::NX;
    constexpr int NQ = (W::QSLOTS + WAVES * 64 - 1) / (WAVES * 64);  // query slots per thread
    static_assert(NACC % WAVES == 0, "waves must divide the output tiles");
    __shared__ uint4 qlds[W::QLDS_U4];
    __shared__ uint4 pbuf[WAVES][W::P_U4][64];
    __shared__ float sm[WAVES][16];
    __shared__ float sl[WAVES][16];
    __shared__ float2 s_tab[STEP ? 128 : 1];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int split = blockIdx.x, hg = blockIdx.y, kvh = blockIdx.z;
    const int nsplit = gridDim.x, nhg = gridDim.y;
    // A decode step's launch: the workgroup of one split (the last, which has the fewest positions)
    // also norms and rotates the token's key, scores it against every query row of the group and
    // appends its row.  Uniform over the workgroup.
    const bool with_new = STEP && split == sp.token_split;

    const int64_t blk_elems = (int64_t)W::BLK * D;
    const KV *kplane = k_tiled + (size_t)kvh * plane_elems;
    const KV *vplane = v_tiled + (size_t)kvh * plane_elems;
    const RowGroup rows{kvh, hg, hpk, Hq, n_tok, kv_len0};
    const int64_t limit = rows.limit(n);          // this lane's row sees positions [0, limit)
    const int64_t limit_min = rows.limit_min();   // below it no row of the group is masked
    const bool all_rows = rows.full();
    const int64_t nblk = (rows.limit_max() + W::BLK - 1) / W::BLK;
    const int64_t b0 = (int64_t)split * blocks_per_split;
    int64_t b1 = b0 + blocks_per_split;
    if (b1 > nblk) b1 = nblk;
    const size_t pid = ((size_t)kvh * nhg + hg) * nsplit + split;
    if (fm.rec && fm.n_zero > 0 && threadIdx.x == 0) {   // clear the other set's used records
        const int nwg = gridDim.x * gridDim.y * gridDim.z;
        for (int i = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x; i < fm.n_zero; i += nwg)
            fm.zero[i] = 0ull;
    }
    if (with_new && b0 >= b1) {
        // no positions for this split (an empty cache): its partial weighs nothing, the token is all there is
        if (wave == 0 && g == 0) {
            const __amdgpu_buffer_rsrc_t mlb = buffer_of(part_ml + pid * 32);
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, neg_inf()), mlb, n * 4, 0, kThrough);
            __builtin_amdgcn_raw_buffer_store_b32(0u, mlb, (16 + n) * 4, 0, kThrough);
        }
        StepQuery<KV, D, WAVES * 64> sq;
        sq.request(sp, rows);
        HeadRotor<sq.EPS, D>::table(sq.freq, sp.pos, sp.rotary_dim, s_tab);
        __syncthreads();
        sq.finish(sp, rows, qscale, plane_elems, true, qlds, nhg, s_tab);
        return;
    }
    if (b0 >= b1) {  // a split that lies wholly beyond what this group's rows may see
        // Its rows of part_o stay unwritten: the merge gives a split whose maximum is -inf the
        // weight 0 by selection, so whatever bytes the workspace holds there never enter a sum.
        if (wave == 0 && g == 0) {
            const __amdgpu_buffer_rsrc_t mlb = buffer_of(part_ml + pid * 32);
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, neg_inf()), mlb, n * 4, 0, kThrough);
            __builtin_amdgcn_raw_buffer_store_b32(0u, mlb, (16 + n) * 4, 0, kThrough);
        }
    } else {

    // ---- requests, in the order they are needed (loads return in order) ---------
    // Every load below is unconditional (indices are clamped instead), so that the
    // compiler can count outstanding loads exactly and wait for the query without
    // waiting for the cache.
    float4 qraw[NQ][W::QRAW_F4];
    StepQuery<KV, D, WAVES * 64> sq;
    if (STEP) {
        sq.request(sp, rows);
        __builtin_amdgcn_s_barrier();
    } else {
#pragma unroll
        for (int i = 0; i < NQ; i++) {
            int slot = threadIdx.x + i * WAVES * 64;
            if (slot >= W::QSLOTS) slot = W::QSLOTS - 1;
            W::load_q_slot(qraw[i], q, slot, rows);
        }
        // A CU returns load data in request order across its waves: hold the bulk requests
        // back until every wave's query request is queued, or a late wave's query would
        // sit behind its siblings' cache blocks.
        __builtin_amdgcn_s_barrier();
    }
    uint4 kreg[NLOAD];
    uint4 vreg[WAVES][TPW];
    // loads [i0, i1) of this wave's K block of the super-block starting at sb
    auto load_k_part = [&](int64_t sb, int i0, int i1) {
        int64_t blk = sb + wave;
        if (blk > b1 - 1) blk = b1 - 1;  // a wave without a block re-reads the last one and ignores it
        const uint4 *p = (const uint4 *)(kplane + blk * blk_elems) + lane;
#pragma unroll
        for (int i = i0; i < i1; i++) kreg[i] = stream_load(p + i * 64);
    };
    auto load_k = [&](int64_t sb) { load_k_part(sb, 0, NLOAD); };
    // V of blocks [j0, j1) of the super-block starting at sb
    auto load_v = [&](int64_t sb, int j0, int j1) {
#pragma unroll
        for (int j = j0; j < j1; j++) {
            int64_t blk = sb + j;
            if (blk > b1 - 1) blk = b1 - 1;
            const uint4 *p = (const uint4 *)(vplane + blk * blk_elems) + lane + (wave * TPW) * 64;
#pragma unroll
            for (int t = 0; t < TPW; t++) vreg[j][t] = stream_load(p + t * 64);
        }
    };
    // A wave issues in order, and a CU accepts only so many outstanding loads: requesting
    // all of V here would keep the wave stuck in the issue stage long after its K has
    // arrived.  So only kVEarly blocks of V go out now, the rest once the scores are under way.
    constexpr int kVEarly = WAVES / 4;
    if (STEP) {
        // Three quarters of the K block are requested first (measured against a quarter, half, all and
        // none of it: 18.5 us per step against 20.1, 18.9, 19.1 and 20.3): enough to keep the memory pipeline full while
        // the first wave forms the rotation table and every wave norms and rotates its share of
        // the query (a wave cannot compute while its requests wait for room in the queue, which
        // the full set would do for microseconds).  The rest follows when the query is in LDS.
        load_k_part(b0, 0, NLOAD * 3 / 4);
        HeadRotor<sq.EPS, D>::table(sq.freq, sp.pos, sp.rotary_dim, s_tab);
        __syncthreads();
        sq.finish(sp, rows, qscale, plane_elems, with_new, qlds, nhg, s_tab);
        load_k_part(b0, NLOAD * 3 / 4, NLOAD);
        load_v(b0, 0, kVEarly);
    } else {
        load_k(b0);
        load_v(b0, 0, kVEarly);
#pragma unroll
        for (int i = 0; i < NQ; i++) {
            const int slot = threadIdx.x + i * WAVES * 64;
            if (slot < W::QSLOTS) W::store_q_slot(qlds, qraw[i], slot, qscale);
        }
    }
    __syncthreads();

    f32x4 o[TPW];
#pragma unroll
    for (int t = 0; t < TPW; t++) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = neg_inf(), l_run = 0.f;

    // One super-block.  `more` is a compile-time constant at both call sites so that
    // each path has a fixed sequence of loads.
    auto super_block = [&](int64_t sb, auto more_tag, auto first_tag) {
        constexpr bool more = decltype(more_tag)::value;
        constexpr int v_issued = decltype(first_tag)::value ? kVEarly : WAVES;  // V blocks already requested
        const int64_t blk = sb + wave;
        const bool have = blk < b1;
        // ---- phase 1: this wave's block of scores ------------------------------
        float x[NX];
        float m_loc = neg_inf();
        {
            typename W::Scores sc;
            W::scores(kreg, qlds, lane, sc);
            W::unpack(sc, x);
        }
        if (v_issued < WAVES) load_v(sb, v_issued, WAVES);
        if (more) load_k(sb + WAVES);  // the K registers are free again
        if (!have || !all_rows || (blk + 1) * W::BLK > limit_min) {  // a block some row must not see in full
#pragma unroll
            for (int e = 0; e < NX; e++)
                if (!have || W::pos_of(blk, g, e) >= limit) x[e] = neg_inf();
        }
#pragma unroll
        for (int e = 0; e < NX; e++) m_loc = fmaxf(m_loc, x[e]);
        m_loc = fmaxf(m_loc, lane_xor(m_loc, 16));
        m_loc = fmaxf(m_loc, lane_xor(m_loc, 32));
        if (g == 0) sm[wave][n] = m_loc;
        __syncthreads();
        float m_new = m_run;
#pragma unroll
        for (int w = 0; w < WAVES; w++) m_new = fmaxf(m_new, sm[w][n]);
        // a row that has seen nothing yet (its limit lies further on, or it is padding) keeps -inf
        const float m_ref = (m_new == neg_inf()) ? 0.f : m_new;
        const float alpha = fast_exp2(m_run - m_ref);
        m_run = m_new;
        float psum = 0.f;
        {
            float e[NX];
#pragma unroll
            for (int i = 0; i < NX; i++) {
                e[i] = fast_exp2(x[i] - m_ref);  // 0 for masked positions
                psum += e[i];
            }
            uint4 p[W::P_U4];
            W::pack_probs(e, p);
#pragma unroll
            for (int i = 0; i < W::P_U4; i++) pbuf[wave][i][lane] = p[i];
        }
        l_run = l_run * alpha + psum;
        __syncthreads();
        // ---- phase 2: every block of the super-block, this wave's output tiles --
        if (__any(alpha != 1.0f)) {  // the running max moved
#pragma unroll
            for (int t = 0; t < TPW; t++) {
                o[t][0] *= alpha; o[t][1] *= alpha; o[t][2] *= alpha; o[t][3] *= alpha;
            }
        }
#pragma unroll
        for (int j = 0; j < WAVES; j++) {
            // a block past the end contributes probabilities that are all zero
            uint4 p[W::P_U4];
#pragma unroll
            for (int i = 0; i < W::P_U4; i++) p[i] = pbuf[j][i][lane];
#pragma unroll
            for (int t = 0; t < TPW; t++) o[t] = W::pv(vreg[j][t], p, o[t]);
        }
        if (more) load_v(sb + WAVES, 0, WAVES);
    };
    if (b0 + WAVES < b1) {
        super_block(b0, std::true_type{}, std::true_type{});
        int64_t sb = b0 + WAVES;
        for (; sb + WAVES < b1; sb += WAVES) super_block(sb, std::true_type{}, std::false_type{});
        super_block(sb, std::false_type{}, std::false_type{});
    } else {
        super_block(b0, std::false_type{}, std::true_type{});
    }

    // ---- one partial per workgroup -----------------------------------------------
    l_run += lane_xor(l_run, 16);
    l_run += lane_xor(l_run, 32);
    if (g == 0) sl[wave][n] = l_run;
    // stores that go through to memory: the partial is read by whichever workgroup merges the group
    const __amdgpu_buffer_rsrc_t ob = buffer_of(part_o + pid * 16 * D);
#pragma unroll
    for (int t = 0; t < TPW; t++) {
        // tile dt, lane group g, element i is channel 16 dt + 4g + i of head n
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o[t]), ob,
                                               (n * D + 16 * (wave * TPW + t) + 4 * g) * 4, 0, kThrough);
    }
    __syncthreads();
    if (wave == 0 && g == 0) {
        float lsum = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) lsum += sl[w][n];
        const __amdgpu_buffer_rsrc_t mlb = buffer_of(part_ml + pid * 32);
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, m_run), mlb, n * 4, 0, kThrough);
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, lsum), mlb, (16 + n) * 4, 0, kThrough);
    }
    }  // a split with positions

    if (!fm.rec) return;   // partials only (uniform over the launch)

    // ---- ticket, and the merge by whoever it falls to -----------------------------------------
    constexpr int TEAMS = WAVES / 4;                 // 256-thread teams of the many-split merge
    constexpr int PER_ROW = D / 64;                  // 64-output units per row
    constexpr int UNITS = 16 * PER_ROW;              // units of a row group
    __shared__ float4 acc4[TEAMS][2][16][16];
    __shared__ unsigned int s_own;                   // chunks this workgroup merges (bit set), 0: none
    const size_t pid0 = ((size_t)kvh * nhg + hg) * nsplit;
    const MergeOut mo{fm.gate, fm.out, hpk, Hq, n_tok, D, D, nullptr, nullptr, 0, nhg};
    const bool few = nsplit <= kFewSplits;
    // chunks of the many-split merge: a power of two, at most one per split, at most 32, and
    // not finer than what the workgroup's teams merge in one pass
    int nchunks = UNITS / TEAMS < kMaxMergeChunks ? UNITS / TEAMS : kMaxMergeChunks;
    while (nchunks > nsplit) nchunks >>= 1;
    const bool helper = !few && split < nchunks;

    // The partial was written with stores that go through to memory: once every wave has counted
    // its own off it is visible device-wide, and the ticket is taken after that.
    wait_for_stores();
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long *rec = fm.rec + (size_t)kvh * nhg + hg;
        const unsigned long long one = 1ull << 32, bit = helper ? (1ull << split) : 0ull;
        const unsigned long long old = __hip_atomic_fetch_add(rec, one + bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned int own = 0;
        if ((int)(old >> 32) == nsplit - 1) {
            // the last arrival: every chunk no helper held at this moment (its own included)
            const unsigned int all = few ? 1u : (nchunks == 32 ? 0xffffffffu : (1u << nchunks) - 1u);
            own = all & ~(unsigned int)old;
        } else if (helper) {
            bool complete = false;
            for (int i = 0; i < fm.wait && !complete; i++) {
                __builtin_amdgcn_s_sleep(2);
                complete = (int)(__hip_atomic_load(rec, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 32) == nsplit;
            }
            if (!complete) {
                // give the chunk back; if the last arrival has been in the meantime, it left the chunk to us
                const unsigned long long was = __hip_atomic_fetch_add(rec, 0ull - bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                complete = (int)(was >> 32) == nsplit;
            }
            if (complete) own = (unsigned int)bit;
        }
        s_own = own;
    }
    __syncthreads();
    unsigned int own = s_own;
    if (own == 0) return;
    // every split's partial is in memory from here on; the reader's loads go there for it
    const PartialsThrough rd(part_o, part_ml, pid0, D);

    if (few) {
        // the whole group in passes of WAVES * UPW units, every request of a pass in flight at once
        if (nsplit <= 8) {
            constexpr int UPW = 8;
            for (int u0 = 0; u0 < UNITS; u0 += WAVES * UPW)
                merge_few_units<8, UPW>(rd, nsplit, kvh, hg, u0 + wave * UPW, UNITS, mo, lane);
        } else {
            constexpr int UPW = 4;
            for (int u0 = 0; u0 < UNITS; u0 += WAVES * UPW)
                merge_few_units<16, UPW>(rd, nsplit, kvh, hg, u0 + wave * UPW, UNITS, mo, lane);
        }
        return;
    }
    const int team = threadIdx.x >> 8, ttid = threadIdx.x & 255;
    const int upc = UNITS / nchunks;                 // units of a chunk, consecutive: a power of two
    while (own) {
        const int c = __builtin_ctz(own);
        own &= own - 1;
        // a chunk's units lie in one row when upc <= PER_ROW, else it is whole rows; a team
        // takes spans of up to two units (128 channels) of one row at a time
        constexpr int SPAN = PER_ROW >= 2 ? 2 : 1;   // units per team pass, at most
        const int span = upc / TEAMS < SPAN ? 1 : SPAN;
        for (int u0 = c * upc; u0 < (c + 1) * upc; u0 += TEAMS * span) {
            const int u = u0 + team * span;
            const bool in = u < (c + 1) * upc;
            const int nn = (in ? u : 0) / PER_ROW, c0 = ((in ? u : 0) % PER_ROW) * 64;
            const int64_t orow = mo.row(kvh, hg * 16 + nn);
            const bool active = in && orow >= 0;
            if (span == 2)
                merge_span<2>(rd, nsplit, D, active, nn, c0, orow, fm.gate, fm.out, ttid, acc4[team], D);
            else
                merge_span<1>(rd, nsplit, D, active, nn, c0, orow, fm.gate, fm.out, ttid, acc4[team], D);
        }
    }
}


// The token a decode step has just appended, as one more split of the merge (MergeOut), and
// where the gate rows lie.
struct MergeExtra {
    int gate_stride;
    const float *new_score, *new_v;
    int new_bf16;
};

// The same merge as a launch of its own.  TOK: the launch takes a decode step's new token as
// one more split (MergeExtra); without it none of that code is compiled in.
// grid (n_tok * Hq, D/64), 256 threads: one 64-output unit per workgroup.
template <bool TOK>
__global__ __launch_bounds__(256) void sdpa_merge_kernel(
    const float *__restrict__ part_o, const float *__restrict__ part_ml, int nsplit, int hpk,
    int Hq, int nhg, int D, const float *__restrict__ gate, float *__restrict__ out, MergeExtra ex) {
    __shared__ float4 acc4[1][16][16];
    // blockIdx.x = token * Hq + head; its row in the kv head's row list is token*hpk + head%hpk
    const int h = blockIdx.x % Hq, tok = blockIdx.x / Hq;
    const int kvh = h / hpk, rr = tok * hpk + h % hpk, hg = rr / 16, n = rr % 16;
    const size_t pid0 = ((size_t)kvh * nhg + hg) * nsplit;
    if constexpr (TOK) {
        const int c = blockIdx.y * 64 + (threadIdx.x & 63);
        merge_span<1, true>(PartialsPlain(part_o, part_ml, pid0, D), nsplit, D, true, n, blockIdx.y * 64, blockIdx.x, gate,
                            out, threadIdx.x, acc4, ex.gate_stride, ex.new_score + ((size_t)kvh * nhg + hg) * 16 + n,
                            ex.new_v + (size_t)kvh * D + c, ex.new_bf16);
    } else {
        merge_span<1>(PartialsPlain(part_o, part_ml, pid0, D), nsplit, D, true, n, blockIdx.y * 64, blockIdx.x, gate, out,
                      threadIdx.x, acc4, D);
    }
}

// Few splits (at most NS = 8 or 16, what a launch over many layers or row groups ends up
// with): one wave per 64 outputs of a (token, head) row, four such units per workgroup.
template <int NS, bool TOK>
__global__ __launch_bounds__(256) void sdpa_merge_few_kernel(
    const float *__restrict__ part_o, const float *__restrict__ part_ml, int nsplit, int hpk,
    int Hq, int nhg, int D, int n_units, const float *__restrict__ gate, float *__restrict__ out, MergeExtra ex) {
    const int lane = threadIdx.x & 63;
    const int unit = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= n_units) return;   // whole waves; there is no barrier below
    const int per_row = D / 64, bx = unit / per_row, by = unit % per_row;
    const int h = bx % Hq, tok = bx / Hq;
    const int kvh = h / hpk, rr = tok * hpk + h % hpk, hg = rr / 16, n = rr % 16;
    const size_t pid0 = ((size_t)kvh * nhg + hg) * nsplit;
    const int u = n * per_row + by;   // the unit's index inside its row group
    const MergeOut mo{gate, out, hpk, Hq, (int)(((int64_t)n_units / per_row) / Hq), D,
                      TOK ? ex.gate_stride : D, TOK ? ex.new_score : nullptr, TOK ? ex.new_v : nullptr,
                      TOK ? ex.new_bf16 : 0, nhg};
    merge_few_units<NS, 1, TOK>(PartialsPlain(part_o, part_ml, pid0, D), nsplit, kvh, hg, u, u + 1, mo, lane);
}

static void launch_merge_kernels(hipStream_t stream, const float *part_o, const float *part_ml, int splits, int hpk,
                                 int Hq, int nhg, int D, int n_tok, const float *gate, float *out,
                                 const MergeExtra *extra = nullptr) {
    const MergeExtra ex = extra ? *extra : MergeExtra{D, nullptr, nullptr, 0};
    const int n_units = n_tok * Hq * (D / 64);
    const dim3 few((n_units + 3) / 4);
#define MFA_MERGE(TOKK)                                                                                                 \
    do {                                                                                                                \
        if (splits <= 8)                                                                                                \
            hipLaunchKernelGGL((sdpa_merge_few_kernel<8, TOKK>), few, dim3(256), 0, stream, part_o, part_ml, splits, hpk, \
                               Hq, nhg, D, n_units, gate, out, ex);                                                     \
        else if (splits <= 16)                                                                                          \
            hipLaunchKernelGGL((sdpa_merge_few_kernel<16, TOKK>), few, dim3(256), 0, stream, part_o, part_ml, splits,   \
                               hpk, Hq, nhg, D, n_units, gate, out, ex);                                                \
        else                                                                                                            \
            hipLaunchKernelGGL(sdpa_merge_kernel<TOKK>, dim3(n_tok * Hq, D / 64), dim3(256), 0, stream, part_o, part_ml, \
                               splits, hpk, Hq, nhg, D, gate, out, ex);                                                 \
    } while (0)
    if (extra) MFA_MERGE(true); else MFA_MERGE(false);
#undef MFA_MERGE
}

int launch_sdpa_merge(hipStream_t stream, const SdpaWorkspace &ws, int splits, int hpk, int Hq, int nhg, int D,
                      int n_tok, const float *gate, float *out) {
    if (splits < 1 || splits > kMaxSplits || D % 64 != 0)
        return fail(MFA_ERR_INVALID, "merge: %d splits (1..%d), width %d (multiple of 64)", splits, kMaxSplits, D);
    launch_merge_kernels(stream, ws.part_o, ws.part_ml, splits, hpk, Hq, nhg, D, n_tok, gate, out);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

bool sdpa_shape_supported(int kv_dtype, int head_dim) {
    if (kv_dtype != MFA_KV_F32 && kv_dtype != MFA_KV_BF16) return false;
    return head_dim == 64 || head_dim == 128 || head_dim == 256;
}

static int blk_of(int kv_dtype) { return kv_dtype == MFA_KV_BF16 ? 32 : 16; }

// Partition of the cache's position blocks over workgroups.  A workgroup has 8 waves
// (super-blocks of 8 blocks) when that still gives every CU a workgroup, else 4;
// head_dim 64 has only 4 output tiles, hence 4 waves.  n_tok > 1 (a prompt chunk)
// multiplies the row groups, which already fill the machine, so the cache is split less.
struct SplitPlan {
    int splits;
    int waves;
    int nhg;      // 16-row groups per kv head
    int64_t bps;  // blocks per split
};

static SplitPlan plan_splits(int kv_dtype, int Hq, int Hkv, int D, int n_tok, int64_t kv_len,
                             int num_cus, int forced) {
    const int hpk = Hq / Hkv;
    SplitPlan p;
    p.nhg = (int)(((int64_t)n_tok * hpk + 15) / 16);
    const int64_t nblk = (kv_len + blk_of(kv_dtype) - 1) / blk_of(kv_dtype);
    int64_t target = forced > 0 ? forced : (num_cus / ((int64_t)Hkv * p.nhg));
    if (target < 1) target = 1;
    // Up to head_dim 128 two 8-wave workgroups fit a CU (<= 128 registers): give every CU two
    // where each still gets a whole pass of 8 blocks (f32, d=128, 32K: 25.6 -> 23.5 us).
    if (forced <= 0 && D <= 128 && nblk >= 8 * 2 * target) target *= 2;
    if (target > kMaxSplits) target = kMaxSplits;
    p.bps = (nblk + target - 1) / target;
    if (p.bps < 1) p.bps = 1;
    p.waves = (p.bps >= 8 && D >= 128) ? 8 : 4;
    // Whole super-blocks only (one block per wave and pass): a pass with idle waves costs as
    // much as a full one, and fewer workgroups of full passes measured 12-18 % faster than
    // one workgroup per CU with a ragged last pass (kv_len 20K-48K at 2 kv heads).
    if (forced <= 0) p.bps = (p.bps + p.waves - 1) / p.waves * p.waves;
    p.splits = (int)((nblk + p.bps - 1) / p.bps);
    if (p.splits < 1) p.splits = 1;
    return p;
}

int sdpa_pick_splits(int kv_dtype, int Hq, int Hkv, int D, int64_t kv_len, int num_cus, int forced) {
    return plan_splits(kv_dtype, Hq, Hkv, D, 1, kv_len, num_cus, forced).splits;
}

// The most splits a decode launch makes at any cache length up to max_len: the plan's split count
// is not monotonic in the length (whole passes per workgroup), its target is.
int sdpa_max_splits(int kv_dtype, int Hq, int Hkv, int D, int64_t max_len, int num_cus, int forced) {
    if (forced > 0) return forced < kMaxSplits ? forced : kMaxSplits;
    const int hpk = Hq / Hkv;
    const int64_t nhg = (hpk + 15) / 16, nblk = (max_len + blk_of(kv_dtype) - 1) / blk_of(kv_dtype);
    int64_t target = num_cus / ((int64_t)Hkv * nhg);
    if (target < 1) target = 1;
    if (D <= 128 && nblk >= 8 * 2 * target) target *= 2;
    if (target > kMaxSplits) target = kMaxSplits;
    return (int)(target < nblk ? target : (nblk > 0 ? nblk : 1));
}

size_t sdpa_workspace_o_elems(int Hq, int Hkv, int D, int splits, int n_tok) {
    const int64_t nhg = ((int64_t)n_tok * (Hq / Hkv) + 15) / 16;
    return (size_t)Hkv * nhg * splits * 16 * D;
}
size_t sdpa_workspace_ml_elems(int Hq, int Hkv, int splits, int n_tok) {
    const int64_t nhg = ((int64_t)n_tok * (Hq / Hkv) + 15) / 16;
    return (size_t)Hkv * nhg * splits * 32;
}

template <typename KV, int D, int WAVES, bool STEP>
static void launch_partial(hipStream_t stream, dim3 grid, const void *k, const void *v,
                           size_t plane_elems, const float *q, int hpk, int Hq, int n_tok,
                           int64_t kv_len0, int bps, float qscale, float *po, float *pml, const FusedMerge &fm,
                           const StepPrologue &sp) {
    hipLaunchKernelGGL((sdpa_partial_kernel<KV, D, WAVES, STEP>), grid, dim3(WAVES * 64), 0, stream,
                       (const KV *)k, (const KV *)v, plane_elems, q, hpk, Hq, n_tok, kv_len0, bps,
                       qscale, po, pml, fm, sp);
}

template <typename KV, int D, bool STEP>
static void launch_partial_w(int waves, hipStream_t stream, dim3 grid, const void *k, const void *v,
                             size_t plane_elems, const float *q, int hpk, int Hq, int n_tok,
                             int64_t kv_len0, int bps, float qscale, float *po, float *pml, const FusedMerge &fm,
                             const StepPrologue &sp) {
    if constexpr (D >= 128) {
        if (waves == 8) {
            launch_partial<KV, D, 8, STEP>(stream, grid, k, v, plane_elems, q, hpk, Hq, n_tok, kv_len0, bps,
                                           qscale, po, pml, fm, sp);
            return;
        }
    }
    launch_partial<KV, D, 4, STEP>(stream, grid, k, v, plane_elems, q, hpk, Hq, n_tok, kv_len0, bps, qscale,
                                   po, pml, fm, sp);
}

// dtype and width dispatch of the split-K launch
template <bool STEP>
static void launch_partial_any(int kv_dtype, int D, int waves, hipStream_t stream, dim3 grid, const void *k,
                               const void *v, size_t plane_elems, const float *q, int hpk, int Hq, int n_tok,
                               int64_t kv_len0, int bps, float qscale, float *po, float *pml, const FusedMerge &fm,
                               const StepPrologue &sp) {
#define MFA_LAUNCH(KV, DD)                                                                                  \
    launch_partial_w<KV, DD, STEP>(waves, stream, grid, k, v, plane_elems, q, hpk, Hq, n_tok, kv_len0, bps, \
                                   qscale, po, pml, fm, sp)
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
}

bool sdpa_step_supported(int kv_dtype, int Hq, int Hkv, int D, int rotary_dim) {
    if (!sdpa_shape_supported(kv_dtype, D) || Hq % Hkv != 0) return false;
    return head_rotor_applies(kv_dtype, D, rotary_dim);
}

// One decode token of a full-attention layer from its raw projections in two launches: the
// split-K launch norms and rotates the query heads itself, attends to the len0 positions the
// cache holds, and the workgroup of the last split (the one with the fewest positions) also scores
// and appends the token; the merge adds the token as one more split.  out: [Hq * D].
int launch_sdpa_step(hipStream_t stream, int kv_dtype, int Hq, int Hkv, int D, int64_t len0, size_t plane_elems,
                     void *k_tiled, void *v_tiled, const float *q_proj, const float *k_in, const float *v_in,
                     const uint16_t *q_norm, const uint16_t *k_norm, const float *inv_freq, int rotary_dim,
                     float eps, int32_t pos, float *new_score, float *out, const SdpaWorkspace &ws, int num_cus,
                     int forced_splits) {
    if (!sdpa_step_supported(kv_dtype, Hq, Hkv, D, rotary_dim))
        return fail(MFA_ERR_SHAPE, "attention step: shape not supported by the two-launch form");
    if (len0 < 0 || pos < 0) return fail(MFA_ERR_INVALID, "attention step: negative position");
    const int hpk = Hq / Hkv;
    SplitPlan plan = plan_splits(kv_dtype, Hq, Hkv, D, 1, len0 > 0 ? len0 : 1, num_cus, forced_splits);
    while (forced_splits <= 0 && plan.splits > 1 && (sdpa_workspace_o_elems(Hq, Hkv, D, plan.splits, 1) > ws.part_o_elems ||
                                                     sdpa_workspace_ml_elems(Hq, Hkv, plan.splits, 1) > ws.part_ml_elems))
        plan = plan_splits(kv_dtype, Hq, Hkv, D, 1, len0 > 0 ? len0 : 1, num_cus, (plan.splits + 1) / 2);
    if (sdpa_workspace_o_elems(Hq, Hkv, D, plan.splits, 1) > ws.part_o_elems ||
        sdpa_workspace_ml_elems(Hq, Hkv, plan.splits, 1) > ws.part_ml_elems)
        return fail(MFA_ERR_INVALID, "sdpa: split-K workspace too small for %d splits", plan.splits);
    const float qscale = (1.0f / sqrtf((float)D)) * kLog2e;
    const FusedMerge fm{nullptr, nullptr, 0, 0, nullptr, nullptr};
    const StepPrologue sp{q_proj, k_in, v_in, q_norm, k_norm, inv_freq, rotary_dim, eps, pos, len0, new_score,
                          k_tiled, v_tiled, plan.splits - 1};
    // rows see positions [0, len0): one token whose own position is not in the cache yet
    launch_partial_any<true>(kv_dtype, D, plan.waves, stream, dim3(plan.splits, plan.nhg, Hkv), k_tiled, v_tiled,
                             plane_elems, nullptr, hpk, Hq, 1, len0 - 1, (int)plan.bps, qscale, ws.part_o, ws.part_ml,
                             fm, sp);
    MFA_HIP(hipGetLastError());
    const MergeExtra ex{2 * D, new_score, v_in, kv_dtype == MFA_KV_BF16 ? 1 : 0};
    launch_merge_kernels(stream, ws.part_o, ws.part_ml, plan.splits, hpk, Hq, plan.nhg, D, 1, q_proj + D, out, &ex);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

// n_tok query tokens against a cache of kv_len positions that already holds them: token t
// (t = 0 is position kv_len - n_tok) attends to positions [0, kv_len - n_tok + t].
// q, gate, out: [n_tok, Hq*D].  n_tok = 1 is decode.
int launch_sdpa(hipStream_t stream, int kv_dtype, int Hq, int Hkv, int D, int n_tok, int64_t kv_len,
                size_t plane_elems, const void *k_tiled, const void *v_tiled, const float *q,
                const float *gate, float *out, const SdpaWorkspace &ws, int num_cus,
                int forced_splits, int partial_only) {
    if (!sdpa_shape_supported(kv_dtype, D))
        return fail(MFA_ERR_SHAPE, "sdpa: head_dim %d / kv dtype %d not supported", D, kv_dtype);
    if (n_tok <= 0 || kv_len < n_tok)
        return fail(MFA_ERR_INVALID, "sdpa: kv_len must be > 0 (got %lld for %d tokens)", (long long)kv_len, n_tok);
    const int hpk = Hq / Hkv;
    SplitPlan plan = plan_splits(kv_dtype, Hq, Hkv, D, n_tok, kv_len, num_cus, forced_splits);
    // never exceed the workspace: a split count shrinks to fit, except one forced for a single
    // token, which is used as given or refused
    while ((forced_splits <= 0 || n_tok > 1) && plan.splits > 1 && (sdpa_workspace_o_elems(Hq, Hkv, D, plan.splits, n_tok) > ws.part_o_elems ||
                               sdpa_workspace_ml_elems(Hq, Hkv, plan.splits, n_tok) > ws.part_ml_elems))
        plan = plan_splits(kv_dtype, Hq, Hkv, D, n_tok, kv_len, num_cus, (plan.splits + 1) / 2);
    if (sdpa_workspace_o_elems(Hq, Hkv, D, plan.splits, n_tok) > ws.part_o_elems ||
        sdpa_workspace_ml_elems(Hq, Hkv, plan.splits, n_tok) > ws.part_ml_elems)
        return fail(MFA_ERR_INVALID, "sdpa: split-K workspace too small for %d splits", plan.splits);
    if (plan.nhg > 65535) return fail(MFA_ERR_SHAPE, "sdpa: too many query rows in one call");
    // scores are produced in log2 units: q is pre-multiplied by (1/sqrt(D)) * log2(e)
    const float qscale = (1.0f / sqrtf((float)D)) * kLog2e;
    const int64_t kv_len0 = kv_len - n_tok;
    dim3 grid(plan.splits, plan.nhg, Hkv);
    // The merge runs inside this launch when the workspace carries ticket records for every row
    // group; otherwise (or when asked for) it is a second launch.
    FusedMerge fm{nullptr, nullptr, 0, 0, gate, out};
    TicketRecords *tk = ws.tickets;
    const size_t groups = (size_t)Hkv * plan.nhg;
    const bool fused = !partial_only && !ws.separate_merge && tk && tk->dev && groups <= tk->cap;
    if (fused) {
        fm.rec = tk->dev + (size_t)tk->cur * tk->cap;
        fm.zero = tk->dev + (size_t)(tk->cur ^ 1) * tk->cap;
        fm.n_zero = (int)tk->used[tk->cur ^ 1];
        fm.wait = ws.merge_wait;
    }
    launch_partial_any<false>(kv_dtype, D, plan.waves, stream, grid, k_tiled, v_tiled, plane_elems, q, hpk, Hq, n_tok,
                              kv_len0, (int)plan.bps, qscale, ws.part_o, ws.part_ml, fm, StepPrologue{});
    MFA_HIP(hipGetLastError());
    if (fused) {   // this set is in use now, the other one is clean again
        tk->used[tk->cur] = groups;
        tk->used[tk->cur ^ 1] = 0;
        tk->cur ^= 1;
        return MFA_OK;
    }
    if (partial_only) return MFA_OK;
    launch_merge_kernels(stream, ws.part_o, ws.part_ml, plan.splits, hpk, Hq, plan.nhg, D, n_tok, gate, out);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
