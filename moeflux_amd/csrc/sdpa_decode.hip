// Split-K flash-decode GQA attention with the sigmoid output gate, for gfx950.
//
// Replaces the reference's four-kernel chain attn_scores_batched /
// attn_softmax_batched / attn_values_batched / sigmoid_gate
// (crates/moeflux/shaders/shaders.metal:976-1134, encoded at
// crates/moeflux/src/riir/linear_attn_forward.rs:850-902) and its CPU fallback
// sdpa_cpu (crates/moeflux/src/riir/sdpa.rs:63-172) with two launches:
//
//   sdpa_partial_kernel  grid (splits, 16-row groups, kv heads), 4 waves.
//     A workgroup streams its share of the cache: K and V pass through a ring of 1 KiB loads
//     per wave (16 for bf16 caches of head_dim 256, else 8), each consumed by the matrix core as
//     it arrives and replaced by the next request, so a CU keeps 32-64 KiB in flight and its
//     four waves, reading side by side, sweep
//     one contiguous run of memory (measured on 64 MiB: 10.8 us per launch in this pattern,
//     12.8 us with a workgroup's whole share requested at once, 11.5-12 us with one contiguous
//     run per wave).  The up to 16 query heads that share the kv head are the N dimension of the
//     matrix instruction, so lane % 16 is the head index throughout.  The cache is consumed in
//     passes of whole chunks of 64 positions; the chunk count of a pass is a compile-time
//     constant (so ring slots are registers), the main loop takes passes of 4 (f32: 2) chunks and
//     the tail one pass of whatever is left, chosen among the compiled forms:
//       K phase  wave w owns the 16-position sub-tile w of every chunk:
//                S^T[pos, head] += K[pos, k-step] . Q[head, k-step] per load, the query operands
//                in registers; while the last K loads are consumed the first V loads go out.
//       exchange the waves' maxima meet in LDS, every wave forms the same running max, and
//                the probabilities go to LDS already in operand order (two LDS barriers per
//                pass; they wait for LDS only, the ring stays in flight).
//       V phase  wave w owns the output tiles w, w + 4, ...:
//                O^T[d, head] += V^T[d, pos] . P^T[pos, head] per load, over all positions of
//                the pass, so nothing is summed across waves at the end; while the last V
//                loads are consumed the next pass's first K loads go out.
//     Each byte of K and V is read exactly once.  bf16 caches use v_mfma_f32_16x16x32_bf16
//     with the f32 query and the f32 probabilities each split into a bf16 high and low part
//     (two instructions, products exact to ~2^-17); f32 caches use v_mfma_f32_16x16x4_f32.
//     The query is pre-multiplied by scale*log2 e so a probability is one v_exp_f32.  One
//     (max, sum, O[16, D]) partial per workgroup is written.
//   sdpa_merge_kernel / sdpa_merge_few_kernel: the log-sum-exp merge of the partials, the
//     normalisation and the sigmoid gate.
#include "attn_prologue.h"
#include "sdpa_merge.h"

namespace mfa {

static constexpr int kMaxSplits = 1024;
static constexpr int kWaves = 4;     // waves of a split-K workgroup

// part_o:  [kv head][head group][split][16 heads][D]
// part_ml: [kv head][head group][split][2][16]   (max in log2 units, then sum)

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
struct NoPrologue {};          // what the plain launch carries in its place

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


// LDS-only barrier: every LDS access of the wave has completed, then the workgroup meets.  Unlike
// __syncthreads() it places no wait on the vector-memory counter, so the ring's loads stay in flight.
__device__ inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// 1 KiB loads a wave keeps in flight.  Eight (32 KiB per CU) is where a plain streaming read of 64 MiB
// is fastest; the widest heads take sixteen, which also keeps the memory system busy while a
// workgroup stages its query and exchanges its probabilities (bf16, head_dim 256, 32768 positions:
// 13.2 us per launch with 8, 12.75 with 16, 12.9 with 32; 14.9 with 4).
__host__ __device__ constexpr int ring_depth(bool bf16, int D) { return bf16 && D == 256 ? 16 : 8; }

// Shape constants of the streaming kernel.  A pass takes NCH chunks; its K is NCH * NK loads per
// wave, its V as many.  The unified sequence of a wave's loads (K of a pass, its V, K of the next
// pass, ...) runs through the ring with load number i in slot i % R, which holds as long as a pass
// is at least one ring of K (MINCH chunks) and two of its phases are whole rings (chunk counts that
// are multiples of GRAN): then every pass begins at slot 0 again.
template <typename KV, int D, bool STEP = false> struct Stream {
    using W = Wave<KV, D>;
    static constexpr int R = ring_depth(sizeof(KV) == 2, D);
    static constexpr int CH = KvTile<KV>::KCH;              // positions of a K chunk
    static constexpr int NK = W::KSTEPS;                    // K loads per chunk and wave (one per k-step)
    static constexpr int VB = CH / W::BLK;                  // V blocks per chunk
    static constexpr int TPW = W::NACC / kWaves;            // output tiles per wave
    static constexpr int NV = VB * TPW;                     // V loads per chunk and wave
    static constexpr int GRAN = (2 * NK) % R == 0 ? 1 : R / (2 * NK);   // chunk counts of a pass are multiples of this
    static constexpr int MINCH = (R + NK - 1) / NK < GRAN ? GRAN : (R + NK - 1) / NK;   // chunks of the smallest pass
    // A share of a single unit is less than a ring of K where MINCH > GRAN; then its K and V together
    // are exactly one ring, requested whole before the query is staged (the short form).
    static constexpr bool HAS_SHORT = MINCH > GRAN;
    // A workgroup's share is streamed in passes of MAIN chunks until at most GMAX are left, which
    // are one last pass: one exchange of maxima and probabilities per pass, and a share a little
    // larger than the others' (a cache just past a multiple of the workgroups' shares) still is
    // a single pass.
    static constexpr int MAIN = sizeof(KV) == 2 ? 4 : 2;
    static constexpr int GMAX = sizeof(KV) == 2 ? 6 : (D == 256 ? 2 : 3);
    static constexpr int KCH_U4 = CH * D * (int)sizeof(KV) / 16;      // 16-byte words of a chunk of K
    static constexpr int VBLK_U4 = W::BLK * D * (int)sizeof(KV) / 16;  // of a block of V
    static_assert(NV == NK && W::NACC % kWaves == 0, "K and V of a chunk are the same number of loads");
    static_assert(!HAS_SHORT || 2 * GRAN * NK == R, "the short form fills the ring exactly");
    static_assert(MAIN % GRAN == 0 && GMAX % GRAN == 0 && MAIN >= MINCH && GMAX - MAIN + GRAN >= MINCH,
                  "every pass of a long share is a whole form");
};

// Calls f with the smallest of the chunk counts N, N + STEP, ... <= END that is at least `want`
// (END if none is), as a compile-time constant.
template <int N, int END, int STEP, typename F> __device__ __attribute__((always_inline)) inline void with_form(int want, F &&f) {
    if constexpr (N + STEP > END) {
        f(std::integral_constant<int, N>{});
    } else {
        if (want <= N) f(std::integral_constant<int, N>{});
        else with_form<N + STEP, END, STEP>(want, f);
    }
}

template <typename KV, int D, bool STEP>
__global__ __launch_bounds__(kWaves * 64) void sdpa_partial_kernel(
    const KV *__restrict__ k_tiled, const KV *__restrict__ v_tiled, size_t plane_elems,
    const float *__restrict__ q, int hpk, int Hq, int n_tok, int64_t kv_len0,
    int units_base, int units_rem, float qscale, float *__restrict__ part_o, float *__restrict__ part_ml,
    std::conditional_t<STEP, StepPrologue, NoPrologue> sp) {
    using W = Wave<KV, D>;
    using S = Stream<KV, D, STEP>;
    constexpr int NK = S::NK, NV = S::NV, TPW = S::TPW, VB = S::VB, kRing = S::R;
    constexpr int NT = kWaves * 64;
    constexpr int NQ = (W::QSLOTS + NT - 1) / NT;  // query slots per thread
    __shared__ uint4 qlds[W::QLDS_U4];
    __shared__ uint4 pbuf[S::GMAX * VB][W::P_U4][64];
    __shared__ float sm[kWaves][16];
    __shared__ float sl[kWaves][16];
    __shared__ float2 s_tab[STEP ? 128 : 1];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int hg = blockIdx.y, kvh = blockIdx.z;
    const int nsplit = gridDim.x, nhg = gridDim.y;
    const int split = blockIdx.x;
    // A decode step's launch: the workgroup of one split (the last, which has the fewest positions)
    // also norms and rotates the token's key, scores it against every query row of the group and
    // appends its row.  Uniform over the workgroup.
    bool with_new = false;
    if constexpr (STEP) with_new = split == sp.token_split;

    const RowGroup rows{kvh, hg, hpk, Hq, n_tok, kv_len0};
    const int64_t limit = rows.limit(n);          // this lane's row sees positions [0, limit)
    // This split's chunks [c0, c1): the plan hands out units of GRAN chunks, the first units_rem
    // splits one unit more than the others; a group whose rows end earlier stops there.
    const int64_t nchunk = (rows.limit_max() + S::CH - 1) / S::CH;
    const int64_t u0 = (int64_t)split * units_base + (split < units_rem ? split : units_rem);
    const int64_t c0 = u0 * S::GRAN;
    int64_t c1 = (u0 + units_base + (split < units_rem ? 1 : 0)) * S::GRAN;
    if (c1 > nchunk) c1 = nchunk;
    const size_t pid = ((size_t)kvh * nhg + hg) * nsplit + split;
    if constexpr (STEP) {
        if (with_new && c0 >= c1) {
            // no positions for this split (an empty cache): its partial weighs nothing, the token is all there is
            if (wave == 0 && g == 0) {
                const __amdgpu_buffer_rsrc_t mlb = buffer_of(part_ml + pid * 32);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, neg_inf()), mlb, n * 4, 0, kThrough);
                __builtin_amdgcn_raw_buffer_store_b32(0u, mlb, (16 + n) * 4, 0, kThrough);
            }
            StepQuery<KV, D, NT> sq;
            sq.request(sp, rows);
            HeadRotor<sq.EPS, D>::table(sq.freq, sp.pos, sp.rotary_dim, s_tab);
            __syncthreads();
            sq.finish(sp, rows, qscale, plane_elems, true, qlds, nhg, s_tab);
            return;
        }
    }
    if (c0 >= c1) {  // a split that lies wholly beyond what this group's rows may see
        // Its rows of part_o stay unwritten: the merge gives a split whose maximum is -inf the
        // weight 0 by selection, so whatever bytes the workspace holds there never enter a sum.
        if (wave == 0 && g == 0) {
            const __amdgpu_buffer_rsrc_t mlb = buffer_of(part_ml + pid * 32);
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, neg_inf()), mlb, n * 4, 0, kThrough);
            __builtin_amdgcn_raw_buffer_store_b32(0u, mlb, (16 + n) * 4, 0, kThrough);
        }
        return;
    }

    // ---- requests, in the order they are needed (loads return in order) ---------
    // Every load below is unconditional (indices are clamped instead), so that the
    // compiler can count outstanding loads exactly and wait for the query without
    // waiting for the cache.
    float4 qraw[NQ][W::QRAW_F4];
    StepQuery<KV, D, NT> sq;
    if constexpr (STEP) {
        sq.request(sp, rows);
    } else {
#pragma unroll
        for (int i = 0; i < NQ; i++) {
            int slot = threadIdx.x + i * NT;
            if (slot >= W::QSLOTS) slot = W::QSLOTS - 1;
            W::load_q_slot(qraw[i], q, slot, rows);
        }
    }
    // A CU returns load data in request order across its waves: hold the cache requests
    // back until every wave's query request is queued, or a late wave's query would
    // sit behind its siblings' cache data.
    __builtin_amdgcn_s_barrier();

    // Piece (k-step s, sub-tile `wave`) of a chunk's K and piece (tile 4t + wave) of a block's V
    // are 16-byte word s * 256 (t * 256) + wave * 64 + lane of the chunk (block): the four waves'
    // loads of one step are 4 KiB side by side, consecutive steps follow each other in memory.
    const uint4 *kbase = reinterpret_cast<const uint4 *>(k_tiled + (size_t)kvh * plane_elems) + wave * 64 + lane;
    const uint4 *vbase = reinterpret_cast<const uint4 *>(v_tiled + (size_t)kvh * plane_elems) + wave * 64 + lane;
    const int64_t cmax = c1 - 1, vmax = c1 * VB - 1;   // requests past the split's end re-read its last chunk / block
    auto k_load = [&](int64_t chunk, int s) {
        const int64_t c = chunk < cmax ? chunk : cmax;
        return stream_load(kbase + c * S::KCH_U4 + s * 256);
    };
    auto v_load = [&](int64_t blk, int t) {
        const int64_t b = blk < vmax ? blk : vmax;
        return stream_load(vbase + b * S::VBLK_U4 + t * 256);
    };
    uint4 ring[kRing];
    constexpr int kHead = kRing < 8 ? kRing : 8;   // of the ring's first requests, those made before the query is staged
    // The ring's first filling is the first kRing loads of the share's sequence: K of its first
    // chunks, or, for a share of one unit where that is half a ring, its K and then its V.
    const bool short_share = S::HAS_SHORT && c1 - c0 <= S::GRAN;
    auto first_load = [&](int i) __attribute__((always_inline)) {
        constexpr int KS = S::GRAN * NK;   // K loads of the short form
        if (S::HAS_SHORT && i >= KS) {
            const int64_t kc = (c0 + i / NK < cmax ? c0 + i / NK : cmax) * S::KCH_U4 + (i % NK) * 256;
            const int64_t vb0 = c0 * VB + (i - KS) / TPW;
            const int64_t vc = (vb0 < vmax ? vb0 : vmax) * S::VBLK_U4 + ((i - KS) % TPW) * 256;
            return stream_load(short_share ? vbase + vc : kbase + kc);
        }
        return k_load(c0 + i / NK, i % NK);
    };
#pragma unroll
    for (int i = 0; i < kHead; i++) {
        ring[i] = first_load(i);
        __builtin_amdgcn_sched_barrier(0);   // in ring order: loads return in the order of their requests
    }

    // The rest of the ring follows when the first part has had time to arrive (a wave that asks for
    // more than the CU's queue holds sits in the issue stage until data returns, and can do nothing
    // else): in a decode step between the rotation table and the norms, which take as long again.
    auto rest_of_ring = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = kHead; i < kRing; i++) {
            ring[i] = first_load(i);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    if constexpr (STEP) {
        HeadRotor<sq.EPS, D>::table(sq.freq, sp.pos, sp.rotary_dim, s_tab);
        lds_barrier();
        rest_of_ring();
        sq.finish(sp, rows, qscale, plane_elems, with_new, qlds, nhg, s_tab);
    } else {
#pragma unroll
        for (int i = 0; i < NQ; i++) {
            const int slot = threadIdx.x + i * NT;
            if (slot < W::QSLOTS) W::store_q_slot(qlds, qraw[i], slot, qscale);
        }
        rest_of_ring();
    }
    lds_barrier();
    uint4 qr[W::QREGS];
#pragma unroll
    for (int i = 0; i < W::QREGS; i++) qr[i] = qlds[i * 64 + lane];

    f32x4 o[TPW];
#pragma unroll
    for (int t = 0; t < TPW; t++) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = neg_inf(), l_run = 0.f;

    // One pass over NCH chunks starting at chunk cb; the ring holds the pass's first K loads.
    // NCH and MORE (another pass follows) are compile-time constants at every call site, so each
    // form is a fixed sequence of loads.
    auto pass = [&](int64_t cb, auto nch_tag, auto more_tag) __attribute__((always_inline)) {
        constexpr int NCH = decltype(nch_tag)::value;
        constexpr bool MORE = decltype(more_tag)::value;
        constexpr int KL = NCH * NK, VL = NCH * NV;
        constexpr int VO = KL % kRing;   // ring slot of the pass's first V load
        static_assert((KL + VL) % kRing == 0 && (KL >= kRing || (!MORE && KL + VL == kRing)),
                      "a ring of K at least and the next pass begins at slot 0, or the whole share in one ring");
        // ---- K phase: this wave's sub-tile of every chunk ----------------------------------
        f32x4 sc[NCH];
#pragma unroll
        for (int c = 0; c < NCH; c++) sc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < KL; i++) {
            sc[i / NK] = W::score_step(ring[i % kRing], qr, i % NK, sc[i / NK]);
            if (i + kRing < KL) ring[i % kRing] = k_load(cb + (i + kRing) / NK, (i + kRing) % NK);
            else if (i + kRing - KL < VL) ring[i % kRing] = v_load(cb * VB + (i + kRing - KL) / TPW, (i + kRing - KL) % TPW);
            // the request stays here, a ring's length ahead of its use (left alone the scheduler
            // sinks it to just before the use, and the ring runs one or two deep)
            __builtin_amdgcn_sched_barrier(0);
        }
        float x[4 * NCH];
        float m_loc = neg_inf();
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            // positions 4g .. 4g+3 of sub-tile `wave` of chunk cb + c: the first `nv` of them exist for
            // this lane's row (none in a chunk past the split's end, whose loads re-read the last one)
            const int64_t chunk = cb + c;
            int64_t room = limit - (chunk * S::CH + 16 * wave + 4 * g);
            if (chunk >= c1) room = 0;
            const int nv = room < 0 ? 0 : room > 4 ? 4 : (int)room;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                x[4 * c + r] = r < nv ? sc[c][r] : neg_inf();
                m_loc = fmaxf(m_loc, x[4 * c + r]);
            }
        }
        m_loc = rows_max(m_loc);
        if (g == 0) sm[wave][n] = m_loc;
        lds_barrier();
        float m_new = m_run;
#pragma unroll
        for (int w = 0; w < kWaves; w++) m_new = fmaxf(m_new, sm[w][n]);
        // a row that has seen nothing yet (its limit lies further on, or it is padding) keeps -inf
        const float m_ref = (m_new == neg_inf()) ? 0.f : m_new;
        const float alpha = fast_exp2(m_run - m_ref);
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            float e[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                e[r] = fast_exp2(x[4 * c + r] - m_ref);  // 0 for masked positions
                psum += e[r];
            }
            // sub-tile `wave` of chunk c is half wave % 2 of V block 2c + wave / 2 (bf16), V block 4c + wave (f32)
            W::store_probs(pbuf[c * VB + (wave * VB) / 4], lane, wave & 1, e);
        }
        l_run = l_run * alpha + psum;
        lds_barrier();
        // ---- V phase: every position of the pass, this wave's output tiles -----------------
        if (__any(alpha != 1.0f)) {  // the running max moved
#pragma unroll
            for (int t = 0; t < TPW; t++) {
                o[t][0] *= alpha; o[t][1] *= alpha; o[t][2] *= alpha; o[t][3] *= alpha;
            }
        }
        uint4 p[W::P_U4];
#pragma unroll
        for (int i = 0; i < VL; i++) {
            if (i % TPW == 0) {
#pragma unroll
                for (int j = 0; j < W::P_U4; j++) p[j] = pbuf[i / TPW][j][lane];
            }
            o[i % TPW] = W::pv(ring[(VO + i) % kRing], p, o[i % TPW]);
            if (i + kRing < VL) ring[(VO + i) % kRing] = v_load(cb * VB + (i + kRing) / TPW, (i + kRing) % TPW);
            else if (MORE) ring[(VO + i) % kRing] = k_load(cb + NCH + (i + kRing - VL) / NK, (i + kRing - VL) % NK);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    int64_t cb = c0;
    for (; c1 - cb > S::GMAX; cb += S::MAIN) pass(cb, std::integral_constant<int, S::MAIN>{}, std::true_type{});
    // the last pass, in the smallest form that holds what is left (a form's chunks past the split's
    // end re-read its last chunk and are masked)
    if (short_share) {
        if constexpr (S::HAS_SHORT) pass(cb, std::integral_constant<int, S::GRAN>{}, std::false_type{});
    } else {
        with_form<S::MINCH, S::GMAX, S::GRAN>((int)(c1 - cb), [&](auto nch) __attribute__((always_inline)) { pass(cb, nch, std::false_type{}); });
    }

    // ---- one partial per workgroup -----------------------------------------------
    l_run = rows_sum(l_run);
    if (g == 0) sl[wave][n] = l_run;
    const __amdgpu_buffer_rsrc_t ob = buffer_of(part_o + pid * 16 * D);
#pragma unroll
    for (int t = 0; t < TPW; t++) {
        // tile dt = 4t + wave, lane group g, element i is channel 16 dt + 4g + i of head n
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, o[t]), ob,
                                               (n * D + 16 * (kWaves * t + wave) + 4 * g) * 4, 0, kThrough);
    }
    lds_barrier();
    if (wave == 0 && g == 0) {
        float lsum = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; w++) lsum += sl[w][n];
        const __amdgpu_buffer_rsrc_t mlb = buffer_of(part_ml + pid * 32);
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, m_run), mlb, n * 4, 0, kThrough);
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, lsum), mlb, (16 + n) * 4, 0, kThrough);
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
    if (kv_dtype != MFA_KV_BF16 && kv_dtype != MFA_KV_F32) return false;
    return head_dim == 64 || head_dim == 128 || head_dim == 256;
}

// chunks of a unit of the plan (Stream::GRAN)
static int unit_chunks(int kv_dtype, int D) {
    const int nk = kv_dtype == MFA_KV_BF16 ? D / 32 : D / 16, ring = ring_depth(kv_dtype == MFA_KV_BF16, D);
    return (2 * nk) % ring == 0 ? 1 : ring / (2 * nk);
}

// chunks of the kernel's smallest pass (Stream::MINCH)
static int min_pass_chunks(int kv_dtype, int D) {
    const int nk = kv_dtype == MFA_KV_BF16 ? D / 32 : D / 16, ring = ring_depth(kv_dtype == MFA_KV_BF16, D);
    const int m = (ring + nk - 1) / nk, g = unit_chunks(kv_dtype, D);
    return m < g ? g : m;
}

// Partition of the cache over workgroups, in units of chunks of 64 positions (pairs of chunks at
// head_dim 64 of a bf16 cache): `splits` workgroups per row group, the first `rem` of them `base + 1` units,
// the others `base`.  The shares differ by at most one unit at every length, so the time of a
// launch follows the length smoothly.  n_tok > 1 (a prompt chunk) multiplies the row groups,
// which already fill the machine, so the cache is split less.
struct SplitPlan {
    int splits;
    int nhg;      // 16-row groups per kv head
    int base, rem;
};

// workgroups the plan aims at per (kv head, row group): every CU one, or two where a workgroup's
// registers and LDS leave room and each still streams a few units
static int64_t split_target(int Hq, int Hkv, int D, int64_t nhg, int64_t nunits, int num_cus, int wgs_per_cu) {
    int64_t target = (int64_t)num_cus / ((int64_t)Hkv * nhg);
    if (target < 1) target = 1;
    if (wgs_per_cu > 1 && nunits >= 2 * wgs_per_cu * target) target *= wgs_per_cu;
    if (target > kMaxSplits) target = kMaxSplits;
    (void)Hq; (void)D;
    return target;
}

static constexpr int g_wgs_per_cu = 1;

static SplitPlan plan_splits(int kv_dtype, int Hq, int Hkv, int D, int n_tok, int64_t kv_len,
                             int num_cus, int forced) {
    const int hpk = Hq / Hkv;
    SplitPlan p;
    p.nhg = (int)(((int64_t)n_tok * hpk + 15) / 16);
    const int64_t nchunk = (kv_len + kKvChunk - 1) / kKvChunk;
    const int U = unit_chunks(kv_dtype, D);
    int64_t nunits = (nchunk + U - 1) / U;
    if (nunits < 1) nunits = 1;
    int64_t target = forced > 0 ? forced : split_target(Hq, Hkv, D, p.nhg, nunits, num_cus, g_wgs_per_cu);
    if (target > kMaxSplits) target = kMaxSplits;
    if (target > nunits) target = nunits;
    // the automatic plan keeps a share at least the kernel's smallest pass of whole rings: shares of a
    // single unit (the short form) on twice the workgroups measured slower (12 layers of 8192
    // positions, head_dim 256, bf16: 128 x 1 chunk against 64 x 2 chunks, +0.5 us per layer)
    const int64_t min_units = (min_pass_chunks(kv_dtype, D) + U - 1) / U;
    if (forced <= 0 && target > 1 && nunits / target < min_units) target = nunits / min_units > 1 ? nunits / min_units : 1;
    p.splits = (int)target;
    p.base = (int)(nunits / target);
    p.rem = (int)(nunits % target);
    return p;
}

int sdpa_pick_splits(int kv_dtype, int Hq, int Hkv, int D, int64_t kv_len, int num_cus, int forced) {
    return plan_splits(kv_dtype, Hq, Hkv, D, 1, kv_len, num_cus, forced).splits;
}

// The most splits a decode launch makes at any cache length up to max_len: the plan's split
// count never falls as the length grows.
int sdpa_max_splits(int kv_dtype, int Hq, int Hkv, int D, int64_t max_len, int num_cus, int forced) {
    if (forced > 0) return forced < kMaxSplits ? forced : kMaxSplits;
    return plan_splits(kv_dtype, Hq, Hkv, D, 1, max_len > 0 ? max_len : 1, num_cus, 0).splits;
}

size_t sdpa_workspace_o_elems(int Hq, int Hkv, int D, int splits, int n_tok) {
    const int64_t nhg = ((int64_t)n_tok * (Hq / Hkv) + 15) / 16;
    return (size_t)Hkv * nhg * splits * 16 * D;
}
size_t sdpa_workspace_ml_elems(int Hq, int Hkv, int splits, int n_tok) {
    const int64_t nhg = ((int64_t)n_tok * (Hq / Hkv) + 15) / 16;
    return (size_t)Hkv * nhg * splits * 32;
}

template <typename KV, int D, bool STEP, typename SP>
static void launch_partial(hipStream_t stream, dim3 grid, const void *k, const void *v, size_t plane_elems,
                           const float *q, int hpk, int Hq, int n_tok, int64_t kv_len0, const SplitPlan &plan,
                           float qscale, float *po, float *pml, const SP &sp) {
    hipLaunchKernelGGL((sdpa_partial_kernel<KV, D, STEP>), grid, dim3(kWaves * 64), 0, stream, (const KV *)k,
                       (const KV *)v, plane_elems, q, hpk, Hq, n_tok, kv_len0, plan.base, plan.rem, qscale, po, pml, sp);
}

// dtype and width dispatch of the split-K launch
template <bool STEP, typename SP>
static void launch_partial_any(int kv_dtype, int D, hipStream_t stream, dim3 grid, const void *k, const void *v,
                               size_t plane_elems, const float *q, int hpk, int Hq, int n_tok, int64_t kv_len0,
                               const SplitPlan &plan, float qscale, float *po, float *pml, const SP &sp) {
#define MFA_LAUNCH(KV, DD) \
    launch_partial<KV, DD, STEP>(stream, grid, k, v, plane_elems, q, hpk, Hq, n_tok, kv_len0, plan, qscale, po, pml, sp)
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

// A plan that fits the workspace: an automatic split count shrinks to fit; one forced for a
// single token is used as given or refused.
static int fit_plan(SplitPlan &plan, int kv_dtype, int Hq, int Hkv, int D, int n_tok, int64_t kv_len, int num_cus,
                    int forced_splits, const SdpaWorkspace &ws) {
    auto fits = [&](const SplitPlan &p) {
        return sdpa_workspace_o_elems(Hq, Hkv, D, p.splits, n_tok) <= ws.part_o_elems &&
               sdpa_workspace_ml_elems(Hq, Hkv, p.splits, n_tok) <= ws.part_ml_elems;
    };
    plan = plan_splits(kv_dtype, Hq, Hkv, D, n_tok, kv_len, num_cus, forced_splits);
    while ((forced_splits <= 0 || n_tok > 1) && plan.splits > 1 && !fits(plan))
        plan = plan_splits(kv_dtype, Hq, Hkv, D, n_tok, kv_len, num_cus, (plan.splits + 1) / 2);
    if (!fits(plan)) return fail(MFA_ERR_INVALID, "sdpa: split-K workspace too small for %d splits", plan.splits);
    if (plan.nhg > 65535 || Hkv > 65535) return fail(MFA_ERR_SHAPE, "sdpa: too many query rows in one call");
    return MFA_OK;
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
    SplitPlan plan;
    MFA_TRY(fit_plan(plan, kv_dtype, Hq, Hkv, D, 1, len0 > 0 ? len0 : 1, num_cus, forced_splits, ws));
    const float qscale = (1.0f / sqrtf((float)D)) * kLog2e;
    const StepPrologue sp{q_proj, k_in, v_in, q_norm, k_norm, inv_freq, rotary_dim, eps, pos, len0, new_score,
                          k_tiled, v_tiled, plan.splits - 1};
    // rows see positions [0, len0): one token whose own position is not in the cache yet
    launch_partial_any<true>(kv_dtype, D, stream, dim3(plan.splits, plan.nhg, Hkv), k_tiled, v_tiled, plane_elems,
                             nullptr, hpk, Hq, 1, len0 - 1, plan, qscale, ws.part_o, ws.part_ml, sp);
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
                int forced_splits, int partial_only, SdpaMergeTask *defer_merge) {
    if (defer_merge) defer_merge->n_units = 0;
    if (!sdpa_shape_supported(kv_dtype, D))
        return fail(MFA_ERR_SHAPE, "sdpa: head_dim %d / kv dtype %d not supported", D, kv_dtype);
    if (n_tok <= 0 || kv_len < n_tok)
        return fail(MFA_ERR_INVALID, "sdpa: kv_len must be > 0 (got %lld for %d tokens)", (long long)kv_len, n_tok);
    const int hpk = Hq / Hkv;
    SplitPlan plan;
    MFA_TRY(fit_plan(plan, kv_dtype, Hq, Hkv, D, n_tok, kv_len, num_cus, forced_splits, ws));
    // scores are produced in log2 units: q is pre-multiplied by (1/sqrt(D)) * log2(e)
    const float qscale = (1.0f / sqrtf((float)D)) * kLog2e;
    launch_partial_any<false>(kv_dtype, D, stream, dim3(plan.splits, plan.nhg, Hkv), k_tiled, v_tiled, plane_elems, q,
                              hpk, Hq, n_tok, kv_len - n_tok, plan, qscale, ws.part_o, ws.part_ml, NoPrologue{});
    MFA_HIP(hipGetLastError());
    if (partial_only) return MFA_OK;
    if (defer_merge && plan.splits <= 16) {
        *defer_merge = SdpaMergeTask{ws.part_o, ws.part_ml, gate, out, plan.splits, hpk, Hq, plan.nhg, D, n_tok * Hq * (D / 64)};
        return MFA_OK;
    }
    launch_merge_kernels(stream, ws.part_o, ws.part_ml, plan.splits, hpk, Hq, plan.nhg, D, n_tok, gate, out);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
