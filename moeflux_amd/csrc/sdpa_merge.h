// Log-sum-exp merge of split-K partials: the device code of the merge kernels.
//
// Partials of one row group (16 query rows that share a kv head) lie at
//   part_o  [pid0 + split][16 rows][D]      part_ml [pid0 + split][2][16]  (max in log2 units, sum)
// and are read through a reader (PartialsPlain, sdpa_wave.h) by indices
// relative to the group's first split.  A row's result is  sum_s w_s O_s / sum_s w_s l_s  with  w_s = 2^(m_s - max_s m_s), times
// the sigmoid of the row's gate.  A split whose maximum is -inf (no row of the group could see
// its positions) gets the weight 0 by selection and its rows are never added, whatever bytes
// they hold.  The carried (max, denominator, accumulator) triple is the reference's own scheme
// for combining passes over a long cache (shaders.metal:1821-1987, gpu_mla.rs:186-268).
#pragma once
#include "gdn_device.h"
#include "sdpa_wave.h"

namespace mfa {

// Where the merged rows of a launch go: out and gate are [n_tok, Hq, D].
struct MergeOut {
    const float *gate;   // may be null: no gate
    float *out;
    int hpk, Hq, n_tok, D;
    int gate_stride;     // floats between the gate rows of consecutive heads (D, or 2 D inside a q projection)
    // One more split that is a single position, the token a decode step has just appended:
    // its score per row (log2 units, [kv head][row group][16]) and its value row ([Hkv * D] as
    // projected; rounded here as the cache holds it).  Null: none.
    const float *new_score, *new_v;
    int new_bf16, nhg;
    // (callers are the TOK instantiations, where both pointers are set: no branch around the loads)
    __device__ float token_score(int kvh, int hg, int n) const { return new_score[((size_t)kvh * nhg + hg) * 16 + n]; }
    __device__ float token_value(int kvh, int c) const {
        const float v = new_v[(size_t)kvh * D + c];
        return new_bf16 ? bf16_bits_to_f32(f32_to_bf16_bits(v)) : v;
    }
    // row rr of kv head kvh's row list (token rr / hpk, head rr % hpk of the group) -> row of out, or -1
    __device__ int64_t row(int kvh, int rr) const {
        if (rr >= n_tok * hpk) return -1;
        return (int64_t)(rr / hpk) * Hq + kvh * hpk + rr % hpk;
    }
};

__device__ inline float merge_gate(const float *gate, float x) { return gate ? 1.0f / (1.0f + expf(-x)) : 1.0f; }

static constexpr int kMergeRows = 8;  // partial rows a thread keeps in flight

// Many splits.  A team of 256 threads (ttid = 0..255) combines channels [c0, c0 + 64 NU) of row n:
// 16 lanes x float4 cover 64 channels of one split's row, 16 such rows per pass.  Every wave forms
// the overall maximum and the denominator by itself (lane reads the (max, sum) of splits lane,
// lane + 64, ..., and the maxima of the splits whose rows it combines), so nothing waits for
// another wave until the 16 row sums meet in LDS, and every request - split statistics, rows,
// gate - is made before the first value is used: one memory round trip and one barrier.
// Called by whole workgroups with a uniform `active` per team; contains two workgroup barriers.
template <int NU, bool TOK = false, typename Reader>
__device__ inline void merge_span(const Reader &rd, int nsplit, int D, bool active, int n, int c0, int64_t orow,
                                  const float *gate, float *out, int ttid, float4 (*acc4)[16][16],
                                  int gate_stride, const float *tok_score_at = nullptr, const float *tok_value_at = nullptr,
                                  int tok_bf16 = 0) {
    constexpr int R = kMergeRows / NU;
    const int lane = ttid & 63, dl = ttid & 15, sg = ttid >> 4;
    // split s of row n: maximum at statistic 32 s + n, sum at 32 s + n + 16
    float ms[4], ls[4];   // splits lane + 64 r (the first 256; beyond that, see the loops below)
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int s = lane + 64 * r;
        const bool ok = active && s < nsplit;
        ms[r] = ok ? rd.stat(s * 32 + n) : neg_inf();
        ls[r] = ok ? rd.stat(s * 32 + n + 16) : 0.f;
    }
    float mo[R];          // maxima of the splits whose rows this thread combines
    float4 rows[NU][R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int s = sg + 16 * r;
        const bool ok = active && s < nsplit;
        mo[r] = ok ? rd.stat(s * 32 + n) : neg_inf();
#pragma unroll
        for (int u = 0; u < NU; u++)
            rows[u][r] = ok ? rd.row4((s * 16 + n) * D + c0 + 64 * u + dl * 4) : float4{0.f, 0.f, 0.f, 0.f};
    }
    const bool writer = active && ttid < 64 * NU;
    const float gt_in = (gate && writer) ? gate[orow * gate_stride + c0 + ttid] : 0.f;
    // TOK: the row's score against the new token and this thread's element of the token's value row,
    // requested with everything else (no branch: both addresses are valid for every thread)
    float tok_score = neg_inf(), tok_value = 0.f;
    if constexpr (TOK) {
        tok_score = *tok_score_at;
        const float v = *tok_value_at;
        tok_value = tok_bf16 ? bf16_bits_to_f32(f32_to_bf16_bits(v)) : v;
    }

    float m = fmaxf(fmaxf(ms[0], ms[1]), fmaxf(ms[2], ms[3]));
    if (active)
        for (int s = lane + 256; s < nsplit; s += 64) m = fmaxf(m, rd.stat(s * 32 + n));
    const float M = TOK ? fmaxf(wave_max(m), tok_score) : wave_max(m);
    auto weight = [&](float ms_) { return (ms_ == neg_inf()) ? 0.f : fast_exp2(ms_ - M); };
    float den = 0.f;
#pragma unroll
    for (int r = 0; r < 4; r++) den += weight(ms[r]) * ls[r];
    if (active)
        for (int s = lane + 256; s < nsplit; s += 64) den += weight(rd.stat(s * 32 + n)) * rd.stat(s * 32 + n + 16);
    den = group_sum<64>(den);
    if (TOK) den += weight(tok_score);   // the single position's sum is 1

    float4 acc[NU];
#pragma unroll
    for (int u = 0; u < NU; u++) acc[u] = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float w = weight(mo[r]);
        if (w != 0.f) {   // a split without rows left its part of part_o unwritten
#pragma unroll
            for (int u = 0; u < NU; u++) {
                acc[u].x += w * rows[u][r].x; acc[u].y += w * rows[u][r].y;
                acc[u].z += w * rows[u][r].z; acc[u].w += w * rows[u][r].w;
            }
        }
    }
    if (active)
        for (int s = sg + 16 * R; s < nsplit; s += 16) {
            const float w = weight(rd.stat(s * 32 + n));
            if (w != 0.f) {
#pragma unroll
                for (int u = 0; u < NU; u++) {
                    const float4 v = rd.row4((s * 16 + n) * D + c0 + 64 * u + dl * 4);
                    acc[u].x += w * v.x; acc[u].y += w * v.y; acc[u].z += w * v.z; acc[u].w += w * v.w;
                }
            }
        }
#pragma unroll
    for (int u = 0; u < NU; u++) acc4[u][sg][dl] = acc[u];
    __syncthreads();
    if (writer) {
        // thread -> one scalar output: span u, float4 lane t/4, component t%4
        const int u = ttid >> 6, t = ttid & 63, ql = t >> 2, qc = t & 3;
        float sum = 0.f;
#pragma unroll
        for (int x = 0; x < 16; x++) sum += ((const float *)&acc4[u][x][ql])[qc];
        if (TOK) sum += weight(tok_score) * tok_value;
        out[orow * D + c0 + ttid] = (sum / den) * merge_gate(gate, gt_in);
    }
    __syncthreads();   // acc4 may be written again by the next call
}

// Few splits (at most NS = 8 or 16).  One wave combines UPW units of 64 outputs (unit u of a row
// group: row u / (D/64), channels 64 (u % (D/64)) ...): lane = channel, lane s also holds split
// s's (max, sum); a lane's output is the weighted sum of one float per split, all of them - for
// all the wave's units - requested before the first use.  No LDS, no barrier.
template <int NS, int UPW, bool TOK = false, typename Reader>
__device__ inline void merge_few_units(const Reader &rd, int nsplit, int kvh, int hg, int u_first, int u_end,
                                       const MergeOut &mo, int lane) {
    const int D = mo.D, per_row = D / 64;
    const int sl = lane < nsplit ? lane : nsplit - 1;
    float m_in[UPW], l_in[UPW], gt_in[UPW], ts_in[UPW], tv_in[UPW], rows[UPW][NS];
    int64_t orow[UPW];
    int ch[UPW];
#pragma unroll
    for (int i = 0; i < UPW; i++) {
        int u = u_first + i;
        orow[i] = u < u_end ? mo.row(kvh, hg * 16 + u / per_row) : -1;
        if (orow[i] < 0) u = 0;                    // nothing to do: harmless addresses
        const int n = u / per_row;
        ch[i] = (u % per_row) * 64 + lane;
        m_in[i] = rd.stat(sl * 32 + n);
        l_in[i] = rd.stat(sl * 32 + n + 16);
#pragma unroll
        for (int s = 0; s < NS; s++) rows[i][s] = rd.row1(((s < nsplit ? s : nsplit - 1) * 16 + n) * D + ch[i]);
        gt_in[i] = (mo.gate && orow[i] >= 0) ? mo.gate[orow[i] * mo.gate_stride + ch[i]] : 0.f;
        ts_in[i] = TOK ? mo.token_score(kvh, hg, n) : neg_inf();
        tv_in[i] = TOK ? mo.token_value(kvh, ch[i]) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < UPW; i++) {
        const float ms = lane < nsplit ? m_in[i] : neg_inf();
        const float M = TOK ? fmaxf(wave_max(ms), ts_in[i]) : wave_max(ms);
        const float w = (ms == neg_inf()) ? 0.f : fast_exp2(ms - M);
        const float wt = (!TOK || ts_in[i] == neg_inf()) ? 0.f : fast_exp2(ts_in[i] - M);
        const float den = group_sum<64>(w * (lane < nsplit ? l_in[i] : 0.f)) + wt;
        float acc = wt * tv_in[i];
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const float ws = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, w), s));
            if (ws != 0.f) acc += ws * rows[i][s];   // 0 for s >= nsplit and for a split without rows (unwritten)
        }
        if (orow[i] >= 0) mo.out[orow[i] * D + ch[i]] = (acc / den) * merge_gate(mo.gate, gt_in[i]);
    }
}

// One 64-output unit of a deferred merge (what a wave of sdpa_merge_few_kernel<16> does), for
// launches that carry such a merge in workgroups of their own.
__device__ inline void sdpa_merge_unit(const SdpaMergeTask &t, int unit, int lane) {
    const int per_row = t.D / 64, bx = unit / per_row, by = unit % per_row;
    const int h = bx % t.Hq, tok = bx / t.Hq;
    const int kvh = h / t.hpk, rr = tok * t.hpk + h % t.hpk, hg = rr / 16, n = rr % 16;
    const size_t pid0 = ((size_t)kvh * t.nhg + hg) * t.nsplit;
    const int u = n * per_row + by;
    const MergeOut mo{t.gate, t.out, t.hpk, t.Hq, (t.n_units / per_row) / t.Hq, t.D, t.D, nullptr, nullptr, 0, t.nhg};
    merge_few_units<16, 1, false>(PartialsPlain(t.part_o, t.part_ml, pid0, t.D), t.nsplit, kvh, hg, u, u + 1, mo, lane);
}

}  // namespace mfa
