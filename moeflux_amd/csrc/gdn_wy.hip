// The delta rule over a prompt chunk in blocked form, on the matrix cores.
//
// The reference steps the recurrence token by token (crates/moeflux/src/riir/
// linear_attn.rs:373-411; eval_prompt is a token loop, riir/mod.rs:1196-1214):
//   S <- g_t S;  d_t = beta_t (v_t - S k_t);  S <- S + d_t k_t^T;  o_t = S q_t.
// For a block of C = 64 tokens that starts from state S0, with L_t = sum_{i<=t} log g_i,
//   A[i][j] = beta_i e^{L_i-L_j} (k_i . k_j)  (j < i),      T = (I + A)^-1,
//   W  = T diag(beta e^L) K,   U = T diag(beta) V,   M[i][j] = e^{L_i-L_j} (q_i . k_j)  (j <= i),
//   D  = U - W S0^T                      (the d_t of the block, one row per token)
//   O  = diag(e^L) Q S0^T + M D
//   S' = e^{L_C} S0 + D^T diag(e^{L_C-L}) K
// are the same d_t, o_t and final state (exact arithmetic; f32 rounding differs at 1e-6).
// A token whose decay is zero (the reference's exp underflows, or its softplus overflows) starts L
// afresh: factors across it are exactly 0, as they are token by token.
// Everything before D depends on the inputs only and is computed for all blocks of the
// chunk at once (gdn_wy_kernel, one workgroup per (block, value head)); the four
// products that involve the state run block after block with the state in registers
// (gdn_wy_recur_kernel, one workgroup per 16 rows of a head's state, rows being
// independent).  All products are v_mfma_f32_16x16x4_f32.
//
// Operand conventions of that instruction (lane l, m = n = l % 16, g = l / 16):
// A[m][g], B[g][n] in; D[4g+i][n], i = 0..3, out.  A contraction over 16 values is done as
// 4 instructions i = 0..3 in which lane group g contributes value number 4g+i: then one
// float4 (values 4g..4g+3) feeds the four instructions, and a D tile can be used as the
// B operand of a contraction over its rows without moving data between lanes.
#include <type_traits>

#include "gdn_device.h"

namespace mfa {

typedef __attribute__((ext_vector_type(4))) float wy_f32x4;

static constexpr int kC = 64;  // tokens per block

__device__ inline wy_f32x4 mfma4(float4 a, float4 b, wy_f32x4 acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, acc, 0, 0, 0);
    return acc;
}
__device__ inline float4 lds_f4(const float *p) {
    const gdn_f32x4 v = *reinterpret_cast<const gdn_f32x4 *>(p);
    return float4{v.x, v.y, v.z, v.w};
}
// Value head served by the workgroups with x index bx.  Workgroups go to the 8 XCDs in turn, so with a
// head count that is a multiple of 8 a head's workgroups share an XCD and its L2; heads that share a
// k head (and read the same q and k inputs) are given x indices 8 apart, the same XCD, so that the
// second reader of a line finds it in that L2 (block precompute 22.3 -> 21.6 us per 512 tokens).
__device__ inline int wy_head_of(int bx, int Hk, int Hv) {
    const int r = Hv / Hk;
    if (Hv % 8 != 0 || (Hv / 8) % r != 0) return bx;
    const int x = bx & 7, j = bx >> 3;
    return (x + 8 * (j / r)) * r + j % r;
}
__device__ inline float4 as_f4(wy_f32x4 v) { return float4{v[0], v[1], v[2], v[3]}; }
// a 16-byte load kept as a vector register value (members of a struct of operands)
__device__ inline wy_f32x4 load_v4(const float *p) { return *reinterpret_cast<const wy_f32x4 *>(p); }

// Per (block, value head) outputs, block-major then head, each cut into 16x16 tiles that
// are stored the way the recurrence kernel's lanes read them, 16 bytes per lane and
// 1 KiB per tile (a row-major matrix read as an A operand has neighbouring lanes 512
// bytes apart, which the memory pipeline serves at a fraction of its rate):
//   Wt [token tile w][col tile c], Qt likewise, Mt [w][token tile tau], Kt [col tile c][tau]
//   (= diag(e^{L_C-L}) K transposed): lane (m, g) holds X[16 row-tile + m][16 col-tile + 4g + i];
//   Ut [w][col tile c]: lane (n, g) holds U[16w + 4g + i][16c + n]  (a D tile as computed);
//   eL [64] (e^{L_t}; eL[63] = e^{L_C} because padded tokens do not decay).
// Tokens past the end of the chunk are padded with beta = 0, log g = 0, k = q = v = 0.
//
// grid (Hv, blocks), one wave per 16 columns of K (DK/16 waves: two per SIMD at DK = 128, so that one
// has matrix work while the other waits for LDS or stores a tile).
// FUSED: the block's inputs come straight from the layer's inputs (WyInputs): what
// gdn_chunk_pre_kernel computes for the token-by-token form is done here per (block, value head) -
// conv + SiLU of the head's q, k and v channels, the per-token q/k norm, the decay's logarithm and
// beta - so the chunk needs no launch and no arrays for them.  A k-head's q and k are formed by
// each of the value heads that share it.
template <int DK, bool FUSED>
__global__ __launch_bounds__(DK * 4) void gdn_wy_kernel(
    int Hk, int Hv, int T, const float *__restrict__ qn, const float *__restrict__ kn,
    const float *__restrict__ vv, const float *__restrict__ lg, const float *__restrict__ bg,
    float *__restrict__ Wt, float *__restrict__ Qt, float *__restrict__ Ut, float *__restrict__ Mt,
    float *__restrict__ Kt, float *__restrict__ eLc, WyInputs in) {
    constexpr int DV = DK;
    constexpr int NK = DK / 16;
    constexpr int LDK = DK + 4;  // row strides chosen so that 16-byte row reads by 8 lanes hit all banks
    constexpr int LDC = kC + 4;
    constexpr int NW = NK;        // waves
    constexpr int NTHR = 64 * NW;
    constexpr int NCT = 1;        // 16-wide column tiles of W (and of U) per wave
    __shared__ __align__(16) float sK[kC][LDK];
    __shared__ __align__(16) float sQ[kC][LDK];  // q^, later v (FUSED: q^ only)
    __shared__ __align__(16) float sV[FUSED ? kC : 1][LDK];
    __shared__ __align__(16) float sA[kC][LDC];
    __shared__ __align__(16) float sT[kC][LDC];
    __shared__ __align__(16) float sL[kC], sB[kC], sCw[kC], sKd[kC];
    __shared__ int sR[kC];

    // heads along x: a head's blocks are produced on the XCD whose L2 the recurrence kernel
    // (heads along x as well) will read them through
    const int vh = wy_head_of(blockIdx.x, Hk, Hv), blk = blockIdx.y, kh = vh / (Hv / Hk);
    const int t0 = blk * kC;
    const int nt = (T - t0 < kC) ? T - t0 : kC;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 15, g = lane >> 4;
    const size_t slot = (size_t)blk * Hv + vh;

    // ---- phase 0: k^, q^ of the block, cumulative log decay, beta ---------------------
    // Everything the block reads is requested here, in the order of use (loads return in the
    // order of their requests): the gates, k^ and q^, and v, which waits in registers for phase 2.
    float lg_in = 0.f, bg_in = 0.f;
    constexpr int NLV = kC * (DV / 4) / NTHR;
    float4 va[FUSED ? 1 : NLV];
    if constexpr (FUSED) {
        constexpr int NCONV = 2 * DK + DV, TT = 16;          // channels of the head; tokens per run
        constexpr int NU = NCONV * (kC / TT) / NTHR;          // (channel, run) units per thread
        static_assert(NCONV * (kC / TT) % NTHR == 0, "whole units per thread");
        const int C = 2 * Hk * DK + Hv * DV;
        float a_in = 0.f, b_in = 0.f, al_in = 0.f, dt_in = 0.f;
        if (wave == 0 && lane < nt) {
            a_in = in.alpha[(size_t)(t0 + lane) * Hv + vh];
            b_in = in.beta[(size_t)(t0 + lane) * Hv + vh];
            al_in = in.a_log[vh];
            dt_in = bf16_bits_to_f32(in.dt_bias[vh]);
        }
        // conv + SiLU (linear_attn.rs:132-154) of channel c over a run of 16 tokens per unit.
        // First every request of every unit: a run's TT + 3 inputs, oldest first, are rows of the
        // chunk, or ring slots for inputs from before it.  Every load is unconditional (the address
        // is selected; rows past the chunk's end re-read its last row and only feed outputs that
        // are zeroed below), so all of a thread's requests are in flight at once instead of one
        // memory round trip per input or per unit.
        // (Conv width 4 only; the launcher sends other widths through the separate first kernel.)
        float xs[NU][TT + 3];
        uint2 wbits[NU];
        const float *blk_rows = in.qkv + (size_t)t0 * C;   // the block's first row: offsets from here fit 32 bits
#pragma unroll
        for (int u = 0; u < NU; u++) {
            const int unit = tid + u * NTHR, c = unit % NCONV, run = unit / NCONV;
            const int ch = c < DK ? kh * DK + c : c < 2 * DK ? Hk * DK + kh * DK + (c - DK) : 2 * Hk * DK + vh * DV + (c - 2 * DK);
            wbits[u] = *(const uint2 *)(in.conv_w + (unsigned)ch * 4u);
#pragma unroll
            for (int j = 0; j < TT + 3; j++) {
                const int rel = TT * run - 3 + j;          // row relative to the block's first
                const int idx = t0 + rel;
                const int last = T - 1 - t0;
                if (rel < 0) {                              // compile-time for all but the first run
                    const int off = (idx < 0 ? ((in.step_mod + idx + 4) & 3) : rel) * C + ch;
                    xs[u][j] = (idx < 0 ? in.ring : blk_rows)[off];
                } else {
                    xs[u][j] = blk_rows[(rel > last ? last : rel) * C + ch];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < NU; u++) {
            const int unit = tid + u * NTHR, c = unit % NCONV, run = unit / NCONV;
            const int tr = t0 + TT * run;
            int ntr = T - tr;
            ntr = ntr < 0 ? 0 : ntr > TT ? TT : ntr;
            const float wt[4] = {bf16_bits_to_f32((uint16_t)(wbits[u].x & 0xffffu)), bf16_bits_to_f32((uint16_t)(wbits[u].x >> 16)),
                                 bf16_bits_to_f32((uint16_t)(wbits[u].y & 0xffffu)), bf16_bits_to_f32((uint16_t)(wbits[u].y >> 16))};
            float(*dst)[LDK] = c < DK ? sQ : c < 2 * DK ? sK : sV;
            const int cc = c < DK ? c : c < 2 * DK ? c - DK : c - 2 * DK;
#pragma unroll
            for (int i = 0; i < TT; i++) {
                float acc = 0.f;
#pragma unroll
                for (int k = 0; k < 4; k++) acc = fmaf(xs[u][i + k], wt[k], acc);
                dst[TT * run + i][cc] = i < ntr ? silu_f(acc) : 0.f;
            }
        }
        if (wave == 0 && lane < nt) {
            // shaders.metal:1321-1326; the decay enters as its logarithm
            const float a_cap = expf(al_in);
            const float sp = logf(1.0f + expf(a_in + dt_in));
            lg_in = -a_cap * sp;
            bg_in = 1.0f / (1.0f + expf(-b_in));
        }
        __syncthreads();
        // per-token norm of q and k (infer.m:2655-2667: x * inv_rms, then q *= (1/sqrt(dk))^2,
        // k *= 1/sqrt(dk)): NTHR / (2 kC) lanes per (token, q|k) row, in place
        constexpr int LPP = NTHR / (2 * kC), EPL = DK / LPP;   // lanes per row, elements per lane
        static_assert(LPP == 2 || LPP == 4, "lanes per normed row");
        {
            const int p = tid / LPP, sub = tid % LPP, tt = p % kC;
            const bool is_q = p < kC;
            float *row = (is_q ? sQ[tt] : sK[tt]) + EPL * sub;
            float4 x[EPL / 4];
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < EPL / 4; i++) {
                x[i] = lds_f4(row + 4 * i);
                ss += x[i].x * x[i].x + x[i].y * x[i].y + x[i].z * x[i].z + x[i].w * x[i].w;
            }
            ss = dpp_add<0xB1>(ss);
            if (LPP == 4) ss = dpp_add<0x4E>(ss);
            const float inv_scale = 1.0f / sqrtf((float)DK);
            const float inv_rms = 1.0f / sqrtf(ss / (float)DK + 1e-6f);
            const float sc = is_q ? inv_scale * inv_scale : inv_scale;
#pragma unroll
            for (int i = 0; i < EPL / 4; i++) {
                float4 y = {x[i].x * inv_rms, x[i].y * inv_rms, x[i].z * inv_rms, x[i].w * inv_rms};
                y.x *= sc; y.y *= sc; y.z *= sc; y.w *= sc;
                *(float4 *)(row + 4 * i) = y;
            }
        }
    } else {
    if (wave == 0 && lane < nt) {
        lg_in = lg[(size_t)(t0 + lane) * Hv + vh];
        bg_in = bg[(size_t)(t0 + lane) * Hv + vh];
    }
    {
        constexpr int NL = kC * (DK / 4) / NTHR;
        float4 a[NL], b[NL];
#pragma unroll
        for (int u = 0; u < NL; u++) {
            const int i = tid + u * NTHR, tt = i / (DK / 4), x = (i % (DK / 4)) * 4;
            const size_t src = ((size_t)(t0 + (tt < nt ? tt : nt - 1)) * Hk + kh) * DK + x;
            a[u] = load_f4(kn + src);
            b[u] = load_f4(qn + src);
        }
#pragma unroll
        for (int u = 0; u < NLV; u++) {
            const int i = tid + u * NTHR, tt = i / (DV / 4), x = (i % (DV / 4)) * 4;
            va[u] = load_f4(vv + ((size_t)(t0 + (tt < nt ? tt : nt - 1)) * Hv + vh) * DV + x);
        }
#pragma unroll
        for (int u = 0; u < NL; u++) {
            const int i = tid + u * NTHR, tt = i / (DK / 4), x = (i % (DK / 4)) * 4;
            const float keep = tt < nt ? 1.f : 0.f;  // padded tokens are zero rows
            *(float4 *)&sK[tt][x] = float4{a[u].x * keep, a[u].y * keep, a[u].z * keep, a[u].w * keep};
            *(float4 *)&sQ[tt][x] = float4{b[u].x * keep, b[u].y * keep, b[u].z * keep, b[u].w * keep};
        }
    }
    }
    if (wave == 0) {
        // Cumulative log decay, restarted after every token whose decay is zero: where the
        // reference's exp() underflows (log g below log FLT_MIN; -inf when its softplus overflows,
        // linear_attn.rs:357-370) the token forgets everything before it, and no factor e^{L_i-L_j}
        // may be formed across it (-inf - -inf).  sR[t] is the last such token up to and
        // including t (-1: none); a pair (row, col) decays to exactly 0 when sR[row] > col.
        const bool dead = lg_in < -87.3f;
        float l = dead ? 0.f : lg_in;
        bool seg = dead;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const float u = __shfl_up(l, d, 64);
            const int su = __shfl_up((int)seg, d, 64);
            if (lane >= d) {
                if (!seg) l += u;
                seg = seg || su;
            }
        }
        const unsigned long long kills = __ballot(dead) & ((2ull << lane) - 1ull);
        const int r = kills ? 63 - __builtin_clzll(kills) : -1;
        const float b = bg_in;
        const float el = r >= 0 ? 0.f : expf(l);      // decay since the block's first token
        sL[lane] = l;
        sR[lane] = r;
        sB[lane] = b;
        sCw[lane] = b * el;
        eLc[slot * kC + lane] = el;
        sKd[lane] = __shfl(r, 63, 64) > lane ? 0.f : expf(__shfl(l, 63, 64) - l);  // e^{L_C - L_t}
    }
    __syncthreads();

    // ---- phase 1: the lower tiles of K K^T (-> A) and of Q K^T (-> M) -----------------
    // 10 tiles (I, J <= I) each; 20 jobs of DK/4 instructions dealt round the waves.
#pragma unroll
    for (int r = 0; r < (20 + NW - 1) / NW; r++) {
        const int job = wave + NW * r;
        if (job >= 20) break;   // uniform over the wave
        const int kind = job / 10, idx = job % 10;
        const int I = idx >= 6 ? 3 : idx >= 3 ? 2 : idx >= 1 ? 1 : 0;
        const int J = idx - I * (I + 1) / 2;
        wy_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        if (kind == 0) {
#pragma unroll
            for (int s = 0; s < DK / 16; s++)
                acc = mfma4(lds_f4(&sK[16 * I + m][16 * s + 4 * g]), lds_f4(&sK[16 * J + m][16 * s + 4 * g]), acc);
            // lane (n = m, g) holds rows 16I + 4g + i of column 16J + n
            const int col = 16 * J + m;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = 16 * I + 4 * g + i;
                const float dl = sL[row] - sL[col];
                const float d = sR[row] > col ? 0.f : __builtin_amdgcn_exp2f((dl < 0.f ? dl : 0.f) * 1.4426950408889634f);  // v_exp_f32: 1 ulp
                sA[row][col] = (col < row) ? sB[row] * d * acc[i] : 0.f;
            }
        } else {
            // the tile transposed (k^ as the A side): lane (n = m, g) then holds columns 16J + 4g + i of
            // row 16I + n, which is this lane's 16 bytes of tile (I, J) in A-operand order
#pragma unroll
            for (int s = 0; s < DK / 16; s++)
                acc = mfma4(lds_f4(&sK[16 * J + m][16 * s + 4 * g]), lds_f4(&sQ[16 * I + m][16 * s + 4 * g]), acc);
            const int row = 16 * I + m;
            wy_f32x4 mv;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int col = 16 * J + 4 * g + i;
                const float dl = sL[row] - sL[col];
                const float d = sR[row] > col ? 0.f : __builtin_amdgcn_exp2f((dl < 0.f ? dl : 0.f) * 1.4426950408889634f);
                mv[i] = (col <= row) ? d * acc[i] : 0.f;
            }
            *reinterpret_cast<wy_f32x4 *>(Mt + ((slot * 4 + I) * 4 + J) * 256 + lane * 4) = mv;
        }
    }
    for (int i = tid; i < 4 * NK * 64; i += NTHR) {  // q^ tiles, before v takes its place
        const int tile = i >> 6, l = i & 63, w = tile / NK, c = tile % NK;
        *(float4 *)(Qt + (slot * 4 * NK + tile) * 256 + l * 4) = lds_f4(&sQ[16 * w + (l & 15)][16 * c + 4 * (l >> 4)]);
    }
    __syncthreads();

    // ---- phase 2: diag(e^{L_C - L}) K transposed goes out, v comes in, and
    //      T = (I + A)^-1 by blocks of 16: the diagonal blocks by forward substitution (one
    //      per wave, a column per lane), the blocks below them level by level from
    //      T_IJ = -T_II sum_{J <= K < I} A_IK T_KJ on the matrix cores -----------------------
    {
#pragma unroll
        for (int u = 0; u < NK * 4 * 64 / NTHR; u++) {
            const int i = tid + u * NTHR, tile = i >> 6, l = i & 63, c = tile >> 2, tau = tile & 3;
            const int kk = 16 * c + (l & 15), j4 = 16 * tau + 4 * (l >> 4);
            const float4 e = lds_f4(&sKd[j4]);
            const float4 o = {e.x * sK[j4 + 0][kk], e.y * sK[j4 + 1][kk], e.z * sK[j4 + 2][kk], e.w * sK[j4 + 3][kk]};
            *(float4 *)(Kt + (slot * NK * 4 + tile) * 256 + l * 4) = o;
        }
        if constexpr (!FUSED) {
#pragma unroll
            for (int u = 0; u < NLV; u++) {
                const int i = tid + u * NTHR, tt = i / (DV / 4), x = (i % (DV / 4)) * 4;
                const float keep = tt < nt ? 1.f : 0.f;
                *(float4 *)&sQ[tt][x] = float4{va[u].x * keep, va[u].y * keep, va[u].z * keep, va[u].w * keep};
            }
        }
    }
    if (wave < 4) {
        // block `wave`; the four lane groups compute the same 16 columns, group 0 stores
        const int r0 = 16 * wave;
        float t[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float acc = (i == m) ? 1.f : 0.f;
#pragma unroll
            for (int j4 = 0; j4 < i; j4 += 4) {
                const float4 a = lds_f4(&sA[r0 + i][r0 + j4]);  // the same address in every lane
                acc = fmaf(-a.x, t[j4], acc);
                if (j4 + 1 < i) acc = fmaf(-a.y, t[j4 + 1], acc);
                if (j4 + 2 < i) acc = fmaf(-a.z, t[j4 + 2], acc);
                if (j4 + 3 < i) acc = fmaf(-a.w, t[j4 + 3], acc);
            }
            t[i] = acc;
            if (g == 0) sT[r0 + i][r0 + m] = acc;
        }
    }
    __syncthreads();
#pragma unroll
    for (int lvl = 1; lvl < 4; lvl++) {
        if (wave < 4 - lvl) {  // block (I, J) = (wave + lvl, wave)
            const int I = wave + lvl, J = wave;
            wy_f32x4 x = {0.f, 0.f, 0.f, 0.f};
            for (int K = J; K < I; K++) {
                float4 bt;
                bt.x = sT[16 * K + 4 * g + 0][16 * J + m];
                bt.y = sT[16 * K + 4 * g + 1][16 * J + m];
                bt.z = sT[16 * K + 4 * g + 2][16 * J + m];
                bt.w = sT[16 * K + 4 * g + 3][16 * J + m];
                x = mfma4(lds_f4(&sA[16 * I + m][16 * K + 4 * g]), bt, x);
            }
            // x is held as rows 4g+i of column m: already the B operand of T_II x
            wy_f32x4 r = {0.f, 0.f, 0.f, 0.f};
            r = mfma4(lds_f4(&sT[16 * I + m][16 * I + 4 * g]), as_f4(x), r);
#pragma unroll
            for (int i = 0; i < 4; i++) sT[16 * I + 4 * g + i][16 * J + m] = -r[i];
        }
        __syncthreads();
    }

    // ---- phase 3: W = T diag(beta e^L) K and U = T diag(beta) V -------------------------
    // Wave w owns column tiles NCT*w .. of both; the K and V operands of those columns are
    // read once and serve all four token tiles.
    float bK[4][NCT][4], bV[4][NCT][4];
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
        for (int ct = 0; ct < NCT; ct++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                bK[s][ct][i] = sK[16 * s + 4 * g + i][16 * (NCT * wave + ct) + m];
                bV[s][ct][i] = (FUSED ? sV : sQ)[16 * s + 4 * g + i][16 * (NCT * wave + ct) + m];
            }
#pragma unroll
    for (int tau = 0; tau < 4; tau++) {
        wy_f32x4 aw4[NCT], au4[NCT];
#pragma unroll
        for (int ct = 0; ct < NCT; ct++) aw4[ct] = au4[ct] = wy_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s <= tau; s++) {
            const float4 t4 = lds_f4(&sT[16 * tau + m][16 * s + 4 * g]);
            const float4 cw = lds_f4(&sCw[16 * s + 4 * g]), cb = lds_f4(&sB[16 * s + 4 * g]);
            const float4 tw = {t4.x * cw.x, t4.y * cw.y, t4.z * cw.z, t4.w * cw.w};
            const float4 tu = {t4.x * cb.x, t4.y * cb.y, t4.z * cb.z, t4.w * cb.w};
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) {
                // W transposed (K as the A side): lane (n = m, g) then holds columns 16c + 4g + i of
                // token 16 tau + n, its 16 bytes of the tile in A-operand order
                aw4[ct] = mfma4(float4{bK[s][ct][0], bK[s][ct][1], bK[s][ct][2], bK[s][ct][3]}, tw, aw4[ct]);
                au4[ct] = mfma4(tu, float4{bV[s][ct][0], bV[s][ct][1], bV[s][ct][2], bV[s][ct][3]}, au4[ct]);
            }
        }
#pragma unroll
        for (int ct = 0; ct < NCT; ct++) {
            const wy_f32x4 aw = aw4[ct], au = au4[ct];
            const size_t tile = (slot * 4 + tau) * NK + NCT * wave + ct;
            // U as computed (a D tile), W in A-operand order
            *reinterpret_cast<wy_f32x4 *>(Ut + tile * 256 + lane * 4) = au;
            *reinterpret_cast<wy_f32x4 *>(Wt + tile * 256 + lane * 4) = aw;
        }
    }
}

// grid (Hv, DV/16), 256 threads.  The 16 rows of the state are kept by every wave, in the
// layout of a D tile per 16 columns (lane (n, g): S[row0+n][16c+4g+i]), which is also the B
// operand of a contraction over the columns.  Wave w serves tokens 16w .. 16w+15 of each
// block and the column tiles (DK/64)*w .. of the state update.
template <int DK>
__global__ __launch_bounds__(256) void gdn_wy_recur_kernel(
    int Hk, int Hv, int T, const float *__restrict__ Wt, const float *__restrict__ Qt,
    const float *__restrict__ Ut, const float *__restrict__ Mt, const float *__restrict__ Kt,
    const float *__restrict__ eLc, float *__restrict__ ssm, float *__restrict__ o_raw) {
    constexpr int DV = DK;
    constexpr int NK = DK / 16;   // column tiles of the state
    constexpr int NKW = NK / 4;   // of which a wave updates
    __shared__ wy_f32x4 s_d[4][64];    // D tiles of the block, by token tile
    __shared__ wy_f32x4 s_st[NK][64];  // the updated state

    const int vh = wy_head_of(blockIdx.x, Hk, Hv), row0 = blockIdx.y * 16;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = lane & 15, g = lane >> 4;
    float *srow = ssm + ((size_t)vh * DV + row0 + m) * DK + 4 * g;
    wy_f32x4 st[NK];
#pragma unroll
    for (int c = 0; c < NK; c++) {
        const float4 v = load_f4(srow + 16 * c);
        st[c] = wy_f32x4{v.x, v.y, v.z, v.w};
    }

    // A block's operands live in registers and are requested one block ahead, all of them
    // before the block's first barrier: the W and q^ rows of this wave's tokens and its U
    // entries into the registers the block has just consumed, its M rows, e^L and the K
    // columns of its share of the update into a second set (two blocks per loop pass,
    // the sets swapping roles).  Requests past the last block re-read it.
    const int nblk = (T + kC - 1) / kC;
    struct Late {
        wy_f32x4 mt[4], kd[NKW][4], el;
        float elc;
    };
    float4 pw[NK], pq[NK], pu;
    auto slot_of = [&](int blk) { return (size_t)(blk < nblk ? blk : nblk - 1) * Hv + vh; };
    // The requests for the next block are issued between the matrix instructions of the
    // first product (an instruction occupies the matrix core for 32 clocks, the wave's issue
    // slot for a few), column tile by column tile as its W and q^ registers come free;
    // the second set's 6 + 4*NKW requests are spread over the same loop.
    auto fetch_wq = [&](int blk, int c) __attribute__((always_inline)) {
        const size_t off = (slot_of(blk) * 4 + wave) * NK * 256 + lane * 4;
        pw[c] = load_f4(Wt + off + c * 256);
        pq[c] = load_f4(Qt + off + c * 256);
    };
    auto fetch_u = [&](int blk) __attribute__((always_inline)) {
        pu = load_f4(Ut + ((slot_of(blk) * 4 + wave) * NK + blockIdx.y) * 256 + lane * 4);
    };
    constexpr int NLATE = 6 + 4 * NKW;                 // requests of a Late set
    constexpr int LATE_PER_C = (NLATE + NK - 1) / NK;  // of which per column tile
    auto fetch_late = [&](Late &p, int blk, int j) __attribute__((always_inline)) {
        const size_t slot = slot_of(blk);
        if (j < 4) p.mt[j] = load_v4(Mt + ((slot * 4 + wave) * 4 + (j <= wave ? j : wave)) * 256 + lane * 4);
        else if (j == 4) p.el = load_v4(eLc + slot * kC + 16 * wave + 4 * g);
        else if (j == 5) p.elc = eLc[slot * kC + kC - 1];
        else if (j < NLATE) {
            const int kt = (j - 6) / 4, tau = (j - 6) % 4;
            p.kd[kt][tau] = load_v4(Kt + ((slot * NK + NKW * wave + kt) * 4 + tau) * 256 + lane * 4);
        }
    };
    auto block = [&](int blk, const Late &cur, Late &nxt) __attribute__((always_inline)) {
        const int t0 = blk * kC;
        // ---- W S0^T and Q S0^T for this wave's 16 tokens ------------------------------
        wy_f32x4 p1 = {0.f, 0.f, 0.f, 0.f}, p2 = p1;
#pragma unroll
        for (int c = 0; c < NK; c++) {
            p1 = mfma4(pw[c], as_f4(st[c]), p1);
            p2 = mfma4(pq[c], as_f4(st[c]), p2);
            fetch_wq(blk + 1, c);
#pragma unroll
            for (int u = 0; u < LATE_PER_C; u++) fetch_late(nxt, blk + 1, c * LATE_PER_C + u);
            // keep this column tile's requests between its matrix instructions (left to itself the
            // scheduler gathers all requests at the end of the product, where nothing hides their issue)
            __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 2 + LATE_PER_C, 0);
        }
        // ---- D = U - W S0^T: lane (n, g) holds tokens 16w+4g+i of state row row0+n ----
        wy_f32x4 d;
        d[0] = pu.x - p1[0]; d[1] = pu.y - p1[1]; d[2] = pu.z - p1[2]; d[3] = pu.w - p1[3];
        fetch_u(blk + 1);
        s_d[wave][lane] = d;
        __syncthreads();
        // ---- O = diag(e^L) Q S0^T + M D ------------------------------------------------
        wy_f32x4 o = cur.el * p2;
#pragma unroll
        for (int tau = 0; tau < 4; tau++)
            if (tau <= wave) o = mfma4(as_f4(cur.mt[tau]), as_f4(s_d[tau][lane]), o);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int t = t0 + 16 * wave + 4 * g + i;
            if (t < T) o_raw[((size_t)t * Hv + vh) * DV + row0 + m] = o[i];
        }
        // ---- S' = e^{L_C} S0 + D^T diag(e^{L_C-L}) K, column tiles NKW*w .. ------------
        // (written out per wave so that the state tile is a compile-time register choice)
        auto update = [&](auto wtag) __attribute__((always_inline)) {
            constexpr int w = decltype(wtag)::value;
#pragma unroll
            for (int kt = 0; kt < NKW; kt++) {
                constexpr int c0 = NKW * w;
                wy_f32x4 acc = st[c0 + kt] * cur.elc;
#pragma unroll
                for (int tau = 0; tau < 4; tau++)
                    acc = mfma4(as_f4(cur.kd[kt][tau]), as_f4(s_d[tau][lane]), acc);
                s_st[c0 + kt][lane] = acc;
            }
        };
        if (wave == 0) update(std::integral_constant<int, 0>{});
        else if (wave == 1) update(std::integral_constant<int, 1>{});
        else if (wave == 2) update(std::integral_constant<int, 2>{});
        else update(std::integral_constant<int, 3>{});
        __syncthreads();
#pragma unroll
        for (int c = 0; c < NK; c++) st[c] = s_st[c][lane];
    };
    Late la, lb;
#pragma unroll
    for (int c = 0; c < NK; c++) fetch_wq(0, c);
    fetch_u(0);
#pragma unroll
    for (int j = 0; j < NLATE; j++) fetch_late(la, 0, j);
    for (int blk = 0; blk < nblk; blk += 2) {
        block(blk, la, lb);
        if (blk + 1 < nblk) block(blk + 1, lb, la);  // uniform over the workgroup
    }
    if (wave == 0) {
#pragma unroll
        for (int c = 0; c < NK; c++) {
            gdn_f32x4 v = {st[c][0], st[c][1], st[c][2], st[c][3]};
            *reinterpret_cast<gdn_f32x4 *>(srow + 16 * c) = v;
        }
    }
}

size_t gdn_wy_scratch_elems(int Hv, int dk, int dv, int T) {
    const size_t nblk = ((size_t)T + kC - 1) / kC;
    return nblk * Hv * (3 * (size_t)kC * dk + (size_t)kC * dv + (size_t)kC * kC + kC);
}

// o_raw [T, Hv*dv].  The blocks' inputs come from the layer's inputs (`in`; qn .. bg are then unused
// and may be null) or, when in is null, from qn, kn [T, Hk, dk]; vv [T, Hv, dv]; lg, bg [T, Hv] (log
// decay, beta gate) as gdn_chunk_pre_kernel leaves them.
int launch_gdn_wy(hipStream_t s, int Hk, int Hv, int dk, int dv, int T, const float *qn, const float *kn,
                  const float *vv, const float *lg, const float *bg, float *scratch, float *ssm,
                  float *o_raw, const WyInputs *in) {
    if (dk != dv || (dk != 64 && dk != 128))
        return fail(MFA_ERR_SHAPE, "gdn blocked form: dk=%d dv=%d not supported", dk, dv);
    const size_t nblk = ((size_t)T + kC - 1) / kC;
    if (nblk > 65535) return fail(MFA_ERR_SHAPE, "gdn blocked form: too many tokens in one call");
    const size_t slots = nblk * Hv;
    float *Wt = scratch;
    float *Qt = Wt + slots * kC * dk;
    float *Kt = Qt + slots * kC * dk;
    float *Ut = Kt + slots * kC * dk;
    float *Mt = Ut + slots * kC * dv;
    float *eLc = Mt + slots * kC * kC;
    const WyInputs none{};
#define MFA_WY(DKK, FU)                                                                                             \
    hipLaunchKernelGGL((gdn_wy_kernel<DKK, FU>), dim3(Hv, (unsigned)nblk), dim3(DKK * 4), 0, s, Hk, Hv, T, qn, kn, vv, \
                       lg, bg, Wt, Qt, Ut, Mt, Kt, eLc, in ? *in : none)
    if (dk == 128) {
        if (in) MFA_WY(128, true); else MFA_WY(128, false);
        hipLaunchKernelGGL((gdn_wy_recur_kernel<128>), dim3(Hv, dv / 16), dim3(256), 0, s, Hk, Hv, T, Wt, Qt, Ut,
                           Mt, Kt, eLc, ssm, o_raw);
    } else {
        if (in) MFA_WY(64, true); else MFA_WY(64, false);
        hipLaunchKernelGGL((gdn_wy_recur_kernel<64>), dim3(Hv, dv / 16), dim3(256), 0, s, Hk, Hv, T, Wt, Qt, Ut,
                           Mt, Kt, eLc, ssm, o_raw);
    }
#undef MFA_WY
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
