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
__device__ inline float4 as_f4(wy_f32x4 v) { return float4{v[0], v[1], v[2], v[3]}; }

// Per (block, value head) outputs, block-major then head:
//   Wc [64][DK], Uc [64][DV], Mc [64][64], KdT [DK][64] (= diag(e^{L_C-L}) K, transposed),
//   eL [64] (e^{L_t}; eL[63] = e^{L_C} because padded tokens do not decay).
// Tokens past the end of the chunk are padded with beta = 0, log g = 0, k = q = v = 0.
//
// grid (blocks, Hv), 256 threads.
template <int DK>
__global__ __launch_bounds__(256) void gdn_wy_kernel(
    int Hk, int Hv, int T, const float *__restrict__ qn, const float *__restrict__ kn,
    const float *__restrict__ vv, const float *__restrict__ lg, const float *__restrict__ bg,
    float *__restrict__ Wc, float *__restrict__ Uc, float *__restrict__ Mc, float *__restrict__ KdT,
    float *__restrict__ eLc) {
    constexpr int DV = DK;
    constexpr int LDK = DK + 4;  // row strides chosen so that 16-byte row reads by 8 lanes hit all banks
    constexpr int LDC = kC + 4;
    constexpr int NCT = DK / 64;  // 16-wide column tiles of W (and of U) per wave
    __shared__ __align__(16) float sK[kC][LDK];
    __shared__ __align__(16) float sQ[kC][LDK];  // q^, later v
    __shared__ __align__(16) float sA[kC][LDC];
    __shared__ __align__(16) float sT[kC][LDC];
    __shared__ __align__(16) float sL[kC], sB[kC], sCw[kC];

    const int blk = blockIdx.x, vh = blockIdx.y, kh = vh / (Hv / Hk);
    const int t0 = blk * kC;
    const int nt = (T - t0 < kC) ? T - t0 : kC;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 15, g = lane >> 4;
    const size_t slot = (size_t)blk * Hv + vh;

    // ---- phase 0: k^, q^ of the block, cumulative log decay, beta ---------------------
    for (int i = tid; i < kC * (DK / 4); i += 256) {
        const int tt = i / (DK / 4), x = (i % (DK / 4)) * 4;
        float4 a = {0.f, 0.f, 0.f, 0.f}, b = a;
        if (tt < nt) {
            const size_t src = ((size_t)(t0 + tt) * Hk + kh) * DK + x;
            a = load_f4(kn + src);
            b = load_f4(qn + src);
        }
        *(float4 *)&sK[tt][x] = a;
        *(float4 *)&sQ[tt][x] = b;
    }
    if (wave == 0) {
        float l = lane < nt ? lg[(size_t)(t0 + lane) * Hv + vh] : 0.f;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const float u = __shfl_up(l, d, 64);
            if (lane >= d) l += u;
        }
        const float b = lane < nt ? bg[(size_t)(t0 + lane) * Hv + vh] : 0.f;
        sL[lane] = l;
        sB[lane] = b;
        sCw[lane] = b * expf(l);
        eLc[slot * kC + lane] = expf(l);
    }
    __syncthreads();

    // ---- phase 1: the lower tiles of K K^T (-> A) and of Q K^T (-> M) -----------------
    // 10 tiles (I, J <= I) each; 20 jobs of DK/4 instructions over 4 waves.
#pragma unroll 1
    for (int r = 0; r < 5; r++) {
        const int job = wave * 5 + r, kind = job / 10, idx = job % 10;
        const int I = idx >= 6 ? 3 : idx >= 3 ? 2 : idx >= 1 ? 1 : 0;
        const int J = idx - I * (I + 1) / 2;
        const float(*X)[LDK] = kind ? sQ : sK;
        wy_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < DK / 16; s++)
            acc = mfma4(lds_f4(&X[16 * I + m][16 * s + 4 * g]), lds_f4(&sK[16 * J + m][16 * s + 4 * g]), acc);
        // lane (n = m, g) holds rows 16I + 4g + i of column 16J + n
        const int col = 16 * J + m;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = 16 * I + 4 * g + i;
            const float dl = sL[row] - sL[col];
            const float d = expf(dl < 0.f ? dl : 0.f);
            if (kind == 0) sA[row][col] = (col < row) ? sB[row] * d * acc[i] : 0.f;
            else Mc[slot * kC * kC + (size_t)row * kC + col] = (col <= row) ? d * acc[i] : 0.f;
        }
    }
    __syncthreads();

    // ---- phase 2: T = (I + A)^-1 by forward substitution, one column per lane of wave 0;
    //      the other waves write diag(e^{L_C - L}) K transposed and bring in v --------------
    if (wave == 0) {
        float t[kC];
#pragma unroll
        for (int i = 0; i < kC; i++) {
            float acc = (i == lane) ? 1.f : 0.f;
#pragma unroll
            for (int j4 = 0; j4 < i; j4 += 4) {
                const float4 a = lds_f4(&sA[i][j4]);  // the same address in every lane
                acc = fmaf(-a.x, t[j4], acc);
                if (j4 + 1 < i) acc = fmaf(-a.y, t[j4 + 1], acc);
                if (j4 + 2 < i) acc = fmaf(-a.z, t[j4 + 2], acc);
                if (j4 + 3 < i) acc = fmaf(-a.w, t[j4 + 3], acc);
            }
            t[i] = acc;
            sT[i][lane] = acc;
        }
    } else {
        const float lc = sL[kC - 1];
        for (int i = tid - 64; i < DK * (kC / 4); i += 192) {
            const int kk = i % DK, j4 = (i / DK) * 4;
            float4 o;
            o.x = expf(lc - sL[j4 + 0]) * sK[j4 + 0][kk];
            o.y = expf(lc - sL[j4 + 1]) * sK[j4 + 1][kk];
            o.z = expf(lc - sL[j4 + 2]) * sK[j4 + 2][kk];
            o.w = expf(lc - sL[j4 + 3]) * sK[j4 + 3][kk];
            *(float4 *)(KdT + slot * DK * kC + (size_t)kk * kC + j4) = o;
        }
        for (int i = tid - 64; i < kC * (DV / 4); i += 192) {
            const int tt = i / (DV / 4), x = (i % (DV / 4)) * 4;
            float4 a = {0.f, 0.f, 0.f, 0.f};
            if (tt < nt) a = load_f4(vv + ((size_t)(t0 + tt) * Hv + vh) * DV + x);
            *(float4 *)&sQ[tt][x] = a;
        }
    }
    __syncthreads();

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
                bV[s][ct][i] = sQ[16 * s + 4 * g + i][16 * (NCT * wave + ct) + m];
            }
#pragma unroll
    for (int tau = 0; tau < 4; tau++) {
        wy_f32x4 aw[NCT], au[NCT];
#pragma unroll
        for (int ct = 0; ct < NCT; ct++) aw[ct] = au[ct] = wy_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s <= tau; s++) {
            const float4 t4 = lds_f4(&sT[16 * tau + m][16 * s + 4 * g]);
            const float4 cw = lds_f4(&sCw[16 * s + 4 * g]), cb = lds_f4(&sB[16 * s + 4 * g]);
            const float4 tw = {t4.x * cw.x, t4.y * cw.y, t4.z * cw.z, t4.w * cw.w};
            const float4 tu = {t4.x * cb.x, t4.y * cb.y, t4.z * cb.z, t4.w * cb.w};
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) {
                aw[ct] = mfma4(tw, float4{bK[s][ct][0], bK[s][ct][1], bK[s][ct][2], bK[s][ct][3]}, aw[ct]);
                au[ct] = mfma4(tu, float4{bV[s][ct][0], bV[s][ct][1], bV[s][ct][2], bV[s][ct][3]}, au[ct]);
            }
        }
#pragma unroll
        for (int ct = 0; ct < NCT; ct++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const size_t row = 16 * tau + 4 * g + i, col = 16 * (NCT * wave + ct) + m;
                Wc[slot * kC * DK + row * DK + col] = aw[ct][i];
                Uc[slot * kC * DV + row * DV + col] = au[ct][i];
            }
    }
}

// grid (Hv, DV/16), 256 threads.  The 16 rows of the state are kept by every wave, in the
// layout of a D tile per 16 columns (lane (n, g): S[row0+n][16c+4g+i]), which is also the B
// operand of a contraction over the columns.  Wave w serves tokens 16w .. 16w+15 of each
// block and the column tiles (DK/64)*w .. of the state update.
template <int DK>
__global__ __launch_bounds__(256) void gdn_wy_recur_kernel(
    int Hk, int Hv, int T, const float *__restrict__ qn, const float *__restrict__ Wc,
    const float *__restrict__ Uc, const float *__restrict__ Mc, const float *__restrict__ KdT,
    const float *__restrict__ eLc, float *__restrict__ ssm, float *__restrict__ o_raw) {
    constexpr int DV = DK;
    constexpr int NK = DK / 16;   // column tiles of the state
    constexpr int NKW = NK / 4;   // of which a wave updates
    __shared__ wy_f32x4 s_d[4][64];    // D tiles of the block, by token tile
    __shared__ wy_f32x4 s_st[NK][64];  // the updated state

    const int vh = blockIdx.x, kh = vh / (Hv / Hk), row0 = blockIdx.y * 16;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = lane & 15, g = lane >> 4;
    float *srow = ssm + ((size_t)vh * DV + row0 + m) * DK + 4 * g;
    wy_f32x4 st[NK];
#pragma unroll
    for (int c = 0; c < NK; c++) {
        const float4 v = load_f4(srow + 16 * c);
        st[c] = wy_f32x4{v.x, v.y, v.z, v.w};
    }

    const int nblk = (T + kC - 1) / kC;
    for (int blk = 0; blk < nblk; blk++) {
        const int t0 = blk * kC;
        const size_t slot = (size_t)blk * Hv + vh;
        const float *Wb = Wc + slot * kC * DK, *Ub = Uc + slot * kC * DV, *Mb = Mc + slot * kC * kC;
        const float *Kb = KdT + slot * DK * kC, *eL = eLc + slot * kC;
        // ---- W S0^T and Q S0^T for this wave's 16 tokens ------------------------------
        const int tq = t0 + 16 * wave + m;  // the token whose q^ row this lane supplies
        const float *qrow = qn + ((size_t)(tq < T ? tq : T - 1) * Hk + kh) * DK + 4 * g;
        const float *wrow = Wb + (size_t)(16 * wave + m) * DK + 4 * g;
        wy_f32x4 p1 = {0.f, 0.f, 0.f, 0.f}, p2 = p1;
#pragma unroll
        for (int c = 0; c < NK; c++) {
            const float4 aw = load_f4(wrow + 16 * c);
            float4 aq = load_f4(qrow + 16 * c);
            if (tq >= T) aq = float4{0.f, 0.f, 0.f, 0.f};
            p1 = mfma4(aw, as_f4(st[c]), p1);
            p2 = mfma4(aq, as_f4(st[c]), p2);
        }
        // ---- D = U - W S0^T: lane (n, g) holds tokens 16w+4g+i of state row row0+n ----
        wy_f32x4 d;
#pragma unroll
        for (int i = 0; i < 4; i++)
            d[i] = Ub[(size_t)(16 * wave + 4 * g + i) * DV + row0 + m] - p1[i];
        s_d[wave][lane] = d;
        __syncthreads();
        // ---- O = diag(e^L) Q S0^T + M D ------------------------------------------------
        const float4 el = load_f4(eL + 16 * wave + 4 * g);
        wy_f32x4 o = {el.x * p2[0], el.y * p2[1], el.z * p2[2], el.w * p2[3]};
        for (int tau = 0; tau <= wave; tau++)
            o = mfma4(load_f4(Mb + (size_t)(16 * wave + m) * kC + 16 * tau + 4 * g), as_f4(s_d[tau][lane]), o);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int t = t0 + 16 * wave + 4 * g + i;
            if (t < T) o_raw[((size_t)t * Hv + vh) * DV + row0 + m] = o[i];
        }
        // ---- S' = e^{L_C} S0 + D^T diag(e^{L_C-L}) K, column tiles NKW*w .. ------------
        const float elc = eL[kC - 1];
#pragma unroll
        for (int kt = 0; kt < NKW; kt++) {
            const int c = NKW * wave + kt;
            wy_f32x4 acc;
            // st[c] with a runtime c: pick it without indexing the register array
            wy_f32x4 cur = st[0];
#pragma unroll
            for (int cc = 1; cc < NK; cc++)
                if (cc == c) cur = st[cc];
            acc = wy_f32x4{elc * cur[0], elc * cur[1], elc * cur[2], elc * cur[3]};
#pragma unroll
            for (int tau = 0; tau < 4; tau++)
                acc = mfma4(load_f4(Kb + (size_t)(16 * c + m) * kC + 16 * tau + 4 * g), as_f4(s_d[tau][lane]), acc);
            s_st[c][lane] = acc;
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < NK; c++) st[c] = s_st[c][lane];
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
    return nblk * Hv * ((size_t)kC * dk + (size_t)kC * dv + (size_t)kC * kC + (size_t)dk * kC + kC);
}

// qn, kn [T, Hk, dk]; vv [T, Hv, dv]; lg, bg [T, Hv] (log decay, beta gate); o_raw [T, Hv*dv].
int launch_gdn_wy(hipStream_t s, int Hk, int Hv, int dk, int dv, int T, const float *qn, const float *kn,
                  const float *vv, const float *lg, const float *bg, float *scratch, float *ssm,
                  float *o_raw) {
    if (dk != dv || (dk != 64 && dk != 128))
        return fail(MFA_ERR_SHAPE, "gdn blocked form: dk=%d dv=%d not supported", dk, dv);
    const size_t nblk = ((size_t)T + kC - 1) / kC;
    if (nblk > 65535) return fail(MFA_ERR_SHAPE, "gdn blocked form: too many tokens in one call");
    const size_t slots = nblk * Hv;
    float *Wc = scratch;
    float *Uc = Wc + slots * kC * dk;
    float *Mc = Uc + slots * kC * dv;
    float *KdT = Mc + slots * kC * kC;
    float *eLc = KdT + slots * dk * kC;
    if (dk == 128) {
        hipLaunchKernelGGL((gdn_wy_kernel<128>), dim3((unsigned)nblk, Hv), dim3(256), 0, s, Hk, Hv, T, qn, kn, vv,
                           lg, bg, Wc, Uc, Mc, KdT, eLc);
        hipLaunchKernelGGL((gdn_wy_recur_kernel<128>), dim3(Hv, dv / 16), dim3(256), 0, s, Hk, Hv, T, qn, Wc, Uc,
                           Mc, KdT, eLc, ssm, o_raw);
    } else {
        hipLaunchKernelGGL((gdn_wy_kernel<64>), dim3((unsigned)nblk, Hv), dim3(256), 0, s, Hk, Hv, T, qn, kn, vv,
                           lg, bg, Wc, Uc, Mc, KdT, eLc);
        hipLaunchKernelGGL((gdn_wy_recur_kernel<64>), dim3(Hv, dv / 16), dim3(256), 0, s, Hk, Hv, T, qn, Wc, Uc,
                           Mc, KdT, eLc, ssm, o_raw);
    }
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
