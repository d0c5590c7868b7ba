// Wave-level building blocks shared by the decode and the prompt-chunk attention kernels:
// the 16-row query groups, and per cache dtype the MFMA operand handling for
// S^T = K Q^T (lane % 16 = query row) and O^T = V^T P^T over one block of positions.
#pragma once
#include <type_traits>

#include "mfa_internal.h"

namespace mfa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;

static constexpr float kLog2e = 1.4426950408889634f;

__device__ inline float neg_inf() { return -__builtin_huge_valf(); }
__device__ inline float lane_xor(float v, int mask) { return __shfl_xor(v, mask, 64); }
// Maximum / sum of a value over the four lanes l % 16 + 16 g, g = 0 .. 3, in every one of them.
// v_permlane16_swap / v_permlane32_swap (vector ALU, no trip through the LDS crossbar) exchange the odd
// rows of 16 lanes (the upper 32 lanes) of their first register with the even rows (the lower 32) of
// the second: given the same value in both, a lane then holds its own value in one register and that
// of lane l ^ 16 (l ^ 32) in the other, and the sum adds the two numbers a lane exchange would.
// As inline assembly with two registers of their own: given one value for both operands, the
// builtin's two results come out as one register.  (The instruction reads its operands two wait
// states after a vector ALU write at the earliest; the compiler does not see into the assembly, so
// the wait states stand on both sides of it.)
__device__ inline void rows_swap16(float &a, float &b) { asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b)); }
__device__ inline void rows_swap32(float &a, float &b) { asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b)); }
__device__ inline float rows_max(float v) {
    float a = v, b = v;
    rows_swap16(a, b);
    a = b = fmaxf(a, b);
    rows_swap32(a, b);
    return fmaxf(a, b);
}
__device__ inline float rows_sum(float v) {
    float a = v, b = v;
    rows_swap16(a, b);
    a = b = a + b;
    rows_swap32(a, b);
    return a + b;
}
__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// (a, b) -> packed bf16 pair, round to nearest even (v_cvt_pk_bf16_f32)
__device__ inline uint32_t pack_bf16(float a, float b) {
    f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
// x = hi + lo + O(2^-17 x): hi = bf16(x), lo = bf16(x - hi); x - hi is exact in f32.
__device__ inline void split_pair(float a, float b, uint32_t &hi, uint32_t &lo) {
    hi = pack_bf16(a, b);
    const float ah = __builtin_bit_cast(float, hi << 16);
    const float bh = __builtin_bit_cast(float, hi & 0xffff0000u);
    lo = pack_bf16(a - ah, b - bh);
}
__device__ inline bf16x8 as_bf16x8(uint4 u) { return __builtin_bit_cast(bf16x8, u); }

// 16-byte load of cache data that is read exactly once per launch: non-temporal, so
// that it does not displace the query, the probabilities and the partials in L2.
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
// The same as one register-valued load (a uint4 assignment is a struct copy, which the
// compiler may leave as a memcpy into a stack slot).
__device__ inline uint4 vec_load(const uint4 *p) {
    return __builtin_bit_cast(uint4, *reinterpret_cast<const u32x4 *>(p));
}
__device__ inline uint4 stream_load(const uint4 *p) {
    return __builtin_bit_cast(uint4, __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p)));
}

// Split-K partials are written with stores that go through to memory (scope bits sc0 sc1): they
// are read by the merge launch, whose workgroups run on other XCDs with L2s of their own, and
// leaving 4 MB of them dirty in the writers' L2s until the end of the launch, to be written back
// in one burst, measured slower.
static constexpr int kThrough = 16;   // cache policy of the buffer instructions: sc1 (device scope)
__device__ inline __amdgpu_buffer_rsrc_t buffer_of(const void *base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, 0xffffffff, 0x00020000);
}

// Reader of one row group's partials, by element index relative to the group's first split:
// rows at (split * 16 + row) * D + channel, statistics at split * 32 + row (+ 16 for the sum).
struct PartialsPlain {
    const float *o, *ml;
    __device__ PartialsPlain(const float *part_o, const float *part_ml, size_t pid0, int D)
        : o(part_o + pid0 * 16 * D), ml(part_ml + pid0 * 32) {}
    __device__ float stat(int i) const { return ml[i]; }
    __device__ float row1(int i) const { return o[i]; }
    __device__ float4 row4(int i) const { return *(const float4 *)(o + i); }
};

// The 16 rows a workgroup serves.  Row rr = 16*hg + n of kv head kvh is query head
// rr % hpk (within the kv head's group) of token rr / hpk: one token in decode, the
// n_tok tokens of a prompt chunk otherwise.  Token t sees positions [0, kv_len0 + t].
struct RowGroup {
    int kvh, hg, hpk, Hq, n_tok;
    int64_t kv_len0;  // cache length before the first of the n_tok tokens was appended
    __device__ bool valid(int n) const { return hg * 16 + n < n_tok * hpk; }
    __device__ size_t q_row(int n) const {
        const int rr = hg * 16 + n;
        return (size_t)(rr / hpk) * Hq + kvh * hpk + rr % hpk;
    }
    __device__ int64_t limit(int n) const { return valid(n) ? kv_len0 + (hg * 16 + n) / hpk + 1 : 0; }
    // smallest and largest limit among the valid rows (uniform over the workgroup)
    __device__ int64_t limit_min() const { return kv_len0 + (hg * 16) / hpk + 1; }
    __device__ int64_t limit_max() const {
        int last = hg * 16 + 15;
        if (last > n_tok * hpk - 1) last = n_tok * hpk - 1;
        return kv_len0 + last / hpk + 1;
    }
    __device__ bool full() const { return hg * 16 + 15 < n_tok * hpk; }
};

// Per-dtype pieces of the kernels.  Common shape: the K of a 16-position sub-tile is KSTEPS
// 1 KiB pieces (one per k-step), a V block is NACC = D/16 1 KiB pieces, piece `dt` being the
// 16-wide output tile dt.  (NLOAD: pieces of K that cover the positions of one V block.)
template <typename KV, int D> struct Wave;

// ---------------------------------------------------------------------------
// bf16 cache: blocks of 32 positions (64*D bytes of K and of V each)
// ---------------------------------------------------------------------------
template <int D> struct Wave<uint16_t, D> {
    static constexpr int BLK = 32;
    static constexpr int KSTEPS = D / 32;   // MFMA k-steps per 16-position sub-tile
    static constexpr int NACC = D / 16;     // 16-wide output tiles of O^T
    static constexpr int NLOAD = D / 16;    // 1 KiB loads of K per block
    static constexpr int QSLOTS = KSTEPS * 64;   // (k-step, lane) operand slots of the query
    static constexpr int QLDS_U4 = QSLOTS * 2;   // hi and lo
    static constexpr int QRAW_F4 = 2;            // float4 loads per slot
    static constexpr int P_U4 = 2;               // hi and lo probability operands per lane

    __device__ static void load_q_slot(float4 (&raw)[QRAW_F4], const float *q, int slot,
                                       const RowGroup &rows) {
        const int s = slot >> 6, lane = slot & 63, n = lane & 15, g = lane >> 4;
        const float4 z = {0.f, 0.f, 0.f, 0.f};
        raw[0] = raw[1] = z;
        if (rows.valid(n)) {
            const float *p = q + rows.q_row(n) * D + 8 * (4 * s + g);
            raw[0] = *(const float4 *)p;
            raw[1] = *(const float4 *)(p + 4);
        }
    }
    // Query operands in LDS: [k-step][hi|lo][lane] of 16 bytes.
    __device__ static void store_q_slot(uint4 *qlds, const float4 (&raw)[QRAW_F4], int slot, float qscale) {
        const int s = slot >> 6, lane = slot & 63;
        uint4 hi, lo;
        split_pair(raw[0].x * qscale, raw[0].y * qscale, hi.x, lo.x);
        split_pair(raw[0].z * qscale, raw[0].w * qscale, hi.y, lo.y);
        split_pair(raw[1].x * qscale, raw[1].y * qscale, hi.z, lo.z);
        split_pair(raw[1].z * qscale, raw[1].w * qscale, hi.w, lo.w);
        qlds[(s * 2 + 0) * 64 + lane] = hi;
        qlds[(s * 2 + 1) * 64 + lane] = lo;
    }

    // The same operands kept in registers by a wave that owns its row group: per k-step a
    // high and a low bf16 part.
    static constexpr int QREGS = KSTEPS * 2;
    __device__ static void load_q_regs(uint4 (&qr)[QREGS], const float *q, int lane, const RowGroup &rows,
                                       float qscale) {
        const int n = lane & 15, g = lane >> 4;
        const bool ok = rows.valid(n);
        const float *p = q + (ok ? rows.q_row(n) : 0) * D + 8 * g;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            float4 a = *(const float4 *)(p + 32 * s), b = *(const float4 *)(p + 32 * s + 4);
            if (!ok) a = b = float4{0.f, 0.f, 0.f, 0.f};
            split_pair(a.x * qscale, a.y * qscale, qr[2 * s].x, qr[2 * s + 1].x);
            split_pair(a.z * qscale, a.w * qscale, qr[2 * s].y, qr[2 * s + 1].y);
            split_pair(b.x * qscale, b.y * qscale, qr[2 * s].z, qr[2 * s + 1].z);
            split_pair(b.z * qscale, b.w * qscale, qr[2 * s].w, qr[2 * s + 1].w);
        }
    }

    struct Scores {
        f32x4 s[2];
    };

    // K load li = 2*s + sub: both 16-position sub-tiles of a k-step share one read of
    // the query operands.  Scores come out in log2 units.
    __device__ static void scores(const uint4 (&kreg)[NLOAD], const uint4 *qlds, int lane, Scores &sc) {
        sc.s[0] = f32x4{0.f, 0.f, 0.f, 0.f};
        sc.s[1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            const bf16x8 qh = as_bf16x8(qlds[(s * 2 + 0) * 64 + lane]);
            const bf16x8 ql = as_bf16x8(qlds[(s * 2 + 1) * 64 + lane]);
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                const bf16x8 a = as_bf16x8(kreg[2 * s + sub]);
                sc.s[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qh, sc.s[sub], 0, 0, 0);
                sc.s[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, ql, sc.s[sub], 0, 0, 0);
            }
        }
    }

    // HI_ONLY: the query's low parts are all zero (a query that is exact in bf16), so their
    // products are left out; the result is the same number.
    template <bool HI_ONLY = false>
    __device__ static void scores_reg(const uint4 (&kreg)[NLOAD], const uint4 (&qr)[QREGS], Scores &sc) {
        sc.s[0] = f32x4{0.f, 0.f, 0.f, 0.f};
        sc.s[1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                const bf16x8 a = as_bf16x8(kreg[2 * s + sub]);
                sc.s[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, as_bf16x8(qr[2 * s]), sc.s[sub], 0, 0, 0);
                if constexpr (!HI_ONLY)
                    sc.s[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, as_bf16x8(qr[2 * s + 1]), sc.s[sub], 0, 0, 0);
            }
        }
    }
    // whether every low part of this lane's query operands is zero
    __device__ static bool q_low_parts_zero(const uint4 (&qr)[QREGS]) {
        unsigned any = 0;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) any |= (qr[2 * s + 1].x | qr[2 * s + 1].y | qr[2 * s + 1].z | qr[2 * s + 1].w) & 0x7fff7fffu;
        return any == 0;
    }
    static constexpr bool kScaleAfter = true;   // scores leave the matrix core unscaled (prompt-chunk kernel)

    // One 1 KiB piece of K (16 positions x the 32 channels of k-step s) against the query
    // operands in registers: the piece's share of S^T[16 positions, 16 rows].
    __device__ static f32x4 score_step(uint4 kpiece, const uint4 (&qr)[QREGS], int s, f32x4 acc) {
        const bf16x8 a = as_bf16x8(kpiece);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, as_bf16x8(qr[2 * s]), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, as_bf16x8(qr[2 * s + 1]), acc, 0, 0, 0);
        return acc;
    }
    // The probabilities of one 16-position sub-tile (lane (n, g): positions 4g .. 4g+3 of query
    // row n) as this lane's half of the value product's operand: the sub-tile is half `h` of a
    // 32-position V block, whose operand slots 4h .. 4h+3 of lane group g are those positions.
    __device__ static void store_probs(uint4 (*pblk)[64], int lane, int h, const float (&e)[4]) {
        uint2 hi, lo;
        split_pair(e[0], e[1], hi.x, lo.x);
        split_pair(e[2], e[3], hi.y, lo.y);
        reinterpret_cast<uint2 *>(&pblk[0][lane])[h] = hi;
        reinterpret_cast<uint2 *>(&pblk[1][lane])[h] = lo;
    }

    static constexpr int NX = 8;  // scores per lane: row 4g+i of sub-tile `sub` is position 16*sub + 4g + i
    __device__ static void unpack(const Scores &sc, float (&x)[NX]) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            x[i] = sc.s[0][i];
            x[4 + i] = sc.s[1][i];
        }
    }
    __device__ static int64_t pos_of(int64_t blk, int g, int e) {
        return blk * BLK + 16 * (e >> 2) + 4 * g + (e & 3);
    }
    // probabilities -> operand registers (slot e of lane group g is position pos_of(.., g, e))
    __device__ static void pack_probs(const float (&e)[NX], uint4 (&p)[P_U4]) {
        split_pair(e[0], e[1], p[0].x, p[1].x);
        split_pair(e[2], e[3], p[0].y, p[1].y);
        split_pair(e[4], e[5], p[0].z, p[1].z);
        split_pair(e[6], e[7], p[0].w, p[1].w);
    }
    __device__ static f32x4 pv(uint4 vreg, const uint4 (&p)[P_U4], f32x4 acc) {
        const bf16x8 a = as_bf16x8(vreg);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, as_bf16x8(p[0]), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, as_bf16x8(p[1]), acc, 0, 0, 0);
        return acc;
    }
};

// ---------------------------------------------------------------------------
// f32 cache: blocks of 16 positions (64*D bytes of K and of V each)
// ---------------------------------------------------------------------------
template <int D> struct Wave<float, D> {
    static constexpr int BLK = 16;
    static constexpr int KSTEPS = D / 16;  // 1 KiB loads of K per block (4 MFMAs each)
    static constexpr int NACC = D / 16;
    static constexpr int NLOAD = D / 16;
    static constexpr int QSLOTS = KSTEPS * 64;
    static constexpr int QLDS_U4 = QSLOTS;
    static constexpr int QRAW_F4 = 1;
    static constexpr int P_U4 = 1;

    __device__ static void load_q_slot(float4 (&raw)[QRAW_F4], const float *q, int slot,
                                       const RowGroup &rows) {
        const int s = slot >> 6, lane = slot & 63, n = lane & 15, g = lane >> 4;
        raw[0] = float4{0.f, 0.f, 0.f, 0.f};
        if (rows.valid(n)) raw[0] = *(const float4 *)(q + rows.q_row(n) * D + 4 * (4 * s + g));
    }
    // Query operands in LDS: [k-step][lane] float4; lane (n, g) holds q[n][4(4s+g) .. +3].
    __device__ static void store_q_slot(uint4 *qlds, const float4 (&raw)[QRAW_F4], int slot, float qscale) {
        float4 v = raw[0];
        v.x *= qscale; v.y *= qscale; v.z *= qscale; v.w *= qscale;
        qlds[slot] = __builtin_bit_cast(uint4, v);
    }

    static constexpr int QREGS = KSTEPS;
    __device__ static void load_q_regs(uint4 (&qr)[QREGS], const float *q, int lane, const RowGroup &rows,
                                       float qscale) {
        const int n = lane & 15, g = lane >> 4;
        const bool ok = rows.valid(n);
        const float *p = q + (ok ? rows.q_row(n) : 0) * D + 4 * g;
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            float4 v = *(const float4 *)(p + 16 * s);
            if (!ok) v = float4{0.f, 0.f, 0.f, 0.f};
            v.x *= qscale; v.y *= qscale; v.z *= qscale; v.w *= qscale;
            qr[s] = __builtin_bit_cast(uint4, v);
        }
    }

    struct Scores {
        f32x4 s;
    };

    __device__ static void scores(const uint4 (&kreg)[NLOAD], const uint4 *qlds, int lane, Scores &sc) {
        sc.s = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            const float4 a = __builtin_bit_cast(float4, kreg[s]);
            const float4 b = __builtin_bit_cast(float4, qlds[s * 64 + lane]);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, sc.s, 0, 0, 0);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, sc.s, 0, 0, 0);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, sc.s, 0, 0, 0);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, sc.s, 0, 0, 0);
        }
    }

    template <bool HI_ONLY = false>   // an f32 query has no parts
    __device__ static void scores_reg(const uint4 (&kreg)[NLOAD], const uint4 (&qr)[QREGS], Scores &sc) {
        sc.s = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KSTEPS; s++) {
            const float4 a = __builtin_bit_cast(float4, kreg[s]);
            const float4 b = __builtin_bit_cast(float4, qr[s]);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, sc.s, 0, 0, 0);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, sc.s, 0, 0, 0);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, sc.s, 0, 0, 0);
            sc.s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, sc.s, 0, 0, 0);
        }
    }

    __device__ static bool q_low_parts_zero(const uint4 (&)[QREGS]) { return false; }
    static constexpr bool kScaleAfter = false;   // the query carries the scale

    // One 1 KiB piece of K (16 positions x the 16 channels of k-step s).
    __device__ static f32x4 score_step(uint4 kpiece, const uint4 (&qr)[QREGS], int s, f32x4 acc) {
        const float4 a = __builtin_bit_cast(float4, kpiece);
        const float4 b = __builtin_bit_cast(float4, qr[s]);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, acc, 0, 0, 0);
        return acc;
    }
    // A 16-position sub-tile is one V block: the four probabilities are the lane's operand.
    __device__ static void store_probs(uint4 (*pblk)[64], int lane, int, const float (&e)[4]) {
        pblk[0][lane] = __builtin_bit_cast(uint4, float4{e[0], e[1], e[2], e[3]});
    }

    static constexpr int NX = 4;  // row 4g+i is position 4g + i
    __device__ static void unpack(const Scores &sc, float (&x)[NX]) {
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = sc.s[i];
    }
    __device__ static int64_t pos_of(int64_t blk, int g, int e) { return blk * BLK + 4 * g + e; }
    __device__ static void pack_probs(const float (&e)[NX], uint4 (&p)[P_U4]) {
        p[0] = __builtin_bit_cast(uint4, float4{e[0], e[1], e[2], e[3]});
    }
    // V load of tile dt: lane (m, g) holds V[pos 4g+j][16 dt + m], j = 0..3; MFMA j
    // contracts the four positions {4g+j}.
    __device__ static f32x4 pv(uint4 vreg, const uint4 (&p)[P_U4], f32x4 acc) {
        const float4 a = __builtin_bit_cast(float4, vreg);
        const float4 b = __builtin_bit_cast(float4, p[0]);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, acc, 0, 0, 0);
        return acc;
    }
};

}  // namespace mfa
