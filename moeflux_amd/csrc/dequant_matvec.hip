// 4-bit group-64 affine dequantising matrix-vector product: the projections either side
// of the attention core (q/k/v_proj, o_proj, in_proj_qkv/z/a/b, out_proj).
//
// Replaces dequant_matvec_4bit_v3 (crates/moeflux/shaders/shaders.metal:251-340; encoder
// gpu_matvec.rs; CPU form cpu_matvec.rs:83-160): out[r] = sum_c (nibble(r,c)*scale + bias)*x[c],
// W packed 8 nibbles per u32 (nibble n at bits 4n..4n+3 is input 8*word + n), one bf16 scale
// and bias per 64 inputs.
//
// Bound: HBM, 0.5625 bytes per weight (4 bits + 2 x bf16 per 64).  At that rate the VALU
// work per weight matters (16 T weights/s at 8 TB/s against 39 T lane-instructions/s), so the
// multiply-adds run on the matrix pipeline and the vector ALU only converts:
//   * A nibble n becomes the bf16 number 1 + n/16 (exponent bits of 1.0, n in the top four
//     mantissa bits): two nibbles per shift + and-or, exact, one instruction per weight.
//   * x is split into three bf16 parts by truncation (x = h + m + l exactly), which sit in
//     three columns of the B operand; a 16x16x32 instruction therefore gives, per row,
//     sum (1 + n/16) x exactly up to f32 accumulation.
//   * One instruction covers 32 inputs per lane group, i.e. two scale groups of 64 per four
//     instructions: columns 0..2 carry the first group's x (zero elsewhere), columns 3..5 the
//     second's, so the two groups' sums stay apart in one accumulator tile.
//   * Per group g and row r:  out += 16 s (D - X_g) + b X_g  with X_g = sum x over the group;
//     D is about 1.5 X_g, so the subtraction costs no more than two bits.
// A workgroup owns 16 rows (the M side of the tile); its waves split the inputs in runs of
// 1024, each lane requesting its 8 x 16 bytes of weights before anything else, and x, the
// scales and the biases are staged in LDS while those requests are in flight.
#include <type_traits>

#include "gdn_device.h"

namespace mfa {

static constexpr int kMvMaxSpecs = 8;

struct MatvecSpecs {
    const uint32_t *w[kMvMaxSpecs];
    const uint16_t *scales[kMvMaxSpecs];
    const uint16_t *biases[kMvMaxSpecs];
    const float *x[kMvMaxSpecs];
    float *out[kMvMaxSpecs];
    int out_dim[kMvMaxSpecs];
    int in_dim[kMvMaxSpecs];
};

typedef unsigned int mv_u32x4 __attribute__((ext_vector_type(4)));

typedef __attribute__((ext_vector_type(8))) __bf16 mv_bf16x8;
typedef __attribute__((ext_vector_type(4))) float mv_f32x4;

struct MatvecTiles {
    int first[kMvMaxSpecs + 1];  // first 16-row tile of every product, and the total
};

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void dequant_matvec_mfma_kernel(MatvecSpecs sp, MatvecTiles tl, int n_specs) {
    constexpr int NTHR = WAVES * 64;
    constexpr int KP = WAVES * 1024;   // inputs covered by the workgroup (in_dim padded)
    constexpr int G = KP / 64;         // scale groups
    constexpr int STEPS = 8;           // 128-input steps per wave
    __shared__ __attribute__((aligned(16))) uint16_t xs[3][KP];       // bf16 parts of x; within a run of 8 inputs the order is 0,4,1,5,2,6,3,7
    __shared__ __attribute__((aligned(16))) uint16_t zeros[128 * STEPS + 128];  // what the other lanes of the B operand read
    // scales and biases of the tile's rows as stored (bf16), [group][row]; + 4: the staging writes walk the groups
    __shared__ __attribute__((aligned(8))) uint16_t sc_l[G][16 + 4], bi_l[G][16 + 4];
    __shared__ float xsum[G];
    __shared__ __attribute__((aligned(16))) float red[WAVES][16];

    int s = 0;
    while (s + 1 < n_specs && (int)blockIdx.x >= tl.first[s + 1]) s++;
    const int row0 = ((int)blockIdx.x - tl.first[s]) * 16;
    const int in_dim = sp.in_dim[s], out_dim = sp.out_dim[s];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int nchunk = in_dim >> 5, groups = in_dim >> 6, words = in_dim >> 3;

    // ---- weights: row n of the tile, 32-input chunk 4 S + g of step S; all requested now ----
    mv_u32x4 w[STEPS];
    {
        const uint32_t *wrow = sp.w[s] + (size_t)min(row0 + n, out_dim - 1) * words;
#pragma unroll
        for (int st = 0; st < STEPS; st++) {
            const int c = 4 * (wave * STEPS + st) + g;
            w[st] = *reinterpret_cast<const mv_u32x4 *>(wrow + (c < nchunk ? c : 0) * 4);  // past the row: any chunk, x is 0 there
        }
    }
    // ---- stage x (a run of 8 inputs per thread and pass), the scales and the biases; every
    //      request first, so that the workgroup pays one round trip, not one per pass ----
    {
        constexpr int XP = KP / 8 / NTHR;       // passes over x
        constexpr int SP = 16 * G / NTHR;   // passes over the (row, group) pairs
        const float *x = sp.x[s];
        const uint16_t *S = sp.scales[s], *B = sp.biases[s];
        float4 xa[XP], xb4[XP];
        uint16_t sraw[SP], braw[SP];
#pragma unroll
        for (int p = 0; p < XP; p++) {
            const int r = tid + p * NTHR;
            const int at = 8 * r < in_dim ? 8 * r : 0;
            xa[p] = load_f4(x + at);
            xb4[p] = load_f4(x + at + 4);
        }
#pragma unroll
        for (int p = 0; p < SP; p++) {
            const int i = tid + p * NTHR;
            const int r = i / G, gg = i % G;
            const size_t at = (size_t)min(row0 + r, out_dim - 1) * groups + (gg < groups ? gg : 0);
            sraw[p] = S[at];
            braw[p] = B[at];
        }
#pragma unroll
        for (int i = tid; i < (128 * STEPS + 128) / 8; i += NTHR) *reinterpret_cast<mv_u32x4 *>(&zeros[8 * i]) = mv_u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int p = 0; p < XP; p++) {
            const int r = tid + p * NTHR;
            const bool live = 8 * r < in_dim;
            const float4 a = xa[p], b = xb4[p];
            float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            uint32_t hb[8], mb[8], lb[8];
#pragma unroll
            for (int e = 0; e < 8; e++) {   // v = h + m + l, each a bf16 number (upper 16 bits)
                if (!live) v[e] = 0.f;
                hb[e] = __builtin_bit_cast(uint32_t, v[e]);
                const float r1 = v[e] - __builtin_bit_cast(float, hb[e] & 0xffff0000u);
                mb[e] = __builtin_bit_cast(uint32_t, r1);
                lb[e] = __builtin_bit_cast(uint32_t, r1 - __builtin_bit_cast(float, mb[e] & 0xffff0000u));
            }
            const uint32_t hi16 = 0x07060302u;  // (upper half of the second operand, upper half of the first)
            mv_u32x4 ph, pm, pl;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                ph[e] = __builtin_amdgcn_perm(hb[e + 4], hb[e], hi16);
                pm[e] = __builtin_amdgcn_perm(mb[e + 4], mb[e], hi16);
                pl[e] = __builtin_amdgcn_perm(lb[e + 4], lb[e], hi16);
            }
            *reinterpret_cast<mv_u32x4 *>(&xs[0][8 * r]) = ph;
            *reinterpret_cast<mv_u32x4 *>(&xs[1][8 * r]) = pm;
            *reinterpret_cast<mv_u32x4 *>(&xs[2][8 * r]) = pl;
            float sum = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
            sum = group_sum<8>(sum);
            if ((tid & 7) == 0) xsum[r >> 3] = sum;
        }
#pragma unroll
        for (int p = 0; p < SP; p++) {
            const int i = tid + p * NTHR;
            const int r = i / G, gg = i % G;
            sc_l[gg][r] = gg < groups ? sraw[p] : (uint16_t)0;
            bi_l[gg][r] = gg < groups ? braw[p] : (uint16_t)0;
        }
    }
    __syncthreads();

    // B operand: lane (column n, input octet g) reads part n % 3 of x if column n belongs to the
    // scale group that octet g lies in (columns 0..2: octets 0, 1; columns 3..5: octets 2, 3), else zeros
    const bool mine = n < 6 && (n / 3) == (g >> 1);
    const uint16_t *xb = (mine ? &xs[n % 3][128 * STEPS * wave] : &zeros[0]) + 32 * g;
    const int gsel = n >= 3 ? 1 : 0;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};   // rows 4g + i of the tile, this lane's column's share
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        mv_f32x4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t ww = w[st][j];
            mv_u32x4 a;   // nibbles (0,4), (1,5), (2,6), (3,7) as bf16 pairs 1 + n/16
            a[0] = ((ww << 3) & 0x00780078u) | 0x3F803F80u;
            a[1] = ((ww >> 1) & 0x00780078u) | 0x3F803F80u;
            a[2] = ((ww >> 5) & 0x00780078u) | 0x3F803F80u;
            a[3] = ((ww >> 9) & 0x00780078u) | 0x3F803F80u;
            const mv_bf16x8 b = *reinterpret_cast<const mv_bf16x8 *>(xb + 128 * st + 8 * j);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mv_bf16x8, a), b, d, 0, 0, 0);
        }
        // out += 16 s D: the scales of rows 4g .. 4g + 3 in this lane's group
        const uint2 sb = *reinterpret_cast<const uint2 *>(&sc_l[2 * (wave * STEPS + st) + gsel][4 * g]);
        acc[0] = fmaf(16.f * __builtin_bit_cast(float, sb.x << 16), d[0], acc[0]);
        acc[1] = fmaf(16.f * __builtin_bit_cast(float, sb.x & 0xffff0000u), d[1], acc[1]);
        acc[2] = fmaf(16.f * __builtin_bit_cast(float, sb.y << 16), d[2], acc[2]);
        acc[3] = fmaf(16.f * __builtin_bit_cast(float, sb.y & 0xffff0000u), d[3], acc[3]);
    }
    {   // the X_g terms of this wave's 16 groups, one group per column lane
        const int gg = 16 * wave + n;
        const uint2 sb = *reinterpret_cast<const uint2 *>(&sc_l[gg][4 * g]);
        const uint2 bb = *reinterpret_cast<const uint2 *>(&bi_l[gg][4 * g]);
        const float xg = xsum[gg];
        const float sv[4] = {__builtin_bit_cast(float, sb.x << 16), __builtin_bit_cast(float, sb.x & 0xffff0000u),
                             __builtin_bit_cast(float, sb.y << 16), __builtin_bit_cast(float, sb.y & 0xffff0000u)};
        const float bv[4] = {__builtin_bit_cast(float, bb.x << 16), __builtin_bit_cast(float, bb.x & 0xffff0000u),
                             __builtin_bit_cast(float, bb.y << 16), __builtin_bit_cast(float, bb.y & 0xffff0000u)};
#pragma unroll
        for (int i = 0; i < 4; i++) acc[i] = fmaf(bv[i] - 16.f * sv[i], xg, acc[i]);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] = group_sum<16>(acc[i]);
    if (n == 0) *reinterpret_cast<mv_f32x4 *>(&red[wave][4 * g]) = mv_f32x4{acc[0], acc[1], acc[2], acc[3]};
    __syncthreads();
    if (tid < 16 && row0 + tid < out_dim) {
        float v = 0.f;
#pragma unroll
        for (int k = 0; k < WAVES; k++) v += red[k][tid];
        sp.out[s][row0 + tid] = v;
    }
}

// Device pointers; one launch for up to 8 products (the reference batches a layer's
// projections into one command buffer, full_attn_forward.rs:193-227).
int launch_dequant_matvec_4bit(hipStream_t stream, int n, const uint32_t *const *w, const uint16_t *const *scales,
                               const uint16_t *const *biases, const float *const *x, float *const *out,
                               const int *out_dim, const int *in_dim, int num_cus) {
    if (n <= 0 || n > kMvMaxSpecs) return fail(MFA_ERR_INVALID, "dequant matvec: 1 to %d products per call (got %d)", kMvMaxSpecs, n);
    MatvecSpecs sp{};
    int max_out = 0, max_in = 0;
    for (int i = 0; i < n; i++) {
        if (!w[i] || !scales[i] || !biases[i] || !x[i] || !out[i]) return fail(MFA_ERR_INVALID, "dequant matvec: NULL pointer in product %d", i);
        if (out_dim[i] <= 0 || in_dim[i] <= 0) return fail(MFA_ERR_INVALID, "dequant matvec: non-positive shape in product %d", i);
        if (in_dim[i] % 64 != 0) return fail(MFA_ERR_INVALID, "dequant matvec: in_dim %d is not a multiple of the group size 64", in_dim[i]);
        if (in_dim[i] > 8192) return fail(MFA_ERR_SHAPE, "dequant matvec: in_dim %d > 8192 not supported", in_dim[i]);
        sp.w[i] = w[i]; sp.scales[i] = scales[i]; sp.biases[i] = biases[i]; sp.x[i] = x[i]; sp.out[i] = out[i];
        sp.out_dim[i] = out_dim[i]; sp.in_dim[i] = in_dim[i];
        max_out = out_dim[i] > max_out ? out_dim[i] : max_out;
        max_in = in_dim[i] > max_in ? in_dim[i] : max_in;
    }
    MatvecTiles tl{};
    for (int i = 0; i < n; i++) tl.first[i + 1] = tl.first[i] + (out_dim[i] + 15) / 16;
    for (int i = n + 1; i <= kMvMaxSpecs; i++) tl.first[i] = tl.first[n];
    const dim3 grid(tl.first[n]);
    (void)max_out;
    (void)num_cus;
    if (max_in <= 1024) hipLaunchKernelGGL((dequant_matvec_mfma_kernel<1>), grid, dim3(64), 0, stream, sp, tl, n);
    else if (max_in <= 2048) hipLaunchKernelGGL((dequant_matvec_mfma_kernel<2>), grid, dim3(128), 0, stream, sp, tl, n);
    else if (max_in <= 4096) hipLaunchKernelGGL((dequant_matvec_mfma_kernel<4>), grid, dim3(256), 0, stream, sp, tl, n);
    else hipLaunchKernelGGL((dequant_matvec_mfma_kernel<8>), grid, dim3(512), 0, stream, sp, tl, n);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
