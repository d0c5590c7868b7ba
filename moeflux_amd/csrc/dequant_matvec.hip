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
//     three rows of the other operand; a 16x16x32 instruction therefore gives, per row of W,
//     sum (1 + n/16) x exactly up to f32 accumulation.
//   * One instruction covers 32 inputs per lane group, i.e. two scale groups of 64 per four
//     instructions: operand rows 0..2 carry the first group's x (zero elsewhere), rows 4..6 the
//     second's, so the two groups' sums stay apart in one accumulator tile.
//   * Per group g and row r:  out += 16 s (D - X_g) + b X_g  with X_g = sum x over the group;
//     D is about 1.5 X_g, so the subtraction costs no more than two bits.
#include <cstdint>
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

// Eight consecutive bf16 scales (or biases) of one row, groups first .. first + 7, as stored.
// ALIGNED: every row starts on a 16-byte boundary and has a multiple of 8 groups.
template <bool ALIGNED>
__device__ inline mv_u32x4 load_sb8(const uint16_t *row, int first, int groups) {
    if constexpr (ALIGNED) return *reinterpret_cast<const mv_u32x4 *>(row + (first < groups ? first : 0));
    uint32_t e[8];
#pragma unroll
    for (int i = 0; i < 8; i++) e[i] = first + i < groups ? row[first + i] : 0u;
    return mv_u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
}

// The product a tile belongs to, found and read with compile-time indices only (the tables
// stay in scalar registers; an index computed at run time would be looked up lane by lane).
struct Product {
    const uint32_t *w;
    const uint16_t *scales, *biases;
    const float *x;
    float *out;
    int out_dim, in_dim, first;
};
__device__ inline Product mv_product_of(const MatvecSpecs &sp, const MatvecTiles &tl, int t) {
    int s = 0;   // first[] does not decrease and is padded with the total
#pragma unroll
    for (int i = 1; i < kMvMaxSpecs; i++) s += t >= tl.first[i] ? 1 : 0;
    s = __builtin_amdgcn_readfirstlane(s);
    Product q;
    q.w = sp.w[0]; q.scales = sp.scales[0]; q.biases = sp.biases[0]; q.x = sp.x[0]; q.out = sp.out[0];
    q.out_dim = sp.out_dim[0]; q.in_dim = sp.in_dim[0]; q.first = tl.first[0];
#pragma unroll
    for (int i = 1; i < kMvMaxSpecs; i++) {
        const bool hit = s == i;
        q.w = hit ? sp.w[i] : q.w;
        q.scales = hit ? sp.scales[i] : q.scales;
        q.biases = hit ? sp.biases[i] : q.biases;
        q.x = hit ? sp.x[i] : q.x;
        q.out = hit ? sp.out[i] : q.out;
        q.out_dim = hit ? sp.out_dim[i] : q.out_dim;
        q.in_dim = hit ? sp.in_dim[i] : q.in_dim;
        q.first = hit ? tl.first[i] : q.first;
    }
    return q;
}

// One workgroup per TILES tiles of 16 rows (TILES = 1 is what is launched: with two, x is read
// and split half as often, but fewer waves fit a CU and the launch as a whole was slower); its
// waves split the inputs in runs of 1024, and each wave stages the part of x it uses itself.
//
// The weights are the B side of the matrix instruction (column = row of the tile) and the
// parts of x the A side: row 0..2 of A are the three parts of x restricted to the first scale
// group of a 128-input step, rows 4..6 the same for the second group.  Lane (n, g) of the
// result then holds, for g = 0 and g = 1, the three partial sums of row n of the tile over
// scale group g of the step - and needs only its own row's scale to finish it.  Lanes
// (n, 2) and (n, 3), whose results are zero, add the bias terms b X_g of the even and odd groups.
//
// Loads come back in the order they were asked for, so the order of the requests is the order
// of use: x (staged in LDS while everything else is on its way), the row's scales and biases
// (16 bytes per lane straight into registers), then the 8 x 16 bytes of weights per lane.
template <int WAVES, bool SB16, int TILES, bool TILED>
__device__ __forceinline__ void dequant_matvec_body(const MatvecSpecs &sp, const MatvecTiles &tl) {
    constexpr int KP = WAVES * 1024;   // inputs covered by the workgroup (in_dim padded)
    constexpr int G = KP / 64;         // scale groups
    constexpr int STEPS = 8;           // 128-input steps per wave
    __shared__ __attribute__((aligned(16))) uint16_t xs[3][KP];       // bf16 parts of x; within a run of 8 inputs the order is 0,4,1,5,2,6,3,7
    __shared__ __attribute__((aligned(16))) uint16_t zeros[128 * STEPS + 128];  // what the other lanes of the A operand read
    __shared__ float xsum[G];
    __shared__ float red[WAVES][16 * TILES];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int t = blockIdx.x;
    const Product q = mv_product_of(sp, tl, t);

    mv_u32x4 w[TILES][STEPS];   // row n of tile T, 32-input chunk 4 S + g of step S
    // The scales (lanes g < 2) or biases (the others) of row n for the wave's 16 groups.  From the file's
    // order: q0 groups 16 wave .. + 7, q1 the next eight.  TILED: q0 alone, the eight groups of this
    // lane's parity (2 e + g % 2, e = 0 .. 7), which are the ones it uses.
    mv_u32x4 q0[TILES], q1[TILES];
    auto fetch = [&]() __attribute__((always_inline)) {
        const int in_dim = q.in_dim, out_dim = q.out_dim;
        const int nchunk = in_dim >> 5, groups = in_dim >> 6, words = in_dim >> 3;
        // the scales before the weights: the first step of the product needs them, and loads
        // come back in the order they were asked for
#pragma unroll
        for (int T = 0; T < TILES; T++) {
            if constexpr (TILED) {
                const int nruns = (in_dim + 1023) >> 10, tile = (t - q.first) * TILES + T;
                const size_t at = (((size_t)tile * nruns + (wave < nruns ? wave : 0)) * (STEPS + 1)) * 64 + lane;
                q0[T] = *reinterpret_cast<const mv_u32x4 *>(q.w + at * 4);
                q1[T] = q0[T];
            } else {
                const int row = min(((t - q.first) * TILES + T) * 16 + n, out_dim - 1);
                const uint16_t *sb = (g < 2 ? q.scales : q.biases) + (size_t)row * groups;
                q0[T] = load_sb8<SB16>(sb, 16 * wave, groups);
                q1[T] = load_sb8<SB16>(sb, 16 * wave + 8, groups);
            }
        }
#pragma unroll
        for (int st = 0; st < STEPS; st++) {
            const int c = 4 * (wave * STEPS + st) + g;
#pragma unroll
            for (int T = 0; T < TILES; T++) {
                if constexpr (TILED) {
                    // [tile][run of 1024 inputs][scales and biases, then the steps][lane]: a wave's
                    // requests are 9 KiB in one piece, each of them 1 KiB
                    const int nruns = (in_dim + 1023) >> 10, tile = (t - q.first) * TILES + T;
                    const size_t at = (((size_t)tile * nruns + (wave < nruns ? wave : 0)) * (STEPS + 1) + 1 + st) * 64 + lane;
                    w[T][st] = *reinterpret_cast<const mv_u32x4 *>(q.w + at * 4);
                } else {
                    const int row = min(((t - q.first) * TILES + T) * 16 + n, out_dim - 1);
                    w[T][st] = *reinterpret_cast<const mv_u32x4 *>(q.w + (size_t)row * words + (c < nchunk ? c : 0) * 4);  // past the row: any chunk, x is 0 there
                }
            }
        }
    };
    // x of product s: three bf16 parts by truncation (x = h + m + l exactly) and the group sums
    constexpr int XP = 2;       // passes, a run of 8 inputs per lane and pass
    float4 xa[XP], xb4[XP];
    auto request_x = [&]() __attribute__((always_inline)) {
        const float *x = q.x;
        const int in_dim = q.in_dim;
#pragma unroll
        for (int p = 0; p < XP; p++) {
            const int r = 128 * wave + lane + 64 * p;   // a wave stages the 1024 inputs it will use itself
            const int at = 8 * r < in_dim ? 8 * r : 0;
            xa[p] = load_f4(x + at);
            xb4[p] = load_f4(x + at + 4);
        }
    };
    auto stage_x = [&]() __attribute__((always_inline)) {
        const int in_dim = q.in_dim;
#pragma unroll
        for (int p = 0; p < XP; p++) {
            const int r = 128 * wave + lane + 64 * p;   // a wave stages the 1024 inputs it will use itself
            mv_u32x4 ph = {0u, 0u, 0u, 0u}, pm = ph, pl = ph;
            float sum = 0.f;
            if (8 * r < in_dim) {   // past the end of x: zeros
                const float4 a = xa[p], b = xb4[p];
                const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
                uint32_t hb[8], mb[8], lb[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {   // v = h + m + l, each a bf16 number (upper 16 bits)
                    hb[e] = __builtin_bit_cast(uint32_t, v[e]);
                    const float r1 = v[e] - __builtin_bit_cast(float, hb[e] & 0xffff0000u);
                    mb[e] = __builtin_bit_cast(uint32_t, r1);
                    lb[e] = __builtin_bit_cast(uint32_t, r1 - __builtin_bit_cast(float, mb[e] & 0xffff0000u));
                }
                const uint32_t hi16 = 0x07060302u;  // (upper half of the second operand, upper half of the first)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    ph[e] = __builtin_amdgcn_perm(hb[e + 4], hb[e], hi16);
                    pm[e] = __builtin_amdgcn_perm(mb[e + 4], mb[e], hi16);
                    pl[e] = __builtin_amdgcn_perm(lb[e + 4], lb[e], hi16);
                }
                sum = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
            }
            *reinterpret_cast<mv_u32x4 *>(&xs[0][8 * r]) = ph;
            *reinterpret_cast<mv_u32x4 *>(&xs[1][8 * r]) = pm;
            *reinterpret_cast<mv_u32x4 *>(&xs[2][8 * r]) = pl;
            sum = group_sum<8>(sum);
            if ((tid & 7) == 0) xsum[r >> 3] = sum;
        }
    };

    // A operand: lane (part row n, input octet g) reads part n % 4 of x if row n belongs to the
    // scale group that octet g lies in (rows 0..2: octets 0, 1; rows 4..6: octets 2, 3), else zeros
    const bool mine = n < 8 && (n & 3) < 3 && (n >> 2) == (g >> 1);
    const uint16_t *xb = (mine ? &xs[n & 3][128 * STEPS * wave] : &zeros[0]) + 32 * g;
    const int half = g & 1, sh = half ? 0 : 16;
    const float *xs_g = &xsum[16 * wave + half];
    request_x();
    fetch();
    // (every wave writes all of the zeros: no wave then has to wait for another before its product)
#pragma unroll
    for (int i = lane; i < (128 * STEPS + 128) / 8; i += 64) *reinterpret_cast<mv_u32x4 *>(&zeros[8 * i]) = mv_u32x4{0u, 0u, 0u, 0u};
    stage_x();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // (x & mask) | bits in one instruction; it takes one constant from a scalar register and one
    // from a vector register, which the compiler will not arrange by itself for two literals
    uint32_t nib_mask = 0x00780078u, one_one = 0x3F803F80u;
    asm volatile("" : "+s"(nib_mask), "+v"(one_one));
    auto and_or = [](uint32_t x, uint32_t mask, uint32_t bits) __attribute__((always_inline)) {
        uint32_t r;
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(mask), "v"(bits));
        return r;
    };
    float acc[TILES];
#pragma unroll
    for (int T = 0; T < TILES; T++) acc[T] = 0.f;
#pragma unroll
    for (int st = 0; st < STEPS; st++) {
        mv_f32x4 d[TILES];
#pragma unroll
        for (int T = 0; T < TILES; T++) d[T] = mv_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const mv_bf16x8 b = *reinterpret_cast<const mv_bf16x8 *>(xb + 128 * st + 8 * j);
#pragma unroll
            for (int T = 0; T < TILES; T++) {
                const uint32_t ww = w[T][st][j];
                mv_u32x4 a;   // nibbles (0,4), (1,5), (2,6), (3,7) as bf16 pairs 1 + n/16
                a[0] = and_or(ww << 3, nib_mask, one_one);
                a[1] = and_or(ww >> 1, nib_mask, one_one);
                a[2] = and_or(ww >> 5, nib_mask, one_one);
                a[3] = and_or(ww >> 9, nib_mask, one_one);
                d[T] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b, __builtin_bit_cast(mv_bf16x8, a), d[T], 0, 0, 0);
            }
        }
        // group 2 st + half of this wave's 16: its scale (lanes g < 2) or bias (the others) for row n
        const float xg = xs_g[2 * st];
#pragma unroll
        for (int T = 0; T < TILES; T++) {
            // file order: element 2 st + half of the wave's 16; TILED: element st of the lane's 8
            const uint32_t word = TILED ? q0[T][st >> 1] : st < 4 ? q0[T][st & 3] : q1[T][st & 3];
            const float val = __builtin_bit_cast(float, (word << (TILED ? ((st & 1) ? 0 : 16) : sh)) & 0xffff0000u);
            const float dsum = (d[T][0] + d[T][1]) + d[T][2];   // sum (1 + nibble/16) x over the group
            acc[T] = fmaf(val, g < 2 ? 16.f * (dsum - xg) : xg, acc[T]);   // 16 s (D - X_g)  |  b X_g
        }
    }
#pragma unroll
    for (int T = 0; T < TILES; T++) {
        acc[T] += __shfl_xor(acc[T], 16, 64);
        acc[T] += __shfl_xor(acc[T], 32, 64);
        if (g == 0) red[wave][16 * T + n] = acc[T];
    }
    __syncthreads();
    const int row = (t - q.first) * 16 * TILES + tid;
    if (tid < 16 * TILES && row < q.out_dim) {
        float v = 0.f;
#pragma unroll
        for (int k = 0; k < WAVES; k++) v += red[k][tid];
        q.out[row] = v;
    }
}

template <int WAVES, bool SB16, bool TILED>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(5, 8))) void dequant_matvec_mfma_kernel(MatvecSpecs sp, MatvecTiles tl) {
    dequant_matvec_body<WAVES, SB16, 1, TILED>(sp, tl);
}

// Weights, scales and biases re-ordered for the kernel above, once, when a model is loaded: for every
// 16-row tile and every run of 1024 inputs the 9 x 64 x 16 bytes its wave requests, in request order.
// First the scales and biases: lane (n, g) gets the eight bf16 values of row n for groups
// 16 run + 2 e + g % 2, e = 0 .. 7 (scales for g < 2, biases for the others), the ones it multiplies
// with.  Then the weights by step, then lane: row lane % 16, 32-input chunk 4 (8 run + step) +
// lane / 16.  Rows past out_dim repeat the last row, chunks and groups past in_dim are zero.
// grid (runs, tiles), 576 threads.
__global__ __launch_bounds__(576) void matvec_tile_weights_kernel(const uint32_t *__restrict__ w, const uint16_t *__restrict__ scales,
                                                                  const uint16_t *__restrict__ biases, uint32_t *__restrict__ tiled,
                                                                  int out_dim, int in_dim) {
    const int run = blockIdx.x, tile = blockIdx.y, nruns = gridDim.x;
    const int i = threadIdx.x >> 6, lane = threadIdx.x & 63;   // request 0: scales and biases; 1 .. 8: steps
    const int row = min(16 * tile + (lane & 15), out_dim - 1);
    const int g = lane >> 4;
    mv_u32x4 v = {0u, 0u, 0u, 0u};
    if (i == 0) {
        const int groups = in_dim >> 6;
        const uint16_t *sb = (g < 2 ? scales : biases) + (size_t)row * groups;
        uint32_t e[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int grp = 16 * run + 2 * k + (g & 1);
            e[k] = grp < groups ? sb[grp] : 0u;
        }
        v = mv_u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
    } else {
        const int c = 4 * (8 * run + (i - 1)) + g;
        if (c < (in_dim >> 5)) v = *reinterpret_cast<const mv_u32x4 *>(w + (size_t)row * (in_dim >> 3) + 4 * c);
    }
    *reinterpret_cast<mv_u32x4 *>(tiled + ((((size_t)tile * nruns + run) * 9 + i) * 64 + lane) * 4) = v;
}

size_t matvec_tiled_words(int out_dim, int in_dim) {
    return (size_t)((out_dim + 15) / 16) * ((in_dim + 1023) / 1024) * 9 * 64 * 4;
}

int launch_matvec_tile_weights(hipStream_t stream, int out_dim, int in_dim, const uint32_t *w, const uint16_t *scales,
                               const uint16_t *biases, uint32_t *tiled) {
    if (!w || !scales || !biases || !tiled) return fail(MFA_ERR_INVALID, "matvec tiling: NULL argument");
    if (out_dim <= 0 || in_dim <= 0 || in_dim % 64 != 0)
        return fail(MFA_ERR_INVALID, "matvec tiling: out_dim %d, in_dim %d (a multiple of 64)", out_dim, in_dim);
    if ((uintptr_t)w % 16 != 0 || (uintptr_t)tiled % 16 != 0)
        return fail(MFA_ERR_INVALID, "matvec tiling: weights must be 16-byte aligned");
    if ((out_dim + 15) / 16 > 65535) return fail(MFA_ERR_SHAPE, "matvec tiling: out_dim %d too large", out_dim);
    hipLaunchKernelGGL(matvec_tile_weights_kernel, dim3((in_dim + 1023) / 1024, (out_dim + 15) / 16), dim3(576), 0, stream,
                       w, scales, biases, tiled, out_dim, in_dim);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

// Device pointers; one launch for up to 8 products (the reference batches a layer's
// projections into one command buffer, full_attn_forward.rs:193-227).
int launch_dequant_matvec_4bit(hipStream_t stream, int n, const uint32_t *const *w, const uint16_t *const *scales,
                               const uint16_t *const *biases, const float *const *x, float *const *out,
                               const int *out_dim, const int *in_dim, int num_cus, bool tiled) {
    if (n <= 0 || n > kMvMaxSpecs) return fail(MFA_ERR_INVALID, "dequant matvec: 1 to %d products per call (got %d)", kMvMaxSpecs, n);
    MatvecSpecs sp{};
    int max_out = 0, max_in = 0;
    bool sb16 = true;   // scale and bias rows can be read 16 bytes at a time in every product
    for (int i = 0; i < n; i++) {
        if (!w[i] || !x[i] || !out[i] || (!tiled && (!scales[i] || !biases[i]))) return fail(MFA_ERR_INVALID, "dequant matvec: NULL pointer in product %d", i);
        if (out_dim[i] <= 0 || in_dim[i] <= 0) return fail(MFA_ERR_INVALID, "dequant matvec: non-positive shape in product %d", i);
        if (in_dim[i] % 64 != 0) return fail(MFA_ERR_INVALID, "dequant matvec: in_dim %d is not a multiple of the group size 64", in_dim[i]);
        if (in_dim[i] > 16384) return fail(MFA_ERR_SHAPE, "dequant matvec: in_dim %d > 16384 not supported", in_dim[i]);
        sp.w[i] = w[i]; sp.scales[i] = scales[i]; sp.biases[i] = biases[i]; sp.x[i] = x[i]; sp.out[i] = out[i];
        sp.out_dim[i] = out_dim[i]; sp.in_dim[i] = in_dim[i];
        if ((uintptr_t)w[i] % 16 != 0 || (uintptr_t)x[i] % 16 != 0)
            return fail(MFA_ERR_INVALID, "dequant matvec: weights and x of product %d must be 16-byte aligned", i);
        if (!tiled && ((in_dim[i] / 64) % 8 != 0 || (uintptr_t)scales[i] % 16 != 0 || (uintptr_t)biases[i] % 16 != 0)) sb16 = false;
        max_out = out_dim[i] > max_out ? out_dim[i] : max_out;
        max_in = in_dim[i] > max_in ? in_dim[i] : max_in;
    }
    MatvecTiles tl{};
    for (int i = 0; i < n; i++) tl.first[i + 1] = tl.first[i] + (out_dim[i] + 15) / 16;
    for (int i = n + 1; i <= kMvMaxSpecs; i++) tl.first[i] = tl.first[n];
    const dim3 grid(tl.first[n]);
    (void)max_out;
    (void)num_cus;
#define MV_LAUNCH(W)                                                                                              \
    do {                                                                                                          \
        if (sb16 && tiled) hipLaunchKernelGGL((dequant_matvec_mfma_kernel<W, true, true>), grid, dim3(W * 64), 0, stream, sp, tl);   \
        else if (sb16) hipLaunchKernelGGL((dequant_matvec_mfma_kernel<W, true, false>), grid, dim3(W * 64), 0, stream, sp, tl);      \
        else if (tiled) hipLaunchKernelGGL((dequant_matvec_mfma_kernel<W, false, true>), grid, dim3(W * 64), 0, stream, sp, tl);     \
        else hipLaunchKernelGGL((dequant_matvec_mfma_kernel<W, false, false>), grid, dim3(W * 64), 0, stream, sp, tl);               \
    } while (0)
    if (max_in <= 1024) MV_LAUNCH(1);
    else if (max_in <= 2048) MV_LAUNCH(2);
    else if (max_in <= 4096) MV_LAUNCH(4);
    else if (max_in <= 8192) MV_LAUNCH(8);
    else MV_LAUNCH(16);
#undef MV_LAUNCH
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
