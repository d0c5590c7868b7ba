// 4-bit group-64 affine dequantising matrix-vector product: the projections either side
// of the attention core (q/k/v_proj, o_proj, in_proj_qkv/z/a/b, out_proj).
//
// Replaces dequant_matvec_4bit_v3 (crates/moeflux/shaders/shaders.metal:251-340; encoder
// gpu_matvec.rs; CPU form cpu_matvec.rs:83-160): out[r] = sum_c (nibble(r,c)*scale + bias)*x[c],
// W packed 8 nibbles per u32 (nibble n at bits 4n..4n+3 is input 8*word + n), one bf16 scale
// and bias per 64 inputs.
//
// Bound: HBM, 0.5625 bytes per weight (4 bits + 2 x bf16 per 64).  At that rate the VALU
// work per weight matters (16 T weights/s at 8 TB/s against 39 T lane-instructions/s): per
// u32 the kernel spends two masks, eight byte->float conversions and eight FMAs, using
//   sum (n s + b) x = s sum n x + b sum x
// so scale and bias are applied once per lane and row, and the high nibbles are converted as
// 16 n against x/16 (exact) to save their shift.
//
// A wave owns a run of rows.  Lane l always handles the same 16-byte column chunks
// (l, l+64, ...), so its slice of x (32 floats per chunk) and the slice's sum stay in
// registers for all of the wave's rows; a row's weights are requested one row ahead.
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

template <int N, typename F> __device__ __forceinline__ void mv_static_for(F &&f) {
    if constexpr (N > 0) {
        mv_static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// sum over the 8 nibbles of `w` of nibble * x: low nibbles of each byte against xl, high
// nibbles (left in place, i.e. 16 * nibble) against xh = x / 16.
__device__ inline float dot8(uint32_t w, const float *xl, const float *xh, float acc) {
    uint32_t lo = w & 0x0F0F0F0Fu, hi = w & 0xF0F0F0F0u;
    // keep the two masked words as they are: the byte selects below then map onto
    // v_cvt_f32_ubyte0..3 (one instruction per nibble) instead of a bit-field extract each
    asm volatile("" : "+v"(lo), "+v"(hi));
    acc = fmaf((float)(lo & 0xFFu), xl[0], acc);
    acc = fmaf((float)(hi & 0xFFu), xh[0], acc);
    acc = fmaf((float)((lo >> 8) & 0xFFu), xl[1], acc);
    acc = fmaf((float)((hi >> 8) & 0xFFu), xh[1], acc);
    acc = fmaf((float)((lo >> 16) & 0xFFu), xl[2], acc);
    acc = fmaf((float)((hi >> 16) & 0xFFu), xh[2], acc);
    acc = fmaf((float)(lo >> 24), xl[3], acc);
    acc = fmaf((float)(hi >> 24), xh[3], acc);
    return acc;
}

// grid (ceil(max out_dim / (4 * ROWS)), n_specs), 256 threads; NCH = ceil(in_dim / 2048).
template <int NCH, int ROWS>
__global__ __launch_bounds__(256) void dequant_matvec_4bit_kernel(MatvecSpecs sp) {
    const int s = blockIdx.y;
    const int in_dim = sp.in_dim[s], out_dim = sp.out_dim[s];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row0 = (blockIdx.x * 4 + wave) * ROWS;
    if (row0 >= out_dim) return;
    const int n16 = in_dim >> 5;  // 16-byte chunks (32 inputs) per row
    const int groups = in_dim >> 6;
    const uint32_t *W = sp.w[s];
    const uint16_t *S = sp.scales[s], *B = sp.biases[s];
    const float *x = sp.x[s];

    // this lane's slice of x: even inputs (low nibbles) as they are, odd inputs / 16
    float xl[NCH][16], xh[NCH][16], sumx[NCH];
    bool live[NCH];
#pragma unroll
    for (int c = 0; c < NCH; c++) {
        const int ch = lane + 64 * c;
        live[c] = ch < n16;
        sumx[c] = 0.f;
#pragma unroll
        for (int u = 0; u < 8; u++) {
            float4 v = {0.f, 0.f, 0.f, 0.f};
            if (live[c]) v = load_f4(x + (size_t)ch * 32 + 4 * u);
            // word u/2 of the chunk, bytes 2(u%2) and 2(u%2)+1: inputs 8(u/2) + 4(u%2) + {0,1,2,3}
            xl[c][2 * u] = v.x;
            xh[c][2 * u] = v.y * 0.0625f;
            xl[c][2 * u + 1] = v.z;
            xh[c][2 * u + 1] = v.w * 0.0625f;
            sumx[c] += (v.x + v.y) + (v.z + v.w);
        }
    }
    auto fetch = [&](int r, mv_u32x4 (&w)[NCH], float (&sc)[NCH], float (&bi)[NCH]) __attribute__((always_inline)) {
        if (r > out_dim - 1) r = out_dim - 1;  // past the end: re-read the last row, never stored
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            const int ch = live[c] ? lane + 64 * c : 0;
            w[c] = *reinterpret_cast<const mv_u32x4 *>(W + (size_t)r * (in_dim >> 3) + (size_t)ch * 4);
            sc[c] = bf16_bits_to_f32(S[(size_t)r * groups + (ch >> 1)]);
            bi[c] = bf16_bits_to_f32(B[(size_t)r * groups + (ch >> 1)]);
        }
    };
    auto row = [&](int r, const mv_u32x4 (&w)[NCH], const float (&sc)[NCH], const float (&bi)[NCH]) __attribute__((always_inline)) {
        float tot = 0.f;
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            const float a0 = dot8(w[c][0], &xl[c][0], &xh[c][0], 0.f);
            const float a1 = dot8(w[c][1], &xl[c][4], &xh[c][4], 0.f);
            const float a2 = dot8(w[c][2], &xl[c][8], &xh[c][8], 0.f);
            const float a3 = dot8(w[c][3], &xl[c][12], &xh[c][12], 0.f);
            const float part = fmaf(sc[c], (a0 + a1) + (a2 + a3), bi[c] * sumx[c]);
            tot += live[c] ? part : 0.f;
        }
        tot = group_sum<64>(tot);
        if (lane == 0 && r < out_dim) sp.out[s][r] = tot;
    };
    // weights of rows i + 1 and i + 2 are in flight while row i is summed
    mv_u32x4 w[3][NCH];
    float sc[3][NCH], bi[3][NCH];
    fetch(row0, w[0], sc[0], bi[0]);
    fetch(row0 + 1, w[1], sc[1], bi[1]);
    mv_static_for<ROWS>([&](auto it) __attribute__((always_inline)) {
        constexpr int i = decltype(it)::value;
        if (i + 2 < ROWS) fetch(row0 + i + 2, w[(i + 2) % 3], sc[(i + 2) % 3], bi[(i + 2) % 3]);
        row(row0 + i, w[i % 3], sc[i % 3], bi[i % 3]);
    });
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
    // rows per wave: as many as still leave every CU about two workgroups
    const int rows = max_out >= 8 * 4 * 2 * num_cus ? 8 : max_out >= 4 * 4 * 2 * num_cus ? 4 : 2;
    const dim3 grid((max_out + 4 * rows - 1) / (4 * rows), n);
#define MFA_MV(NCH)                                                                                          \
    if (rows == 8) hipLaunchKernelGGL((dequant_matvec_4bit_kernel<NCH, 8>), grid, dim3(256), 0, stream, sp);      \
    else if (rows == 4) hipLaunchKernelGGL((dequant_matvec_4bit_kernel<NCH, 4>), grid, dim3(256), 0, stream, sp); \
    else hipLaunchKernelGGL((dequant_matvec_4bit_kernel<NCH, 2>), grid, dim3(256), 0, stream, sp)
    if (max_in <= 2048) { MFA_MV(1); } else if (max_in <= 4096) { MFA_MV(2); } else { MFA_MV(4); }
#undef MFA_MV
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
