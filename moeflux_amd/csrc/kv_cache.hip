// Maintenance of the tiled device KV cache: scatter rows in (append / import),
// gather rows out (export), zero a range (truncate).  The reference's cache is
// row-major [len, kv_dim] f32 (crates/moeflux/src/riir/state.rs:33-74); these
// kernels are the seam between that layout and the tiled one (KvTile).
#include "mfa_internal.h"

namespace mfa {

template <typename KV, typename SRC> __device__ inline KV convert_kv(SRC x);
template <> __device__ inline float convert_kv<float, float>(float x) { return x; }
template <> __device__ inline uint16_t convert_kv<uint16_t, float>(float x) { return f32_to_bf16_bits(x); }
template <> __device__ inline uint16_t convert_kv<uint16_t, uint16_t>(uint16_t x) { return x; }
template <> __device__ inline float convert_kv<float, uint16_t>(uint16_t x) { return bf16_bits_to_f32(x); }

template <typename KV, typename SRC>
__global__ void kv_scatter_kernel(const SRC *__restrict__ k_rows, const SRC *__restrict__ v_rows,
                                  KV *__restrict__ k_tiled, KV *__restrict__ v_tiled,
                                  size_t plane_elems, int Hkv, int D, int64_t pos0,
                                  int64_t n_rows) {
    const int64_t kv_dim = (int64_t)Hkv * D;
    const int64_t total = n_rows * kv_dim;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / kv_dim;
        const int c = (int)(i % kv_dim);
        const int kvh = c / D, x = c % D;
        const int64_t pos = pos0 + r;
        k_tiled[(size_t)kvh * plane_elems + KvTile<KV>::k_off(pos, x, D)] = convert_kv<KV, SRC>(k_rows[i]);
        v_tiled[(size_t)kvh * plane_elems + KvTile<KV>::v_off(pos, x, D)] = convert_kv<KV, SRC>(v_rows[i]);
    }
}

template <typename KV>
__global__ void kv_gather_kernel(const KV *__restrict__ k_tiled, const KV *__restrict__ v_tiled,
                                 float *__restrict__ k_rows, float *__restrict__ v_rows,
                                 size_t plane_elems, int Hkv, int D, int64_t n_rows) {
    const int64_t kv_dim = (int64_t)Hkv * D;
    const int64_t total = n_rows * kv_dim;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t r = i / kv_dim;
        const int c = (int)(i % kv_dim);
        const int kvh = c / D, x = c % D;
        k_rows[i] = convert_kv<float, KV>(k_tiled[(size_t)kvh * plane_elems + KvTile<KV>::k_off(r, x, D)]);
        v_rows[i] = convert_kv<float, KV>(v_tiled[(size_t)kvh * plane_elems + KvTile<KV>::v_off(r, x, D)]);
    }
}

template <typename KV>
__global__ void kv_zero_kernel(KV *__restrict__ k_tiled, KV *__restrict__ v_tiled,
                               size_t plane_elems, int Hkv, int D, int64_t pos0, int64_t pos1) {
    const int64_t kv_dim = (int64_t)Hkv * D;
    const int64_t total = (pos1 - pos0) * kv_dim;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t pos = pos0 + i / kv_dim;
        const int c = (int)(i % kv_dim);
        const int kvh = c / D, x = c % D;
        k_tiled[(size_t)kvh * plane_elems + KvTile<KV>::k_off(pos, x, D)] = (KV)0;
        v_tiled[(size_t)kvh * plane_elems + KvTile<KV>::v_off(pos, x, D)] = (KV)0;
    }
}

static int grid_for(int64_t total, int block) {
    int64_t gsz = (total + block - 1) / block;
    if (gsz > 65536) gsz = 65536;
    if (gsz < 1) gsz = 1;
    return (int)gsz;
}

int launch_kv_scatter(hipStream_t stream, int kv_dtype, int src_is_bf16, int Hkv, int D,
                      size_t plane_elems, int64_t pos0, int64_t n_rows, const void *k_rows,
                      const void *v_rows, void *k_tiled, void *v_tiled) {
    if (n_rows <= 0) return MFA_OK;
    const int64_t total = n_rows * Hkv * D;
    const int grid = grid_for(total, 256);
    if (kv_dtype == MFA_KV_BF16 && src_is_bf16)
        hipLaunchKernelGGL((kv_scatter_kernel<uint16_t, uint16_t>), dim3(grid), dim3(256), 0, stream,
                           (const uint16_t *)k_rows, (const uint16_t *)v_rows, (uint16_t *)k_tiled,
                           (uint16_t *)v_tiled, plane_elems, Hkv, D, pos0, n_rows);
    else if (kv_dtype == MFA_KV_BF16)
        hipLaunchKernelGGL((kv_scatter_kernel<uint16_t, float>), dim3(grid), dim3(256), 0, stream,
                           (const float *)k_rows, (const float *)v_rows, (uint16_t *)k_tiled,
                           (uint16_t *)v_tiled, plane_elems, Hkv, D, pos0, n_rows);
    else if (src_is_bf16)
        hipLaunchKernelGGL((kv_scatter_kernel<float, uint16_t>), dim3(grid), dim3(256), 0, stream,
                           (const uint16_t *)k_rows, (const uint16_t *)v_rows, (float *)k_tiled,
                           (float *)v_tiled, plane_elems, Hkv, D, pos0, n_rows);
    else
        hipLaunchKernelGGL((kv_scatter_kernel<float, float>), dim3(grid), dim3(256), 0, stream,
                           (const float *)k_rows, (const float *)v_rows, (float *)k_tiled,
                           (float *)v_tiled, plane_elems, Hkv, D, pos0, n_rows);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_kv_gather(hipStream_t stream, int kv_dtype, int Hkv, int D, size_t plane_elems,
                     int64_t n_rows, const void *k_tiled, const void *v_tiled, float *k_rows,
                     float *v_rows) {
    if (n_rows <= 0) return MFA_OK;
    const int grid = grid_for(n_rows * Hkv * D, 256);
    if (kv_dtype == MFA_KV_BF16)
        hipLaunchKernelGGL((kv_gather_kernel<uint16_t>), dim3(grid), dim3(256), 0, stream,
                           (const uint16_t *)k_tiled, (const uint16_t *)v_tiled, k_rows, v_rows,
                           plane_elems, Hkv, D, n_rows);
    else
        hipLaunchKernelGGL((kv_gather_kernel<float>), dim3(grid), dim3(256), 0, stream,
                           (const float *)k_tiled, (const float *)v_tiled, k_rows, v_rows,
                           plane_elems, Hkv, D, n_rows);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

int launch_kv_zero(hipStream_t stream, int kv_dtype, int Hkv, int D, size_t plane_elems,
                   int64_t pos0, int64_t pos1, void *k_tiled, void *v_tiled) {
    if (pos1 <= pos0) return MFA_OK;
    const int grid = grid_for((pos1 - pos0) * Hkv * D, 256);
    if (kv_dtype == MFA_KV_BF16)
        hipLaunchKernelGGL((kv_zero_kernel<uint16_t>), dim3(grid), dim3(256), 0, stream,
                           (uint16_t *)k_tiled, (uint16_t *)v_tiled, plane_elems, Hkv, D, pos0, pos1);
    else
        hipLaunchKernelGGL((kv_zero_kernel<float>), dim3(grid), dim3(256), 0, stream,
                           (float *)k_tiled, (float *)v_tiled, plane_elems, Hkv, D, pos0, pos1);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

// Plain 16-byte-per-lane device copy (mfa_debug_copy_dev): a kernel of known traffic,
// nbytes read and nbytes written, against which hardware memory counters are scaled.
__global__ void plain_copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

int launch_plain_copy(hipStream_t stream, void *dst, const void *src, size_t nbytes) {
    if (nbytes % 16 != 0) return fail(MFA_ERR_INVALID, "copy size must be a multiple of 16 bytes");
    if (nbytes == 0) return MFA_OK;
    hipLaunchKernelGGL(plain_copy_kernel, dim3(grid_for((int64_t)(nbytes / 16), 256)), dim3(256), 0, stream,
                       (const uint4 *)src, (uint4 *)dst, nbytes / 16);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

// Streaming read of nbytes and nothing else (mfa_debug_read_dev): every workgroup reads one
// contiguous share, eight 16-byte loads per lane in flight, each wave-level load 1 KiB
// contiguous and non-temporal - the access pattern of the decode kernel without its arithmetic
// or its partials.  Its time is what the memory system allows a launch of that size.
__global__ __launch_bounds__(256) void plain_read_kernel(const uint4 *__restrict__ src, size_t n_per_block, size_t n,
                                                         uint4 *__restrict__ sink) {
    typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
    const size_t base = (size_t)blockIdx.x * n_per_block;
    size_t end = base + n_per_block;
    if (end > n) end = n;
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (size_t i = base + threadIdx.x; i < end; i += 256 * 8) {
        u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const size_t j = i + (size_t)u * 256;
            v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src) + (j < end ? j : i));
        }
#pragma unroll
        for (int u = 0; u < 8; u++) acc ^= v[u];
    }
    // never true for the buffers this is run on (the store keeps the loads alive)
    if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u && acc.z == 0x0fedcba9u) sink[blockIdx.x] = __builtin_bit_cast(uint4, acc);
}

int launch_plain_read(hipStream_t stream, const void *src, size_t nbytes, int workgroups, void *sink) {
    if (nbytes % 16 != 0 || nbytes == 0) return fail(MFA_ERR_INVALID, "read size must be a positive multiple of 16 bytes");
    if (workgroups <= 0 || workgroups > 65536) return fail(MFA_ERR_INVALID, "1 to 65536 workgroups (got %d)", workgroups);
    const size_t n = nbytes / 16;
    const size_t per = (n + workgroups - 1) / workgroups;
    hipLaunchKernelGGL(plain_read_kernel, dim3(workgroups), dim3(256), 0, stream, (const uint4 *)src, per, n, (uint4 *)sink);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

}  // namespace mfa
