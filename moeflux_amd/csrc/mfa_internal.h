// Internal declarations shared by the translation units of libmoeflux_attn_hip.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <string>
#include <utility>
#include <vector>

#include "moeflux_attn.h"

namespace mfa {

// ---- error plumbing --------------------------------------------------------
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);

#define MFA_HIP(expr)                                                                  \
    do {                                                                               \
        hipError_t _e = (expr);                                                        \
        if (_e != hipSuccess)                                                          \
            return ::mfa::fail(MFA_ERR_HIP, "%s failed: %s (%s:%d)", #expr,            \
                               hipGetErrorString(_e), __FILE__, __LINE__);             \
    } while (0)

#define MFA_TRY(expr)              \
    do {                           \
        int _rc = (expr);          \
        if (_rc != MFA_OK) return _rc; \
    } while (0)

// ---- small device helpers ---------------------------------------------------
__host__ __device__ inline float bf16_bits_to_f32(uint16_t b) {
    union { uint32_t u; float f; } c;
    c.u = ((uint32_t)b) << 16;
    return c.f;
}

// round-to-nearest-even; NaN stays NaN.
__host__ __device__ inline uint16_t f32_to_bf16_bits(float f) {
    union { uint32_t u; float f; } c;
    c.f = f;
    uint32_t u = c.u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// ---- KV cache tiling ---------------------------------------------------------
// The device KV cache is stored in the order the attention kernels' MFMA operands
// consume it, so that every wave-level load is one contiguous 1 KiB run that goes
// straight from HBM into matrix-core operand registers, and so that the four waves of a
// decode workgroup, reading side by side, sweep memory in one contiguous stream.
//
// One plane per (layer, K|V, kv head).  K is grouped in chunks of 64 positions (KCH), V in
// blocks of 32 (bf16) or 16 (f32) positions (BLK); a chunk and a block are contiguous.
//
// K, chunk of 64 positions, element (p, x) with p in [0,64), x in [0,D).  A 1 KiB piece holds
// 16 positions (sub-tile p/16) of one MFMA k-step; the four sub-tiles of a k-step are adjacent:
//   bf16: [step = x/32][sub = p/16][part = (x%32)/8][row = p%16][e = x%8]
//   f32:  [step = x/16][sub = p/16][part = (x%16)/4][row = p%16][e = x%4]
// V, element (p, x) of a block:
//   bf16, 32 positions: [dt = x/16][g = (p%16)/4][m = x%16][e = 4*(p/16) + p%4]
//   f32,  16 positions: [dt = x/16][g = p/4][m = x%16][j = p%4]
template <typename T> struct KvTile;

template <> struct KvTile<uint16_t> {
    static constexpr int BLK = 32;
    static constexpr int KCH = 64;
    __host__ __device__ static inline int64_t k_off(int64_t pos, int x, int D) {
        const int64_t ch = pos / 64;
        const int p = (int)(pos % 64);
        return ch * 64 * D + (((int64_t)(x / 32) * 4 + p / 16) * 4 + (x % 32) / 8) * 128 + (p % 16) * 8 + (x % 8);
    }
    __host__ __device__ static inline int64_t v_off(int64_t pos, int x, int D) {
        const int64_t blk = pos / 32;
        const int p = (int)(pos % 32);
        const int g = (p % 16) / 4;
        const int e = 4 * (p / 16) + (p % 4);
        return blk * 32 * D + (((int64_t)(x / 16) * 4 + g) * 16 + (x % 16)) * 8 + e;
    }
};

template <> struct KvTile<float> {
    static constexpr int BLK = 16;
    static constexpr int KCH = 64;
    __host__ __device__ static inline int64_t k_off(int64_t pos, int x, int D) {
        const int64_t ch = pos / 64;
        const int p = (int)(pos % 64);
        return ch * 64 * D + (((int64_t)(x / 16) * 4 + p / 16) * 4 + (x % 16) / 4) * 64 + (p % 16) * 4 + (x % 4);
    }
    __host__ __device__ static inline int64_t v_off(int64_t pos, int x, int D) {
        const int64_t blk = pos / 16;
        const int p = (int)(pos % 16);
        return blk * 16 * D + ((((int64_t)(x / 16)) * 4 + p / 4) * 16 + (x % 16)) * 4 + (p % 4);
    }
};

// positions the planes are padded to (whole K chunks, which are whole V blocks)
static constexpr int kKvChunk = 64;

// ---- context ----------------------------------------------------------------
struct LinearWeights {
    uint16_t *conv_w = nullptr;  // [C, K] bf16
    float *a_log = nullptr;      // [Hv]
    uint16_t *dt_bias = nullptr; // [Hv] bf16
    uint16_t *norm_w = nullptr;  // [dv] bf16
    bool set = false;
};

struct FullLayer {
    void *k = nullptr;  // [Hkv] planes, tiled (see KvTile)
    void *v = nullptr;
    int32_t len = 0;
    uint16_t *q_norm = nullptr;  // [head_dim] bf16, per-head RMS norm weights of q and k
    uint16_t *k_norm = nullptr;
    bool norms_set = false;
};

struct LinearLayer {
    float *conv_ring = nullptr; // [K, C] ring of the last K inputs (slot = step % K)
    float *ssm = nullptr;       // [Hv, dv, dk]
    int64_t step = 0;           // tokens consumed since the last reset/import
    LinearWeights w;
};

// The state at one sequence position, kept on the device (checkpoint.hip).
struct Checkpoint {
    int32_t pos = 0;
    char *buf = nullptr;              // one allocation: K prefixes, V prefixes, rings, recurrent states
    size_t bytes = 0;                 // bytes in use
    size_t cap = 0;                   // bytes allocated
    std::vector<int32_t> full_len;    // cache length of every full-attention layer
    std::vector<int64_t> lin_step;    // ring position of every linear layer
};

struct Ctx {
    mfa_config cfg{};
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    std::vector<int> kind;      // per layer: 1 = full attention, 0 = linear
    std::vector<int> slot;      // index into full / lin
    std::vector<FullLayer> full;
    std::vector<LinearLayer> lin;
    std::vector<void *> slabs;  // device allocations behind full[] and lin[] (layer-major)
    int32_t sweep_per_layer = 0; // 1: the token sweep launches layer by layer
    // rotation of q and k ahead of the attention core: 1 / theta^(2i/rotary_dim) on the device
    float *inv_freq = nullptr;
    int32_t rotary_dim = 0;
    float *qg_stage = nullptr;   // q and gate of mfa_full_attn_step, 2 * q_dim floats
    float *step_score = nullptr; // the new token's score per query row of the two-launch attention step
    int32_t step_launches = 2;   // launches of mfa_full_attn_step: 2 (prologue inside the attention launch) or 3
    float *qg_chunk = nullptr;   // the same for a chunk of tokens (mfa_prefill_full_attn), grown on demand
    size_t qg_chunk_elems = 0;
    int64_t cap_pad = 0;        // kv capacity rounded up to whole K chunks
    size_t plane_elems = 0;     // elements of one (layer, K|V, kv head) plane
    // split-K workspace
    float *part_o = nullptr;
    float *part_ml = nullptr;
    size_t part_o_elems = 0, part_ml_elems = 0;
    int32_t forced_splits = 0;
    int32_t partial_only = 0;
    // scratch of the Gated-DeltaNet chunk kernels (grown on demand)
    float *gdn_scratch = nullptr;
    size_t gdn_scratch_elems = 0;
    // host-pointer staging
    float *stage = nullptr;
    size_t stage_elems = 0;
    float *pinned = nullptr;
    size_t pinned_elems = 0;
    int num_cus = 256;
    // checkpoints by position, least recently stored first (checkpoint.hip)
    std::vector<Checkpoint> checkpoints;
    size_t max_checkpoints = 4;       // DEFAULT_MAX_CHECKPOINTS, riir/mod.rs:105-109
    // buffers of evicted or replaced checkpoints, kept for the next store (buffer, bytes allocated)
    std::vector<std::pair<char *, size_t>> checkpoint_pool;

    int conv_dim() const {
        return 2 * cfg.linear_num_k_heads * cfg.linear_key_dim +
               cfg.linear_num_v_heads * cfg.linear_value_dim;
    }
    int q_dim() const { return cfg.num_attn_heads * cfg.head_dim; }
    int kv_dim() const { return cfg.num_kv_heads * cfg.head_dim; }
    int v_total() const { return cfg.linear_num_v_heads * cfg.linear_value_dim; }
    size_t kv_elem_size() const { return cfg.kv_dtype == MFA_KV_BF16 ? 2 : 4; }
};

inline Ctx *as_ctx(mfa_ctx *c) { return reinterpret_cast<Ctx *>(c); }

int full_layer(Ctx *c, int32_t layer, FullLayer **out);
int linear_layer(Ctx *c, int32_t layer, LinearLayer **out);
int ensure_stage(Ctx *c, size_t elems);
// The staging buffer a context keeps between calls is at most this many floats (256 MiB): the bulk
// entry points (snapshot, cache import and export), whose staging grows with the cache length, call
// release_stage_beyond_cap once their work on the stream has completed.
static constexpr size_t kStageCap = ((size_t)256 << 20) / sizeof(float);
int release_stage_beyond_cap(Ctx *c);
// api.hip: device-to-device halves of the state export and import calls (no synchronisation)
int kv_export_to(Ctx *c, FullLayer *f, float *k_dev, float *v_dev);
int kv_import_from(Ctx *c, FullLayer *f, int32_t len, const float *k_dev, const float *v_dev);
int linear_export_to(Ctx *c, LinearLayer *l, float *conv_dev);
int linear_import_from(Ctx *c, LinearLayer *l, const float *conv_dev);

// ---- kernel launchers (device pointers, asynchronous on `stream`) ------------

// sdpa_decode.hip
struct SdpaWorkspace {
    float *part_o;
    float *part_ml;
    size_t part_o_elems, part_ml_elems;
};
bool sdpa_shape_supported(int kv_dtype, int head_dim);
// Number of splits the launcher will use (for workspace sizing pass kv_len = capacity).
int sdpa_max_splits(int kv_dtype, int Hq, int Hkv, int D, int64_t max_len, int num_cus, int forced);
int sdpa_pick_splits(int kv_dtype, int Hq, int Hkv, int D, int64_t kv_len, int num_cus, int forced);
size_t sdpa_workspace_o_elems(int Hq, int Hkv, int D, int splits, int n_tok = 1);
size_t sdpa_workspace_ml_elems(int Hq, int Hkv, int splits, int n_tok = 1);
// n_tok query tokens (q, gate, out: [n_tok, Hq*D]) against a cache of kv_len positions that
// already holds them; token t attends to positions [0, kv_len - n_tok + t].  n_tok = 1 is decode.
// A merge of split-K partials that its caller will run inside a later launch on the same stream
// (n_units == 0: nothing deferred).  Only merges of at most 16 splits are handed over.
struct SdpaMergeTask {
    const float *part_o = nullptr, *part_ml = nullptr, *gate = nullptr;
    float *out = nullptr;
    int nsplit = 0, hpk = 0, Hq = 0, nhg = 0, D = 0, n_units = 0;
};
int launch_sdpa(hipStream_t stream, int kv_dtype, int Hq, int Hkv, int D, int n_tok, int64_t kv_len,
                size_t plane_elems, const void *k_tiled, const void *v_tiled, const float *q,
                const float *gate, float *out, const SdpaWorkspace &ws, int num_cus,
                int forced_splits, int partial_only = 0, SdpaMergeTask *defer_merge = nullptr);
// One decode token of a full-attention layer from its raw projections in two launches (the
// attention launch norms and rotates the query itself and appends the token; the merge takes
// the token as one more split).  len0: cache length before the call.
bool sdpa_step_supported(int kv_dtype, int Hq, int Hkv, int D, int rotary_dim);
int launch_sdpa_step(hipStream_t stream, int kv_dtype, int Hq, int Hkv, int D, int64_t len0, size_t plane_elems,
                     void *k_tiled, void *v_tiled, const float *q_proj, const float *k_in, const float *v_in,
                     const uint16_t *q_norm, const uint16_t *k_norm, const float *inv_freq, int rotary_dim,
                     float eps, int32_t pos, float *new_score, float *out, const SdpaWorkspace &ws, int num_cus,
                     int forced_splits);
// Log-sum-exp merge of partials laid out [kv head][16-row group][split][16][D] (+ (max, sum) per row),
// normalisation, and the sigmoid gate when `gate` is not null.  out, gate: [n_tok, Hq*D].
int launch_sdpa_merge(hipStream_t stream, const SdpaWorkspace &ws, int splits, int hpk, int Hq, int nhg, int D,
                      int n_tok, const float *gate, float *out);
// mla_sdpa.hip: one query token of H heads against a latent cache [L, R] + rotary keys [L, P].
struct MlaPlan {
    int splits;     // workgroups along the cache
    int bps;        // 16-position blocks per split
    int nhg;        // 16-head groups
    int nwg_heads;  // workgroups along the heads (4 groups each)
};
bool mla_shape_supported(int kv_lora_rank, int qk_rope_head_dim);
MlaPlan mla_plan(int H, int L, int num_cus, int forced_splits = 0);
size_t mla_workspace_o_elems(const MlaPlan &p, int R);
size_t mla_workspace_ml_elems(const MlaPlan &p);
int launch_mla_sdpa_folded(hipStream_t stream, int H, int R, int P, int L, float softmax_scale,
                           const float *q_prime, const float *q_pe, const float *latent, const float *rope_k,
                           float *out, const SdpaWorkspace &ws, const MlaPlan &plan);
// dequant_matvec.hip: up to 8 four-bit dequantising matrix-vector products in one launch.
int launch_dequant_matvec_4bit(hipStream_t stream, int n, const uint32_t *const *w, const uint16_t *const *scales,
                               const uint16_t *const *biases, const float *const *x, float *const *out,
                               const int *out_dim, const int *in_dim, int num_cus = 256, bool tiled = false);
// The weight order the tiled form of the kernel reads (words of the re-ordered copy, and the copy itself).
size_t matvec_tiled_words(int out_dim, int in_dim);
int launch_matvec_tile_weights(hipStream_t stream, int out_dim, int in_dim, const uint32_t *w, const uint16_t *scales,
                               const uint16_t *biases, uint32_t *tiled);
// attn_prologue.hip: q/gate split, per-head norms, rotation, cache append of one token.
int launch_attn_prologue(hipStream_t s, int kv_dtype, int Hq, int Hkv, int D, int rotary_dim, float eps, int n_tok,
                         int32_t pos, int64_t cache_pos, size_t plane_elems, const uint16_t *q_norm,
                         const uint16_t *k_norm, const float *inv_freq, const float *q_proj, const float *k_in,
                         const float *v_in, float *q_out, float *gate_out, void *k_tiled, void *v_tiled);
// sdpa_prefill.hip: the same contract for a chunk whose rows fill the machine without
// splitting the cache (no workspace, one launch).
bool sdpa_prefill_applies(int kv_dtype, int Hq, int Hkv, int n_tok, int64_t kv_len, int num_cus);
int launch_sdpa_prefill(hipStream_t stream, int kv_dtype, int Hq, int Hkv, int D, int n_tok, int64_t kv_len,
                        size_t plane_elems, const void *k_tiled, const void *v_tiled, const float *q,
                        const float *gate, float *out, int num_cus);
// Scatter `n_rows` row-major rows ([n_rows, Hkv*D], f32 or bf16 source) into the
// tiled planes starting at position pos0.
int launch_kv_scatter(hipStream_t stream, int kv_dtype, int src_is_bf16, int Hkv, int D,
                      size_t plane_elems, int64_t pos0, int64_t n_rows, const void *k_rows,
                      const void *v_rows, void *k_tiled, void *v_tiled);
// Gather positions [0, n_rows) back to row-major f32.
int launch_kv_gather(hipStream_t stream, int kv_dtype, int Hkv, int D, size_t plane_elems,
                     int64_t n_rows, const void *k_tiled, const void *v_tiled, float *k_rows,
                     float *v_rows);
// Zero positions [pos0, pos1) of every plane.
int launch_kv_zero(hipStream_t stream, int kv_dtype, int Hkv, int D, size_t plane_elems,
                   int64_t pos0, int64_t pos1, void *k_tiled, void *v_tiled);

int launch_plain_copy(hipStream_t stream, void *dst, const void *src, size_t nbytes);
// A launch that only reads nbytes (sink: 16 bytes per workgroup, never written in practice).
int launch_plain_read(hipStream_t stream, const void *src, size_t nbytes, int workgroups, void *sink);

// sdpa_static.hip: looks up, once per device, the device address of the file-scope scratch array
// of mfa_sdpa_decode_static_dev; `device` must be the current device.
int static_scratch_init(int device);

// checkpoint.hip
void drop_checkpoints(Ctx *c);   // frees every stored checkpoint (reset, destroy)

// attn_kernels.hip (the four reference kernels, one launch each)
int launch_attn_scores(hipStream_t s, int Hq, int Hkv, int D, int L, int stride, const float *q,
                       const float *k, float scale, float *scores);
int launch_attn_softmax(hipStream_t s, int Hq, int L, int stride, float *scores);
int launch_attn_values(hipStream_t s, int Hq, int Hkv, int D, int L, int stride,
                       const float *scores, const float *v, float *out);
int launch_sigmoid_gate(hipStream_t s, int dim, const float *gate, float *x);

// gdn.hip
bool gdn_shape_supported(int Hk, int Hv, int dk, int dv, int K);
int launch_gdn_step(hipStream_t s, int Hk, int Hv, int dk, int dv, int K, float eps,
                    const LinearWeights &w, float *conv_ring, int64_t step, float *ssm,
                    const float *qkv_in, const float *z, const float *alpha, const float *beta,
                    float *out, int n_layers = 1, const SdpaMergeTask *merge = nullptr);
// gdn_chunk.hip: T tokens through one layer (three launches); scratch holds
// gdn_chunk_scratch_elems floats.
size_t gdn_chunk_scratch_elems(int Hk, int Hv, int dk, int dv, int T);
// gdn_wy.hip: the recurrence of a chunk in blocked form (blocks of 64 tokens) on the matrix
// cores, from the per-token operands the chunk's first kernel prepares.
size_t gdn_wy_scratch_elems(int Hv, int dk, int dv, int T);
// The layer's inputs, for blocks of the blocked form that compute their own operands from them.
struct WyInputs {
    const float *qkv;          // [T, C] the chunk's conv inputs
    const float *ring;         // [K, C] conv history (input number s in slot s % K)
    const uint16_t *conv_w;    // [C, K] bf16
    const float *a_log;        // [Hv]
    const uint16_t *dt_bias;   // [Hv] bf16
    const float *alpha, *beta; // [T, Hv]
    int K, step_mod;
};
int launch_gdn_wy(hipStream_t s, int Hk, int Hv, int dk, int dv, int T, const float *qn, const float *kn,
                  const float *vv, const float *lg, const float *bg, float *scratch, float *ssm,
                  float *o_raw, const WyInputs *in = nullptr);
int launch_gdn_chunk(hipStream_t s, int Hk, int Hv, int dk, int dv, int K, float eps, int T,
                     const LinearWeights &w, float *conv_ring, int64_t step, float *ssm,
                     const float *qkv_in, const float *z, const float *alpha, const float *beta,
                     float *scratch, float *out);
int launch_conv1d_step(hipStream_t s, int C, int K, float *conv_state, const float *in,
                       const uint16_t *w, float *out);
int launch_rms_norm_qk(hipStream_t s, int Hk, int dk, float *q, float *k);
int launch_rms_norm_bare(hipStream_t s, int dim, float eps, const float *x, float *out);
int launch_decay_beta(hipStream_t s, int Hv, const float *alpha, const float *beta,
                      const float *a_log, const uint16_t *dt_bias, float *g, float *b);
int launch_delta_net_step(hipStream_t s, int Hv, int Hk, int dk, int dv, const float *g,
                          const float *b, const float *q, const float *k, const float *v,
                          float *ssm, float *out);
int launch_gated_rms_norm(hipStream_t s, int H, int dim, float eps, const float *x,
                          const float *z, const uint16_t *w, float *out);
// ring <-> time-major conversion of the conv state
int launch_conv_ring_export(hipStream_t s, int C, int K, int64_t step, const float *ring,
                            float *state_out);
int launch_conv_ring_import(hipStream_t s, int C, int K, const float *state, float *ring);

}  // namespace mfa
