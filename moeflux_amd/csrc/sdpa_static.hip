// Decode attention for callers that cannot allocate: the split-K partials of
// mfa_sdpa_decode_static_dev live in a file-scope device array instead of the context's
// workspace, so the call makes no hipMalloc / hipFree whatever the cache length (code under HIP
// graph capture, tight serving loops, harnesses that forbid allocation).  Every GPU the library
// runs on holds its own copy of the array (8.25 MiB) until the process ends; its device address
// is looked up once per device, when the first context on that device is created, and kept.
// Kernels and host code use that address, never the array's name.
#include "mfa_internal.h"

namespace mfa {

// partial outputs [kv head][row group][split][16][D] f32, then the (max, sum) pairs
static constexpr size_t kStaticOElems = (size_t)2 << 20;    // 8 MiB
static constexpr size_t kStaticMlElems = (size_t)64 << 10;  // 256 KiB
static __device__ __align__(256) float scratch[kStaticOElems + kStaticMlElems];

static constexpr int kMaxDevices = 64;
static float *g_scratch_ptr[kMaxDevices];   // device address of `scratch` on each device, once looked up

// The device address of this device's copy of the array; `device` must be the current device.
int static_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return fail(MFA_ERR_INVALID, "device %d out of range", device);
    if (g_scratch_ptr[device]) return MFA_OK;
    void *p = nullptr;
    MFA_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(MFA_ERR_HIP, "no device address for the static scratch array");
    g_scratch_ptr[device] = (float *)p;
    return MFA_OK;
}

size_t static_scratch_bytes() { return sizeof(float) * (kStaticOElems + kStaticMlElems); }

}  // namespace mfa

using namespace mfa;

extern "C" int mfa_sdpa_decode_static_dev(mfa_ctx *ctx, int32_t layer, const float *q_dev, const float *q_gate_dev,
                                          float *out_dev) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q_dev || !q_gate_dev || !out_dev) return fail(MFA_ERR_INVALID, "NULL argument");
    if (f->len <= 0) return fail(MFA_ERR_INVALID, "kv_len must be > 0 (got %d)", f->len);
    float *base = (c->device >= 0 && c->device < kMaxDevices) ? g_scratch_ptr[c->device] : nullptr;
    if (!base) return fail(MFA_ERR_HIP, "the static scratch array was not set up for device %d", c->device);
    const mfa_config &g = c->cfg;
    // the partials of the split plan this call will use must fit the array: nothing grows here
    const int splits = sdpa_pick_splits(g.kv_dtype, g.num_attn_heads, g.num_kv_heads, g.head_dim, f->len, c->num_cus,
                                        c->forced_splits);
    const size_t need_o = sdpa_workspace_o_elems(g.num_attn_heads, g.num_kv_heads, g.head_dim, splits);
    const size_t need_ml = sdpa_workspace_ml_elems(g.num_attn_heads, g.num_kv_heads, splits);
    if (need_o > kStaticOElems || need_ml > kStaticMlElems)
        return fail(MFA_ERR_INVALID,
                    "mfa_sdpa_decode_static_dev: %d splits of %d kv heads need %zu bytes of partials, the static "
                    "scratch holds %zu (use mfa_sdpa_decode_dev, or fewer splits: mfa_set_num_splits)",
                    splits, g.num_kv_heads, (need_o + need_ml) * sizeof(float), static_scratch_bytes());
    SdpaWorkspace ws{base, base + kStaticOElems, kStaticOElems, kStaticMlElems};
    return launch_sdpa(c->stream, g.kv_dtype, g.num_attn_heads, g.num_kv_heads, g.head_dim, 1, f->len, c->plane_elems,
                       f->k, f->v, q_dev, q_gate_dev, out_dev, ws, c->num_cus, c->forced_splits, 0);
}
