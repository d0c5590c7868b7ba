// Host side of libmoeflux_attn_hip: context, state operations and the extern "C"
// entry points declared in include/moeflux_attn.h.
#include <cstdarg>
#include <cstring>
#include <new>

#include "mfa_internal.h"

namespace mfa {

static thread_local std::string g_last_error;

void set_error(const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

int full_layer(Ctx *c, int32_t layer, FullLayer **out) {
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    if (layer < 0 || layer >= c->cfg.num_layers)
        return fail(MFA_ERR_LAYER, "layer %d out of range [0, %d)", layer, c->cfg.num_layers);
    if (c->kind[layer] != 1)
        return fail(MFA_ERR_LAYER, "layer %d is a linear-attention layer", layer);
    *out = &c->full[c->slot[layer]];
    return MFA_OK;
}

int linear_layer(Ctx *c, int32_t layer, LinearLayer **out) {
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    if (layer < 0 || layer >= c->cfg.num_layers)
        return fail(MFA_ERR_LAYER, "layer %d out of range [0, %d)", layer, c->cfg.num_layers);
    if (c->kind[layer] != 0)
        return fail(MFA_ERR_LAYER, "layer %d is a full-attention layer", layer);
    *out = &c->lin[c->slot[layer]];
    return MFA_OK;
}

int ensure_stage(Ctx *c, size_t elems) {
    if (elems <= c->stage_elems) return MFA_OK;
    MFA_HIP(hipStreamSynchronize(c->stream));
    if (c->stage) MFA_HIP(hipFree(c->stage));
    c->stage = nullptr;
    c->stage_elems = 0;
    MFA_HIP(hipMalloc((void **)&c->stage, elems * sizeof(float)));
    c->stage_elems = elems;
    return MFA_OK;
}

int release_stage_beyond_cap(Ctx *c) {
    if (c->stage_elems <= kStageCap) return MFA_OK;
    MFA_HIP(hipFree(c->stage));
    c->stage = nullptr;
    c->stage_elems = 0;
    // (hipMemGetInfo shows the bytes again once another command has followed the stream's last one:
    // the runtime keeps a freed buffer alive as long as the last command submitted refers to it)
    return MFA_OK;
}

static SdpaWorkspace workspace(Ctx *c) {
    return SdpaWorkspace{c->part_o, c->part_ml, c->part_o_elems, c->part_ml_elems};
}

static int h2d(Ctx *c, void *dst, const void *src, size_t bytes) {
    MFA_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, c->stream));
    return MFA_OK;
}
static int d2h_sync(Ctx *c, void *dst, const void *src, size_t bytes) {
    MFA_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, c->stream));
    MFA_HIP(hipStreamSynchronize(c->stream));
    return MFA_OK;
}

static void destroy(Ctx *c) {
    if (!c) return;
    (void)hipSetDevice(c->device);
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    drop_checkpoints(c);
    for (void *p : c->slabs)
        if (p) (void)hipFree(p);
    if (c->part_o) (void)hipFree(c->part_o);
    if (c->part_ml) (void)hipFree(c->part_ml);
    if (c->stage) (void)hipFree(c->stage);
    if (c->gdn_scratch) (void)hipFree(c->gdn_scratch);
    if (c->qg_chunk) (void)hipFree(c->qg_chunk);
    if (c->ev0) (void)hipEventDestroy(c->ev0);
    if (c->ev1) (void)hipEventDestroy(c->ev1);
    if (c->stream) (void)hipStreamDestroy(c->stream);
    delete c;
}

// A zero-filled device allocation owned by the context until it is destroyed.
static int slab_alloc(Ctx *c, size_t bytes, char **out) {
    void *p = nullptr;
    MFA_HIP(hipMalloc(&p, bytes ? bytes : 4));
    c->slabs.push_back(p);
    MFA_HIP(hipMemsetAsync(p, 0, bytes, c->stream));
    *out = (char *)p;
    return MFA_OK;
}

// The frequency table of rope.rs:99-103, with the host's powf (the reference computes the
// same expression with its libm on every call), uploaded once.
static int set_rope(Ctx *c, float theta, int32_t rotary_dim) {
    if (!c->inv_freq) return fail(MFA_ERR_LAYER, "the context has no full-attention layer");
    if (!(theta > 0.f) || rotary_dim <= 0 || rotary_dim > c->cfg.head_dim || (rotary_dim & 1))
        return fail(MFA_ERR_INVALID, "rope: theta %g, rotary_dim %d (even, in (0, head_dim])", (double)theta, rotary_dim);
    std::vector<float> f((size_t)rotary_dim / 2);
    for (int i = 0; i < rotary_dim / 2; i++) f[i] = 1.0f / powf(theta, (float)(2 * i) / (float)rotary_dim);
    MFA_HIP(hipMemcpyAsync(c->inv_freq, f.data(), f.size() * sizeof(float), hipMemcpyHostToDevice, c->stream));
    MFA_HIP(hipStreamSynchronize(c->stream));
    c->rotary_dim = rotary_dim;
    return MFA_OK;
}

static int validate(const mfa_config *cfg, bool *has_full, bool *has_lin) {
    if (!cfg) return fail(MFA_ERR_INVALID, "NULL config");
    if (cfg->num_layers <= 0 || cfg->full_attn_interval <= 0)
        return fail(MFA_ERR_INVALID, "num_layers and full_attn_interval must be positive");
    *has_full = false;
    *has_lin = false;
    for (int i = 0; i < cfg->num_layers; i++) {
        if ((i + 1) % cfg->full_attn_interval == 0) *has_full = true;
        else *has_lin = true;
    }
    if (*has_full) {
        if (cfg->num_attn_heads <= 0 || cfg->num_kv_heads <= 0 || cfg->head_dim <= 0 ||
            cfg->kv_capacity <= 0)
            return fail(MFA_ERR_INVALID, "non-positive full-attention shape");
        if (cfg->num_attn_heads % cfg->num_kv_heads != 0)
            return fail(MFA_ERR_INVALID, "num_attn_heads %d is not a multiple of num_kv_heads %d",
                        cfg->num_attn_heads, cfg->num_kv_heads);
        if (!sdpa_shape_supported(cfg->kv_dtype, cfg->head_dim))
            return fail(MFA_ERR_SHAPE, "head_dim %d / kv_dtype %d not supported (64, 128, 256; f32, bf16)",
                        cfg->head_dim, cfg->kv_dtype);
    }
    if (*has_lin) {
        if (cfg->linear_num_k_heads <= 0 || cfg->linear_num_v_heads <= 0 ||
            cfg->linear_key_dim <= 0 || cfg->linear_value_dim <= 0 || cfg->conv_kernel_size <= 0)
            return fail(MFA_ERR_INVALID, "non-positive linear-attention shape");
        if (cfg->linear_num_v_heads % cfg->linear_num_k_heads != 0)
            return fail(MFA_ERR_INVALID, "linear_num_v_heads %d is not a multiple of linear_num_k_heads %d",
                        cfg->linear_num_v_heads, cfg->linear_num_k_heads);
        if (!gdn_shape_supported(cfg->linear_num_k_heads, cfg->linear_num_v_heads,
                                 cfg->linear_key_dim, cfg->linear_value_dim, cfg->conv_kernel_size))
            return fail(MFA_ERR_SHAPE, "linear-attention shape dk=%d dv=%d K=%d not supported",
                        cfg->linear_key_dim, cfg->linear_value_dim, cfg->conv_kernel_size);
    }
    return MFA_OK;
}

static int create(const mfa_config *cfg, Ctx **out) {
    bool has_full, has_lin;
    MFA_TRY(validate(cfg, &has_full, &has_lin));
    int ndev = 0;
    MFA_HIP(hipGetDeviceCount(&ndev));
    if (ndev <= 0) return fail(MFA_ERR_HIP, "no HIP device");
    Ctx *c = new (std::nothrow) Ctx();
    if (!c) return fail(MFA_ERR_INVALID, "out of host memory");
    *out = c;
    c->cfg = *cfg;
    MFA_HIP(hipGetDevice(&c->device));
    hipDeviceProp_t prop;
    MFA_HIP(hipGetDeviceProperties(&prop, c->device));
    c->num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    MFA_TRY(static_scratch_init(c->device));
    MFA_HIP(hipStreamCreate(&c->stream));
    MFA_HIP(hipEventCreate(&c->ev0));
    MFA_HIP(hipEventCreate(&c->ev1));
    c->kind.resize(cfg->num_layers);
    c->slot.resize(cfg->num_layers);
    int nfull = 0, nlin = 0;
    for (int i = 0; i < cfg->num_layers; i++) {
        const bool full = (i + 1) % cfg->full_attn_interval == 0;  // variants.rs:258-264
        c->kind[i] = full ? 1 : 0;
        c->slot[i] = full ? nfull++ : nlin++;
    }
    c->full.resize(nfull);
    c->lin.resize(nlin);
    if (nfull) {
        c->cap_pad = ((int64_t)cfg->kv_capacity + kKvChunk - 1) / kKvChunk * kKvChunk;
        c->plane_elems = (size_t)c->cap_pad * cfg->head_dim;
        const size_t bytes = c->plane_elems * cfg->num_kv_heads * c->kv_elem_size();
        // One allocation for all layers' K planes and one for their V planes, layer-major:
        // plane (layer, kv head) sits at index layer * Hkv + kv head, so a launch over all
        // layers is a launch over nfull * Hkv kv heads.
        char *kslab, *vslab;
        MFA_TRY(slab_alloc(c, bytes * nfull, &kslab));
        MFA_TRY(slab_alloc(c, bytes * nfull, &vslab));
        char *norms;
        MFA_TRY(slab_alloc(c, (size_t)nfull * 2 * cfg->head_dim * 2, &norms));
        for (int i = 0; i < nfull; i++) {
            c->full[i].k = kslab + (size_t)i * bytes;
            c->full[i].v = vslab + (size_t)i * bytes;
            c->full[i].q_norm = (uint16_t *)norms + (size_t)(2 * i) * cfg->head_dim;
            c->full[i].k_norm = (uint16_t *)norms + (size_t)(2 * i + 1) * cfg->head_dim;
        }
        char *rope;
        MFA_TRY(slab_alloc(c, (size_t)cfg->head_dim * sizeof(float), &rope));
        c->inv_freq = (float *)rope;
        char *qg;
        MFA_TRY(slab_alloc(c, 2 * (size_t)cfg->num_attn_heads * cfg->head_dim * sizeof(float), &qg));
        c->qg_stage = (float *)qg;
        char *sc;
        MFA_TRY(slab_alloc(c, (size_t)cfg->num_kv_heads * ((cfg->num_attn_heads / cfg->num_kv_heads + 15) / 16) * 16 * sizeof(float), &sc));
        c->step_score = (float *)sc;
        // variants.rs:245-250, 369: a quarter of the head is rotated, theta = 1e7
        MFA_TRY(set_rope(c, 1.0e7f, cfg->head_dim / 4));
        // room for the most splits any cache length up to the capacity gets
        int splits = sdpa_max_splits(cfg->kv_dtype, cfg->num_attn_heads, cfg->num_kv_heads,
                                     cfg->head_dim, cfg->kv_capacity, c->num_cus, 0);
        if (splits < 128) splits = 128;
        c->part_o_elems = sdpa_workspace_o_elems(cfg->num_attn_heads, cfg->num_kv_heads, cfg->head_dim, splits);
        c->part_ml_elems = sdpa_workspace_ml_elems(cfg->num_attn_heads, cfg->num_kv_heads, splits);
        MFA_HIP(hipMalloc((void **)&c->part_o, c->part_o_elems * sizeof(float)));
        MFA_HIP(hipMalloc((void **)&c->part_ml, c->part_ml_elems * sizeof(float)));
    }
    if (nlin) {
        const size_t C = (size_t)c->conv_dim(), K = (size_t)cfg->conv_kernel_size;
        const size_t ssm = (size_t)cfg->linear_num_v_heads * cfg->linear_value_dim * cfg->linear_key_dim;
        const int Hv = cfg->linear_num_v_heads;
        // Layer-major slabs, each layer's part at a fixed stride, so that one launch can
        // step every linear layer (the kernels offset by layer index * stride).
        const size_t dv = (size_t)cfg->linear_value_dim;
        char *ring, *state, *cw, *al, *dt, *nw;
        MFA_TRY(slab_alloc(c, nlin * K * C * sizeof(float), &ring));
        MFA_TRY(slab_alloc(c, nlin * ssm * sizeof(float), &state));
        MFA_TRY(slab_alloc(c, nlin * C * K * 2, &cw));
        MFA_TRY(slab_alloc(c, nlin * Hv * sizeof(float), &al));
        MFA_TRY(slab_alloc(c, nlin * Hv * 2, &dt));
        MFA_TRY(slab_alloc(c, nlin * dv * 2, &nw));
        for (int i = 0; i < nlin; i++) {
            LinearLayer &l = c->lin[i];
            l.conv_ring = (float *)ring + (size_t)i * K * C;
            l.ssm = (float *)state + (size_t)i * ssm;
            l.w.conv_w = (uint16_t *)cw + (size_t)i * C * K;
            l.w.a_log = (float *)al + (size_t)i * Hv;
            l.w.dt_bias = (uint16_t *)dt + (size_t)i * Hv;
            l.w.norm_w = (uint16_t *)nw + (size_t)i * dv;
        }
    }
    MFA_HIP(hipStreamSynchronize(c->stream));
    return MFA_OK;
}

static int reset_linear(Ctx *c, LinearLayer &l) {
    const size_t C = (size_t)c->conv_dim(), K = (size_t)c->cfg.conv_kernel_size;
    const size_t ssm = (size_t)c->cfg.linear_num_v_heads * c->cfg.linear_value_dim * c->cfg.linear_key_dim;
    MFA_HIP(hipMemsetAsync(l.conv_ring, 0, K * C * sizeof(float), c->stream));
    MFA_HIP(hipMemsetAsync(l.ssm, 0, ssm * sizeof(float), c->stream));
    l.step = 0;
    return MFA_OK;
}

// KvCache::truncate (state.rs:60-74): no-op unless 0 <= new_len <= len; zero the dropped rows.
static int truncate_full(Ctx *c, FullLayer &f, int32_t new_len) {
    if (new_len < 0 || new_len > f.len) return MFA_OK;
    if (new_len < f.len)
        MFA_TRY(launch_kv_zero(c->stream, c->cfg.kv_dtype, c->cfg.num_kv_heads, c->cfg.head_dim,
                               c->plane_elems, new_len, f.len, f.k, f.v));
    f.len = new_len;
    return MFA_OK;
}

// Grows the split-K workspace to at least the given element counts (never shrinks it).
static int ensure_workspace_elems(Ctx *c, size_t need_o, size_t need_ml) {
    if (need_o <= c->part_o_elems && need_ml <= c->part_ml_elems) return MFA_OK;
    MFA_HIP(hipStreamSynchronize(c->stream));
    if (need_o > c->part_o_elems) {
        if (c->part_o) MFA_HIP(hipFree(c->part_o));
        c->part_o = nullptr;
        c->part_o_elems = 0;
        MFA_HIP(hipMalloc((void **)&c->part_o, need_o * sizeof(float)));
        c->part_o_elems = need_o;
    }
    if (need_ml > c->part_ml_elems) {
        if (c->part_ml) MFA_HIP(hipFree(c->part_ml));
        c->part_ml = nullptr;
        c->part_ml_elems = 0;
        MFA_HIP(hipMalloc((void **)&c->part_ml, need_ml * sizeof(float)));
        c->part_ml_elems = need_ml;
    }
    return MFA_OK;
}

// The split-K workspace is sized for decode at create time; a prompt chunk has n_tok times
// the rows and grows it on first use.
// `layers` > 1 sizes it for one launch over that many layers (layers * Hkv kv heads).
static int ensure_workspace(Ctx *c, int n_tok, int64_t kv_len, int layers = 1) {
    const mfa_config &g = c->cfg;
    const int Hq = g.num_attn_heads * layers, Hkv = g.num_kv_heads * layers;
    // decode: room for the most splits any length up to kv_len gets (a shorter cache can be split more)
    int splits = sdpa_max_splits(g.kv_dtype, Hq, Hkv, g.head_dim, kv_len, c->num_cus, c->forced_splits);
    if (n_tok > 1) splits = 1;  // the launcher splits a chunk less; one split always fits its plan
    return ensure_workspace_elems(c, sdpa_workspace_o_elems(Hq, Hkv, g.head_dim, splits, n_tok),
                                  sdpa_workspace_ml_elems(Hq, Hkv, splits, n_tok));
}

// What sdpa_dev could still refuse for n_tok tokens over a cache of kv_len positions, checked
// (and the split-K workspace grown) while the cache is as the caller left it.
static int sdpa_prepare(Ctx *c, int n_tok, int64_t kv_len) {
    const mfa_config &g = c->cfg;
    if (!c->forced_splits && !c->partial_only &&
        sdpa_prefill_applies(g.kv_dtype, g.num_attn_heads, g.num_kv_heads, n_tok, kv_len, c->num_cus))
        return MFA_OK;   // one launch, no workspace
    const int64_t nhg = ((int64_t)n_tok * (g.num_attn_heads / g.num_kv_heads) + 15) / 16;
    if (nhg > 65535) return fail(MFA_ERR_SHAPE, "sdpa: too many query rows in one call");
    if (n_tok > 1) MFA_TRY(ensure_workspace(c, n_tok, kv_len));
    return MFA_OK;
}

// n_tok tokens whose K/V rows are already in the cache (the last n_tok positions).
static int sdpa_dev(Ctx *c, FullLayer *f, int n_tok, const float *q, const float *gate, float *out) {
    if (f->len <= 0) return fail(MFA_ERR_INVALID, "kv_len must be > 0 (got %d)", f->len);
    if (!c->forced_splits && !c->partial_only &&
        sdpa_prefill_applies(c->cfg.kv_dtype, c->cfg.num_attn_heads, c->cfg.num_kv_heads, n_tok, f->len,
                             c->num_cus))
        return launch_sdpa_prefill(c->stream, c->cfg.kv_dtype, c->cfg.num_attn_heads, c->cfg.num_kv_heads,
                                   c->cfg.head_dim, n_tok, f->len, c->plane_elems, f->k, f->v, q, gate, out,
                                   c->num_cus);
    if (n_tok > 1) MFA_TRY(ensure_workspace(c, n_tok, f->len));
    return launch_sdpa(c->stream, c->cfg.kv_dtype, c->cfg.num_attn_heads, c->cfg.num_kv_heads,
                       c->cfg.head_dim, n_tok, f->len, c->plane_elems, f->k, f->v, q, gate, out,
                       workspace(c), c->num_cus, c->forced_splits, c->partial_only);
}

static int sdpa_decode_dev(Ctx *c, FullLayer *f, const float *q, const float *gate, float *out) {
    return sdpa_dev(c, f, 1, q, gate, out);
}

static int kv_append_dev(Ctx *c, FullLayer *f, const float *k, const float *v, int64_t rows) {
    if ((int64_t)f->len + rows > c->cfg.kv_capacity)
        return fail(MFA_ERR_OVERFLOW, "kv cache overflow: len %d + %lld > capacity %d", f->len,
                    (long long)rows, c->cfg.kv_capacity);
    MFA_TRY(launch_kv_scatter(c->stream, c->cfg.kv_dtype, 0, c->cfg.num_kv_heads, c->cfg.head_dim,
                              c->plane_elems, f->len, rows, k, v, f->k, f->v));
    f->len += (int32_t)rows;
    return MFA_OK;
}

static int gdn_step_dev(Ctx *c, LinearLayer *l, const float *qkv, const float *z,
                        const float *alpha, const float *beta, float *out) {
    if (!l->w.set) return fail(MFA_ERR_INVALID, "linear layer weights not set (mfa_set_linear_weights)");
    MFA_TRY(launch_gdn_step(c->stream, c->cfg.linear_num_k_heads, c->cfg.linear_num_v_heads,
                            c->cfg.linear_key_dim, c->cfg.linear_value_dim, c->cfg.conv_kernel_size,
                            c->cfg.rms_norm_eps, l->w, l->conv_ring, l->step, l->ssm, qkv, z, alpha,
                            beta, out));
    l->step++;
    return MFA_OK;
}

// A scratch device allocation for the stateless hooks.
struct DevBuf {
    void *p = nullptr;
    ~DevBuf() { if (p) (void)hipFree(p); }
    int alloc(size_t bytes) {
        MFA_HIP(hipMalloc(&p, bytes ? bytes : 4));
        return MFA_OK;
    }
    int upload(const void *src, size_t bytes) {
        MFA_TRY(alloc(bytes));
        MFA_HIP(hipMemcpy(p, src, bytes, hipMemcpyHostToDevice));
        return MFA_OK;
    }
    int download(void *dst, size_t bytes) {
        MFA_HIP(hipDeviceSynchronize());
        MFA_HIP(hipMemcpy(dst, p, bytes, hipMemcpyDeviceToHost));
        return MFA_OK;
    }
    template <typename T> T *as() { return reinterpret_cast<T *>(p); }
};

static int sdpa_stateless(int kv_dtype, int32_t kv_len, int32_t Hq, int32_t Hkv, int32_t D,
                          const float *q, const float *gate, const void *k, const void *v,
                          float *out) {
    if (!q || !gate || !k || !v || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (kv_len <= 0) return fail(MFA_ERR_INVALID, "kv_len must be > 0 (got %d)", kv_len);
    if (Hq <= 0 || Hkv <= 0 || D <= 0) return fail(MFA_ERR_INVALID, "non-positive shape");
    if (Hq % Hkv != 0) return fail(MFA_ERR_INVALID, "num_attn_heads %d %% num_kv_heads %d != 0", Hq, Hkv);
    if (!sdpa_shape_supported(kv_dtype, D)) return fail(MFA_ERR_SHAPE, "head_dim %d not supported", D);
    const size_t es = kv_dtype == MFA_KV_BF16 ? 2 : 4;
    const int64_t cap = ((int64_t)kv_len + kKvChunk - 1) / kKvChunk * kKvChunk;
    const size_t plane = (size_t)cap * D;
    const size_t qd = (size_t)Hq * D, rows = (size_t)kv_len * Hkv * D;
    int ncu = 256;
    {
        int dev = 0;
        hipDeviceProp_t prop;
        MFA_HIP(hipGetDevice(&dev));
        MFA_HIP(hipGetDeviceProperties(&prop, dev));
        if (prop.multiProcessorCount > 0) ncu = prop.multiProcessorCount;
    }
    DevBuf dq, dg, dout, kr, vr, kt, vt, po, pml;
    MFA_TRY(dq.upload(q, qd * 4));
    MFA_TRY(dg.upload(gate, qd * 4));
    MFA_TRY(dout.alloc(qd * 4));
    MFA_TRY(kr.upload(k, rows * es));
    MFA_TRY(vr.upload(v, rows * es));
    MFA_TRY(kt.alloc(plane * Hkv * es));
    MFA_TRY(vt.alloc(plane * Hkv * es));
    MFA_HIP(hipMemsetAsync(kt.p, 0, plane * Hkv * es, nullptr));
    MFA_HIP(hipMemsetAsync(vt.p, 0, plane * Hkv * es, nullptr));
    MFA_TRY(launch_kv_scatter(nullptr, kv_dtype, kv_dtype == MFA_KV_BF16, Hkv, D, plane, 0, kv_len,
                              kr.p, vr.p, kt.p, vt.p));
    const int splits = sdpa_pick_splits(kv_dtype, Hq, Hkv, D, kv_len, ncu, 0);
    SdpaWorkspace ws;
    ws.part_o_elems = sdpa_workspace_o_elems(Hq, Hkv, D, splits);
    ws.part_ml_elems = sdpa_workspace_ml_elems(Hq, Hkv, splits);
    MFA_TRY(po.alloc(ws.part_o_elems * 4));
    MFA_TRY(pml.alloc(ws.part_ml_elems * 4));
    ws.part_o = po.as<float>();
    ws.part_ml = pml.as<float>();
    MFA_TRY(launch_sdpa(nullptr, kv_dtype, Hq, Hkv, D, 1, kv_len, plane, kt.p, vt.p, dq.as<float>(),
                        dg.as<float>(), dout.as<float>(), ws, ncu, 0));
    return dout.download(out, qd * 4);
}

// Device-to-device halves of the export and import calls, enqueued on the context's stream without
// a synchronisation, for callers that move the state of many layers at once (the snapshot).
// k_dev, v_dev: [len, num_kv_heads * head_dim] f32; conv_dev: [(K-1) * C] f32, oldest input first.
int kv_export_to(Ctx *c, FullLayer *f, float *k_dev, float *v_dev) {
    if (f->len == 0) return MFA_OK;
    return launch_kv_gather(c->stream, c->cfg.kv_dtype, c->cfg.num_kv_heads, c->cfg.head_dim, c->plane_elems,
                            f->len, f->k, f->v, k_dev, v_dev);
}
int kv_import_from(Ctx *c, FullLayer *f, int32_t len, const float *k_dev, const float *v_dev) {
    MFA_TRY(truncate_full(c, *f, 0));
    if (len > 0)
        MFA_TRY(launch_kv_scatter(c->stream, c->cfg.kv_dtype, 0, c->cfg.num_kv_heads, c->cfg.head_dim,
                                  c->plane_elems, 0, len, k_dev, v_dev, f->k, f->v));
    f->len = len;
    return MFA_OK;
}
int linear_export_to(Ctx *c, LinearLayer *l, float *conv_dev) {
    return launch_conv_ring_export(c->stream, c->conv_dim(), c->cfg.conv_kernel_size, l->step, l->conv_ring, conv_dev);
}
int linear_import_from(Ctx *c, LinearLayer *l, const float *conv_dev) {
    MFA_TRY(launch_conv_ring_import(c->stream, c->conv_dim(), c->cfg.conv_kernel_size, conv_dev, l->conv_ring));
    l->step = 0;
    return MFA_OK;
}

}  // namespace mfa

using namespace mfa;

extern "C" {

mfa_ctx *mfa_ctx_create(const mfa_config *cfg) {
    Ctx *c = nullptr;
    const int rc = create(cfg, &c);
    if (rc != MFA_OK) {
        const std::string keep = g_last_error;
        destroy(c);
        g_last_error = keep;
        return nullptr;
    }
    return reinterpret_cast<mfa_ctx *>(c);
}

void mfa_ctx_destroy(mfa_ctx *ctx) { destroy(as_ctx(ctx)); }

const char *mfa_last_error_string(void) { return g_last_error.c_str(); }

int mfa_sync(mfa_ctx *ctx) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    MFA_HIP(hipStreamSynchronize(c->stream));
    return MFA_OK;
}

void *mfa_stream(mfa_ctx *ctx) { return ctx ? (void *)as_ctx(ctx)->stream : nullptr; }

int mfa_set_linear_weights(mfa_ctx *ctx, int32_t layer, const uint16_t *conv_w_bf16,
                           const float *a_log, const uint16_t *dt_bias_bf16,
                           const uint16_t *norm_w_bf16) {
    Ctx *c = as_ctx(ctx);
    LinearLayer *l;
    MFA_TRY(linear_layer(c, layer, &l));
    if (!conv_w_bf16 || !a_log || !dt_bias_bf16 || !norm_w_bf16)
        return fail(MFA_ERR_INVALID, "NULL weight pointer");
    const size_t C = (size_t)c->conv_dim(), K = (size_t)c->cfg.conv_kernel_size;
    const int Hv = c->cfg.linear_num_v_heads;
    MFA_TRY(h2d(c, l->w.conv_w, conv_w_bf16, C * K * 2));
    MFA_TRY(h2d(c, l->w.a_log, a_log, Hv * sizeof(float)));
    MFA_TRY(h2d(c, l->w.dt_bias, dt_bias_bf16, Hv * 2));
    MFA_TRY(h2d(c, l->w.norm_w, norm_w_bf16, (size_t)c->cfg.linear_value_dim * 2));
    MFA_HIP(hipStreamSynchronize(c->stream));
    l->w.set = true;
    return MFA_OK;
}

int mfa_set_num_splits(mfa_ctx *ctx, int32_t num_splits) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    if (num_splits < 0) return fail(MFA_ERR_INVALID, "num_splits must be >= 0");
    c->forced_splits = num_splits;
    // a forced count is used as given, so the workspace must hold it at any cache length
    if (num_splits > 0 && !c->full.empty()) MFA_TRY(ensure_workspace(c, 1, c->cfg.kv_capacity));
    return MFA_OK;
}

int mfa_set_step_launches(mfa_ctx *ctx, int32_t launches) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    if (launches != 2 && launches != 3) return fail(MFA_ERR_INVALID, "step launches must be 2 or 3 (got %d)", launches);
    c->step_launches = launches;
    return MFA_OK;
}

int mfa_set_partial_only(mfa_ctx *ctx, int32_t on) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    c->partial_only = on ? 1 : 0;
    return MFA_OK;
}

int mfa_set_full_weights(mfa_ctx *ctx, int32_t layer, const uint16_t *q_norm_bf16, const uint16_t *k_norm_bf16) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q_norm_bf16 || !k_norm_bf16) return fail(MFA_ERR_INVALID, "NULL weight pointer");
    MFA_TRY(h2d(c, f->q_norm, q_norm_bf16, (size_t)c->cfg.head_dim * 2));
    MFA_TRY(h2d(c, f->k_norm, k_norm_bf16, (size_t)c->cfg.head_dim * 2));
    MFA_HIP(hipStreamSynchronize(c->stream));
    f->norms_set = true;
    return MFA_OK;
}

int mfa_set_rope(mfa_ctx *ctx, float theta, int32_t rotary_dim) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    return set_rope(c, theta, rotary_dim);
}

/* ---- full attention -------------------------------------------------------- */

int mfa_kv_append_dev(mfa_ctx *ctx, int32_t layer, const float *k_dev, const float *v_dev) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!k_dev || !v_dev) return fail(MFA_ERR_INVALID, "NULL k/v row");
    return kv_append_dev(c, f, k_dev, v_dev, 1);
}

int mfa_kv_append(mfa_ctx *ctx, int32_t layer, const float *k, const float *v) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!k || !v) return fail(MFA_ERR_INVALID, "NULL k/v row");
    if (f->len + 1 > c->cfg.kv_capacity)
        return fail(MFA_ERR_OVERFLOW, "kv cache overflow: len %d at capacity %d", f->len, c->cfg.kv_capacity);
    const size_t kvd = (size_t)c->kv_dim();
    MFA_TRY(ensure_stage(c, 2 * kvd));
    MFA_TRY(h2d(c, c->stage, k, kvd * 4));
    MFA_TRY(h2d(c, c->stage + kvd, v, kvd * 4));
    MFA_TRY(kv_append_dev(c, f, c->stage, c->stage + kvd, 1));
    MFA_HIP(hipStreamSynchronize(c->stream));
    return MFA_OK;
}

int32_t mfa_kv_len(mfa_ctx *ctx, int32_t layer) {
    FullLayer *f;
    const int rc = full_layer(as_ctx(ctx), layer, &f);
    return rc != MFA_OK ? rc : f->len;
}

int mfa_sdpa_decode_dev(mfa_ctx *ctx, int32_t layer, const float *q_dev, const float *q_gate_dev,
                        float *out_dev) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q_dev || !q_gate_dev || !out_dev) return fail(MFA_ERR_INVALID, "NULL argument");
    return sdpa_decode_dev(c, f, q_dev, q_gate_dev, out_dev);
}

int mfa_sdpa_decode(mfa_ctx *ctx, int32_t layer, const float *q, const float *q_gate, float *out) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q || !q_gate || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (f->len <= 0) return fail(MFA_ERR_INVALID, "kv_len must be > 0 (got %d)", f->len);
    const size_t qd = (size_t)c->q_dim();
    MFA_TRY(ensure_stage(c, 3 * qd));
    MFA_TRY(h2d(c, c->stage, q, qd * 4));
    MFA_TRY(h2d(c, c->stage + qd, q_gate, qd * 4));
    MFA_TRY(sdpa_decode_dev(c, f, c->stage, c->stage + qd, c->stage + 2 * qd));
    return d2h_sync(c, out, c->stage + 2 * qd, qd * 4);
}

// Undo the appends of a call that failed after them, keeping the error of the failure.
static void rollback_append(Ctx *c, FullLayer *f, int32_t len0) {
    const std::string keep = g_last_error;
    (void)truncate_full(c, *f, len0);
    g_last_error = keep;
}

// n_tok tokens at positions pos .. pos + n_tok - 1, appended at the end of the layer's cache.
static int prologue_dev(Ctx *c, FullLayer *f, int32_t pos, const float *q_proj, const float *k, const float *v,
                        float *q_out, float *gate_out, int32_t n_tok = 1) {
    if (!f->norms_set) return fail(MFA_ERR_INVALID, "q/k norm weights not set (mfa_set_full_weights)");
    if ((int64_t)f->len + n_tok > c->cfg.kv_capacity)
        return fail(MFA_ERR_OVERFLOW, "kv cache overflow: len %d + %d > capacity %d", f->len, n_tok, c->cfg.kv_capacity);
    MFA_TRY(launch_attn_prologue(c->stream, c->cfg.kv_dtype, c->cfg.num_attn_heads, c->cfg.num_kv_heads,
                                 c->cfg.head_dim, c->rotary_dim, c->cfg.rms_norm_eps, n_tok, pos, f->len, c->plane_elems,
                                 f->q_norm, f->k_norm, c->inv_freq, q_proj, k, v, q_out, gate_out, f->k, f->v));
    f->len += n_tok;
    return MFA_OK;
}

// One token through a full-attention layer from its raw projections.  Two launches where the
// shape allows (and no measurement switch asks otherwise): the attention launch norms and
// rotates its own query heads and appends the token, the merge takes the token as one more
// split.  Otherwise three: prologue, attention, merge.
static int full_attn_step_dev(Ctx *c, FullLayer *f, int32_t pos, const float *q_proj, const float *k, const float *v,
                              float *out) {
    const mfa_config &g = c->cfg;
    const size_t qd = (size_t)c->q_dim();
    const int32_t len0 = f->len;
    if (c->step_launches == 2 && !c->partial_only &&
        sdpa_step_supported(g.kv_dtype, g.num_attn_heads, g.num_kv_heads, g.head_dim, c->rotary_dim)) {
        if (!f->norms_set) return fail(MFA_ERR_INVALID, "q/k norm weights not set (mfa_set_full_weights)");
        if (pos < 0) return fail(MFA_ERR_INVALID, "attention prologue: pos %d < 0", pos);
        if ((int64_t)f->len + 1 > g.kv_capacity)
            return fail(MFA_ERR_OVERFLOW, "kv cache overflow: len %d + 1 > capacity %d", f->len, g.kv_capacity);
        MFA_TRY(launch_sdpa_step(c->stream, g.kv_dtype, g.num_attn_heads, g.num_kv_heads, g.head_dim, f->len,
                                 c->plane_elems, f->k, f->v, q_proj, k, v, f->q_norm, f->k_norm, c->inv_freq,
                                 c->rotary_dim, g.rms_norm_eps, pos, c->step_score, out, workspace(c), c->num_cus,
                                 c->forced_splits));
        f->len += 1;
        return MFA_OK;
    }
    MFA_TRY(prologue_dev(c, f, pos, q_proj, k, v, c->qg_stage, c->qg_stage + qd));
    const int rc = sdpa_decode_dev(c, f, c->qg_stage, c->qg_stage + qd, out);
    if (rc != MFA_OK) rollback_append(c, f, len0);
    return rc;
}

int mfa_attn_prologue_dev(mfa_ctx *ctx, int32_t layer, int32_t pos, const float *q_proj_out_dev,
                          const float *k_dev, const float *v_dev, float *q_out_dev, float *q_gate_out_dev) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q_proj_out_dev || !k_dev || !v_dev || !q_out_dev || !q_gate_out_dev)
        return fail(MFA_ERR_INVALID, "NULL argument");
    return prologue_dev(c, f, pos, q_proj_out_dev, k_dev, v_dev, q_out_dev, q_gate_out_dev);
}

int mfa_attn_prologue(mfa_ctx *ctx, int32_t layer, int32_t pos, const float *q_proj_out, const float *k,
                      const float *v, float *q_out, float *q_gate_out) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q_proj_out || !k || !v || !q_out || !q_gate_out) return fail(MFA_ERR_INVALID, "NULL argument");
    const size_t qd = (size_t)c->q_dim(), kd = (size_t)c->kv_dim();
    MFA_TRY(ensure_stage(c, 4 * qd + 2 * kd));
    float *qp = c->stage, *kk = qp + 2 * qd, *vv = kk + kd, *qo = vv + kd, *go = qo + qd;
    MFA_TRY(h2d(c, qp, q_proj_out, 2 * qd * 4));
    MFA_TRY(h2d(c, kk, k, kd * 4));
    MFA_TRY(h2d(c, vv, v, kd * 4));
    MFA_TRY(prologue_dev(c, f, pos, qp, kk, vv, qo, go));
    MFA_HIP(hipMemcpyAsync(q_out, qo, qd * 4, hipMemcpyDeviceToHost, c->stream));
    return d2h_sync(c, q_gate_out, go, qd * 4);
}

int mfa_full_attn_step_dev(mfa_ctx *ctx, int32_t layer, int32_t pos, const float *q_proj_out_dev,
                           const float *k_dev, const float *v_dev, float *out_dev) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q_proj_out_dev || !k_dev || !v_dev || !out_dev) return fail(MFA_ERR_INVALID, "NULL argument");
    return full_attn_step_dev(c, f, pos, q_proj_out_dev, k_dev, v_dev, out_dev);
}

int mfa_full_attn_step(mfa_ctx *ctx, int32_t layer, int32_t pos, const float *q_proj_out, const float *k,
                       const float *v, float *out) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q_proj_out || !k || !v || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    const size_t qd = (size_t)c->q_dim(), kd = (size_t)c->kv_dim();
    MFA_TRY(ensure_stage(c, 3 * qd + 2 * kd));
    float *qp = c->stage, *kk = qp + 2 * qd, *vv = kk + kd, *oo = vv + kd;
    MFA_TRY(h2d(c, qp, q_proj_out, 2 * qd * 4));
    MFA_TRY(h2d(c, kk, k, kd * 4));
    MFA_TRY(h2d(c, vv, v, kd * 4));
    MFA_TRY(full_attn_step_dev(c, f, pos, qp, kk, vv, oo));
    return d2h_sync(c, out, oo, qd * 4);
}

int mfa_prefill_full_attn_dev(mfa_ctx *ctx, int32_t layer, int32_t pos0, int32_t T, const float *q_proj_out_dev,
                              const float *k_dev, const float *v_dev, float *out_dev) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q_proj_out_dev || !k_dev || !v_dev || !out_dev) return fail(MFA_ERR_INVALID, "NULL argument");
    if (T <= 0) return fail(MFA_ERR_INVALID, "T must be > 0 (got %d)", T);
    // everything that can fail is checked before the first token is appended
    if (!f->norms_set) return fail(MFA_ERR_INVALID, "q/k norm weights not set (mfa_set_full_weights)");
    if (pos0 < 0 || (int64_t)pos0 + T - 1 > INT32_MAX)
        return fail(MFA_ERR_INVALID, "positions %d .. %lld out of range", pos0, (long long)pos0 + T - 1);
    if ((int64_t)f->len + T > c->cfg.kv_capacity)
        return fail(MFA_ERR_OVERFLOW, "kv cache overflow: len %d + %d > capacity %d", f->len, T, c->cfg.kv_capacity);
    const size_t qd = (size_t)c->q_dim() * T;
    if (2 * qd > c->qg_chunk_elems) {
        MFA_HIP(hipStreamSynchronize(c->stream));
        if (c->qg_chunk) MFA_HIP(hipFree(c->qg_chunk));
        c->qg_chunk = nullptr;
        c->qg_chunk_elems = 0;
        MFA_HIP(hipMalloc((void **)&c->qg_chunk, 2 * qd * sizeof(float)));
        c->qg_chunk_elems = 2 * qd;
    }
    MFA_TRY(sdpa_prepare(c, T, (int64_t)f->len + T));
    // the whole chunk is normed, rotated and appended, then one causal pass: row t sees positions [0, len0 + t]
    const int32_t len0 = f->len;
    const int kSeg = 32768;   // tokens per prologue launch (the grid's second dimension holds 65535)
    int rc = MFA_OK;
    for (int32_t off = 0; off < T && rc == MFA_OK; off += kSeg) {
        const int32_t n = T - off < kSeg ? T - off : kSeg;
        rc = prologue_dev(c, f, pos0 + off, q_proj_out_dev + (size_t)off * 2 * c->q_dim(),
                          k_dev + (size_t)off * c->kv_dim(), v_dev + (size_t)off * c->kv_dim(),
                          c->qg_chunk + (size_t)off * c->q_dim(), c->qg_chunk + qd + (size_t)off * c->q_dim(), n);
    }
    if (rc == MFA_OK) rc = sdpa_dev(c, f, T, c->qg_chunk, c->qg_chunk + qd, out_dev);
    if (rc != MFA_OK) rollback_append(c, f, len0);   // a launch refused after all: the cache is as before the call
    return rc;
}

int mfa_prefill_full_attn(mfa_ctx *ctx, int32_t layer, int32_t pos0, int32_t T, const float *q_proj_out,
                          const float *k, const float *v, float *out) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q_proj_out || !k || !v || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (T <= 0) return fail(MFA_ERR_INVALID, "T must be > 0 (got %d)", T);
    const size_t qd = (size_t)c->q_dim() * T, kvd = (size_t)c->kv_dim() * T;
    MFA_TRY(ensure_stage(c, 3 * qd + 2 * kvd));
    float *qp = c->stage, *dk = qp + 2 * qd, *dv = dk + kvd, *dout = dv + kvd;
    MFA_TRY(h2d(c, qp, q_proj_out, 2 * qd * 4));
    MFA_TRY(h2d(c, dk, k, kvd * 4));
    MFA_TRY(h2d(c, dv, v, kvd * 4));
    MFA_TRY(mfa_prefill_full_attn_dev(ctx, layer, pos0, T, qp, dk, dv, dout));
    return d2h_sync(c, out, dout, qd * 4);
}

int mfa_prefill_attn_dev(mfa_ctx *ctx, int32_t layer, int32_t T, const float *q_dev,
                         const float *q_gate_dev, const float *k_dev, const float *v_dev,
                         float *out_dev) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q_dev || !q_gate_dev || !k_dev || !v_dev || !out_dev) return fail(MFA_ERR_INVALID, "NULL argument");
    if (T <= 0) return fail(MFA_ERR_INVALID, "T must be > 0 (got %d)", T);
    if ((int64_t)f->len + T > c->cfg.kv_capacity)
        return fail(MFA_ERR_OVERFLOW, "kv cache overflow: len %d + %d > capacity %d", f->len, T,
                    c->cfg.kv_capacity);
    MFA_TRY(sdpa_prepare(c, T, (int64_t)f->len + T));
    // append the whole chunk, then one causal pass: row t sees positions [0, len0 + t]
    const int32_t len0 = f->len;
    int rc = kv_append_dev(c, f, k_dev, v_dev, T);
    if (rc == MFA_OK) rc = sdpa_dev(c, f, T, q_dev, q_gate_dev, out_dev);
    if (rc != MFA_OK) rollback_append(c, f, len0);
    return rc;
}

int mfa_prefill_attn(mfa_ctx *ctx, int32_t layer, int32_t T, const float *q, const float *q_gate,
                     const float *k, const float *v, float *out) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!q || !q_gate || !k || !v || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (T <= 0) return fail(MFA_ERR_INVALID, "T must be > 0 (got %d)", T);
    const size_t qd = (size_t)c->q_dim() * T, kvd = (size_t)c->kv_dim() * T;
    MFA_TRY(ensure_stage(c, 3 * qd + 2 * kvd));
    float *dq = c->stage, *dg = dq + qd, *dout = dg + qd, *dk = dout + qd, *dv = dk + kvd;
    MFA_TRY(h2d(c, dq, q, qd * 4));
    MFA_TRY(h2d(c, dg, q_gate, qd * 4));
    MFA_TRY(h2d(c, dk, k, kvd * 4));
    MFA_TRY(h2d(c, dv, v, kvd * 4));
    MFA_TRY(mfa_prefill_attn_dev(ctx, layer, T, dq, dg, dk, dv, dout));
    return d2h_sync(c, out, dout, qd * 4);
}

/* ---- gated delta net --------------------------------------------------------- */

int mfa_gdn_step_dev(mfa_ctx *ctx, int32_t layer, const float *qkv_in_dev, const float *z_dev,
                     const float *alpha_dev, const float *beta_dev, float *out_dev) {
    Ctx *c = as_ctx(ctx);
    LinearLayer *l;
    MFA_TRY(linear_layer(c, layer, &l));
    if (!qkv_in_dev || !z_dev || !alpha_dev || !beta_dev || !out_dev)
        return fail(MFA_ERR_INVALID, "NULL argument");
    return gdn_step_dev(c, l, qkv_in_dev, z_dev, alpha_dev, beta_dev, out_dev);
}

int mfa_prefill_gdn_dev(mfa_ctx *ctx, int32_t layer, int32_t T, const float *qkv_in_dev,
                        const float *z_dev, const float *alpha_dev, const float *beta_dev,
                        float *out_dev) {
    Ctx *c = as_ctx(ctx);
    LinearLayer *l;
    MFA_TRY(linear_layer(c, layer, &l));
    if (!qkv_in_dev || !z_dev || !alpha_dev || !beta_dev || !out_dev)
        return fail(MFA_ERR_INVALID, "NULL argument");
    if (T <= 0) return fail(MFA_ERR_INVALID, "T must be > 0 (got %d)", T);
    if (T == 1) return gdn_step_dev(c, l, qkv_in_dev, z_dev, alpha_dev, beta_dev, out_dev);
    if (!l->w.set) return fail(MFA_ERR_INVALID, "linear layer weights not set (mfa_set_linear_weights)");
    const mfa_config &g = c->cfg;
    // Long prompts go through in segments, which bounds the scratch (about 57 KB per token
    // at the 16/32-head, 128-wide shape); the ring and the state carry over as between calls.
    const int kSeg = 4096;
    const size_t need = gdn_chunk_scratch_elems(g.linear_num_k_heads, g.linear_num_v_heads,
                                                g.linear_key_dim, g.linear_value_dim, T < kSeg ? T : kSeg);
    if (need > c->gdn_scratch_elems) {
        MFA_HIP(hipStreamSynchronize(c->stream));
        if (c->gdn_scratch) MFA_HIP(hipFree(c->gdn_scratch));
        c->gdn_scratch = nullptr;
        c->gdn_scratch_elems = 0;
        MFA_HIP(hipMalloc((void **)&c->gdn_scratch, need * sizeof(float)));
        c->gdn_scratch_elems = need;
    }
    const size_t C = (size_t)c->conv_dim(), tv = (size_t)c->v_total(), Hv = (size_t)g.linear_num_v_heads;
    for (int off = 0; off < T; off += kSeg) {
        const int n = T - off < kSeg ? T - off : kSeg;
        MFA_TRY(launch_gdn_chunk(c->stream, g.linear_num_k_heads, g.linear_num_v_heads, g.linear_key_dim,
                                 g.linear_value_dim, g.conv_kernel_size, g.rms_norm_eps, n, l->w,
                                 l->conv_ring, l->step, l->ssm, qkv_in_dev + off * C, z_dev + off * tv,
                                 alpha_dev + off * Hv, beta_dev + off * Hv, c->gdn_scratch, out_dev + off * tv));
        l->step += n;
    }
    return MFA_OK;
}

int mfa_prefill_gdn(mfa_ctx *ctx, int32_t layer, int32_t T, const float *qkv_in, const float *z,
                    const float *alpha, const float *beta, float *out) {
    Ctx *c = as_ctx(ctx);
    LinearLayer *l;
    MFA_TRY(linear_layer(c, layer, &l));
    if (!qkv_in || !z || !alpha || !beta || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (T <= 0) return fail(MFA_ERR_INVALID, "T must be > 0 (got %d)", T);
    const size_t C = (size_t)c->conv_dim() * T, tv = (size_t)c->v_total() * T,
                 Hv = (size_t)c->cfg.linear_num_v_heads * T;
    MFA_TRY(ensure_stage(c, C + 2 * tv + 2 * Hv));
    float *dx = c->stage, *dz = dx + C, *dout = dz + tv, *da = dout + tv, *db = da + Hv;
    MFA_TRY(h2d(c, dx, qkv_in, C * 4));
    MFA_TRY(h2d(c, dz, z, tv * 4));
    MFA_TRY(h2d(c, da, alpha, Hv * 4));
    MFA_TRY(h2d(c, db, beta, Hv * 4));
    MFA_TRY(mfa_prefill_gdn_dev(ctx, layer, T, dx, dz, da, db, dout));
    return d2h_sync(c, out, dout, tv * 4);
}

int mfa_gdn_step(mfa_ctx *ctx, int32_t layer, const float *qkv_in, const float *z,
                 const float *alpha, const float *beta, float *out) {
    return mfa_prefill_gdn(ctx, layer, 1, qkv_in, z, alpha, beta, out);
}

/* ---- whole-stack sweep -------------------------------------------------------- */

int mfa_token_sweep_dev(mfa_ctx *ctx, const float *full_q, const float *full_gate, float *full_out,
                        const float *lin_qkv, const float *lin_z, const float *lin_alpha,
                        const float *lin_beta, float *lin_out) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    if (!c->full.empty() && (!full_q || !full_gate || !full_out))
        return fail(MFA_ERR_INVALID, "NULL full-attention argument");
    if (!c->lin.empty() && (!lin_qkv || !lin_z || !lin_alpha || !lin_beta || !lin_out))
        return fail(MFA_ERR_INVALID, "NULL linear-attention argument");
    const size_t qd = (size_t)c->q_dim(), C = (size_t)c->conv_dim(), tv = (size_t)c->v_total(),
                 Hv = (size_t)c->cfg.linear_num_v_heads;
    // The layers' caches, states and weights are layer-major slabs and the inputs are packed
    // per kind, so when the layers of a kind stand at the same position the whole kind is
    // one launch: every linear layer as a second grid dimension, every full-attention
    // layer as n_full * Hkv kv heads.  Results are those of the layer-by-layer loop.
    bool lin_batch = !c->sweep_per_layer && c->lin.size() > 1, full_batch = !c->sweep_per_layer && c->full.size() > 1;
    const int64_t K = c->cfg.conv_kernel_size;
    for (auto &l : c->lin) lin_batch = lin_batch && l.w.set && l.step % K == c->lin[0].step % K;
    for (auto &f : c->full) full_batch = full_batch && f.len > 0 && f.len == c->full[0].len;
    // With both kinds in one launch each, the merge of the attention launch's partials (few splits:
    // the layers themselves fill the machine) rides in the first workgroups of the DeltaNet launch.
    SdpaMergeTask merge;
    if (full_batch) {
        const int n = (int)c->full.size();
        MFA_TRY(ensure_workspace(c, 1, c->full[0].len, n));
        MFA_TRY(launch_sdpa(c->stream, c->cfg.kv_dtype, c->cfg.num_attn_heads * n, c->cfg.num_kv_heads * n,
                            c->cfg.head_dim, 1, c->full[0].len, c->plane_elems, c->full[0].k, c->full[0].v,
                            full_q, full_gate, full_out, workspace(c), c->num_cus, c->forced_splits,
                            c->partial_only, lin_batch ? &merge : nullptr));
    }
    if (lin_batch) {
        LinearLayer &l0 = c->lin[0];
        MFA_TRY(launch_gdn_step(c->stream, c->cfg.linear_num_k_heads, c->cfg.linear_num_v_heads,
                                c->cfg.linear_key_dim, c->cfg.linear_value_dim, c->cfg.conv_kernel_size,
                                c->cfg.rms_norm_eps, l0.w, l0.conv_ring, l0.step, l0.ssm, lin_qkv, lin_z,
                                lin_alpha, lin_beta, lin_out, (int)c->lin.size(), &merge));
        for (auto &l : c->lin) l.step++;
    }
    for (int i = 0; i < c->cfg.num_layers; i++) {
        if (c->kind[i] == 1 ? full_batch : lin_batch) continue;
        const size_t s = (size_t)c->slot[i];
        if (c->kind[i] == 1)
            MFA_TRY(sdpa_decode_dev(c, &c->full[s], full_q + s * qd, full_gate + s * qd, full_out + s * qd));
        else
            MFA_TRY(gdn_step_dev(c, &c->lin[s], lin_qkv + s * C, lin_z + s * tv, lin_alpha + s * Hv,
                                 lin_beta + s * Hv, lin_out + s * tv));
    }
    return MFA_OK;
}

int mfa_set_sweep_per_layer(mfa_ctx *ctx, int32_t on) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    c->sweep_per_layer = on ? 1 : 0;
    return MFA_OK;
}

/* ---- attention over a latent cache -------------------------------------------------- */

static int mla_check(int32_t H, int32_t R, int32_t P, int32_t L) {
    if (H <= 0 || R <= 0 || P <= 0) return fail(MFA_ERR_INVALID, "non-positive shape");
    if (L <= 0) return fail(MFA_ERR_INVALID, "cache_len must be > 0 (got %d)", L);
    if (!mla_shape_supported(R, P))
        return fail(MFA_ERR_SHAPE, "kv_lora_rank %d / qk_rope_head_dim %d not supported (512 / 64)", R, P);
    return MFA_OK;
}

int mfa_mla_sdpa_folded_dev(mfa_ctx *ctx, int32_t num_heads, int32_t kv_lora_rank, int32_t qk_rope_head_dim,
                            int32_t cache_len, float softmax_scale, const float *q_prime, const float *q_pe,
                            const float *latent_cache, const float *rope_k_cache, float *v_combine) {
    Ctx *c = as_ctx(ctx);
    if (!c || !q_prime || !q_pe || !latent_cache || !rope_k_cache || !v_combine)
        return fail(MFA_ERR_INVALID, "NULL argument");
    MFA_TRY(mla_check(num_heads, kv_lora_rank, qk_rope_head_dim, cache_len));
    const MlaPlan plan = mla_plan(num_heads, cache_len, c->num_cus, c->forced_splits);
    MFA_TRY(ensure_workspace_elems(c, mla_workspace_o_elems(plan, kv_lora_rank), mla_workspace_ml_elems(plan)));
    return launch_mla_sdpa_folded(c->stream, num_heads, kv_lora_rank, qk_rope_head_dim, cache_len, softmax_scale,
                                  q_prime, q_pe, latent_cache, rope_k_cache, v_combine, workspace(c), plan);
}

int mfa_mla_sdpa_folded(int32_t num_heads, int32_t kv_lora_rank, int32_t qk_rope_head_dim, int32_t cache_len,
                        float softmax_scale, const float *q_prime, const float *q_pe, const float *latent_cache,
                        const float *rope_k_cache, float *v_combine) {
    if (!q_prime || !q_pe || !latent_cache || !rope_k_cache || !v_combine)
        return fail(MFA_ERR_INVALID, "NULL argument");
    MFA_TRY(mla_check(num_heads, kv_lora_rank, qk_rope_head_dim, cache_len));
    const size_t H = num_heads, R = kv_lora_rank, P = qk_rope_head_dim, L = cache_len;
    int dev = 0;
    hipDeviceProp_t prop;
    MFA_HIP(hipGetDevice(&dev));
    MFA_HIP(hipGetDeviceProperties(&prop, dev));
    const MlaPlan plan = mla_plan(num_heads, cache_len, prop.multiProcessorCount);
    DevBuf dq, dp, dl, dr, dout, dpo, dml;
    MFA_TRY(dq.upload(q_prime, H * R * 4));
    MFA_TRY(dp.upload(q_pe, H * P * 4));
    MFA_TRY(dl.upload(latent_cache, L * R * 4));
    MFA_TRY(dr.upload(rope_k_cache, L * P * 4));
    MFA_TRY(dout.alloc(H * R * 4));
    const size_t no = mla_workspace_o_elems(plan, kv_lora_rank), nml = mla_workspace_ml_elems(plan);
    MFA_TRY(dpo.alloc(no * 4));
    MFA_TRY(dml.alloc(nml * 4));
    const SdpaWorkspace ws{dpo.as<float>(), dml.as<float>(), no, nml};
    MFA_TRY(launch_mla_sdpa_folded(nullptr, num_heads, kv_lora_rank, qk_rope_head_dim, cache_len, softmax_scale,
                                   dq.as<float>(), dp.as<float>(), dl.as<float>(), dr.as<float>(), dout.as<float>(),
                                   ws, plan));
    return dout.download(v_combine, H * R * 4);
}

/* ---- projections ------------------------------------------------------------------- */

static int matvec_dev(mfa_ctx *ctx, int32_t n, const mfa_matvec_spec *specs, bool tiled) {
    Ctx *c = as_ctx(ctx);
    if (!c || !specs) return fail(MFA_ERR_INVALID, "NULL argument");
    if (n <= 0 || n > 8) return fail(MFA_ERR_INVALID, "1 to 8 products per call (got %d)", n);
    const uint32_t *w[8];
    const uint16_t *sc[8], *bi[8];
    const float *x[8];
    float *out[8];
    int od[8], id[8];
    for (int i = 0; i < n; i++) {
        w[i] = specs[i].w_packed; sc[i] = specs[i].scales; bi[i] = specs[i].biases;
        x[i] = specs[i].x; out[i] = specs[i].out; od[i] = specs[i].out_dim; id[i] = specs[i].in_dim;
    }
    return launch_dequant_matvec_4bit(c->stream, n, w, sc, bi, x, out, od, id, c->num_cus, tiled);
}

int mfa_dequant_matvec_4bit_dev(mfa_ctx *ctx, int32_t n, const mfa_matvec_spec *specs) {
    return matvec_dev(ctx, n, specs, false);
}

int mfa_dequant_matvec_4bit_tiled_dev(mfa_ctx *ctx, int32_t n, const mfa_matvec_spec *specs) {
    return matvec_dev(ctx, n, specs, true);
}

int64_t mfa_matvec_tiled_words(int32_t out_dim, int32_t in_dim) {
    if (out_dim <= 0 || in_dim <= 0 || in_dim % 64 != 0) return fail(MFA_ERR_INVALID, "out_dim %d, in_dim %d (a multiple of 64)", out_dim, in_dim);
    return (int64_t)matvec_tiled_words(out_dim, in_dim);
}

int mfa_matvec_tile_weights_dev(mfa_ctx *ctx, int32_t out_dim, int32_t in_dim, const uint32_t *w_packed,
                                const uint16_t *scales, const uint16_t *biases, uint32_t *w_tiled) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    return launch_matvec_tile_weights(c->stream, out_dim, in_dim, w_packed, scales, biases, w_tiled);
}

int mfa_dequant_matvec_4bit(int32_t out_dim, int32_t in_dim, int32_t group_size, const uint32_t *w_packed,
                            const uint16_t *scales, const uint16_t *biases, const float *x, float *out) {
    if (!w_packed || !scales || !biases || !x || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (out_dim <= 0 || in_dim <= 0) return fail(MFA_ERR_INVALID, "non-positive shape");
    if (group_size != 64) return fail(MFA_ERR_SHAPE, "group size %d not supported (64)", group_size);
    if (in_dim % 64 != 0) return fail(MFA_ERR_INVALID, "in_dim %d is not a multiple of the group size 64", in_dim);
    const size_t nw = (size_t)out_dim * (in_dim / 8), ng = (size_t)out_dim * (in_dim / 64);
    DevBuf dw, ds, db, dx, dout;
    MFA_TRY(dw.upload(w_packed, nw * 4));
    MFA_TRY(ds.upload(scales, ng * 2));
    MFA_TRY(db.upload(biases, ng * 2));
    MFA_TRY(dx.upload(x, (size_t)in_dim * 4));
    MFA_TRY(dout.alloc((size_t)out_dim * 4));
    const uint32_t *w[1] = {dw.as<uint32_t>()};
    const uint16_t *sc[1] = {ds.as<uint16_t>()}, *bi[1] = {db.as<uint16_t>()};
    const float *xx[1] = {dx.as<float>()};
    float *oo[1] = {dout.as<float>()};
    MFA_TRY(launch_dequant_matvec_4bit(nullptr, 1, w, sc, bi, xx, oo, &out_dim, &in_dim));
    return dout.download(out, (size_t)out_dim * 4);
}

/* ---- state operations ----------------------------------------------------------- */

int mfa_reset(mfa_ctx *ctx) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    for (auto &f : c->full) MFA_TRY(truncate_full(c, f, 0));
    for (auto &l : c->lin) MFA_TRY(reset_linear(c, l));
    MFA_HIP(hipStreamSynchronize(c->stream));
    drop_checkpoints(c);  // keyed by position: a full clear invalidates every key (riir/mod.rs:1965-1968)
    return MFA_OK;
}

int mfa_truncate(mfa_ctx *ctx, int32_t p0, int32_t p1) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    const int32_t new_len = p0 < 0 ? 0 : p0;
    for (auto &f : c->full) {
        const int32_t end = (p1 < 0 || p1 > f.len) ? f.len : p1;
        MFA_TRY(truncate_full(c, f, new_len < end ? new_len : end));
    }
    for (auto &l : c->lin) MFA_TRY(reset_linear(c, l));
    MFA_HIP(hipStreamSynchronize(c->stream));
    return MFA_OK;
}

int32_t mfa_pos_max(mfa_ctx *ctx) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    int32_t m = -1;
    for (auto &f : c->full) m = f.len > m ? f.len : m;
    return m;
}

int mfa_kv_export(mfa_ctx *ctx, int32_t layer, int32_t max_rows, float *k_out, float *v_out) {
    Ctx *c = as_ctx(ctx);
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (!k_out || !v_out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (max_rows < f->len) return fail(MFA_ERR_INVALID, "buffer holds %d rows, layer has %d", max_rows, f->len);
    if (f->len == 0) return MFA_OK;
    const size_t n = (size_t)f->len * c->kv_dim();
    MFA_TRY(ensure_stage(c, 2 * n));
    MFA_TRY(launch_kv_gather(c->stream, c->cfg.kv_dtype, c->cfg.num_kv_heads, c->cfg.head_dim,
                             c->plane_elems, f->len, f->k, f->v, c->stage, c->stage + n));
    MFA_HIP(hipMemcpyAsync(k_out, c->stage, n * 4, hipMemcpyDeviceToHost, c->stream));
    MFA_TRY(d2h_sync(c, v_out, c->stage + n, n * 4));
    return release_stage_beyond_cap(c);
}


void *mfa_host_alloc(int64_t bytes) {
    if (bytes <= 0) {
        (void)fail(MFA_ERR_INVALID, "host allocation of %lld bytes", (long long)bytes);
        return nullptr;
    }
    void *p = nullptr;
    const hipError_t e = hipHostMalloc(&p, (size_t)bytes, hipHostMallocDefault);
    if (e != hipSuccess) {
        (void)fail(MFA_ERR_HIP, "hipHostMalloc(%lld): %s", (long long)bytes, hipGetErrorString(e));
        return nullptr;
    }
    return p;
}

void mfa_host_free(void *p) {
    if (p) (void)hipHostFree(p);
}

static int kv_import(Ctx *c, int32_t layer, int32_t len, const void *k, const void *v, int src_bf16) {
    FullLayer *f;
    MFA_TRY(full_layer(c, layer, &f));
    if (len < 0) return fail(MFA_ERR_INVALID, "negative length");
    if (len > c->cfg.kv_capacity)
        return fail(MFA_ERR_OVERFLOW, "kv import of %d rows exceeds capacity %d", len, c->cfg.kv_capacity);
    if (len > 0 && (!k || !v)) return fail(MFA_ERR_INVALID, "NULL argument");
    if (src_bf16 && c->cfg.kv_dtype != MFA_KV_BF16)
        return fail(MFA_ERR_INVALID, "bf16 rows need a bf16 cache");
    MFA_TRY(truncate_full(c, *f, 0));
    if (len > 0) {
        const size_t n = (size_t)len * c->kv_dim();
        const size_t es = src_bf16 ? 2 : 4;
        MFA_TRY(ensure_stage(c, 2 * n));
        char *dk = (char *)c->stage, *dv = dk + n * es;
        MFA_TRY(h2d(c, dk, k, n * es));
        MFA_TRY(h2d(c, dv, v, n * es));
        MFA_TRY(launch_kv_scatter(c->stream, c->cfg.kv_dtype, src_bf16, c->cfg.num_kv_heads,
                                  c->cfg.head_dim, c->plane_elems, 0, len, dk, dv, f->k, f->v));
    }
    f->len = len;
    MFA_HIP(hipStreamSynchronize(c->stream));
    return release_stage_beyond_cap(c);
}

int mfa_kv_import(mfa_ctx *ctx, int32_t layer, int32_t len, const float *k, const float *v) {
    return kv_import(as_ctx(ctx), layer, len, k, v, 0);
}

int mfa_kv_import_bf16(mfa_ctx *ctx, int32_t layer, int32_t len, const uint16_t *k,
                       const uint16_t *v) {
    return kv_import(as_ctx(ctx), layer, len, k, v, 1);
}

int mfa_linear_state_export(mfa_ctx *ctx, int32_t layer, float *conv_state_out, float *ssm_state_out) {
    Ctx *c = as_ctx(ctx);
    LinearLayer *l;
    MFA_TRY(linear_layer(c, layer, &l));
    if (!conv_state_out || !ssm_state_out) return fail(MFA_ERR_INVALID, "NULL argument");
    const int C = c->conv_dim(), K = c->cfg.conv_kernel_size;
    const size_t nconv = (size_t)(K - 1) * C;
    const size_t nssm = (size_t)c->cfg.linear_num_v_heads * c->cfg.linear_value_dim * c->cfg.linear_key_dim;
    MFA_TRY(ensure_stage(c, nconv));
    MFA_TRY(launch_conv_ring_export(c->stream, C, K, l->step, l->conv_ring, c->stage));
    MFA_HIP(hipMemcpyAsync(conv_state_out, c->stage, nconv * 4, hipMemcpyDeviceToHost, c->stream));
    return d2h_sync(c, ssm_state_out, l->ssm, nssm * 4);
}

int mfa_linear_state_import(mfa_ctx *ctx, int32_t layer, const float *conv_state,
                            const float *ssm_state) {
    Ctx *c = as_ctx(ctx);
    LinearLayer *l;
    MFA_TRY(linear_layer(c, layer, &l));
    if (!conv_state || !ssm_state) return fail(MFA_ERR_INVALID, "NULL argument");
    const int C = c->conv_dim(), K = c->cfg.conv_kernel_size;
    const size_t nconv = (size_t)(K - 1) * C;
    const size_t nssm = (size_t)c->cfg.linear_num_v_heads * c->cfg.linear_value_dim * c->cfg.linear_key_dim;
    MFA_TRY(ensure_stage(c, nconv));
    MFA_TRY(h2d(c, c->stage, conv_state, nconv * 4));
    MFA_TRY(launch_conv_ring_import(c->stream, C, K, c->stage, l->conv_ring));
    MFA_TRY(h2d(c, l->ssm, ssm_state, nssm * 4));
    l->step = 0;
    MFA_HIP(hipStreamSynchronize(c->stream));
    return MFA_OK;
}

/* ---- diagnostics --------------------------------------------------------------------- */

int64_t mfa_debug_kv_offset(int32_t kv_dtype, int32_t is_v, int64_t pos, int32_t x, int32_t D) {
    if (!sdpa_shape_supported(kv_dtype, D) || pos < 0 || x < 0 || x >= D) return -1;
    if (kv_dtype == MFA_KV_BF16)
        return is_v ? KvTile<uint16_t>::v_off(pos, x, D) : KvTile<uint16_t>::k_off(pos, x, D);
    return is_v ? KvTile<float>::v_off(pos, x, D) : KvTile<float>::k_off(pos, x, D);
}

int32_t mfa_debug_num_splits(int32_t kv_dtype, int32_t Hq, int32_t Hkv, int32_t D, int64_t kv_len,
                             int32_t num_cus, int32_t forced_splits) {
    if (!sdpa_shape_supported(kv_dtype, D) || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || kv_len <= 0 ||
        num_cus <= 0)
        return -1;
    return sdpa_pick_splits(kv_dtype, Hq, Hkv, D, kv_len, num_cus, forced_splits);
}

int32_t mfa_debug_max_splits(int32_t kv_dtype, int32_t Hq, int32_t Hkv, int32_t D, int64_t max_len,
                             int32_t num_cus, int32_t forced_splits) {
    if (!sdpa_shape_supported(kv_dtype, D) || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || max_len <= 0 ||
        num_cus <= 0)
        return -1;
    return sdpa_max_splits(kv_dtype, Hq, Hkv, D, max_len, num_cus, forced_splits);
}

int mfa_debug_copy_dev(mfa_ctx *ctx, void *dst_dev, const void *src_dev, size_t nbytes) {
    Ctx *c = as_ctx(ctx);
    if (!c || !dst_dev || !src_dev) return fail(MFA_ERR_INVALID, "NULL argument");
    return launch_plain_copy(c->stream, dst_dev, src_dev, nbytes);
}

int mfa_debug_read_dev(mfa_ctx *ctx, const void *src_dev, size_t nbytes, int32_t workgroups) {
    Ctx *c = as_ctx(ctx);
    if (!c || !src_dev) return fail(MFA_ERR_INVALID, "NULL argument");
    // the sink is 16 bytes per workgroup: the staging buffer holds them
    MFA_TRY(ensure_stage(c, (size_t)(workgroups > 0 ? workgroups : 1) * 4));
    return launch_plain_read(c->stream, src_dev, nbytes, workgroups, c->stage);
}

int mfa_debug_fill_workspace(mfa_ctx *ctx, uint32_t pattern) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    if (c->part_o) MFA_HIP(hipMemsetD32Async((hipDeviceptr_t)c->part_o, (int)pattern, c->part_o_elems, c->stream));
    if (c->part_ml) MFA_HIP(hipMemsetD32Async((hipDeviceptr_t)c->part_ml, (int)pattern, c->part_ml_elems, c->stream));
    MFA_HIP(hipStreamSynchronize(c->stream));
    return MFA_OK;
}

/* ---- timing ------------------------------------------------------------------------ */

int mfa_timer_start(mfa_ctx *ctx) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    MFA_HIP(hipEventRecord(c->ev0, c->stream));
    return MFA_OK;
}

int mfa_timer_stop(mfa_ctx *ctx, float *elapsed_ms) {
    Ctx *c = as_ctx(ctx);
    if (!c || !elapsed_ms) return fail(MFA_ERR_INVALID, "NULL argument");
    MFA_HIP(hipEventRecord(c->ev1, c->stream));
    MFA_HIP(hipEventSynchronize(c->ev1));
    MFA_HIP(hipEventElapsedTime(elapsed_ms, c->ev0, c->ev1));
    return MFA_OK;
}

/* ---- stateless hooks ------------------------------------------------------------------ */

int mfa_sdpa(int32_t kv_len, int32_t Hq, int32_t Hkv, int32_t D, const float *q,
             const float *q_gate, const float *k_cache, const float *v_cache, float *out) {
    return sdpa_stateless(MFA_KV_F32, kv_len, Hq, Hkv, D, q, q_gate, k_cache, v_cache, out);
}

int mfa_sdpa_bf16kv(int32_t kv_len, int32_t Hq, int32_t Hkv, int32_t D, const float *q,
                    const float *q_gate, const uint16_t *k_cache, const uint16_t *v_cache,
                    float *out) {
    return sdpa_stateless(MFA_KV_BF16, kv_len, Hq, Hkv, D, q, q_gate, k_cache, v_cache, out);
}

int mfa_attn_scores_batched(int32_t Hq, int32_t Hkv, int32_t D, int32_t L, const float *q,
                            const float *k_cache, float scale, float *scores_out) {
    if (!q || !k_cache || !scores_out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (Hq <= 0 || Hkv <= 0 || D <= 0 || L <= 0) return fail(MFA_ERR_INVALID, "non-positive shape");
    if (Hq % Hkv != 0) return fail(MFA_ERR_INVALID, "num_heads %d %% num_kv_heads %d != 0", Hq, Hkv);
    DevBuf dq, dk, ds;
    MFA_TRY(dq.upload(q, (size_t)Hq * D * 4));
    MFA_TRY(dk.upload(k_cache, (size_t)L * Hkv * D * 4));
    MFA_TRY(ds.alloc((size_t)Hq * L * 4));
    MFA_TRY(launch_attn_scores(nullptr, Hq, Hkv, D, L, L, dq.as<float>(), dk.as<float>(), scale, ds.as<float>()));
    return ds.download(scores_out, (size_t)Hq * L * 4);
}

int mfa_attn_softmax_batched(int32_t Hq, int32_t L, float *scores_inout) {
    if (!scores_inout) return fail(MFA_ERR_INVALID, "NULL argument");
    if (Hq <= 0 || L <= 0) return fail(MFA_ERR_INVALID, "non-positive shape");
    DevBuf ds;
    MFA_TRY(ds.upload(scores_inout, (size_t)Hq * L * 4));
    MFA_TRY(launch_attn_softmax(nullptr, Hq, L, L, ds.as<float>()));
    return ds.download(scores_inout, (size_t)Hq * L * 4);
}

int mfa_attn_values_batched(int32_t Hq, int32_t Hkv, int32_t D, int32_t L, const float *scores,
                            const float *v_cache, float *out) {
    if (!scores || !v_cache || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (Hq <= 0 || Hkv <= 0 || D <= 0 || L <= 0) return fail(MFA_ERR_INVALID, "non-positive shape");
    if (Hq % Hkv != 0) return fail(MFA_ERR_INVALID, "num_heads %d %% num_kv_heads %d != 0", Hq, Hkv);
    DevBuf ds, dv, dout;
    MFA_TRY(ds.upload(scores, (size_t)Hq * L * 4));
    MFA_TRY(dv.upload(v_cache, (size_t)L * Hkv * D * 4));
    MFA_TRY(dout.alloc((size_t)Hq * D * 4));
    MFA_TRY(launch_attn_values(nullptr, Hq, Hkv, D, L, L, ds.as<float>(), dv.as<float>(), dout.as<float>()));
    return dout.download(out, (size_t)Hq * D * 4);
}

int mfa_sigmoid_gate(int32_t dim, const float *gate, float *x_inout) {
    if (!gate || !x_inout) return fail(MFA_ERR_INVALID, "NULL argument");
    if (dim <= 0) return fail(MFA_ERR_INVALID, "non-positive dim");
    DevBuf dg, dx;
    MFA_TRY(dg.upload(gate, (size_t)dim * 4));
    MFA_TRY(dx.upload(x_inout, (size_t)dim * 4));
    MFA_TRY(launch_sigmoid_gate(nullptr, dim, dg.as<float>(), dx.as<float>()));
    return dx.download(x_inout, (size_t)dim * 4);
}

int mfa_conv1d_step(int32_t C, int32_t K, float *conv_state_inout, const float *new_input,
                    const uint16_t *weight_bf16, float *out) {
    if (!conv_state_inout || !new_input || !weight_bf16 || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (C <= 0 || K < 2) return fail(MFA_ERR_INVALID, "bad conv shape: channels=%d kernel_size=%d", C, K);
    DevBuf ds, di, dw, dout;
    MFA_TRY(ds.upload(conv_state_inout, (size_t)(K - 1) * C * 4));
    MFA_TRY(di.upload(new_input, (size_t)C * 4));
    MFA_TRY(dw.upload(weight_bf16, (size_t)C * K * 2));
    MFA_TRY(dout.alloc((size_t)C * 4));
    MFA_TRY(launch_conv1d_step(nullptr, C, K, ds.as<float>(), di.as<float>(), dw.as<uint16_t>(), dout.as<float>()));
    MFA_TRY(dout.download(out, (size_t)C * 4));
    return ds.download(conv_state_inout, (size_t)(K - 1) * C * 4);
}

int mfa_rms_norm_qk(int32_t Hk, int32_t dk, float *q_inout, float *k_inout) {
    if (!q_inout || !k_inout) return fail(MFA_ERR_INVALID, "NULL argument");
    if (Hk <= 0 || dk <= 0) return fail(MFA_ERR_INVALID, "non-positive shape");
    DevBuf dq, dkb;
    MFA_TRY(dq.upload(q_inout, (size_t)Hk * dk * 4));
    MFA_TRY(dkb.upload(k_inout, (size_t)Hk * dk * 4));
    MFA_TRY(launch_rms_norm_qk(nullptr, Hk, dk, dq.as<float>(), dkb.as<float>()));
    MFA_TRY(dq.download(q_inout, (size_t)Hk * dk * 4));
    return dkb.download(k_inout, (size_t)Hk * dk * 4);
}

int mfa_rms_norm_bare(int32_t dim, float eps, const float *x, float *out) {
    if (!x || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (dim <= 0) return fail(MFA_ERR_INVALID, "dim must be positive");
    DevBuf dx, dout;
    MFA_TRY(dx.upload(x, (size_t)dim * 4));
    MFA_TRY(dout.alloc((size_t)dim * 4));
    MFA_TRY(launch_rms_norm_bare(nullptr, dim, eps, dx.as<float>(), dout.as<float>()));
    return dout.download(out, (size_t)dim * 4);
}

int mfa_compute_decay_beta(int32_t Hv, const float *alpha, const float *beta, const float *a_log,
                           const uint16_t *dt_bias_bf16, float *g_decay_out, float *beta_gate_out) {
    if (!alpha || !beta || !a_log || !dt_bias_bf16 || !g_decay_out || !beta_gate_out)
        return fail(MFA_ERR_INVALID, "NULL argument");
    if (Hv <= 0) return fail(MFA_ERR_INVALID, "non-positive head count");
    DevBuf da, db, dl, dt, dg, dbo;
    MFA_TRY(da.upload(alpha, (size_t)Hv * 4));
    MFA_TRY(db.upload(beta, (size_t)Hv * 4));
    MFA_TRY(dl.upload(a_log, (size_t)Hv * 4));
    MFA_TRY(dt.upload(dt_bias_bf16, (size_t)Hv * 2));
    MFA_TRY(dg.alloc((size_t)Hv * 4));
    MFA_TRY(dbo.alloc((size_t)Hv * 4));
    MFA_TRY(launch_decay_beta(nullptr, Hv, da.as<float>(), db.as<float>(), dl.as<float>(),
                              dt.as<uint16_t>(), dg.as<float>(), dbo.as<float>()));
    MFA_TRY(dg.download(g_decay_out, (size_t)Hv * 4));
    return dbo.download(beta_gate_out, (size_t)Hv * 4);
}

static int check_delta_shape(int32_t v_heads, int32_t k_heads, int32_t key_dim, int32_t value_dim) {
    if (v_heads <= 0 || k_heads <= 0 || key_dim <= 0 || value_dim <= 0)
        return fail(MFA_ERR_INVALID, "non-positive shape");
    if (v_heads % k_heads != 0)
        return fail(MFA_ERR_INVALID, "v_heads %d is not a multiple of k_heads %d", v_heads, k_heads);
    return MFA_OK;
}

int mfa_gated_delta_net_step(int32_t v_heads, int32_t k_heads, int32_t key_dim, int32_t value_dim,
                             const float *g_decay, const float *beta_gate, const float *q,
                             const float *k, const float *v, float *ssm_state_inout,
                             float *out_values) {
    if (!g_decay || !beta_gate || !q || !k || !v || !ssm_state_inout || !out_values)
        return fail(MFA_ERR_INVALID, "NULL argument");
    MFA_TRY(check_delta_shape(v_heads, k_heads, key_dim, value_dim));
    const size_t nk = (size_t)k_heads * key_dim, nv = (size_t)v_heads * value_dim,
                 ns = nv * key_dim;
    DevBuf dg, db, dq, dk, dv, ds, dout;
    MFA_TRY(dg.upload(g_decay, (size_t)v_heads * 4));
    MFA_TRY(db.upload(beta_gate, (size_t)v_heads * 4));
    MFA_TRY(dq.upload(q, nk * 4));
    MFA_TRY(dk.upload(k, nk * 4));
    MFA_TRY(dv.upload(v, nv * 4));
    MFA_TRY(ds.upload(ssm_state_inout, ns * 4));
    MFA_TRY(dout.alloc(nv * 4));
    MFA_TRY(launch_delta_net_step(nullptr, v_heads, k_heads, key_dim, value_dim, dg.as<float>(),
                                  db.as<float>(), dq.as<float>(), dk.as<float>(), dv.as<float>(),
                                  ds.as<float>(), dout.as<float>()));
    MFA_TRY(dout.download(out_values, nv * 4));
    return ds.download(ssm_state_inout, ns * 4);
}

int mfa_gated_delta_recurrence(const float *a_log, const uint16_t *dt_bias_bf16, const float *alpha,
                               const float *beta, const float *q, const float *k, const float *v,
                               int32_t v_heads, int32_t k_heads, int32_t key_dim, int32_t value_dim,
                               float *ssm_state_inout, float *out_values) {
    if (!a_log || !dt_bias_bf16 || !alpha || !beta || !q || !k || !v || !ssm_state_inout || !out_values)
        return fail(MFA_ERR_INVALID, "NULL argument");
    MFA_TRY(check_delta_shape(v_heads, k_heads, key_dim, value_dim));
    const size_t nk = (size_t)k_heads * key_dim, nv = (size_t)v_heads * value_dim,
                 ns = nv * key_dim;
    DevBuf da, db, dl, dt, dg, dbo, dq, dk, dv, ds, dout;
    MFA_TRY(da.upload(alpha, (size_t)v_heads * 4));
    MFA_TRY(db.upload(beta, (size_t)v_heads * 4));
    MFA_TRY(dl.upload(a_log, (size_t)v_heads * 4));
    MFA_TRY(dt.upload(dt_bias_bf16, (size_t)v_heads * 2));
    MFA_TRY(dg.alloc((size_t)v_heads * 4));
    MFA_TRY(dbo.alloc((size_t)v_heads * 4));
    MFA_TRY(dq.upload(q, nk * 4));
    MFA_TRY(dk.upload(k, nk * 4));
    MFA_TRY(dv.upload(v, nv * 4));
    MFA_TRY(ds.upload(ssm_state_inout, ns * 4));
    MFA_TRY(dout.alloc(nv * 4));
    MFA_TRY(launch_decay_beta(nullptr, v_heads, da.as<float>(), db.as<float>(), dl.as<float>(),
                              dt.as<uint16_t>(), dg.as<float>(), dbo.as<float>()));
    MFA_TRY(launch_delta_net_step(nullptr, v_heads, k_heads, key_dim, value_dim, dg.as<float>(),
                                  dbo.as<float>(), dq.as<float>(), dk.as<float>(), dv.as<float>(),
                                  ds.as<float>(), dout.as<float>()));
    MFA_TRY(dout.download(out_values, nv * 4));
    return ds.download(ssm_state_inout, ns * 4);
}

int mfa_gated_rms_norm(int32_t H, int32_t dim, float eps, const float *x, const float *z,
                       const uint16_t *weight_bf16, float *out) {
    if (!x || !z || !weight_bf16 || !out) return fail(MFA_ERR_INVALID, "NULL argument");
    if (H <= 0 || dim <= 0) return fail(MFA_ERR_INVALID, "non-positive shape");
    const size_t n = (size_t)H * dim;
    DevBuf dx, dz, dw, dout;
    MFA_TRY(dx.upload(x, n * 4));
    MFA_TRY(dz.upload(z, n * 4));
    MFA_TRY(dw.upload(weight_bf16, (size_t)dim * 2));
    MFA_TRY(dout.alloc(n * 4));
    MFA_TRY(launch_gated_rms_norm(nullptr, H, dim, eps, dx.as<float>(), dz.as<float>(),
                                  dw.as<uint16_t>(), dout.as<float>()));
    return dout.download(out, n * 4);
}

}  // extern "C"
