// The per-context state snapshot in the reference's wire format
// (crates/moeflux/src/riir/state_snapshot.rs:1-73; C side infer.m:8525-8700), over the
// device-resident state this library owns.  Little-endian:
//   header   u32 magic 'MFLX' = 0x4D464C58, version, num_layers, full_attn_interval,
//            num_kv_heads, head_dim, linear_conv_bytes = (K-1)*C*4,
//            linear_ssm_bytes = Hv*dv*dk*4, and in version 2 kv_lora_rank, qk_rope_head_dim
//            (both 0 here: no MLA layers);
//   per layer, in layer order
//     full attention   i32 len, len rows of K ([num_kv_heads*head_dim] f32) then len rows of V
//     linear attention conv state [(K-1)*C] f32 (oldest first), recurrent state [Hv*dv*dk] f32.
// Saved as version 2 (what the reference writes); versions 1 and 2 load.  A bf16 cache is
// widened on save and rounded back on load, which is exact for values that were bf16.
#include <cstring>
#include <vector>

#include "mfa_internal.h"

namespace mfa {

static constexpr uint32_t kMagic = 0x4D464C58u;
static constexpr uint32_t kVersion = 2;
static constexpr size_t kHeaderV1 = 8, kHeaderV2 = 10;

static size_t conv_bytes(const Ctx *c) {
    return c->lin.empty() ? 0 : (size_t)(c->cfg.conv_kernel_size - 1) * c->conv_dim() * 4;
}
static size_t ssm_bytes(const Ctx *c) {
    return c->lin.empty() ? 0
                          : (size_t)c->cfg.linear_num_v_heads * c->cfg.linear_value_dim * c->cfg.linear_key_dim * 4;
}
static size_t row_bytes(const Ctx *c) { return c->full.empty() ? 0 : (size_t)c->kv_dim() * 4; }

static void put_u32(uint8_t *p, uint32_t v) {
    p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); p[2] = (uint8_t)(v >> 16); p[3] = (uint8_t)(v >> 24);
}
static uint32_t get_u32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

// The device image the state is assembled in (save) or unpacked from (load): per layer one segment of
// the context's staging buffer, 256-byte aligned, holding K rows then V rows, or the conv state (the
// recurrent state is copied to and from its own allocation).  Offsets in floats.
static constexpr size_t kSegAlign = 64;
static size_t seg_round(size_t elems) { return (elems + kSegAlign - 1) / kSegAlign * kSegAlign; }

// The image is built for runs of consecutive layers whose segments fit kStageCap together (a layer
// larger than that is a run of its own), so the staging buffer a snapshot needs does not grow with
// the number of layers; the runs follow one another on the stream and reuse the buffer in stream
// order.  What a long cache made the buffer grow beyond the cap is given back when the call ends
// (release_stage_beyond_cap).

// seg[i]: image elements of layer i.  Returns the ends of the runs and the largest run.
static std::vector<int> layer_runs(const std::vector<size_t> &seg, size_t *largest) {
    std::vector<int> ends;
    *largest = 0;
    for (size_t i = 0; i < seg.size();) {
        size_t img = seg[i], j = i + 1;
        while (j < seg.size() && img + seg[j] <= kStageCap) img += seg[j++];
        if (img > *largest) *largest = img;
        ends.push_back((int)j);
        i = j;
    }
    return ends;
}


}  // namespace mfa

using namespace mfa;

/* state_size (state_snapshot.rs:184-216) */
int64_t mfa_state_size(mfa_ctx *ctx) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    size_t n = kHeaderV2 * 4;
    for (int i = 0; i < c->cfg.num_layers; i++) {
        if (c->kind[i] == 1) n += 4 + 2 * (size_t)c->full[c->slot[i]].len * row_bytes(c);
        else n += conv_bytes(c) + ssm_bytes(c);
    }
    return (int64_t)n;
}

/* state_save (state_snapshot.rs:218-360): bytes written, or a negative error. */
int64_t mfa_state_save(mfa_ctx *ctx, uint8_t *buf, int64_t buf_len) {
    Ctx *c = as_ctx(ctx);
    if (!c || !buf) return fail(MFA_ERR_INVALID, "NULL argument");
    const int64_t need = mfa_state_size(ctx);
    if (buf_len < need) return fail(MFA_ERR_INVALID, "buffer too small: need %lld bytes, got %lld", (long long)need, (long long)buf_len);
    const uint32_t header[kHeaderV2] = {kMagic, kVersion, (uint32_t)c->cfg.num_layers, (uint32_t)c->cfg.full_attn_interval,
                                        (uint32_t)c->cfg.num_kv_heads, (uint32_t)c->cfg.head_dim,
                                        (uint32_t)conv_bytes(c), (uint32_t)ssm_bytes(c), 0u, 0u};
    // a run's rows are gathered into the device image first, then its copies follow one another on
    // the stream; the host waits once, after the last run
    std::vector<size_t> seg(c->cfg.num_layers);
    for (int i = 0; i < c->cfg.num_layers; i++)
        seg[i] = c->kind[i] == 1 ? seg_round(2 * (size_t)c->full[c->slot[i]].len * c->kv_dim()) : seg_round(conv_bytes(c) / 4);
    size_t largest = 0;
    const std::vector<int> runs = layer_runs(seg, &largest);
    MFA_TRY(ensure_stage(c, largest));
    size_t off = kHeaderV2 * 4;
    int first = 0;
    for (int end : runs) {
        size_t at = 0;
        for (int i = first; i < end; i++) {
            if (c->kind[i] == 1) {
                FullLayer *f = &c->full[c->slot[i]];
                const size_t n = (size_t)f->len * c->kv_dim();
                MFA_TRY(kv_export_to(c, f, c->stage + at, c->stage + at + n));
            } else {
                MFA_TRY(linear_export_to(c, &c->lin[c->slot[i]], c->stage + at));
            }
            at += seg[i];
        }
        at = 0;
        for (int i = first; i < end; i++) {
            if (c->kind[i] == 1) {
                const size_t n = (size_t)c->full[c->slot[i]].len * c->kv_dim();
                off += 4;
                if (n > 0) MFA_HIP(hipMemcpyAsync(buf + off, c->stage + at, 2 * n * 4, hipMemcpyDeviceToHost, c->stream));
                off += 2 * n * 4;
            } else {
                MFA_HIP(hipMemcpyAsync(buf + off, c->stage + at, conv_bytes(c), hipMemcpyDeviceToHost, c->stream));
                MFA_HIP(hipMemcpyAsync(buf + off + conv_bytes(c), c->lin[c->slot[i]].ssm, ssm_bytes(c), hipMemcpyDeviceToHost, c->stream));
                off += conv_bytes(c) + ssm_bytes(c);
            }
            at += seg[i];
        }
        first = end;
    }
    MFA_HIP(hipStreamSynchronize(c->stream));
    MFA_TRY(release_stage_beyond_cap(c));
    // the words the host knows: header and cache lengths
    off = 0;
    for (uint32_t w : header) { put_u32(buf + off, w); off += 4; }
    for (int i = 0; i < c->cfg.num_layers; i++) {
        if (c->kind[i] == 1) {
            const int32_t len = c->full[c->slot[i]].len;
            put_u32(buf + off, (uint32_t)len);
            off += 4 + 2 * (size_t)len * row_bytes(c);
        } else {
            off += conv_bytes(c) + ssm_bytes(c);
        }
    }
    return (int64_t)off;
}

/* state_load (state_snapshot.rs:362-640): header and sizes are checked over the whole buffer
 * before anything is restored, so a bad snapshot leaves the context as it was. */
int mfa_state_load(mfa_ctx *ctx, const uint8_t *buf, int64_t buf_len) {
    Ctx *c = as_ctx(ctx);
    if (!c || !buf) return fail(MFA_ERR_INVALID, "NULL argument");
    if (buf_len < 8) return fail(MFA_ERR_STATE, "snapshot truncated: need 8 bytes, got %lld", (long long)buf_len);
    if (get_u32(buf) != kMagic)
        return fail(MFA_ERR_STATE, "snapshot magic mismatch (got 0x%08X, want 0x%08X)", get_u32(buf), kMagic);
    const uint32_t version = get_u32(buf + 4);
    if (version != 1 && version != 2) return fail(MFA_ERR_STATE, "snapshot version mismatch (got %u, want %u)", version, kVersion);
    const size_t header_bytes = (version == 1 ? kHeaderV1 : kHeaderV2) * 4;
    if ((size_t)buf_len < header_bytes)
        return fail(MFA_ERR_STATE, "snapshot truncated: need %zu header bytes, got %lld", header_bytes, (long long)buf_len);
    const struct { size_t off; const char *field; uint32_t want; } checks[] = {
        {8, "num_layers", (uint32_t)c->cfg.num_layers},
        {12, "full_attn_interval", (uint32_t)c->cfg.full_attn_interval},
        {16, "num_kv_heads", (uint32_t)c->cfg.num_kv_heads},
        {20, "head_dim", (uint32_t)c->cfg.head_dim},
        {24, "linear_conv_bytes", (uint32_t)conv_bytes(c)},
        {28, "linear_ssm_bytes", (uint32_t)ssm_bytes(c)},
        {32, "kv_lora_rank", 0u},
        {36, "qk_rope_head_dim", 0u},
    };
    for (const auto &k : checks) {
        if (k.off >= header_bytes) break;
        // a context without layers of a kind carries zeros for that kind's shape fields
        if (c->full.empty() && (k.off == 16 || k.off == 20)) continue;
        if (get_u32(buf + k.off) != k.want)
            return fail(MFA_ERR_STATE, "snapshot shape mismatch on field '%s' (got %u, want %u)", k.field,
                        get_u32(buf + k.off), k.want);
    }
    // preflight
    size_t q = header_bytes;
    const size_t total = (size_t)buf_len;
    for (int i = 0; i < c->cfg.num_layers; i++) {
        if (c->kind[i] == 1) {
            if (total - q < 4) return fail(MFA_ERR_STATE, "snapshot truncated at layer %d", i);
            const int32_t len = (int32_t)get_u32(buf + q);
            q += 4;
            if (len < 0) return fail(MFA_ERR_STATE, "snapshot layer %d has negative KV length %d", i, len);
            if (len > c->cfg.kv_capacity)
                return fail(MFA_ERR_OVERFLOW, "snapshot layer %d KV length %d exceeds the capacity %d", i, len, c->cfg.kv_capacity);
            const size_t bytes = 2 * (size_t)len * row_bytes(c);
            if (total - q < bytes) return fail(MFA_ERR_STATE, "snapshot truncated at layer %d: need %zu more bytes, got %zu", i, bytes, total - q);
            q += bytes;
        } else {
            const size_t bytes = conv_bytes(c) + ssm_bytes(c);
            if (total - q < bytes) return fail(MFA_ERR_STATE, "snapshot truncated at layer %d: need %zu more bytes, got %zu", i, bytes, total - q);
            q += bytes;
        }
    }
    // restore: a run's bytes go to the device image first (a copy from pageable memory has left the
    // caller's buffer when the call returns), then the kernels unpack them; one wait at the end
    std::vector<size_t> seg(c->cfg.num_layers);
    size_t off = header_bytes;
    for (int i = 0; i < c->cfg.num_layers; i++) {
        if (c->kind[i] == 1) {
            const int32_t len = (int32_t)get_u32(buf + off);
            off += 4 + 2 * (size_t)len * row_bytes(c);
            seg[i] = seg_round(2 * (size_t)len * c->kv_dim());
        } else {
            off += conv_bytes(c) + ssm_bytes(c);
            seg[i] = seg_round(conv_bytes(c) / 4);
        }
    }
    size_t largest = 0;
    const std::vector<int> runs = layer_runs(seg, &largest);
    MFA_TRY(ensure_stage(c, largest));
    off = header_bytes;
    int first = 0;
    for (int end : runs) {
        size_t at = 0;
        for (int i = first; i < end; i++) {
            if (c->kind[i] == 1) {
                const int32_t len = (int32_t)get_u32(buf + off);
                off += 4;
                const size_t n = (size_t)len * c->kv_dim();
                if (n > 0) MFA_HIP(hipMemcpyAsync(c->stage + at, buf + off, 2 * n * 4, hipMemcpyHostToDevice, c->stream));
                MFA_TRY(kv_import_from(c, &c->full[c->slot[i]], len, c->stage + at, c->stage + at + n));
                off += 2 * n * 4;
            } else {
                LinearLayer *l = &c->lin[c->slot[i]];
                MFA_HIP(hipMemcpyAsync(c->stage + at, buf + off, conv_bytes(c), hipMemcpyHostToDevice, c->stream));
                MFA_TRY(linear_import_from(c, l, c->stage + at));
                MFA_HIP(hipMemcpyAsync(l->ssm, buf + off + conv_bytes(c), ssm_bytes(c), hipMemcpyHostToDevice, c->stream));
                off += conv_bytes(c) + ssm_bytes(c);
            }
            at += seg[i];
        }
        first = end;
    }
    MFA_HIP(hipStreamSynchronize(c->stream));
    return release_stage_beyond_cap(c);
}
