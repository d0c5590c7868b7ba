// Checkpoints by sequence position: RsCtx::checkpoint_pos / restore_to / set_max_checkpoints /
// checkpoint_count (crates/moeflux/src/riir/mod.rs:2015-2100; tests/checkpoint_restore.rs).
//
// The reference serialises the whole context into host bytes with state_save and keeps at most
// four such buffers, least recently stored first.  Here a checkpoint never leaves the device: it
// is one allocation that holds, for every full-attention layer, the blocks of the tiled K and V
// planes up to the layer's length (a plane's first blocks are its first bytes, so each plane
// gives one contiguous run), and the conv rings and recurrent states of all linear layers as
// they lie in their slabs.  Storing and restoring are device-to-device copies on the context's
// stream; the keys, the order and the eviction rule are the reference's.
#include <algorithm>

#include "mfa_internal.h"

namespace mfa {

// rows x width16 units of 16 bytes, row r at src + r * src_pitch16 -> dst + r * dst_pitch16
__global__ void copy_rows_kernel(const uint4 *__restrict__ src, size_t src_pitch16, uint4 *__restrict__ dst,
                                 size_t dst_pitch16, size_t width16, size_t rows) {
    const size_t total = rows * width16;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / width16, x = i - r * width16;
        dst[r * dst_pitch16 + x] = src[r * src_pitch16 + x];
    }
}

static int copy_rows(hipStream_t stream, const void *src, size_t src_pitch, void *dst, size_t dst_pitch,
                     size_t width, size_t rows) {
    if (width == 0 || rows == 0) return MFA_OK;
    const size_t total = rows * (width / 16);
    const size_t want = (total + 255) / 256;
    const int grid = (int)(want < 65536 ? want : 65536);
    hipLaunchKernelGGL(copy_rows_kernel, dim3(grid), dim3(256), 0, stream, (const uint4 *)src, src_pitch / 16,
                       (uint4 *)dst, dst_pitch / 16, width / 16, rows);
    MFA_HIP(hipGetLastError());
    return MFA_OK;
}

namespace {

struct Sizes {
    size_t block_bytes;   // one block of one plane
    size_t plane_bytes;   // stride between planes in the K and V slabs
    size_t ring_bytes;    // all linear layers' conv rings
    size_t ssm_bytes;     // all linear layers' recurrent states
    int blk;
};

Sizes sizes_of(const Ctx *c) {
    Sizes s{};
    if (!c->full.empty()) {
        s.blk = kKvChunk;   // K is stored in chunks of 64 positions, which are whole blocks of V
        s.block_bytes = (size_t)s.blk * c->cfg.head_dim * c->kv_elem_size();
        s.plane_bytes = c->plane_elems * c->kv_elem_size();
    }
    if (!c->lin.empty()) {
        const size_t n = c->lin.size();
        s.ring_bytes = n * (size_t)c->cfg.conv_kernel_size * c->conv_dim() * sizeof(float);
        s.ssm_bytes = n * (size_t)c->cfg.linear_num_v_heads * c->cfg.linear_value_dim * c->cfg.linear_key_dim *
                      sizeof(float);
    }
    return s;
}

// bytes of one plane's blocks that hold positions [0, len)
size_t prefix_bytes(const Sizes &s, int32_t len) { return (size_t)((len + s.blk - 1) / s.blk) * s.block_bytes; }

// An evicted or replaced checkpoint's buffer goes back to the pool for the next store: in
// steady state (a rolling set of checkpoints) storing one allocates nothing.  The pool never
// holds more buffers than checkpoints may be kept.
void release(Ctx *c, Checkpoint &k) {
    if (k.buf) {
        if (c->checkpoint_pool.size() < c->max_checkpoints + 1) c->checkpoint_pool.emplace_back(k.buf, k.cap);
        else (void)hipFree(k.buf);
    }
    k.buf = nullptr;
}

// A buffer of at least `bytes`: the smallest pooled one that is large enough, else a new
// allocation with a quarter of headroom (caches grow between stores), for which the largest
// pooled buffer makes room.
int acquire(Ctx *c, size_t bytes, Checkpoint &k) {
    auto &pool = c->checkpoint_pool;
    size_t best = pool.size();
    for (size_t i = 0; i < pool.size(); i++)
        if (pool[i].second >= bytes && (best == pool.size() || pool[i].second < pool[best].second)) best = i;
    if (best != pool.size()) {
        k.buf = pool[best].first;
        k.cap = pool[best].second;
        pool.erase(pool.begin() + best);
        return MFA_OK;
    }
    if (!pool.empty()) {
        size_t big = 0;
        for (size_t i = 1; i < pool.size(); i++)
            if (pool[i].second > pool[big].second) big = i;
        (void)hipFree(pool[big].first);
        pool.erase(pool.begin() + big);
    }
    const size_t cap = ((bytes + bytes / 4) | 255) + 1;
    MFA_HIP(hipMalloc((void **)&k.buf, cap));
    k.cap = cap;
    return MFA_OK;
}

}  // namespace

void drop_checkpoints(Ctx *c) {
    for (auto &k : c->checkpoints)
        if (k.buf) (void)hipFree(k.buf);
    c->checkpoints.clear();
    for (auto &b : c->checkpoint_pool) (void)hipFree(b.first);
    c->checkpoint_pool.clear();
}

}  // namespace mfa

using namespace mfa;

extern "C" {

int mfa_checkpoint_pos(mfa_ctx *ctx, int32_t pos) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    const Sizes s = sizes_of(c);
    const size_t Hkv = (size_t)c->cfg.num_kv_heads;
    Checkpoint k;
    k.pos = pos;
    for (auto &f : c->full) {
        k.full_len.push_back(f.len);
        k.bytes += 2 * Hkv * prefix_bytes(s, f.len);
    }
    for (auto &l : c->lin) k.lin_step.push_back(l.step);
    k.bytes += s.ring_bytes + s.ssm_bytes;
    MFA_TRY(acquire(c, k.bytes, k));
    char *at = k.buf;
    int rc = MFA_OK;
    for (size_t i = 0; i < c->full.size() && rc == MFA_OK; i++) {
        const size_t w = prefix_bytes(s, c->full[i].len);
        rc = copy_rows(c->stream, c->full[i].k, s.plane_bytes, at, w, w, Hkv);
        if (rc == MFA_OK) rc = copy_rows(c->stream, c->full[i].v, s.plane_bytes, at + Hkv * w, w, w, Hkv);
        at += 2 * Hkv * w;
    }
    if (rc == MFA_OK && !c->lin.empty()) {
        rc = launch_plain_copy(c->stream, at, c->lin[0].conv_ring, s.ring_bytes);
        if (rc == MFA_OK) rc = launch_plain_copy(c->stream, at + s.ring_bytes, c->lin[0].ssm, s.ssm_bytes);
    }
    if (rc == MFA_OK && hipStreamSynchronize(c->stream) != hipSuccess) rc = fail(MFA_ERR_HIP, "checkpoint copy failed");
    if (rc != MFA_OK) {
        release(c, k);
        return rc;
    }
    // a checkpoint already stored at this position is replaced and becomes the newest
    auto &cks = c->checkpoints;
    for (size_t i = 0; i < cks.size(); i++)
        if (cks[i].pos == pos) {
            release(c, cks[i]);
            cks.erase(cks.begin() + i);
            break;
        }
    cks.push_back(std::move(k));
    // over the cap: drop the oldest, but never position 0 nor the one just stored
    while (cks.size() > c->max_checkpoints) {
        size_t victim = cks.size();
        for (size_t i = 0; i < cks.size(); i++)
            if (cks[i].pos != 0 && cks[i].pos != pos) {
                victim = i;
                break;
            }
        if (victim == cks.size()) break;
        release(c, cks[victim]);
        cks.erase(cks.begin() + victim);
    }
    return MFA_OK;
}

int mfa_restore_to(mfa_ctx *ctx, int32_t pos) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    auto &cks = c->checkpoints;
    size_t at_i = cks.size();
    for (size_t i = 0; i < cks.size(); i++)
        if (cks[i].pos == pos) at_i = i;
    if (at_i == cks.size()) return fail(MFA_ERR_NO_CHECKPOINT, "no checkpoint stored at position %d", pos);
    const Checkpoint &k = cks[at_i];
    const Sizes s = sizes_of(c);
    const size_t Hkv = (size_t)c->cfg.num_kv_heads;
    // Every copy is issued and waited for before a length or a ring position changes: a
    // failure on the way leaves the context's bookkeeping where it was.
    const char *at = k.buf;
    for (size_t i = 0; i < c->full.size(); i++) {
        FullLayer &f = c->full[i];
        const int32_t len = k.full_len[i];
        // rows past the restored length read as zero, as after a truncation
        if (f.len > len)
            MFA_TRY(launch_kv_zero(c->stream, c->cfg.kv_dtype, c->cfg.num_kv_heads, c->cfg.head_dim, c->plane_elems,
                                   len, f.len, f.k, f.v));
        const size_t w = prefix_bytes(s, len);
        MFA_TRY(copy_rows(c->stream, at, w, f.k, s.plane_bytes, w, Hkv));
        MFA_TRY(copy_rows(c->stream, at + Hkv * w, w, f.v, s.plane_bytes, w, Hkv));
        at += 2 * Hkv * w;
    }
    if (!c->lin.empty()) {
        MFA_TRY(launch_plain_copy(c->stream, c->lin[0].conv_ring, at, s.ring_bytes));
        MFA_TRY(launch_plain_copy(c->stream, c->lin[0].ssm, at + s.ring_bytes, s.ssm_bytes));
    }
    MFA_HIP(hipStreamSynchronize(c->stream));
    for (size_t i = 0; i < c->full.size(); i++) c->full[i].len = k.full_len[i];
    for (size_t i = 0; i < c->lin.size(); i++) c->lin[i].step = k.lin_step[i];
    // later positions will be written afresh from here on: their checkpoints are void
    for (size_t i = cks.size(); i-- > 0;)
        if (cks[i].pos > pos) {
            release(c, cks[i]);
            cks.erase(cks.begin() + i);
        }
    return MFA_OK;
}

int mfa_set_max_checkpoints(mfa_ctx *ctx, int32_t n) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    if (n < 0) return fail(MFA_ERR_INVALID, "max_checkpoints must be >= 0 (got %d)", n);
    c->max_checkpoints = (size_t)n;   // takes effect at the next mfa_checkpoint_pos, as in the reference
    return MFA_OK;
}

int32_t mfa_checkpoint_count(mfa_ctx *ctx) {
    Ctx *c = as_ctx(ctx);
    if (!c) return fail(MFA_ERR_INVALID, "NULL context");
    return (int32_t)c->checkpoints.size();
}

}  // extern "C"
