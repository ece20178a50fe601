// Helpers shared by the C ABI translation units: error reporting, the
// per-call context guard, host-side batch layout checks.
#pragma once

#include <string.h>

#include <algorithm>
#include <new>
#include <string>

#include "ctx.hpp"

namespace bnk {

inline thread_local std::string g_init_err;

inline int fail(bnk_ctx *ctx, int code, const std::string &what)
{
    if (ctx) ctx->err = what;
    else g_init_err = what;
    return code;
}

inline int fail_hip(bnk_ctx *ctx, const char *what, hipError_t e)
{
    return fail(ctx, e == hipErrorOutOfMemory ? BNK_E_NOMEM : BNK_E_HIP,
                std::string(what) + ": " + hipGetErrorString(e));
}

#define HIPCHK(ctx, expr)                                         \
    do {                                                          \
        hipError_t e_ = (expr);                                   \
        if (e_ != hipSuccess) return fail_hip((ctx), #expr, e_);  \
    } while (0)

// Every entry point takes the context lock and makes the context's device
// current for the calling thread.
struct Guard {
    std::unique_lock<std::mutex> lk;
    int rc = BNK_OK;
    explicit Guard(bnk_ctx *ctx)
    {
        if (!ctx) { rc = fail(nullptr, BNK_E_INVAL, "null context"); return; }
        lk = std::unique_lock<std::mutex>(ctx->mu);
        if (!ctx->alive) { rc = fail(ctx, BNK_E_STATE, "context is shut down"); return; }
        hipError_t e = hipSetDevice(ctx->device);
        if (e != hipSuccess) rc = fail_hip(ctx, "hipSetDevice", e);
    }
};

inline uint64_t pkt_off(const bnk_batch *b, uint32_t i)
{
    return b->offsets ? b->offsets[i] : (uint64_t)i * b->stride;
}

struct Span {
    uint64_t lo = UINT64_MAX, hi = 0;
    void add(uint64_t a, uint64_t b) { lo = std::min(lo, a); hi = std::max(hi, b); }
    uint64_t size() const { return hi > lo ? hi - lo : 0; }
};

// Checks that packet i of a host batch occupies [off, off + len + delta)
// inside the arena and accumulates the touched span.  lens come from `src`
// (the input batch) because an output batch only carries a layout.
inline int scan_host_layout(bnk_ctx *ctx, const bnk_batch *lay, const bnk_batch *src, int delta,
                     Span *span, const char *name)
{
    const uint32_t n = src->n;
    for (uint32_t i = 0; i < n; i++) {
        const uint64_t off = pkt_off(lay, i);
        int64_t len = (int64_t)(src->lens ? src->lens[i] : src->len) + delta;
        if (len < 0) len = 0;
        if (off > lay->bytes || (uint64_t)len > lay->bytes - off)
            return fail(ctx, BNK_E_INVAL, std::string(name) + ": packet " + std::to_string(i) +
                                              " lies outside the arena");
        span->add(off, off + (uint64_t)len);
    }
    return BNK_OK;
}

inline int check_batch_common(bnk_ctx *ctx, const bnk_batch *b, const char *name)
{
    if (!b) return fail(ctx, BNK_E_INVAL, std::string(name) + ": null batch");
    if (b->mem != BNK_MEM_HOST && b->mem != BNK_MEM_DEVICE)
        return fail(ctx, BNK_E_INVAL, std::string(name) + ": bad mem kind");
    if (b->n && !b->base) return fail(ctx, BNK_E_INVAL, std::string(name) + ": null arena");
    return BNK_OK;
}


// Host-resident view of a batch staged on the device.
struct Staged {
    uint8_t *d_in = nullptr, *d_out = nullptr;
    const uint64_t *d_in_off = nullptr, *d_out_off = nullptr;
    const uint32_t *d_lens = nullptr, *d_peer = nullptr;
    const uint64_t *d_counters = nullptr;
    Span sin, sout;
    bool in_place = false;
};

inline bool same_layout(const bnk_batch *a, const bnk_batch *b)
{
    if (a->base != b->base) return false;
    if (a->offsets || b->offsets) return a->offsets == b->offsets;
    return a->stride == b->stride;
}

// Copies the rebased offsets of `lay` into pinned staging at `slot` and
// queues the upload.
inline int upload_offsets(bnk_ctx *ctx, const bnk_batch *lay, uint32_t n, uint64_t lo, DevBuf *dst,
                   size_t pin_off, const uint64_t **out)
{
    if (!lay->offsets) { *out = nullptr; return BNK_OK; }
    HIPCHK(ctx, dst->reserve((size_t)n * 8));
    uint64_t *h = reinterpret_cast<uint64_t *>(ctx->pin.as<uint8_t>() + pin_off);
    for (uint32_t i = 0; i < n; i++) h[i] = lay->offsets[i] - lo;
    HIPCHK(ctx, hipMemcpyAsync(dst->p, h, (size_t)n * 8, hipMemcpyHostToDevice, ctx->stream));
    *out = dst->as<uint64_t>();
    return BNK_OK;
}

// Stages a host input batch (and the layout of its output batch) on the
// device.  in_delta/out_delta adjust the per-packet byte counts: seal writes
// len + 16, open writes len - 16.
inline int stage_host(bnk_ctx *ctx, const bnk_batch *in, const bnk_batch *out, int out_delta,
               uint32_t n_keys, Staged *st)
{
    const uint32_t n = in->n;
    int rc = scan_host_layout(ctx, in, in, 0, &st->sin, "in");
    if (rc) return rc;
    rc = scan_host_layout(ctx, out, in, out_delta, &st->sout, "out");
    if (rc) return rc;
    if (in->peer)
        for (uint32_t i = 0; i < n; i++)
            if (in->peer[i] >= n_keys)
                return fail(ctx, BNK_E_RANGE, "peer index " + std::to_string(in->peer[i]) +
                                                  " beyond the key table");
    // pinned staging for the two rebased offset arrays
    HIPCHK(ctx, ctx->pin.reserve((size_t)n * 16 + 64));

    st->in_place = same_layout(in, out);
    if (st->in_place) {
        Span u = st->sin;
        u.add(st->sout.lo, st->sout.hi);
        st->sin = st->sout = u;
    }
    HIPCHK(ctx, ctx->in_arena.reserve(st->sin.size() + 16));
    st->d_in = ctx->in_arena.as<uint8_t>();
    HIPCHK(ctx, hipMemcpyAsync(st->d_in, (const uint8_t *)in->base + st->sin.lo, st->sin.size(),
                               hipMemcpyHostToDevice, ctx->stream));
    if (st->in_place) {
        st->d_out = st->d_in;
    } else {
        HIPCHK(ctx, ctx->out_arena.reserve(st->sout.size() + 16));
        st->d_out = ctx->out_arena.as<uint8_t>();
        // bytes between packets of the output arena must survive the round
        // trip, so the device copy starts from the host's content
        HIPCHK(ctx, hipMemcpyAsync(st->d_out, (const uint8_t *)out->base + st->sout.lo,
                                   st->sout.size(), hipMemcpyHostToDevice, ctx->stream));
    }
    rc = upload_offsets(ctx, in, n, st->sin.lo, &ctx->off_in, 0, &st->d_in_off);
    if (rc) return rc;
    if (st->in_place) {
        st->d_out_off = st->d_in_off;
    } else {
        rc = upload_offsets(ctx, out, n, st->sout.lo, &ctx->off_out, (size_t)n * 8, &st->d_out_off);
        if (rc) return rc;
    }
    if (in->lens) {
        HIPCHK(ctx, ctx->lens.reserve((size_t)n * 4));
        HIPCHK(ctx, hipMemcpyAsync(ctx->lens.p, in->lens, (size_t)n * 4, hipMemcpyHostToDevice,
                                   ctx->stream));
        st->d_lens = ctx->lens.as<uint32_t>();
    }
    if (in->peer) {
        HIPCHK(ctx, ctx->peer.reserve((size_t)n * 4));
        HIPCHK(ctx, hipMemcpyAsync(ctx->peer.p, in->peer, (size_t)n * 4, hipMemcpyHostToDevice,
                                   ctx->stream));
        st->d_peer = ctx->peer.as<uint32_t>();
    }
    if (in->counters) {
        HIPCHK(ctx, ctx->counters.reserve((size_t)n * 8));
        HIPCHK(ctx, hipMemcpyAsync(ctx->counters.p, in->counters, (size_t)n * 8,
                                   hipMemcpyHostToDevice, ctx->stream));
        st->d_counters = ctx->counters.as<uint64_t>();
    }
    return BNK_OK;
}

// Lanes of a wave should run the same number of ChaCha20 blocks: when lengths
// vary, hand packets to lanes in length order.
inline int maybe_sort(bnk_ctx *ctx, const uint32_t *d_lens, uint32_t n, uint32_t tag_bytes,
               const uint32_t **order)
{
    *order = nullptr;
    if (!d_lens || n <= 64) return BNK_OK;
    HIPCHK(ctx, ctx->order.reserve((size_t)n * 4));
    HIPCHK(ctx, ctx->hist.reserve(LEN_BINS * 4));
    HIPCHK(ctx, ctx->cursor.reserve(LEN_BINS * 4));
    HIPCHK(ctx, launch_length_sort(d_lens, n, tag_bytes, ctx->order.as<uint32_t>(),
                                   ctx->hist.as<uint32_t>(), ctx->cursor.as<uint32_t>(),
                                   ctx->stream));
    *order = ctx->order.as<uint32_t>();
    return BNK_OK;
}

// Reads and clears the device status word (waits for the stream).
int take_status(bnk_ctx *ctx, uint32_t *status);
// Maps status bits to an error code (BNK_OK when clear).
int status_to_rc(bnk_ctx *ctx, uint32_t status);

} // namespace bnk
