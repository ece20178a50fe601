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


// Reads and clears the device status word (waits for the stream).
int take_status(bnk_ctx *ctx, uint32_t *status);
// Maps status bits to an error code (BNK_OK when clear).
int status_to_rc(bnk_ctx *ctx, uint32_t status);

} // namespace bnk
