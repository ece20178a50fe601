// Helpers shared by the C ABI translation units: error reporting, the
// per-call context guard, host-side batch layout checks.
#pragma once

#include <string.h>

#include <algorithm>
#include <functional>
#include <initializer_list>
#include <new>
#include <string>

#include "ctx.hpp"

namespace bnk {

inline thread_local std::string g_init_err;

// The error text has a lock of its own: bnk_last_error may be called by a
// thread that does not hold the context lock.
inline int fail(bnk_ctx *ctx, int code, const std::string &what)
{
    if (ctx) {
        std::lock_guard<std::mutex> lk(ctx->err_mu);
        ctx->err = what;
    } else {
        g_init_err = what;
    }
    return code;
}

// For the exception barrier: must not throw itself.
inline int fail_caught(bnk_ctx *ctx, int code, const char *what) noexcept
{
    try {
        return fail(ctx, code, what);
    } catch (...) {
        return code;
    }
}

// Nothing may unwind into a C (cgo) caller: every extern "C" body sits between
// these two.  The context lock (a Guard inside the body) is released by the
// unwinding before the handler runs.
#define BNK_API_TRY try {
#define BNK_API_CATCH(ctx)                                                                   \
    }                                                                                        \
    catch (const std::bad_alloc &) { return bnk::fail_caught((ctx), BNK_E_NOMEM, "out of host memory"); } \
    catch (...) { return bnk::fail_caught((ctx), BNK_E_HIP, "unexpected C++ exception inside the library"); }

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

// Hot-path counters (tally.hip).  A host batch's result bytes are counted on the
// host, a device-resident batch's by a launch behind the batch on ctx->stream
// (the caller holds the context's lock, as for every launch).
enum TallyKind { TALLY_OPEN, TALLY_CHECK, TALLY_DECAP, TALLY_DECAP_CHECK, TALLY_RELAY };
void tally_add(bnk_ctx *ctx, TallySlot slot, uint64_t k);
int tally_results(bnk_ctx *ctx, TallyKind kind, const uint8_t *res, uint32_t n, int mem);
int tally_nonzero(bnk_ctx *ctx, TallySlot slot, const uint32_t *words, uint32_t n, int mem);

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

// Sum of the packet lengths of a host batch.
inline uint64_t host_payload_bytes(const bnk_batch *b)
{
    if (!b->lens) return (uint64_t)b->n * b->len;
    uint64_t sum = 0;
    for (uint32_t i = 0; i < b->n; i++) sum += b->lens[i];
    return sum;
}

// Every index of a host array must name a row of a table with `rows` rows.
inline int check_index_range(bnk_ctx *ctx, const uint32_t *index, uint32_t n, uint32_t rows,
                             const char *what, const char *table)
{
    if (!index) return BNK_OK;
    for (uint32_t i = 0; i < n; i++)
        if (index[i] >= rows)
            return fail(ctx, BNK_E_RANGE,
                        std::string(what) + " " + std::to_string(index[i]) + " beyond " + table);
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


// Host batches up to this size run in place when their arenas are pinned rings
// of the context (no staging copies).  Measured against the chunked copy-engine
// route the crossover lies at about 8 MB of packets, whatever their size.
constexpr uint32_t DIRECT_MAX_PACKETS = 1u << 16;
constexpr uint64_t DIRECT_MAX_BYTES = 8ull << 20;

// Device address of [p, p + bytes) when it lies inside one of the context's
// pinned rings, else null.
inline uint8_t *ring_device_ptr(const bnk_ctx *ctx, const void *p, uint64_t bytes)
{
    const uintptr_t a = (uintptr_t)p;
    for (const bnk_ctx::Ring &r : ctx->rings)
        if (r.dev && a >= r.host && bytes <= r.bytes && a - r.host <= r.bytes - bytes) return r.dev + (a - r.host);
    return nullptr;
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
    rc = check_index_range(ctx, in->peer, n, n_keys, "peer index", "the key table");
    if (rc) return rc;
    // pinned staging for the two rebased offset arrays, and behind them room for
    // one result byte per packet (a copy into pageable memory is slow)
    HIPCHK(ctx, ctx->pin.reserve((size_t)n * 17 + 64));

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
// A launch that gives every packet its own wave has no use for the order.
inline int maybe_sort(bnk_ctx *ctx, AeadArgs *a, uint32_t tag_bytes)
{
    a->order = nullptr;
    if (!a->lens || a->n <= 64 || aead_runs_spread(*a)) return BNK_OK;
    HIPCHK(ctx, ctx->order.reserve((size_t)a->n * 4));
    HIPCHK(ctx, ctx->hist.reserve(LEN_BINS * 4));
    HIPCHK(ctx, ctx->cursor.reserve(LEN_CURSOR_WORDS * 4));
    HIPCHK(ctx, launch_length_sort(a->lens, a->n, tag_bytes, ctx->order.as<uint32_t>(),
                                   ctx->hist.as<uint32_t>(), ctx->cursor.as<uint32_t>(),
                                   ctx->stream));
    a->order = ctx->order.as<uint32_t>();
    return BNK_OK;
}

// ---------------------------------------------------------------------------
// Chunked host batches.  While chunk k is computed, chunk k+1 is on its way up
// and chunk k-1 on its way down (the link is full duplex): three streams, one
// event pair per chunk.  Needs packets laid out in ascending, non-overlapping
// order in both arenas, so that a run of consecutive packets is one contiguous
// span.
// ---------------------------------------------------------------------------
constexpr uint32_t PIPE_MAX_CHUNKS = 16;
constexpr uint64_t PIPE_MIN_CHUNK_BYTES = 4ull << 20;

struct HostPipe {
    bnk_ctx *ctx = nullptr;
    const bnk_batch *in = nullptr, *out = nullptr;
    uint32_t n = 0, chunks = 0, per = 0;
    Span sin, sout;
    bool in_place = false;
    uint64_t row_width = 0; // > 0: the output comes back row by row (uniform layout, see plan)
    uint32_t max_chunks = PIPE_MAX_CHUNKS;
    uint8_t *d_in = nullptr, *d_out = nullptr;
    const uint64_t *d_in_off = nullptr, *d_out_off = nullptr;

    // Bytes packet i occupies from its offset in the input / output arena.
    std::function<uint64_t(uint32_t)> in_ext, out_ext;

    struct Result {
        void *host;
        const void *dev;
        uint32_t elem;
        size_t pin_off;
    };
    std::vector<Result> results;
    size_t pin_used = 0;

    // BNK_OK, an error code, or 1 when the batch does not qualify (too small, or
    // not ascending) and the caller should take the single-shot route.
    // uniform_out_width: the output extent when every packet has the same one
    // and the layout is a uniform stride (then the gaps between output packets
    // never need to be on the device), else 0.
    int plan(uint64_t uniform_out_width)
    {
        n = in->n;
        uint64_t in_end = 0, out_end = 0;
        for (uint32_t i = 0; i < n; i++) {
            const uint64_t io = pkt_off(in, i), ie = in_ext(i), oo = pkt_off(out, i), oe = out_ext(i);
            if (io > in->bytes || ie > in->bytes - io)
                return fail(ctx, BNK_E_INVAL, "in: packet " + std::to_string(i) + " lies outside the arena");
            if (oo > out->bytes || oe > out->bytes - oo)
                return fail(ctx, BNK_E_INVAL, "out: packet " + std::to_string(i) + " lies outside the arena");
            if (io < in_end || oo < out_end) return 1;
            in_end = io + ie;
            out_end = oo + oe;
            sin.add(io, io + ie);
            sout.add(oo, oo + oe);
        }
        const uint32_t by_bytes =
            (uint32_t)std::min<uint64_t>(std::max(sin.size(), sout.size()) / PIPE_MIN_CHUNK_BYTES, max_chunks);
        if (by_bytes < 2 || n < 2u * 64u) return 1;
        chunks = by_bytes;
        per = ((n + chunks - 1u) / chunks + 63u) & ~63u; // whole waves per chunk
        if (!ctx->s_up) HIPCHK(ctx, hipStreamCreateWithFlags(&ctx->s_up, hipStreamNonBlocking));
        if (!ctx->s_down) HIPCHK(ctx, hipStreamCreateWithFlags(&ctx->s_down, hipStreamNonBlocking));
        while (ctx->ev_up.size() < chunks + 1u || ctx->ev_done.size() < chunks) {
            hipEvent_t a, b;
            HIPCHK(ctx, hipEventCreateWithFlags(&a, hipEventDisableTiming));
            ctx->ev_up.push_back(a);
            HIPCHK(ctx, hipEventCreateWithFlags(&b, hipEventDisableTiming));
            ctx->ev_done.push_back(b);
        }
        in_place = same_layout(in, out);
        if (in_place) {
            sin.add(sout.lo, sout.hi);
            sout = sin;
        }
        row_width = (!in_place && !out->offsets) ? uniform_out_width : 0;
        HIPCHK(ctx, ctx->in_arena.reserve(sin.size() + 16));
        d_in = d_out = ctx->in_arena.as<uint8_t>();
        if (!in_place) {
            HIPCHK(ctx, ctx->out_arena.reserve(sout.size() + 16));
            d_out = ctx->out_arena.as<uint8_t>();
        }
        pin_used = (size_t)n * 16; // the two rebased offset arrays
        return BNK_OK;
    }

    // A per-packet result array that comes back chunk by chunk.  Downloads go
    // through pinned staging: a copy into pageable memory would make the
    // runtime wait for it and stall the pipeline.
    void add_result(void *host, const void *dev, uint32_t elem)
    {
        results.push_back(Result{host, dev, elem, pin_used});
        pin_used += ((size_t)n * elem + 15u) & ~size_t(15);
    }

    // Uploads the offset arrays (on the compute stream) and opens the pipeline.
    int begin()
    {
        HIPCHK(ctx, ctx->pin.reserve(pin_used + 64));
        int rc = upload_offsets(ctx, in, n, sin.lo, &ctx->off_in, 0, &d_in_off);
        if (rc) return rc;
        if (in_place) d_out_off = d_in_off;
        else {
            rc = upload_offsets(ctx, out, n, sout.lo, &ctx->off_out, (size_t)n * 8, &d_out_off);
            if (rc) return rc;
        }
        return BNK_OK;
    }
    // After every other whole-batch upload has been queued on the compute stream.
    int open_gate()
    {
        HIPCHK(ctx, hipEventRecord(ctx->ev_up[chunks], ctx->stream));
        HIPCHK(ctx, hipStreamWaitEvent(ctx->s_up, ctx->ev_up[chunks], 0));
        return BNK_OK;
    }

    bool range(uint32_t k, uint32_t *lo, uint32_t *hi) const
    {
        *lo = k * per;
        *hi = std::min(n, *lo + per);
        return *lo < *hi;
    }

    // Queues chunk k's upload and makes the compute stream wait for it.
    int upload(uint32_t k)
    {
        uint32_t lo, hi;
        if (!range(k, &lo, &hi)) return BNK_OK;
        const uint8_t *h_in = (const uint8_t *)in->base;
        const uint8_t *h_out = (const uint8_t *)out->base;
        uint64_t u0 = pkt_off(in, lo), u1 = pkt_off(in, hi - 1) + in_ext(hi - 1);
        const uint64_t o0 = pkt_off(out, lo), o1 = pkt_off(out, hi - 1) + out_ext(hi - 1);
        if (in_place) {
            u0 = std::min(u0, o0);
            u1 = std::max(u1, o1);
        }
        if (u1 > u0)
            HIPCHK(ctx, hipMemcpyAsync(d_in + (u0 - sin.lo), h_in + u0, u1 - u0, hipMemcpyHostToDevice, ctx->s_up));
        // any layout that does not come back row by row first takes the host's
        // output bytes up, so that what lies between packets comes back unchanged
        if (!in_place && !row_width && o1 > o0)
            HIPCHK(ctx, hipMemcpyAsync(d_out + (o0 - sout.lo), h_out + o0, o1 - o0, hipMemcpyHostToDevice, ctx->s_up));
        HIPCHK(ctx, hipEventRecord(ctx->ev_up[k], ctx->s_up));
        HIPCHK(ctx, hipStreamWaitEvent(ctx->stream, ctx->ev_up[k], 0));
        return BNK_OK;
    }

    // After chunk k's kernels have been queued on the compute stream.
    int download(uint32_t k)
    {
        uint32_t lo, hi;
        if (!range(k, &lo, &hi)) return BNK_OK;
        uint8_t *h_out = (uint8_t *)out->base;
        HIPCHK(ctx, hipEventRecord(ctx->ev_done[k], ctx->stream));
        HIPCHK(ctx, hipStreamWaitEvent(ctx->s_down, ctx->ev_done[k], 0));
        uint64_t o0 = pkt_off(out, lo), o1 = pkt_off(out, hi - 1) + out_ext(hi - 1);
        if (in_place) {
            o0 = std::min(o0, pkt_off(in, lo));
            o1 = std::max(o1, pkt_off(in, hi - 1) + in_ext(hi - 1));
        }
        if (row_width)
            HIPCHK(ctx, hipMemcpy2DAsync(h_out + o0, out->stride, d_out + (o0 - sout.lo), out->stride, row_width,
                                         hi - lo, hipMemcpyDeviceToHost, ctx->s_down));
        else if (o1 > o0)
            HIPCHK(ctx, hipMemcpyAsync(h_out + o0, d_out + (o0 - sout.lo), o1 - o0, hipMemcpyDeviceToHost, ctx->s_down));
        for (const Result &r : results)
            HIPCHK(ctx, hipMemcpyAsync(ctx->pin.as<uint8_t>() + r.pin_off + (size_t)lo * r.elem,
                                       (const uint8_t *)r.dev + (size_t)lo * r.elem, (size_t)(hi - lo) * r.elem,
                                       hipMemcpyDeviceToHost, ctx->s_down));
        return BNK_OK;
    }

    // Waits for the last download and hands the result arrays over.
    int finish()
    {
        HIPCHK(ctx, hipStreamSynchronize(ctx->s_down));
        for (const Result &r : results) memcpy(r.host, ctx->pin.as<uint8_t>() + r.pin_off, (size_t)n * r.elem);
        return BNK_OK;
    }
};

// Seal or open of one batch (api.hip).  sort_scratch: null, or device memory of
// LEN_BINS + LEN_CURSOR_WORDS + in->n words for the length grouping of a device-resident batch;
// with it the call allocates nothing and takes device batches only.
int aead_batch(bnk_ctx *ctx, bool open, const bnk_batch *in, const bnk_batch *out, uint8_t *verdict,
               uint32_t *sort_scratch);

// bnk_wg_encap_batch (wg_api.hip), with NoteOutbound at *note_now on the plaintexts first
// when note_now is given; and bnk_wg_decap_batch, with CheckInbound at *check_now on the
// delivered packets afterwards when check_now is given.  The context lock is held.
int wg_encap_impl(bnk_ctx *ctx, const bnk_batch *slots, uint32_t mtu, uint32_t *wire_len, const int64_t *note_now);
int wg_decap_impl(bnk_ctx *ctx, const bnk_batch *wire, const bnk_batch *out, uint8_t *result, uint32_t *out_len,
                  uint32_t *peer, uint64_t *counter, const int64_t *check_now);

// The file-scope device scratch of the entry point that allocates nothing
// (noalloc_api.hip): looks up its address on `device` (which must be current).
int noalloc_setup(bnk_ctx *ctx, int device);
// Drops a context that is being shut down from the record of who used the scratch last.
void noalloc_forget(bnk_ctx *ctx);

// What a small-batch route returns in deferred mode (bnk_ctx::defer) instead of BNK_OK:
// its work is enqueued, its results are not there yet.  Never crosses the C ABI.
constexpr int BNK_DEFERRED = 2;

// Waits for everything enqueued on the context stream so far.
int wait_stream(bnk_ctx *ctx);
// The same in two steps, for a caller that gives up the context lock in between:
// post_ticket enqueues the one-thread launch that ends the work so far and
// returns its number; wait_ticket waits for that number (or a later one).
int post_ticket(bnk_ctx *ctx, uint32_t *ticket);
int wait_ticket(bnk_ctx *ctx, uint32_t ticket);
// The end of a small-batch route whose kernels wrote their results to pinned
// staging: waits for the stream (reading the status words when with_status),
// then copies the results out -- or, when the context is in deferred mode,
// only notes the copies for whoever waits later.
int finish_direct(bnk_ctx *ctx, bool with_status, std::initializer_list<Deferred> copies);
// Reads and clears the device status word (waits for the stream; after_kernel: through
// wait_stream, for a call whose last enqueued operation is a kernel).
int take_status(bnk_ctx *ctx, uint32_t *status, bool after_kernel = false);
// Reads and clears the status words (the stream must have been waited for).
uint32_t read_status_words(bnk_ctx *ctx);
// Maps status bits to an error code (BNK_OK when clear).
int status_to_rc(bnk_ctx *ctx, uint32_t status);

} // namespace bnk
