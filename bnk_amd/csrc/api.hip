// C ABI of libbnkhip.so (see include/bnkhip.h): argument checking, staging of
// host batches through the context's device buffers, kernel launches.
#include "api_common.hpp"

#include <atomic>
#include <chrono>
#include "filter_host.hpp"

using namespace bnk;

namespace {

// Chunked form of a host seal/open batch (see HostPipe).  Returns 1 when the
// batch does not qualify and the caller should take the single-shot route.
int aead_batch_host_chunked(bnk_ctx *ctx, bool open, const bnk_batch *in, const bnk_batch *out,
                            uint8_t *verdict, AeadArgs a)
{
    const uint32_t n = in->n;
    const int out_delta = open ? -16 : 16;
    HostPipe hp;
    hp.ctx = ctx;
    hp.in = in;
    hp.out = out;
    hp.in_ext = [in](uint32_t i) { return (uint64_t)(in->lens ? in->lens[i] : in->len); };
    hp.out_ext = [in, out_delta](uint32_t i) {
        return (uint64_t)std::max<int64_t>((int64_t)(in->lens ? in->lens[i] : in->len) + out_delta, 0);
    };
    int rc = hp.plan(in->lens ? 0 : hp.out_ext(0));
    if (rc) return rc;
    rc = check_index_range(ctx, in->peer, n, a.n_peers, "peer index", "the key table");
    if (rc) return rc;
    if (open) {
        HIPCHK(ctx, ctx->verdict.reserve(n));
        a.verdict = ctx->verdict.as<uint8_t>();
        hp.add_result(verdict, a.verdict, 1);
    }
    rc = hp.begin();
    if (rc) return rc;
    // per-packet arrays go up whole, ahead of everything, on the compute stream
    auto up = [&](DevBuf *dst, const void *src, size_t bytes) -> hipError_t {
        hipError_t e = dst->reserve(bytes);
        if (e != hipSuccess) return e;
        return hipMemcpyAsync(dst->p, src, bytes, hipMemcpyHostToDevice, ctx->stream);
    };
    if (in->lens) {
        HIPCHK(ctx, up(&ctx->lens, in->lens, (size_t)n * 4));
        a.lens = ctx->lens.as<uint32_t>();
        HIPCHK(ctx, ctx->order.reserve((size_t)n * 4));
        HIPCHK(ctx, ctx->hist.reserve(LEN_BINS * 4));
        HIPCHK(ctx, ctx->cursor.reserve(LEN_CURSOR_WORDS * 4));
    }
    if (in->peer) {
        HIPCHK(ctx, up(&ctx->peer, in->peer, (size_t)n * 4));
        a.peer = ctx->peer.as<uint32_t>();
    }
    if (in->counters) {
        HIPCHK(ctx, up(&ctx->counters, in->counters, (size_t)n * 8));
        a.counters = ctx->counters.as<uint64_t>();
    }
    a.in = hp.d_in;
    a.out = hp.d_out;
    a.in_off = hp.d_in_off;
    a.out_off = hp.d_out_off;
    rc = hp.open_gate();
    if (rc) return rc;
    for (uint32_t k = 0; k < hp.chunks; k++) {
        uint32_t lo, hi;
        if (!hp.range(k, &lo, &hi)) break;
        rc = hp.upload(k);
        if (rc) return rc;
        AeadArgs c = a;
        c.first = lo;
        c.n = hi - lo;
        if (a.lens && c.n > 64) {
            HIPCHK(ctx, launch_length_sort(a.lens + lo, c.n, open ? 16 : 0, ctx->order.as<uint32_t>() + lo,
                                           ctx->hist.as<uint32_t>(), ctx->cursor.as<uint32_t>(), ctx->stream));
            c.order = ctx->order.as<uint32_t>() + lo;
        }
        HIPCHK(ctx, open ? launch_aead_open(c, ctx->stream) : launch_aead_seal(c, ctx->stream));
        rc = hp.download(k);
        if (rc) return rc;
    }
    rc = hp.finish();
    if (rc) return rc;
    uint32_t status = 0;
    rc = take_status(ctx, &status);
    if (rc) return rc;
    return status_to_rc(ctx, status);
}

// Small batches whose arenas lie in the context's pinned rings: kernels read
// and write the rings over the link themselves and the per-packet arrays sit
// in pinned staging, so a call is host bookkeeping, two launches and one wait,
// with no copy-engine transfer.  Returns 1 when the batch does not qualify.
int aead_batch_host_direct(bnk_ctx *ctx, bool open, const bnk_batch *in, const bnk_batch *out,
                           uint8_t *verdict, AeadArgs a)
{
    const uint32_t n = in->n;
    if (n > DIRECT_MAX_PACKETS) return 1;
    uint8_t *d_in = ring_device_ptr(ctx, in->base, in->bytes);
    uint8_t *d_out = ring_device_ptr(ctx, out->base, out->bytes);
    if (!d_in || !d_out) return 1;
    Span sin, sout;
    int rc = scan_host_layout(ctx, in, in, 0, &sin, "in");
    if (rc) return rc;
    rc = scan_host_layout(ctx, out, in, open ? -16 : 16, &sout, "out");
    if (rc) return rc;
    // A launch of a wave per packet reads every packet where it lies, so only the
    // packets' own bytes count; a lane per packet first fetches the whole span.
    a.lens = in->lens; // (for aead_runs_spread only whether there is one matters; set properly below)
    const uint64_t moved = aead_runs_spread(a) ? host_payload_bytes(in) : sin.size();
    if (moved > DIRECT_MAX_BYTES) return 1;
    rc = check_index_range(ctx, in->peer, n, a.n_peers, "peer index", "the key table");
    if (rc) return rc;

    // pinned staging: three 8-byte arrays, three 4-byte arrays, verdict bytes
    PinBuf &stage = *ctx->pin_cur;
    HIPCHK(ctx, stage.reserve((size_t)n * 37 + 64));
    uint8_t *pin = stage.as<uint8_t>();
    uint64_t *p_in_off = (uint64_t *)pin, *p_out_off = p_in_off + n, *p_ctr = p_out_off + n;
    uint32_t *p_lens = (uint32_t *)(p_ctr + n), *p_peer = p_lens + n, *p_order = p_peer + n;
    uint8_t *p_verdict = (uint8_t *)(p_order + n);
    // A wave per packet loads each byte once, all loads in flight together, so
    // it reads the ring itself.  A lane per packet walks its packet line by
    // line, a round trip over the link each: for it the span is first fetched
    // into device memory by one wide copy kernel, at the same position within a
    // 128-byte line so that whole lines can be moved.  Either way the output
    // goes straight into the ring, where stores need no round trip.
    a.lens = in->lens ? stage.dev(p_lens) : nullptr;
    if (aead_runs_spread(a)) {
        a.in = d_in + sin.lo;
    } else {
        const uint32_t mis = (uint32_t)((uintptr_t)(d_in + sin.lo) & 127u);
        HIPCHK(ctx, ctx->in_arena.reserve(sin.size() + 160));
        HIPCHK(ctx, launch_pull(d_in + sin.lo, ctx->in_arena.as<uint8_t>() + mis, sin.size(), ctx->stream));
        a.in = ctx->in_arena.as<uint8_t>() + mis;
    }
    a.out = d_out;
    if (in->offsets) {
        for (uint32_t i = 0; i < n; i++) p_in_off[i] = in->offsets[i] - sin.lo;
        a.in_off = stage.dev(p_in_off);
    }
    if (out->offsets) { memcpy(p_out_off, out->offsets, (size_t)n * 8); a.out_off = stage.dev(p_out_off); }
    if (in->counters) { memcpy(p_ctr, in->counters, (size_t)n * 8); a.counters = stage.dev(p_ctr); }
    if (in->peer) { memcpy(p_peer, in->peer, (size_t)n * 4); a.peer = stage.dev(p_peer); }
    if (in->lens) {
        memcpy(p_lens, in->lens, (size_t)n * 4);
        a.lens = stage.dev(p_lens);
        if (n > 64 && !aead_runs_spread(a)) {
            // lanes of a wave should run equal block counts: longest first
            const uint32_t tag = open ? 16 : 0;
            auto blocks = [&](uint32_t i) {
                const uint32_t len = in->lens[i];
                return ((len >= tag ? len - tag : 0u) + 63u) >> 6;
            };
            uint32_t most = 0;
            for (uint32_t i = 0; i < n; i++) most = std::max(most, blocks(i));
            if (most <= 65535) {
                std::vector<uint32_t> at(most + 2, 0);
                for (uint32_t i = 0; i < n; i++) at[most - blocks(i) + 1]++;
                for (uint32_t b = 0; b <= most; b++) at[b + 1] += at[b];
                for (uint32_t i = 0; i < n; i++) p_order[at[most - blocks(i)]++] = i;
                a.order = stage.dev(p_order);
            }
        }
    }
    if (open) a.verdict = stage.dev(p_verdict);
    HIPCHK(ctx, open ? launch_aead_open(a, ctx->stream) : launch_aead_seal(a, ctx->stream));
    // host batches have had their peer indices checked above, so the kernel
    // has nothing to report through the status word
    return finish_direct(ctx, false, {{verdict, p_verdict, open ? (size_t)n : 0}});
}

// Device batches cannot be walked on the host; check what is uniform.
int aead_device_layout_check(bnk_ctx *ctx, bool open, const bnk_batch *in, const bnk_batch *out)
{
    const uint32_t n = in->n;
    if (in->bytes == 0 || out->bytes == 0) return fail(ctx, BNK_E_INVAL, "arena size 0");
    if (!in->offsets && !in->lens && ((uint64_t)(n - 1) * in->stride + in->len > in->bytes))
        return fail(ctx, BNK_E_INVAL, "in: uniform layout exceeds the arena");
    if (!out->offsets && !in->lens) {
        const int64_t ol = (int64_t)in->len + (open ? -16 : 16);
        if ((uint64_t)(n - 1) * out->stride + (uint64_t)std::max<int64_t>(ol, 0) > out->bytes)
            return fail(ctx, BNK_E_INVAL, "out: uniform layout exceeds the arena");
    }
    return BNK_OK;
}

} // namespace

namespace bnk {

// sort_scratch: null, or device memory of LEN_BINS + LEN_CURSOR_WORDS + n words for the
// length grouping of a device-resident batch (then nothing is allocated); its
// first LEN_BINS words must be zeros on the first call and are zeros again
// after every call.
int aead_batch(bnk_ctx *ctx, bool open, const bnk_batch *in, const bnk_batch *out,
               uint8_t *verdict, uint32_t *sort_scratch)
{
    int rc = check_batch_common(ctx, in, "in");
    if (rc) return rc;
    rc = check_batch_common(ctx, out, "out");
    if (rc) return rc;
    if (in->mem != out->mem) return fail(ctx, BNK_E_INVAL, "in and out must use the same mem kind");
    const uint32_t n = in->n;
    if (n == 0) return BNK_OK;
    if (open && !verdict) return fail(ctx, BNK_E_INVAL, "null verdict array");
    const int which = open ? BNK_KEYS_RECV : BNK_KEYS_SEND;
    if (!ctx->d_keys[which] || ctx->n_keys[which] == 0)
        return fail(ctx, BNK_E_STATE, open ? "no receive keys loaded" : "no send keys loaded");
    if (!in->peer && ctx->n_keys[which] < 1) return fail(ctx, BNK_E_RANGE, "empty key table");

    AeadArgs a{};

    a.spread_max = ctx->spread_max;
    a.keys = ctx->d_keys[which];
    a.n_peers = ctx->n_keys[which];
    a.status = ctx->d_status;
    a.counter0 = in->counter0;
    a.n = n;
    a.in_stride = in->stride;
    a.out_stride = out->stride;
    a.len = in->len;

    if (in->mem == BNK_MEM_DEVICE) {
        rc = aead_device_layout_check(ctx, open, in, out);
        if (rc) return rc;
        a.in = (const uint8_t *)in->base;
        a.out = (uint8_t *)out->base;
        a.in_off = in->offsets;
        a.out_off = out->offsets;
        a.lens = in->lens;
        a.peer = in->peer;
        a.counters = in->counters;
        a.verdict = verdict;
        // offsets and lengths in device memory cannot be checked here: the lanes do it
        if (in->offsets || in->lens || out->offsets) {
            a.in_limit = in->bytes;
            a.out_limit = out->bytes;
        }
        if (sort_scratch) {
            // the caller's scratch instead of the context's grow-only buffers
            a.order = nullptr;
            if (a.lens && n > 64 && !aead_runs_spread(a)) {
                // the histogram keeps its place from call to call: it is left all zeros by each grouping
                uint32_t *hist = sort_scratch, *cursor = hist + LEN_BINS, *order = cursor + LEN_CURSOR_WORDS;
                HIPCHK(ctx, launch_length_sort(a.lens, n, open ? 16 : 0, order, hist, cursor, ctx->stream));
                a.order = order;
            }
        } else {
            rc = maybe_sort(ctx, &a, open ? 16 : 0);
            if (rc) return rc;
        }
        // the verdicts are counted by the launch itself where a lane has a packet, else by a
        // launch behind it
        const bool count = open && ctx->tally_on.load(std::memory_order_relaxed);
        if (count && !aead_runs_spread(a)) a.tally = reinterpret_cast<unsigned long long *>(ctx->d_tally);
        HIPCHK(ctx, open ? launch_aead_open(a, ctx->stream) : launch_aead_seal(a, ctx->stream));
        if (count && !a.tally) return tally_results(ctx, TALLY_OPEN, verdict, n, BNK_MEM_DEVICE);
        return BNK_OK;
    }
    if (sort_scratch) return fail(ctx, BNK_E_INVAL, "this entry point takes device-resident batches only");

    rc = aead_batch_host_direct(ctx, open, in, out, verdict, a);
    if (rc != 1) return rc;
    rc = aead_batch_host_chunked(ctx, open, in, out, verdict, a);
    if (rc != 1) return rc;
    Staged st;
    rc = stage_host(ctx, in, out, open ? -16 : 16, ctx->n_keys[which], &st);
    if (rc) return rc;
    a.in = st.d_in;
    a.out = st.d_out;
    a.in_off = st.d_in_off;
    a.out_off = st.d_out_off;
    a.lens = st.d_lens;
    a.peer = st.d_peer;
    a.counters = st.d_counters;
    if (open) {
        HIPCHK(ctx, ctx->verdict.reserve(n));
        a.verdict = ctx->verdict.as<uint8_t>();
    }
    rc = maybe_sort(ctx, &a, open ? 16 : 0);
    if (rc) return rc;
    HIPCHK(ctx, open ? launch_aead_open(a, ctx->stream) : launch_aead_seal(a, ctx->stream));
    HIPCHK(ctx, hipMemcpyAsync((uint8_t *)out->base + st.sout.lo, st.d_out, st.sout.size(),
                               hipMemcpyDeviceToHost, ctx->stream));
    uint8_t *h_verdict = ctx->pin.as<uint8_t>() + (size_t)n * 16 + 64;
    if (open)
        HIPCHK(ctx, hipMemcpyAsync(h_verdict, a.verdict, n, hipMemcpyDeviceToHost, ctx->stream));
    // stage_host has checked the peer indices, so the kernel has nothing to
    // report through the status word: waiting is enough
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    if (open) memcpy(verdict, h_verdict, n);
    return BNK_OK;
}

// Waits for everything enqueued on the context stream so far.  After a short kernel
// hipStreamSynchronize returns 13 us after the launch; a one-thread launch behind the
// work that writes this wait's number into pinned memory, with the host watching that
// word, is seen after 9.6 us.  Why the results are there when the word is: the stream
// runs its kernels one after the other, so the earlier kernels (which wrote verdicts,
// lengths and status words to pinned host memory) have ended, and their stores have
// been released at system scope, before done_word_kernel starts; that kernel fences and
// stores the word with release semantics at system scope; the host reads it with an
// acquire fence before it touches the results.  The watch is bounded: whatever takes
// longer than WAIT_WATCH_US is waited for the ordinary way.  A launch that failed is
// reported by hipGetLastError on either path; a fault inside a kernel ends the process
// on this runtime whichever way the host waits.  BNK_WAIT_SYNC=1 in the environment at
// bnk_init switches the watch off (every wait is hipStreamSynchronize).
constexpr int64_t WAIT_WATCH_US = 100;
int post_ticket(bnk_ctx *ctx, uint32_t *ticket)
{
    const uint32_t seq = ++ctx->wait_seq;
    *ticket = seq;
    HIPCHK(ctx, launch_done_word(ctx->d_status + STATUS_DONE_WORD, seq, ctx->stream));
    return BNK_OK;
}

// May be called without the context lock: it reads the watched word and, past
// the watch, waits for the stream as a whole (which then includes whatever
// other callers have enqueued behind the ticket).
int wait_ticket(bnk_ctx *ctx, uint32_t ticket)
{
    if (!ctx->wait_sync_only) {
        volatile uint32_t *done = ctx->h_status + STATUS_DONE_WORD;
        const auto t0 = std::chrono::steady_clock::now();
        for (;;) {
            for (int spin = 0; spin < 64; spin++) {
                // (numbers are handed out in stream order: a later one also means done)
                if ((int32_t)(*done - ticket) >= 0) {
                    std::atomic_thread_fence(std::memory_order_acquire);
                    HIPCHK(ctx, hipGetLastError());
                    return BNK_OK;
                }
                __builtin_ia32_pause();
            }
            if (std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count() >
                WAIT_WATCH_US)
                break;
        }
    }
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return BNK_OK;
}

int wait_stream(bnk_ctx *ctx)
{
    uint32_t ticket;
    if (ctx->wait_sync_only || post_ticket(ctx, &ticket) != BNK_OK) {
        HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
        return BNK_OK;
    }
    return wait_ticket(ctx, ticket);
}

int finish_direct(bnk_ctx *ctx, bool with_status, std::initializer_list<Deferred> copies)
{
    if (ctx->defer) {
        for (const Deferred &c : copies)
            if (c.bytes) ctx->defer->push_back(c);
        ctx->defer_status = with_status;
        return BNK_DEFERRED;
    }
    uint32_t status = 0;
    if (with_status) {
        if (int rc = take_status(ctx, &status, true)) return rc;
    } else {
        if (int rc = wait_stream(ctx)) return rc;
    }
    for (const Deferred &c : copies)
        if (c.bytes) memcpy(c.dst, c.src, c.bytes);
    return status_to_rc(ctx, status);
}

// Waits for the stream, then reads and clears the status words.  after_kernel: the
// last thing enqueued is a kernel (behind a copy the watched word comes later than the
// copy's own completion does).
int take_status(bnk_ctx *ctx, uint32_t *status, bool after_kernel)
{
    if (after_kernel) {
        if (int rc = wait_stream(ctx)) return rc;
    } else {
        HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    }
    *status = read_status_words(ctx);
    return BNK_OK;
}

uint32_t read_status_words(bnk_ctx *ctx)
{
    volatile uint32_t *h = ctx->h_status;
    const uint32_t status = (h[STATUS_PEER_RANGE] ? STATUS_PEER_RANGE : 0u) |
                            (h[STATUS_FLOWS_FULL] ? STATUS_FLOWS_FULL : 0u) | (h[STATUS_BOUNDS] ? STATUS_BOUNDS : 0u) |
                            (h[STATUS_INTERNAL] ? STATUS_INTERNAL : 0u);
    if (status) {
        h[STATUS_PEER_RANGE] = 0;
        h[STATUS_FLOWS_FULL] = 0;
        h[STATUS_BOUNDS] = 0;
        h[STATUS_INTERNAL] = 0;
    }
    return status;
}

int status_to_rc(bnk_ctx *ctx, uint32_t status)
{
    if (status & STATUS_INTERNAL)
        return fail(ctx, BNK_E_HIP, "a launch for short packets met a packet it does not handle (packets were skipped)");
    if (status & STATUS_BOUNDS)
        return fail(ctx, BNK_E_INVAL, "a packet of a device-resident batch reaches beyond its arena (it was skipped)");
    if (status & STATUS_PEER_RANGE) return fail(ctx, BNK_E_RANGE, "peer index beyond the key table");
    if (status & STATUS_FLOWS_FULL) return fail(ctx, BNK_E_NOMEM, "flow table overflow");
    return BNK_OK;
}

} // namespace bnk

extern "C" {

int bnk_init(int device_ordinal, bnk_ctx **out)
{
    BNK_API_TRY
    if (!out) return fail(nullptr, BNK_E_INVAL, "null out pointer");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(nullptr, BNK_E_NODEV, std::string("no HIP device: ") +
                                              (e != hipSuccess ? hipGetErrorString(e) : "count is 0"));
    if (device_ordinal < 0 || device_ordinal >= count)
        return fail(nullptr, BNK_E_NODEV, "device ordinal out of range");
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device_ordinal);
    if (e != hipSuccess) return fail_hip(nullptr, "hipGetDeviceProperties", e);
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(nullptr, BNK_E_NODEV,
                    std::string("device is ") + prop.gcnArchName + ", this library is built for gfx950");
    bnk_ctx *ctx = new (std::nothrow) bnk_ctx;
    if (!ctx) return fail(nullptr, BNK_E_NOMEM, "out of host memory");
    ctx->device = device_ordinal;
    auto bail = [&](const char *what, hipError_t err) {
        int rc = fail_hip(nullptr, what, err);
        ctx->alive = true;
        bnk_shutdown(ctx);
        return rc;
    };
    if ((e = hipSetDevice(device_ordinal)) != hipSuccess) return bail("hipSetDevice", e);
    if ((e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking)) != hipSuccess)
        return bail("hipStreamCreate", e);
    if ((e = hipEventCreate(&ctx->ev0)) != hipSuccess) return bail("hipEventCreate", e);
    if ((e = hipEventCreate(&ctx->ev1)) != hipSuccess) return bail("hipEventCreate", e);
    for (auto &t : ctx->tally_host) t.store(0, std::memory_order_relaxed);
    if ((e = hipMalloc((void **)&ctx->d_tally, TALLY_SLOTS * TALLY_LANES * 8)) != hipSuccess)
        return bail("hipMalloc", e);
    if ((e = hipMemset(ctx->d_tally, 0, TALLY_SLOTS * TALLY_LANES * 8)) != hipSuccess) return bail("hipMemset", e);
    if ((e = hipEventCreateWithFlags(&ctx->ev_noalloc, hipEventDisableTiming)) != hipSuccess)
        return bail("hipEventCreate", e);
    if ((e = hipHostMalloc((void **)&ctx->h_status, 64, hipHostMallocDefault)) != hipSuccess)
        return bail("hipHostMalloc", e);
    memset(ctx->h_status, 0, 64);
    if (const char *ws = getenv("BNK_WAIT_SYNC")) ctx->wait_sync_only = ws[0] != '\0' && ws[0] != '0';
    if ((e = hipHostGetDevicePointer((void **)&ctx->d_status, ctx->h_status, 0)) != hipSuccess)
        return bail("hipHostGetDevicePointer", e);
    // the length grouping's histogram starts out cleared and every grouping
    // leaves it cleared
    if ((e = ctx->hist.reserve(LEN_BINS * 4)) != hipSuccess) return bail("hipMalloc", e);
    if ((e = ctx->cursor.reserve(LEN_CURSOR_WORDS * 4)) != hipSuccess) return bail("hipMalloc", e);
    if ((e = hipMemsetAsync(ctx->hist.p, 0, LEN_BINS * 4, ctx->stream)) != hipSuccess) return bail("hipMemsetAsync", e);
    if (int rc = noalloc_setup(nullptr, device_ordinal)) {
        ctx->alive = true;
        bnk_shutdown(ctx);
        return rc;
    }
    ctx->filter = filter_create(ctx->stream, prop.multiProcessorCount);
    if (!ctx->filter) return bail("filter state", hipErrorOutOfMemory);
    if ((e = hipStreamSynchronize(ctx->stream)) != hipSuccess) return bail("hipStreamSynchronize", e);
    ctx->alive = true;
    *out = ctx;
    return BNK_OK;
    BNK_API_CATCH(nullptr)
}

void bnk_shutdown(bnk_ctx *ctx)
{
    try {
    if (!ctx) return;
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        if (!ctx->alive) return;
        ctx->alive = false;
        (void)hipSetDevice(ctx->device);
        if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
        noalloc_forget(ctx);
        for (DevBuf *b : {&ctx->in_arena, &ctx->out_arena, &ctx->off_in, &ctx->off_out, &ctx->lens,
                          &ctx->peer, &ctx->counters, &ctx->verdict, &ctx->order, &ctx->hist,
                          &ctx->cursor, &ctx->misc, &ctx->r_plain, &ctx->r_auth, &ctx->r_pass,
                          &ctx->r_keys, &ctx->r_idx, &ctx->r_skeys, &ctx->r_sidx, &ctx->r_tmp,
                          &ctx->r_peer_out, &ctx->r_ctr_base, &ctx->r_ctr_out, &ctx->r_verdict,
                          &ctx->wg_index, &ctx->wg_remote, &ctx->wg_allowed, &ctx->wg_send_ctr,
                          &ctx->wg_peer, &ctx->wg_counter, &ctx->wg_ctlen, &ctx->wg_result,
                          &ctx->wg_outlen, &ctx->wg_padded, &ctx->wg_wirelen, &ctx->wg_skip, &ctx->wg_sctr,
                          &ctx->wg_sval, &ctx->wg_pmax, &ctx->wg_lastb, &ctx->wg_rtable, &ctx->wg_rflags,
                          &ctx->r_heads, &ctx->wg_hash})
            b->release();
        ctx->pin.release();
        for (HostStage &st : ctx->stages) st.pin.release();
        if (ctx->wg_replay) (void)hipFree(ctx->wg_replay);
        if (ctx->d_tally) (void)hipFree(ctx->d_tally);
        for (const bnk_ctx::Ring &r : ctx->rings) (void)hipHostFree(reinterpret_cast<void *>(r.host));
        ctx->rings.clear();
        for (int w = 0; w < 2; w++)
            if (ctx->d_keys[w]) (void)hipFree(ctx->d_keys[w]);
        if (ctx->h_status) (void)hipHostFree(ctx->h_status);
        if (ctx->filter) filter_destroy(ctx->filter);
        for (hipEvent_t e : ctx->ev_up) (void)hipEventDestroy(e);
        for (hipEvent_t e : ctx->ev_done) (void)hipEventDestroy(e);
        if (ctx->s_up) (void)hipStreamDestroy(ctx->s_up);
        if (ctx->s_down) (void)hipStreamDestroy(ctx->s_down);
        if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
        if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
        if (ctx->ev_noalloc) (void)hipEventDestroy(ctx->ev_noalloc);
        if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    }
    delete ctx;
    } catch (...) {
    }
}

const char *bnk_last_error(bnk_ctx *ctx)
{
    // a copy of the caller's own: another thread may fail on the same context
    // while this one reads
    static thread_local std::string copy;
    try {
        if (ctx) {
            std::lock_guard<std::mutex> lk(ctx->err_mu);
            copy = ctx->err;
        } else {
            copy = g_init_err;
        }
    } catch (...) {
        return "out of host memory";
    }
    return copy.c_str();
}

int bnk_ring_alloc(bnk_ctx *ctx, size_t bytes, void **host_pinned)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!host_pinned || bytes == 0) return fail(ctx, BNK_E_INVAL, "bad ring request");
    HIPCHK(ctx, hipHostMalloc(host_pinned, bytes, hipHostMallocDefault));
    void *dev = nullptr;
    if (hipHostGetDevicePointer(&dev, *host_pinned, 0) != hipSuccess) {
        dev = nullptr; // the ring still works through the copying routes
        (void)hipGetLastError();
    }
    try {
        std::lock_guard<std::mutex> rl(ctx->rings_mu);
        ctx->rings.push_back({(uintptr_t)*host_pinned, (uint8_t *)dev, bytes});
    } catch (...) {
        (void)hipHostFree(*host_pinned);
        *host_pinned = nullptr;
        throw;
    }
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_ring_free(bnk_ctx *ctx, void *host_pinned)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!host_pinned) return BNK_OK;
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    {
        std::lock_guard<std::mutex> rl(ctx->rings_mu);
        for (size_t i = 0; i < ctx->rings.size(); i++)
            if (ctx->rings[i].host == (uintptr_t)host_pinned) {
                ctx->rings.erase(ctx->rings.begin() + i);
                break;
            }
    }
    HIPCHK(ctx, hipHostFree(host_pinned));
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_set_spread_max_packets(bnk_ctx *ctx, uint32_t max_packets)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    ctx->spread_max = max_packets;
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_dev_alloc(bnk_ctx *ctx, size_t bytes, void **dev)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!dev || bytes == 0) return fail(ctx, BNK_E_INVAL, "bad device allocation request");
    HIPCHK(ctx, hipMalloc(dev, bytes));
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_dev_free(bnk_ctx *ctx, void *dev)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!dev) return BNK_OK;
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipFree(dev));
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_copy_to_device(bnk_ctx *ctx, void *dev, const void *host, size_t bytes)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (bytes == 0) return BNK_OK;
    if (!dev || !host) return fail(ctx, BNK_E_INVAL, "null pointer");
    HIPCHK(ctx, hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_copy_to_host(bnk_ctx *ctx, void *host, const void *dev, size_t bytes)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (bytes == 0) return BNK_OK;
    if (!dev || !host) return fail(ctx, BNK_E_INVAL, "null pointer");
    HIPCHK(ctx, hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_sync(bnk_ctx *ctx)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    uint32_t status = 0;
    int rc = take_status(ctx, &status);
    if (rc) return rc;
    return status_to_rc(ctx, status);
    BNK_API_CATCH(ctx)
}

void *bnk_stream(bnk_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int bnk_keys_set(bnk_ctx *ctx, int which, const uint8_t *keys32, uint32_t n_peers)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (which != BNK_KEYS_SEND && which != BNK_KEYS_RECV)
        return fail(ctx, BNK_E_INVAL, "bad key table selector");
    if (!keys32 || n_peers == 0) return fail(ctx, BNK_E_INVAL, "empty key table");
    // in-flight work may still read the old table
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    uint32_t *nk = nullptr;
    HIPCHK(ctx, hipMalloc((void **)&nk, (size_t)n_peers * 32));
    hipError_t e = hipMemcpyAsync(nk, keys32, (size_t)n_peers * 32, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(nk);
        return fail_hip(ctx, "key upload", e);
    }
    if (ctx->d_keys[which]) (void)hipFree(ctx->d_keys[which]);
    ctx->d_keys[which] = nk;
    ctx->n_keys[which] = n_peers;
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_aead_seal_batch(bnk_ctx *ctx, const bnk_batch *in, const bnk_batch *out)
{
    BNK_API_TRY
    {
        CoRequest rq{CO_SEAL, in, out, 0, 0, nullptr, nullptr, nullptr, nullptr};
        int crc;
        if (out && coalesce_submit(ctx, rq, &crc)) {
            if (crc == BNK_OK) tally_add(ctx, TALLY_SEALED, in->n);
            return crc;
        }
    }
    Guard g(ctx);
    if (g.rc) return g.rc;
    const int rc = aead_batch(ctx, false, in, out, nullptr, nullptr);
    if (rc == BNK_OK) tally_add(ctx, TALLY_SEALED, in->n);
    return rc;
    BNK_API_CATCH(ctx)
}

int bnk_aead_open_batch(bnk_ctx *ctx, const bnk_batch *in, const bnk_batch *out, uint8_t *verdict)
{
    BNK_API_TRY
    {
        CoRequest rq{CO_OPEN, in, out, 0, 0, verdict, nullptr, nullptr, nullptr};
        int crc;
        if (out && coalesce_submit(ctx, rq, &crc)) {
            if (crc == BNK_OK) (void)tally_results(ctx, TALLY_OPEN, verdict, in->n, BNK_MEM_HOST);
            return crc;
        }
    }
    Guard g(ctx);
    if (g.rc) return g.rc;
    const int rc = aead_batch(ctx, true, in, out, verdict, nullptr);
    // (a device-resident batch has been counted on the device)
    if (rc == BNK_OK && in->mem == BNK_MEM_HOST) return tally_results(ctx, TALLY_OPEN, verdict, in->n, BNK_MEM_HOST);
    return rc;
    BNK_API_CATCH(ctx)
}

} // extern "C"
