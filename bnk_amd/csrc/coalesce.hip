// Merging of small host calls (see coalesce.hpp): joining a window, leading
// one, running its merged batch through the same routines a direct call uses.
#include "api_common.hpp"

using namespace bnk;

namespace {

using Clock = std::chrono::steady_clock;

inline int64_t us_since(Clock::time_point t0)
{
    return std::chrono::duration_cast<std::chrono::microseconds>(Clock::now() - t0).count();
}

// How long a caller watches for its window's end before it sleeps.  A window of
// two thousand packets in pinned rings takes about 100 us.
constexpr int64_t FOLLOWER_SPIN_US = 200;
constexpr uint32_t MAX_IN_FLIGHT = 2;

// Bytes packet i of a call occupies from its offset in the arena it is read
// from (ext_a) and in the one it is written to (ext_b).
inline void extents(CoKind kind, uint32_t len, uint32_t mtu, uint64_t *ext_a, uint64_t *ext_b)
{
    switch (kind) {
    case CO_SEAL:
        *ext_a = len;
        *ext_b = (uint64_t)len + 16u;
        break;
    case CO_OPEN:
        *ext_a = len;
        *ext_b = len >= 16u ? len - 16u : 0u;
        break;
    case CO_ENCAP:
    case CO_NOTE_ENCAP:
        *ext_a = *ext_b = 16ull + len + wg_padding(len, mtu) + 16ull;
        break;
    default: // decapsulation: 32 bytes of a datagram are header and tag
        *ext_a = len;
        *ext_b = len >= 32u ? len - 32u : 0u;
        break;
    }
}

struct RingRef {
    uintptr_t host = 0;
    uint64_t bytes = 0;
};

// The pinned ring an arena lies in (host address and size), if any.
bool find_ring(bnk_ctx *ctx, const void *base, uint64_t bytes, RingRef *out)
{
    const uintptr_t a = (uintptr_t)base;
    std::lock_guard<std::mutex> lk(ctx->rings_mu);
    for (const bnk_ctx::Ring &r : ctx->rings)
        if (r.dev && a >= r.host && bytes <= r.bytes && a - r.host <= r.bytes - bytes) {
            out->host = r.host;
            out->bytes = r.bytes;
            return true;
        }
    return false;
}

int run_window(bnk_ctx *ctx, CoWindow &w)
{
    const uint32_t n = w.n.load(std::memory_order_relaxed);
    bnk_batch A{}, B{};
    A.base = reinterpret_cast<void *>(w.ring_a_host);
    A.bytes = w.ring_a_bytes;
    A.n = n;
    A.mem = BNK_MEM_HOST;
    A.offsets = w.off_a.data();
    if (w.same_len) A.len = w.len0;
    else A.lens = w.lens.data();
    if (w.any_peer) A.peer = w.peer.data();
    B.base = reinterpret_cast<void *>(w.ring_b_host);
    B.bytes = w.ring_b_bytes;
    B.n = n;
    B.mem = BNK_MEM_HOST;
    B.offsets = w.in_place ? w.off_a.data() : w.off_b.data();
    switch (w.kind) {
    case CO_SEAL:
        A.counters = w.counters.data();
        return aead_batch(ctx, false, &A, &B, nullptr, nullptr);
    case CO_OPEN:
        A.counters = w.counters.data();
        w.r8.resize(n);
        return aead_batch(ctx, true, &A, &B, w.r8.data(), nullptr);
    case CO_ENCAP:
    case CO_NOTE_ENCAP:
        w.r32a.resize(n);
        return wg_encap_impl(ctx, &A, w.mtu, w.r32a.data(), w.kind == CO_NOTE_ENCAP ? &w.now : nullptr);
    default:
        w.r8.resize(n);
        w.r32a.resize(n);
        w.r32b.resize(n);
        w.r64.resize(n);
        return wg_decap_impl(ctx, &A, &B, w.r8.data(), w.r32a.data(), w.r32b.data(), w.r64.data(),
                             w.kind == CO_DECAP_FILTER ? &w.now : nullptr);
    }
}

// The first caller of a window: waits for company, then for the context, closes
// the window and runs it.
void lead(bnk_ctx *ctx, const std::shared_ptr<CoWindow> &w, uint32_t expected, uint32_t max_packets)
{
    Coalescer &co = ctx->co;
    const int64_t max_wait = co.max_wait_us.load(std::memory_order_relaxed);
    bool timed_out = false;
    const Clock::time_point t0 = Clock::now();
    Clock::time_point t_locked = t0, t_enqueued = t0;
    if (max_wait > 0) {
        for (;;) {
            // Company worth waiting for: half of the callers that are inside the library
            // right now, so that two windows share them and one is enqueued while the
            // other runs, but no more than are making this kind of call (a caller
            // alone waits for nobody); and never fewer than the application asked
            // for (bnk_set_coalesce's expect_callers).
            uint32_t all = 0;
            for (const auto &c : co.active) all += c.load(std::memory_order_acquire);
            const uint32_t mine = co.active[w->kind].load(std::memory_order_acquire);
            const uint32_t want = std::max(expected, std::min(mine, (all + 1u) / 2u));
            if (w->callers.load(std::memory_order_acquire) >= want ||
                w->n.load(std::memory_order_acquire) >= max_packets || w->closed.load(std::memory_order_acquire))
                break;
            if (us_since(t0) >= max_wait) {
                timed_out = true;
                break;
            }
            for (int spin = 0; spin < 32; spin++) __builtin_ia32_pause();
        }
    }
    // At most two windows are enqueued or running at a time: one on the GPU, one
    // behind it so that the GPU never waits for the host.  While this one waits for
    // its turn it stays open and fills up.
    while (co.in_flight.load(std::memory_order_acquire) >= MAX_IN_FLIGHT)
        for (int spin = 0; spin < 32; spin++) __builtin_ia32_pause();
    // The window's pinned staging is its own from here until its results have been
    // copied out (by this thread, which may be descheduled for a while after the
    // GPU is done: only this thread gives the stage back).
    HostStage *stage = nullptr;
    while (!stage) {
        for (HostStage &st : ctx->stages) {
            bool expect = false;
            if (st.busy.compare_exchange_strong(expect, true, std::memory_order_acq_rel)) {
                stage = &st;
                break;
            }
        }
        if (!stage)
            for (int spin = 0; spin < 32; spin++) __builtin_ia32_pause();
    }
    int rc;
    bool counted = false, ran = false;
    try {
        std::vector<Deferred> copies;
        uint32_t ticket = 0;
        bool with_status = false;
        {
            // May block while another call holds the context: callers keep joining
            // until the lock is ours.
            Guard g(ctx);
            t_locked = Clock::now();
            {
                std::lock_guard<std::mutex> lk(co.mu);
                if (co.open[w->kind] == w) co.open[w->kind].reset();
                w->closed = true;
                const uint32_t callers = w->callers.load(std::memory_order_relaxed);
                const uint32_t n = w->n.load(std::memory_order_relaxed);
                co.stats.batches++;
                if (timed_out) co.stats.timed_out++;
                if (n > co.stats.largest_batch) co.stats.largest_batch = n;
                if (callers > co.stats.largest_callers) co.stats.largest_callers = callers;
            }
            co.in_flight.fetch_add(1, std::memory_order_acq_rel);
            counted = true;
            rc = g.rc;
            if (!rc) {
                ctx->pin_cur = &stage->pin;
                ctx->defer = &copies;
                ctx->defer_status = false;
                rc = run_window(ctx, *w);
                ctx->pin_cur = &ctx->pin;
                ctx->defer = nullptr;
                with_status = ctx->defer_status;
                ran = rc == BNK_DEFERRED;
                if (rc == BNK_DEFERRED) {
                    // (if the launch behind the work fails, wait for the work the ordinary way)
                    if (post_ticket(ctx, &ticket) != BNK_OK) {
                        const hipError_t e = hipStreamSynchronize(ctx->stream);
                        rc = e == hipSuccess ? BNK_OK : fail_hip(ctx, "hipStreamSynchronize", e);
                        if (!rc) {
                            for (const Deferred &c : copies) memcpy(c.dst, c.src, c.bytes);
                            if (with_status) rc = status_to_rc(ctx, read_status_words(ctx));
                        }
                    }
                }
            }
        }
        t_enqueued = Clock::now();
        // the context is free again: the next window is enqueued while this one runs
        if (rc == BNK_DEFERRED) {
            rc = wait_ticket(ctx, ticket);
            if (!rc) {
                for (const Deferred &c : copies) memcpy(c.dst, c.src, c.bytes);
                if (with_status) rc = status_to_rc(ctx, read_status_words(ctx));
            }
        }
    } catch (const std::bad_alloc &) {
        rc = fail_caught(ctx, BNK_E_NOMEM, "out of host memory");
    } catch (...) {
        rc = fail_caught(ctx, BNK_E_HIP, "unexpected C++ exception inside the library");
    }
    stage->busy.store(false, std::memory_order_release);
    if (counted) co.in_flight.fetch_sub(1, std::memory_order_acq_rel);
    {
        const Clock::time_point t_done = Clock::now();
        auto ns = [](Clock::time_point a, Clock::time_point b) {
            return (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(b - a).count();
        };
        std::lock_guard<std::mutex> lk(co.mu);
        co.stats.gather_ns += ns(t0, t_locked);
        co.stats.enqueue_ns += ns(t_locked, t_enqueued);
        co.stats.wait_ns += ns(t_enqueued, t_done);
    }
    // Refusals that are decided before anything runs and that belong to one caller's
    // arguments (or to the context's state, which every caller should hear about
    // in its own name): everyone makes a call of its own.
    if (!ran && (rc == BNK_E_INVAL || rc == BNK_E_RANGE || rc == BNK_E_STATE)) {
        rc = CO_RETRY;
        std::lock_guard<std::mutex> lk(co.mu);
        co.stats.retried++;
    }
    w->rc = rc;
    w->done.store(1, std::memory_order_release);
    {
        std::lock_guard<std::mutex> lk(w->mu);
    }
    w->cv.notify_all();
}

void follow(CoWindow &w)
{
    const Clock::time_point t0 = Clock::now();
    for (;;) {
        for (int spin = 0; spin < 64; spin++) {
            if (w.done.load(std::memory_order_acquire)) return;
            __builtin_ia32_pause();
        }
        if (us_since(t0) > FOLLOWER_SPIN_US) break;
    }
    std::unique_lock<std::mutex> lk(w.mu);
    w.cv.wait(lk, [&] { return w.done.load(std::memory_order_acquire) != 0; });
}

} // namespace

namespace bnk {

bool coalesce_submit(bnk_ctx *ctx, const CoRequest &rq, int *rc_out)
{
    if (!ctx) return false;
    Coalescer &co = ctx->co;
    const uint32_t max_packets = co.max_packets.load(std::memory_order_relaxed);
    if (max_packets == 0) return false;
    const bnk_batch *a = rq.a, *b = rq.b ? rq.b : rq.a;
    // whatever a direct call would refuse is left to the direct call, which says why
    if (!a || !b || a->mem != BNK_MEM_HOST || b->mem != BNK_MEM_HOST || a->n == 0 || !a->base || !b->base)
        return false;
    const uint32_t n = a->n;
    if (n > std::max(128u, max_packets / 4u)) return false; // big enough by itself
    switch (rq.kind) {
    case CO_SEAL: break;
    case CO_OPEN: if (!rq.r8) return false; break;
    case CO_ENCAP:
    case CO_NOTE_ENCAP: if (!rq.r32a) return false; break;
    default: if (!rq.r8 || !rq.r32a || !rq.r32b || !rq.r64) return false; break;
    }
    RingRef ra, rb;
    if (!find_ring(ctx, a->base, a->bytes, &ra) || !find_ring(ctx, b->base, b->bytes, &rb)) return false;
    const uint64_t base_a = (uintptr_t)a->base - ra.host, base_b = (uintptr_t)b->base - rb.host;

    // This call's packets as offsets from the rings' starts, checked against the
    // call's own arenas as a direct call would check them.
    static thread_local std::vector<uint64_t> off_a, off_b;
    off_a.resize(n);
    off_b.resize(n);
    bool same_len = true;
    const uint32_t len0 = a->lens ? a->lens[0] : a->len;
    for (uint32_t i = 0; i < n; i++) {
        const uint32_t len = a->lens ? a->lens[i] : a->len;
        same_len = same_len && len == len0;
        uint64_t ext_a, ext_b;
        extents(rq.kind, len, rq.mtu, &ext_a, &ext_b);
        const uint64_t oa = pkt_off(a, i), ob = pkt_off(b, i);
        if (oa > a->bytes || ext_a > a->bytes - oa || ob > b->bytes || ext_b > b->bytes - ob) return false;
        off_a[i] = base_a + oa;
        off_b[i] = base_b + ob;
    }
    const bool in_place = ra.host == rb.host && base_a == base_b &&
                          (rq.b == nullptr || rq.b == rq.a ||
                           (a->offsets ? a->offsets == b->offsets : (!b->offsets && a->stride == b->stride)));

    std::shared_ptr<CoWindow> w;
    bool leader = false;
    uint32_t first = 0, expected = 1;
    {
        std::lock_guard<std::mutex> lk(co.mu);
        w = co.open[rq.kind];
        if (w) {
            if (w->ring_a_host != ra.host || w->ring_b_host != rb.host || w->mtu != rq.mtu) return false;
            if (w->n.load(std::memory_order_relaxed) + n > max_packets) {
                // full: this call opens the next window
                w->closed = true;
                co.open[rq.kind].reset();
                co.stats.full_windows++;
                w.reset();
            }
        }
        if (!w) {
            w = std::make_shared<CoWindow>();
            w->kind = rq.kind;
            w->mtu = rq.mtu;
            w->ring_a_host = ra.host;
            w->ring_a_bytes = ra.bytes;
            w->ring_b_host = rb.host;
            w->ring_b_bytes = rb.bytes;
            w->len0 = len0;
            co.open[rq.kind] = w;
            leader = true;
            expected = co.expected[rq.kind];
        }
        first = w->n.load(std::memory_order_relaxed);
        w->off_a.insert(w->off_a.end(), off_a.begin(), off_a.end());
        w->off_b.insert(w->off_b.end(), off_b.begin(), off_b.end());
        if (a->lens) w->lens.insert(w->lens.end(), a->lens, a->lens + n);
        else w->lens.insert(w->lens.end(), n, a->len);
        w->same_len = w->same_len && same_len && len0 == w->len0;
        w->in_place = w->in_place && in_place;
        if (rq.kind == CO_SEAL || rq.kind == CO_OPEN || rq.kind == CO_ENCAP || rq.kind == CO_NOTE_ENCAP) {
            if (a->peer) {
                w->peer.resize(first, 0u); // earlier calls without a peer array: peer 0
                w->peer.insert(w->peer.end(), a->peer, a->peer + n);
                w->any_peer = true;
            } else if (w->any_peer) {
                w->peer.insert(w->peer.end(), n, 0u);
            }
        }
        if (rq.kind == CO_SEAL || rq.kind == CO_OPEN) {
            if (a->counters) w->counters.insert(w->counters.end(), a->counters, a->counters + n);
            else
                for (uint32_t i = 0; i < n; i++) w->counters.push_back(a->counter0 + i);
        }
        if (rq.now > w->now) w->now = rq.now;
        co.stats.calls++;
        co.stats.packets += n;
        co.active[rq.kind].fetch_add(1, std::memory_order_acq_rel);
        w->n.store(first + n, std::memory_order_release);
        w->callers.fetch_add(1, std::memory_order_release);
        if (first + n >= max_packets) {
            w->closed = true;
            if (co.open[rq.kind] == w) co.open[rq.kind].reset();
            co.stats.full_windows++;
        }
    }
    if (leader) lead(ctx, w, expected, max_packets);
    else follow(*w);
    co.active[rq.kind].fetch_sub(1, std::memory_order_acq_rel);

    const int rc = w->rc;
    if (rc == CO_RETRY) return false;
    if (rc == BNK_OK) {
        switch (rq.kind) {
        case CO_SEAL: break;
        case CO_OPEN: memcpy(rq.r8, w->r8.data() + first, n); break;
        case CO_ENCAP:
        case CO_NOTE_ENCAP: memcpy(rq.r32a, w->r32a.data() + first, (size_t)n * 4); break;
        default:
            memcpy(rq.r8, w->r8.data() + first, n);
            memcpy(rq.r32a, w->r32a.data() + first, (size_t)n * 4);
            memcpy(rq.r32b, w->r32b.data() + first, (size_t)n * 4);
            memcpy(rq.r64, w->r64.data() + first, (size_t)n * 8);
            break;
        }
    }
    *rc_out = rc;
    return true;
}

} // namespace bnk

extern "C" int bnk_set_coalesce(bnk_ctx *ctx, uint32_t max_packets, uint32_t max_wait_us, uint32_t expect_callers)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (max_packets > DIRECT_MAX_PACKETS) return fail(ctx, BNK_E_INVAL, "window larger than 65536 packets");
    {
        std::lock_guard<std::mutex> lk(ctx->co.mu);
        for (uint32_t &e : ctx->co.expected) e = expect_callers ? expect_callers : 1u;
    }
    ctx->co.max_wait_us.store(max_wait_us, std::memory_order_relaxed);
    ctx->co.max_packets.store(max_packets, std::memory_order_relaxed);
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

extern "C" int bnk_coalesce_stats_get(bnk_ctx *ctx, bnk_coalesce_stats *out)
{
    BNK_API_TRY
    if (!ctx) return fail(nullptr, BNK_E_INVAL, "null context");
    if (!out) return fail(ctx, BNK_E_INVAL, "null stats pointer");
    std::lock_guard<std::mutex> lk(ctx->co.mu);
    *out = ctx->co.stats;
    return BNK_OK;
    BNK_API_CATCH(ctx)
}
