// Load generator with wireguard-go's calling pattern, for the benchmark and
// the many-callers test: T threads, each standing for one per-peer goroutine,
// each handing the library at most 128 packets per call from its own part of
// a pinned ring and blocking until the call returns
// (internal/filter/filter.go:160-186: one Read / Write per batch;
// internal/magicsock/bind.go:326-328: Send "called concurrently by per-peer
// goroutines"; batch size bind.go:372-377).  Uses the public C ABI only.
//
// Two workloads, both a round trip so that every round starts from plaintext
// without the caller copying anything:
//   BNKC_AEAD    seal ring X -> ring Y, open ring Y -> ring X
//   BNKC_TUNNEL  NoteOutbound + encapsulate in place in ring X, then
//                decapsulate (anti-replay windows on) + CheckInbound from ring
//                X into ring Y at the slots' plaintext position; X and Y swap
// The context must hold a peer table that loops back (a peer's remote index is
// its own local index, send key = receive key, allowed address = the inner
// source address this generator writes: 100.64.(t >> 8).(t & 255) for thread
// t's peer t), as bench.py and the test set it up.
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <thread>
#include <vector>

#include "bnk_callers.h"

namespace {

using Clock = std::chrono::steady_clock;

struct Spin {
    // all threads start the timed rounds together
    std::atomic<uint32_t> arrived{0};
    void wait(uint32_t n)
    {
        arrived.fetch_add(1, std::memory_order_acq_rel);
        while (arrived.load(std::memory_order_acquire) < n) std::this_thread::yield();
    }
};

double pct(std::vector<float> &v, double p)
{
    if (v.empty()) return 0;
    const size_t k = std::min(v.size() - 1, (size_t)(p * (double)(v.size() - 1) + 0.5));
    std::nth_element(v.begin(), v.begin() + (long)k, v.end());
    return v[k];
}

// An IPv4 + TCP packet of `len` bytes from thread t's address to 100.112.(t >> 8).(t & 255);
// every 16th goes to port 23, which the rule set of the tunnel workload denies.
void inner_packet(uint8_t *p, uint32_t len, uint32_t t, uint32_t i, uint32_t seed)
{
    uint32_t x = seed * 2654435761u + t * 40503u + i * 9973u + 1u;
    for (uint32_t k = 0; k < len; k++) {
        x = x * 1664525u + 1013904223u;
        p[k] = (uint8_t)(x >> 24);
    }
    if (len < 24) return;
    p[0] = 0x45;
    p[2] = (uint8_t)(len >> 8);
    p[3] = (uint8_t)len;
    p[6] = p[7] = 0;
    p[9] = 6;
    p[12] = 100; p[13] = 64; p[14] = (uint8_t)(t >> 8); p[15] = (uint8_t)t;
    p[16] = 100; p[17] = 112; p[18] = (uint8_t)(t >> 8); p[19] = (uint8_t)t;
    const uint16_t sport = (uint16_t)(40000u + i);
    p[20] = (uint8_t)(sport >> 8); p[21] = (uint8_t)sport;
    const uint16_t dport = (i % 16u == 5u) ? 23 : 8000;
    p[22] = (uint8_t)(dport >> 8);
    p[23] = (uint8_t)dport;
}

// Waits for a point in time: sleeping while it is far, yielding when it is near.
void wait_until(Clock::time_point when)
{
    for (;;) {
        const auto left = when - Clock::now();
        if (left <= std::chrono::nanoseconds(0)) return;
        if (left > std::chrono::microseconds(300)) std::this_thread::sleep_for(left - std::chrono::microseconds(200));
        else std::this_thread::yield();
    }
}

// interval_us > 0: every thread starts its timed round r at a fixed time, r intervals
// after its first (the threads' first rounds spread evenly over one interval), whether
// or not the round before has returned: offered load instead of back-to-back calls.  A
// call's time then counts from when its round was due.
int run(bnk_ctx *ctx, int workload, uint32_t threads, uint32_t packets_per_call, uint32_t payload, uint32_t rounds,
        uint32_t warmup, int64_t now_ns, double interval_us, bnkc_result *out)
{
    if (!ctx || !out || threads == 0 || packets_per_call == 0 || rounds == 0) return BNK_E_INVAL;
    if (workload != BNKC_AEAD && workload != BNKC_TUNNEL) return BNK_E_INVAL;
    if (workload == BNKC_TUNNEL && (payload < 24 || payload > 65000)) return BNK_E_INVAL;
    memset(out, 0, sizeof(*out));
    const uint32_t n = packets_per_call;
    // a slot holds the header's 16 bytes of headroom, the payload, padding and the tag
    const uint32_t slot = (16u + payload + 15u + 16u + 127u) & ~127u;
    const size_t per_thread = (size_t)n * slot, total = per_thread * threads;
    // one ring (as a wireguard-go buffer pool would be one allocation), two halves
    uint8_t *ring[2] = {nullptr, nullptr};
    {
        void *p = nullptr;
        const int rc = bnk_ring_alloc(ctx, 2 * total, &p);
        if (rc) return rc;
        ring[0] = static_cast<uint8_t *>(p);
        ring[1] = ring[0] + total;
        memset(ring[0], 0, 2 * total);
    }
    std::vector<std::vector<uint8_t>> plain(threads);
    for (uint32_t t = 0; t < threads; t++) {
        plain[t].resize((size_t)n * payload);
        for (uint32_t i = 0; i < n; i++) {
            inner_packet(plain[t].data() + (size_t)i * payload, payload, t, i, 7);
            memcpy(ring[0] + t * per_thread + (size_t)i * slot + 16, plain[t].data() + (size_t)i * payload, payload);
        }
    }

    std::atomic<int> first_rc{0};
    std::atomic<uint64_t> mismatches{0}, filtered{0};
    std::vector<std::vector<float>> lat_out(threads), lat_in(threads);
    Spin start;
    std::vector<Clock::time_point> t_begin(threads), t_end(threads);

    auto body = [&](uint32_t t) {
        lat_out[t].reserve(rounds);
        lat_in[t].reserve(rounds);
        std::vector<uint32_t> peer(n, t), wire_len(n), out_len(n), got_peer(n);
        std::vector<uint64_t> got_ctr(n);
        std::vector<uint8_t> res(n);
        uint64_t counter = (uint64_t)t << 40; // AEAD workload: this thread's nonce sequence
        int x = 0;                            // which ring holds the plaintext
        uint64_t bad = 0, dropped = 0;
        for (uint32_t r = 0; r < warmup + rounds; r++) {
            if (r == warmup) {
                start.wait(threads);
                t_begin[t] = Clock::now();
            }
            uint8_t *X = ring[x] + t * per_thread, *Y = ring[x ^ 1] + t * per_thread;
            bnk_batch a{}, b{};
            a.bytes = b.bytes = per_thread;
            a.n = b.n = n;
            a.mem = b.mem = BNK_MEM_HOST;
            a.stride = b.stride = slot;
            int rc;
            bool second = false;
            Clock::time_point c0, c1, c2;
            Clock::time_point due{};
            if (interval_us > 0 && r >= warmup) {
                due = t_begin[t] + std::chrono::duration_cast<Clock::duration>(std::chrono::duration<double, std::micro>(
                                       interval_us * ((double)(r - warmup) + (double)t / (double)threads)));
                wait_until(due);
            }
            if (workload == BNKC_AEAD) {
                a.base = X + 16;
                a.bytes = b.bytes = per_thread - 16;
                a.len = payload;
                a.peer = peer.data();
                a.counter0 = counter;
                b.base = Y + 16;
                c0 = Clock::now();
                rc = bnk_aead_seal_batch(ctx, &a, &b);
                c1 = Clock::now();
                if (!rc) {
                    second = true;
                    bnk_batch ci = a, po = b;
                    ci.base = Y + 16;
                    ci.len = payload + 16;
                    po.base = X + 16;
                    rc = bnk_aead_open_batch(ctx, &ci, &po, res.data());
                }
                c2 = Clock::now();
                counter += n;
                if (!rc)
                    for (uint32_t i = 0; i < n; i++) bad += res[i] != 1;
                // the plaintext is back in X: no swap
            } else {
                a.base = X;
                a.len = payload;
                a.peer = peer.data();
                c0 = Clock::now();
                rc = bnk_wg_note_encap_batch(ctx, &a, 0, now_ns, wire_len.data());
                c1 = Clock::now();
                if (!rc) {
                    second = true;
                    bnk_batch w = a, o = b;
                    w.peer = nullptr;
                    w.len = 0;
                    w.lens = wire_len.data();
                    o.base = Y + 16;
                    o.bytes = per_thread - 16;
                    rc = bnk_wg_decap_filter_batch(ctx, &w, &o, now_ns, res.data(), out_len.data(), got_peer.data(),
                                                   got_ctr.data());
                }
                c2 = Clock::now();
                if (!rc)
                    for (uint32_t i = 0; i < n; i++) {
                        const bool deny = i % 16u == 5u;
                        dropped += res[i] == BNK_WG_FILTERED;
                        bad += res[i] != (deny ? BNK_WG_FILTERED : BNK_WG_OK) || out_len[i] != payload ||
                               got_peer[i] != t;
                    }
                x ^= 1; // the plaintext now lies in Y, at the slots' plaintext position
            }
            if (rc) {
                int zero = 0;
                if (first_rc.compare_exchange_strong(zero, rc))
                    fprintf(stderr, "bnk_callers: thread %u round %u: %s call failed with %d: %s (wire_len[0] %u)\n", t, r,
                            second ? "inbound" : "outbound", rc, bnk_last_error(ctx), wire_len[0]);
                break;
            }
            if (r >= warmup) {
                if (interval_us > 0) c0 = due;
                lat_out[t].push_back(std::chrono::duration<float, std::micro>(c1 - c0).count());
                lat_in[t].push_back(std::chrono::duration<float, std::micro>(c2 - c1).count());
            }
        }
        t_end[t] = Clock::now();
        // every byte of the last round trip against what went in
        const uint8_t *fin = ring[x] + t * per_thread;
        for (uint32_t i = 0; i < n && first_rc.load() == 0; i++)
            bad += memcmp(fin + (size_t)i * slot + 16, plain[t].data() + (size_t)i * payload, payload) != 0;
        mismatches.fetch_add(bad);
        filtered.fetch_add(dropped);
        // a thread that failed early must not leave the others waiting at the start line
        if (first_rc.load() != 0 && start.arrived.load() < threads) start.arrived.fetch_add(threads);
    };

    std::vector<std::thread> th;
    for (uint32_t t = 0; t < threads; t++) th.emplace_back(body, t);
    for (auto &x : th) x.join();

    out->rc = first_rc.load();
    if (out->rc == 0) {
        Clock::time_point b0 = t_begin[0], e1 = t_end[0];
        for (uint32_t t = 1; t < threads; t++) {
            b0 = std::min(b0, t_begin[t]);
            e1 = std::max(e1, t_end[t]);
        }
        out->seconds = std::chrono::duration<double>(e1 - b0).count();
        out->calls = 2ull * threads * rounds;
        out->packets = (uint64_t)threads * rounds * n;
        out->plaintext_bytes = out->packets * payload;
        std::vector<float> lo, li;
        for (uint32_t t = 0; t < threads; t++) {
            lo.insert(lo.end(), lat_out[t].begin(), lat_out[t].end());
            li.insert(li.end(), lat_in[t].begin(), lat_in[t].end());
        }
        out->out_p50_us = pct(lo, 0.50);
        out->out_p99_us = pct(lo, 0.99);
        out->out_max_us = lo.empty() ? 0 : *std::max_element(lo.begin(), lo.end());
        out->in_p50_us = pct(li, 0.50);
        out->in_p99_us = pct(li, 0.99);
        out->in_max_us = li.empty() ? 0 : *std::max_element(li.begin(), li.end());
    }
    out->mismatches = mismatches.load();
    out->filtered = filtered.load();
    bnk_ring_free(ctx, ring[0]);
    return out->rc;
}

} // namespace

extern "C" int bnkc_run(bnk_ctx *ctx, int workload, uint32_t threads, uint32_t packets_per_call, uint32_t payload,
                        uint32_t rounds, uint32_t warmup, int64_t now_ns, bnkc_result *out)
{
    return run(ctx, workload, threads, packets_per_call, payload, rounds, warmup, now_ns, 0.0, out);
}

extern "C" int bnkc_run_paced(bnk_ctx *ctx, int workload, uint32_t threads, uint32_t packets_per_call,
                              uint32_t payload, uint32_t rounds, uint32_t warmup, int64_t now_ns,
                              double gbit_per_s_per_direction, bnkc_result *out)
{
    if (!(gbit_per_s_per_direction > 0)) return BNK_E_INVAL;
    // one round of every thread carries threads x packets x payload bytes each way
    const double interval_us = (double)threads * packets_per_call * payload * 8.0 / (gbit_per_s_per_direction * 1e3);
    return run(ctx, workload, threads, packets_per_call, payload, rounds, warmup, now_ns, interval_us, out);
}
