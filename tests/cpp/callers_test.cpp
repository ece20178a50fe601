// Many threads calling the library the way wireguard-go's per-peer goroutines
// do (at most 128 packets per call, each thread blocking on its own call;
// internal/filter/filter.go:160-186, internal/magicsock/bind.go:326-328), with
// and without the library merging their calls.  Needs a GPU.  Every round of
// every thread is checked by the load generator itself: all packets of a seal
// -> open round trip verify and come back bit for bit; in the tunnel workload
// every datagram is delivered by its own peer with a fresh counter, the ones
// to the denied port are dropped by the inbound filter and only those, and
// the plaintext of the last round equals what went in.  The statistics must
// show that merged calls did share launches.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <random>
#include <vector>

#include "../../bnk_amd/host/bnk_callers.h"

#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            fprintf(stderr, "FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);  \
            exit(1);                                                         \
        }                                                                    \
    } while (0)

static void setup(bnk_ctx *ctx, uint32_t peers)
{
    std::mt19937 rng(99);
    std::vector<uint8_t> keys((size_t)peers * 32);
    for (auto &k : keys) k = (uint8_t)rng();
    CHECK(bnk_keys_set(ctx, BNK_KEYS_SEND, keys.data(), peers) == 0);
    CHECK(bnk_keys_set(ctx, BNK_KEYS_RECV, keys.data(), peers) == 0);
    std::vector<bnk_wg_peer> table(peers);
    for (uint32_t t = 0; t < peers; t++) {
        table[t].local_index = table[t].remote_index = 0x1000u + 37u * t; // loops back
        table[t].allowed_net = 0x64400000u + t;                            // 100.64.(t >> 8).(t & 255)
        table[t].allowed_mask = 0xFFFFFFFFu;
    }
    CHECK(bnk_wg_peers_set(ctx, table.data(), peers) == 0);
    bnk_rule rule{};
    rule.src_net = 0x64400000u; // 100.64.0.0/10
    rule.src_mask = 0xFFC00000u;
    rule.port_first = rule.port_last = 8000;
    rule.proto = 6;
    CHECK(bnk_filter_set_rules(ctx, &rule, 1) == 0);
}

int main()
{
    bnk_ctx *ctx = nullptr;
    if (bnk_init(0, &ctx) != 0) {
        fprintf(stderr, "bnk_init: %s\n", bnk_last_error(nullptr));
        return 1;
    }
    const uint32_t T = 16;
    setup(ctx, T);
    const int64_t now = 1700000000ll * 1000000000ll;
    // how long a window's first caller waits for company, at most (microseconds)
    const uint32_t wait_us = getenv("BNK_TEST_WAIT_US") ? (uint32_t)atoi(getenv("BNK_TEST_WAIT_US")) : 30;
    struct Case {
        int workload;
        uint32_t per_call, payload, rounds;
        const char *name;
    } cases[] = {{BNKC_AEAD, 128, 1420, 40, "seal+open 128x1420"},
                 {BNKC_TUNNEL, 128, 1420, 40, "tunnel 128x1420"},
                 {BNKC_TUNNEL, 37, 60, 40, "tunnel 37x60"},
                 {BNKC_AEAD, 1, 1420, 40, "seal+open 1x1420"}};
    for (const Case &c : cases) {
        for (int merged = 0; merged < 2; merged++) {
            CHECK(bnk_set_coalesce(ctx, merged ? 4096 : 0, wait_us, 0) == 0);
            bnk_coalesce_stats s0{}, s1{};
            CHECK(bnk_coalesce_stats_get(ctx, &s0) == 0);
            bnkc_result r{};
            const int rc = bnkc_run(ctx, c.workload, T, c.per_call, c.payload, c.rounds, 3, now, &r);
            if (rc) fprintf(stderr, "%s: rc %d: %s\n", c.name, rc, bnk_last_error(ctx));
            CHECK(rc == 0);
            CHECK(bnk_coalesce_stats_get(ctx, &s1) == 0);
            const uint64_t calls = s1.calls - s0.calls, batches = s1.batches - s0.batches;
            printf("%-20s %s: %7.1f Gbit/s, out p50 %6.1f p99 %6.1f us, in p50 %6.1f p99 %6.1f us, "
                   "%llu calls in %llu batches, mismatches %llu, filtered %llu\n",
                   c.name, merged ? "merged" : "direct", (double)r.plaintext_bytes * 8e-9 / r.seconds, r.out_p50_us,
                   r.out_p99_us, r.in_p50_us, r.in_p99_us, (unsigned long long)calls, (unsigned long long)batches,
                   (unsigned long long)r.mismatches, (unsigned long long)r.filtered);
            if (batches)
                printf("%-20s         per window: gather %.1f us, enqueue %.1f us, wait %.1f us, %.1f calls\n", "",
                       (double)(s1.gather_ns - s0.gather_ns) * 1e-3 / (double)batches,
                       (double)(s1.enqueue_ns - s0.enqueue_ns) * 1e-3 / (double)batches,
                       (double)(s1.wait_ns - s0.wait_ns) * 1e-3 / (double)batches, (double)calls / (double)batches),
                printf("%-20s         %llu windows went without the company they waited for\n", "",
                       (unsigned long long)(s1.timed_out - s0.timed_out));
            CHECK(r.mismatches == 0);
            if (c.workload == BNKC_TUNNEL) {
                // packets 5, 21, 37, ... of every call go to the denied port
                const uint64_t per = (c.per_call + 10) / 16;
                CHECK(r.filtered == per * T * (c.rounds + 3));
            }
            if (merged) {
                CHECK(calls == 2ull * T * (c.rounds + 3));
                CHECK(2 * batches < calls); // calls did share launches
                CHECK(s1.retried == s0.retried);
            } else {
                CHECK(calls == 0);
            }
        }
    }
    // one thread alone with merging on: every window holds one call and nobody waits
    CHECK(bnk_set_coalesce(ctx, 4096, 30, 0) == 0);
    bnk_coalesce_stats s0{}, s1{};
    CHECK(bnk_coalesce_stats_get(ctx, &s0) == 0);
    bnkc_result r{};
    CHECK(bnkc_run(ctx, BNKC_TUNNEL, 1, 128, 1420, 20, 2, now, &r) == 0);
    CHECK(bnk_coalesce_stats_get(ctx, &s1) == 0);
    CHECK(r.mismatches == 0 && s1.batches - s0.batches == s1.calls - s0.calls && s1.timed_out == s0.timed_out);
    printf("one caller, merging on: out p50 %.1f us, in p50 %.1f us\n", r.out_p50_us, r.in_p50_us);
    // the same callers under an offered load well below what they carry back to back: every
    // round's results right, and the load carried (the rounds take the time they were spread over)
    for (int workload : {BNKC_AEAD, BNKC_TUNNEL}) {
        bnkc_result p{};
        const double offered = workload == BNKC_AEAD ? 8.0 : 5.0;
        CHECK(bnkc_run_paced(ctx, workload, 8, 128, 1420, 60, 3, now, offered, &p) == 0);
        const double carried = (double)p.plaintext_bytes * 8e-9 / p.seconds;
        printf("8 callers offering %.1f Gbit/s each way, merging on: carried %.1f, out p50 %.1f p99 %.1f us\n", offered,
               carried, p.out_p50_us, p.out_p99_us);
        // (the rate only loosely: a busy host may delay a round, and this load is a tenth of what the callers carry)
        CHECK(p.mismatches == 0 && carried > 0.5 * offered && carried < 1.1 * offered);
    }
    bnk_shutdown(ctx);
    printf("callers_test ok\n");
    return 0;
}
