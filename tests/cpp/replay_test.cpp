// CPU-only: the host ReplayFilter against a brute-force model (a set of seen
// counters and the newest one), against the oracle's window, and on the
// counter sequence WireGuard publishes as its self-test.
#include <stdio.h>

#include <random>
#include <set>

#include "../../bnk_amd/host/bnk_host.hpp"
#include "../../oracle/bnk_oracle.h"

using bnk_host::ReplayFilter;

static int failures = 0;
#define EXPECT(cond, msg)                                              \
    do {                                                               \
        if (!(cond)) {                                                 \
            printf("FAIL %s:%d %s\n", __FILE__, __LINE__, msg);        \
            failures++;                                                \
        }                                                              \
    } while (0)

struct Model {
    std::set<uint64_t> seen;
    uint64_t newest = 0;
    bool validate(uint64_t c, uint64_t limit)
    {
        if (c >= limit) return false;
        if (c > newest) {
            newest = c;
            seen.insert(c);
            return true;
        }
        if (newest - c > ReplayFilter::kWindow) return false;
        return seen.insert(c).second;
    }
};

static void selftest_sequence()
{
    const uint64_t LIM = ReplayFilter::kWindow + 1;
    const uint64_t REJ = ReplayFilter::kRejectAfterMessages;
    const struct { uint64_t c; bool ok; } steps[] = {
        {0, true}, {1, true}, {1, false}, {9, true}, {8, true}, {7, true}, {7, false},
        {LIM, true}, {LIM - 1, true}, {LIM - 1, false}, {LIM - 2, true}, {2, true}, {2, false},
        {LIM + 16, true}, {3, false}, {LIM + 16, false}, {LIM * 4, true},
        {LIM * 4 - (LIM - 1), true}, {10, false}, {LIM * 4 - LIM, false},
        {LIM * 4 - (LIM + 1), false}, {LIM * 4 - (LIM - 2), true}, {LIM * 4 + 1 - LIM, false},
        {0, false}, {REJ, false}, {REJ - 1, true}, {REJ, false}, {REJ - 1, false},
        {REJ - 2, true}, {REJ + 1, false}, {REJ + 2, false}, {REJ - 2, false}, {REJ - 3, true},
        {0, false},
    };
    ReplayFilter f;
    bnko_replay o;
    bnko_replay_reset(&o);
    Model m;
    int k = 0;
    for (const auto &s : steps) {
        k++;
        const bool got = f.ValidateCounter(s.c, REJ);
        const bool ora = bnko_replay_validate(&o, s.c, REJ) != 0;
        const bool mod = m.validate(s.c, REJ);
        if (got != s.ok || ora != s.ok || mod != s.ok) {
            printf("FAIL selftest step %d: host %d oracle %d model %d want %d\n", k, got, ora, mod, s.ok);
            failures++;
        }
    }
    // in-order, then reversed: every counter of a fresh window is accepted once
    f.Reset();
    for (uint64_t i = 1; i <= ReplayFilter::kWindow; i++) EXPECT(f.ValidateCounter(i), "in-order counter");
    EXPECT(f.ValidateCounter(0), "0 after a full window in order");
    EXPECT(!f.ValidateCounter(0), "0 twice");
    f.Reset();
    for (uint64_t i = 2; i <= ReplayFilter::kWindow + 1; i++) EXPECT(f.ValidateCounter(i), "in-order counter");
    EXPECT(f.ValidateCounter(1), "oldest counter still inside the window");
    EXPECT(!f.ValidateCounter(0), "counter just outside the window");
    f.Reset();
    for (uint64_t i = ReplayFilter::kWindow + 1; i-- > 0;) EXPECT(f.ValidateCounter(i), "reverse-order counter");
}

static void random_walks()
{
    std::mt19937_64 rng(0x626E6B);
    for (int trial = 0; trial < 40; trial++) {
        ReplayFilter f;
        bnko_replay o;
        bnko_replay_reset(&o);
        Model m;
        uint64_t head = rng() % 1000;
        const uint64_t limit = trial % 5 == 0 ? 60000 : ReplayFilter::kRejectAfterMessages;
        for (int step = 0; step < 20000; step++) {
            uint64_t c;
            switch (rng() % 8) {
            case 0: head += rng() % 20000; c = head; break;             // jump, sometimes past the ring
            case 1: c = head > 9000 ? head - 7900 - rng() % 500 : 0; break; // around the window's edge
            case 2: c = head - (rng() % (head + 1)); break;            // anywhere behind
            default: head += rng() % 3; c = head - rng() % 64 % (head + 1); break; // mild reordering
            }
            const bool got = f.ValidateCounter(c, limit);
            const bool ora = bnko_replay_validate(&o, c, limit) != 0;
            const bool mod = m.validate(c, limit);
            if (got != mod || ora != mod) {
                printf("FAIL trial %d step %d counter %llu: host %d oracle %d model %d\n", trial, step,
                       (unsigned long long)c, got, ora, mod);
                failures++;
                return;
            }
        }
    }
}

int main()
{
    selftest_sequence();
    random_walks();
    if (failures) {
        printf("%d failure(s)\n", failures);
        return 1;
    }
    printf("ok\n");
    return 0;
}
