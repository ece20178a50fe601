// CPU-only: the batch coalescer with a stand-in executor (verdict = low bit of
// the packet's first byte): every caller gets its own verdicts, windows fill
// and flush, a lone caller is released after max_wait, failures reach every
// caller of the window, notes and checks are told apart.
#include <stdio.h>

#include <atomic>
#include <stdexcept>
#include <thread>

#include "../../bnk_amd/host/bnk_coalesce.hpp"

using namespace bnk_host;
using std::chrono::microseconds;
using std::chrono::steady_clock;

static int failures = 0;
#define EXPECT(cond, msg)                                              \
    do {                                                               \
        if (!(cond)) {                                                 \
            printf("FAIL %s:%d %s\n", __FILE__, __LINE__, msg);        \
            failures++;                                                \
        }                                                              \
    } while (0)

static void many_threads_get_their_own_verdicts()
{
    std::atomic<uint64_t> notes{0}, checks{0}, execs{0};
    BatchCoalescer co(
        [&](const uint8_t *const *p, const uint32_t *l, const uint8_t *note, uint32_t n, int64_t now,
            uint8_t *v) {
            execs++;
            if (now != 77) throw std::runtime_error("clock not used");
            for (uint32_t i = 0; i < n; i++) {
                if (note[i]) notes++;
                else {
                    checks++;
                    v[i] = (uint8_t)((p[i][0] & 1) ^ (l[i] & 1));
                }
            }
            std::this_thread::sleep_for(microseconds(300)); // a launch's worth of time
        },
        64, microseconds(2000), [] { return (int64_t)77; });
    constexpr int T = 16, CALLS = 200;
    std::atomic<int> wrong{0};
    std::vector<std::thread> th;
    for (int t = 0; t < T; t++)
        th.emplace_back([&, t] {
            for (int c = 0; c < CALLS; c++) {
                uint8_t a[3] = {(uint8_t)(t * 7 + c), 0, 0}, b[5] = {(uint8_t)(t + c * 3), 0, 0, 0, 0};
                const uint8_t *ptrs[2] = {a, b};
                const uint32_t lens[2] = {3, (uint32_t)(4 + (c & 1))};
                if (c % 5 == 0) {
                    co.Submit(ptrs, lens, 2, true, nullptr);
                } else {
                    uint8_t v[2] = {9, 9};
                    co.Submit(ptrs, lens, 2, false, v);
                    if (v[0] != ((a[0] & 1) ^ 1) || v[1] != ((b[0] & 1) ^ (lens[1] & 1))) wrong++;
                }
            }
        });
    for (auto &x : th) x.join();
    const CoalesceStats st = co.Stats();
    EXPECT(wrong == 0, "every caller got the verdicts of its own packets");
    EXPECT(st.calls == (uint64_t)T * CALLS && st.packets == 2ull * T * CALLS, "call and packet counts");
    EXPECT(notes == 2ull * T * (CALLS / 5) && checks == 2ull * T * (CALLS - CALLS / 5), "notes and checks told apart");
    EXPECT(st.batches == execs && st.batches < st.calls / 4, "calls were merged");
    EXPECT(st.largest_batch > 2 && st.largest_batch <= 64 + 2, "windows close when full");
    printf("coalesced %llu calls into %llu batches (largest %llu, %llu closed full)\n",
           (unsigned long long)st.calls, (unsigned long long)st.batches,
           (unsigned long long)st.largest_batch, (unsigned long long)st.full_flushes);
}

static void lone_caller_waits_at_most_the_window()
{
    BatchCoalescer co([](const uint8_t *const *, const uint32_t *, const uint8_t *, uint32_t n, int64_t,
                         uint8_t *v) { for (uint32_t i = 0; i < n; i++) v[i] = 1; },
                      1000, microseconds(5000));
    uint8_t pkt[1] = {0};
    const uint8_t *p = pkt;
    const uint32_t len = 1;
    uint8_t v = 0;
    const auto t0 = steady_clock::now();
    co.Submit(&p, &len, 1, false, &v);
    const auto us = std::chrono::duration_cast<microseconds>(steady_clock::now() - t0).count();
    EXPECT(v == 1, "verdict delivered");
    EXPECT(us >= 4000 && us < 200000, "released when the window's time is up");
    // a call that fills the window by itself does not wait at all
    BatchCoalescer full([](const uint8_t *const *, const uint32_t *, const uint8_t *, uint32_t, int64_t,
                           uint8_t *) {}, 1, std::chrono::seconds(5));
    const auto t1 = steady_clock::now();
    full.Submit(&p, &len, 1, true, nullptr);
    EXPECT(steady_clock::now() - t1 < std::chrono::seconds(1), "a full window flushes at once");
    EXPECT(full.Stats().full_flushes == 1, "counted as a full flush");
}

static void lone_callers_stop_waiting_for_company()
{
    std::atomic<uint64_t> execs{0};
    BatchCoalescer co([&](const uint8_t *const *, const uint32_t *, const uint8_t *, uint32_t n, int64_t,
                          uint8_t *v) { execs++; for (uint32_t i = 0; i < n; i++) v[i] = 1; },
                      1000, microseconds(40000));
    co.SetSoloWait(microseconds(200));
    uint8_t pkt[1] = {0};
    const uint8_t *p = pkt;
    const uint32_t len = 1;
    uint8_t v = 0;
    auto timed = [&] {
        const auto t0 = steady_clock::now();
        co.Submit(&p, &len, 1, false, &v);
        return std::chrono::duration_cast<microseconds>(steady_clock::now() - t0).count();
    };
    const auto first = timed();  // nothing is known yet: the full window
    const auto second = timed(); // the window before held one call
    const auto third = timed();
    EXPECT(first >= 35000, "the first window waits in full");
    EXPECT(second < 20000 && third < 20000, "a caller that was alone waits the short time only");
    // two callers at once: the follower is merged, and the next window waits in full again
    std::thread other([&] {
        uint8_t q[1] = {1};
        const uint8_t *qp = q;
        uint8_t qv = 0;
        std::this_thread::sleep_for(microseconds(5000));
        co.Submit(&qp, &len, 1, false, &qv);
    });
    BatchCoalescer *c = &co;
    c->SetSoloWait(microseconds(39000)); // long enough for the other thread to turn up
    const uint64_t before = execs;
    (void)timed();
    other.join();
    EXPECT(execs == before + 1, "the follower rode the leader's window");
    c->SetSoloWait(microseconds(200));
    const auto after_pair = timed();
    EXPECT(after_pair >= 35000, "after a shared window the next one waits in full");
    const auto alone_again = timed();
    EXPECT(alone_again < 20000, "and alone again it does not");
}

static void failures_reach_every_caller()
{
    BatchCoalescer co([](const uint8_t *const *, const uint32_t *, const uint8_t *, uint32_t, int64_t,
                         uint8_t *) { throw std::runtime_error("device lost"); },
                      4, microseconds(100000));
    std::atomic<int> caught{0};
    std::vector<std::thread> th;
    for (int t = 0; t < 4; t++)
        th.emplace_back([&] {
            uint8_t pkt[1] = {0};
            const uint8_t *p = pkt;
            const uint32_t len = 1;
            uint8_t v = 0;
            try {
                co.Submit(&p, &len, 1, false, &v);
            } catch (const std::runtime_error &e) {
                if (std::string(e.what()) == "device lost") caught++;
            }
        });
    for (auto &x : th) x.join();
    EXPECT(caught == 4, "all four callers of the window saw the failure");
}

int main()
{
    many_threads_get_their_own_verdicts();
    lone_caller_waits_at_most_the_window();
    lone_callers_stop_waiting_for_company();
    failures_reach_every_caller();
    if (failures) {
        printf("%d failure(s)\n", failures);
        return 1;
    }
    printf("ok\n");
    return 0;
}
