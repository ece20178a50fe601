// Coalescing of small filter calls into GPU-sized batches.
//
// wireguard-go hands the TUN wrapper at most 128 packets per Write, from one
// goroutine per peer (internal/filter/filter.go:171-186 is called once per
// such batch); a GPU launch wants thousands.  Callers that arrive within a
// short window are therefore merged: the first caller of a window becomes its
// leader, waits until the window is full or its time is up, runs one batch for
// everyone and hands each caller its own verdicts.  No background thread.
//
// A caller that has been alone lately should not pay the whole window for
// company that is not coming: when the previous window held a single call, the
// next leader waits only solo_wait (SetSoloWait; by default the full window).
// A follower that turns up within that time is merged as usual and restores
// the full window for the next round.
//
// What changes against calling the filter directly: the packets of one window
// share one `now` (the leader's clock at flush time, at most max_wait later
// than a caller's own), and NoteOutbound calls of a window are applied before
// its CheckInbound calls.  Both are orders the reference could have produced
// itself for calls that overlap in time, which the members of a window do.
#pragma once

#include <stdint.h>

#include <chrono>
#include <condition_variable>
#include <exception>
#include <functional>
#include <memory>
#include <mutex>
#include <vector>

namespace bnk_host {

struct CoalesceStats {
    uint64_t calls = 0, packets = 0, batches = 0, full_flushes = 0, largest_batch = 0;
};

class BatchCoalescer {
public:
    // Runs one merged batch: n packets, note[i] != 0 marks a NoteOutbound
    // packet; verdict[i] is filled for the others.
    using Executor = std::function<void(const uint8_t *const *ptrs, const uint32_t *lens,
                                        const uint8_t *note, uint32_t n, int64_t now_ns,
                                        uint8_t *verdict)>;
    using Clock = std::function<int64_t()>;

    BatchCoalescer(Executor exec, size_t max_packets, std::chrono::microseconds max_wait,
                   Clock clock = nullptr)
        : exec_(std::move(exec)), max_packets_(max_packets ? max_packets : 1), max_wait_(max_wait),
          solo_wait_(max_wait), clock_(std::move(clock))
    {
    }

    // How long a leader waits when the window before its own held one call only.
    void SetSoloWait(std::chrono::microseconds solo_wait)
    {
        std::lock_guard<std::mutex> lk(mu_);
        solo_wait_ = solo_wait < max_wait_ ? solo_wait : max_wait_;
    }

    // Blocks until the window this call joined has run.  verdict may be null
    // for notes.  An executor failure is rethrown in every caller of the window.
    void Submit(const uint8_t *const *ptrs, const uint32_t *lens, uint32_t n, bool note, uint8_t *verdict)
    {
        if (n == 0) return;
        std::unique_lock<std::mutex> lk(mu_);
        if (!open_) open_ = std::make_shared<Window>();
        std::shared_ptr<Window> w = open_;
        const bool leader = w->ptrs.empty();
        const size_t first = w->ptrs.size();
        w->ptrs.insert(w->ptrs.end(), ptrs, ptrs + n);
        w->lens.insert(w->lens.end(), lens, lens + n);
        w->note.insert(w->note.end(), n, note ? 1 : 0);
        w->callers++;
        stats_.calls++;
        stats_.packets += n;
        if (w->ptrs.size() >= max_packets_) {
            // full: later arrivals open the next window
            w->full = true;
            if (open_ == w) open_.reset();
            w->cv.notify_all();
        }
        if (leader) {
            w->cv.wait_for(lk, last_callers_ >= 2 ? max_wait_ : solo_wait_, [&] { return w->full; });
            if (open_ == w) open_.reset();
            last_callers_ = w->callers;
            if (w->full) stats_.full_flushes++;
            stats_.batches++;
            if (w->ptrs.size() > stats_.largest_batch) stats_.largest_batch = w->ptrs.size();
            lk.unlock();
            w->verdict.assign(w->ptrs.size(), 0);
            try {
                exec_(w->ptrs.data(), w->lens.data(), w->note.data(), (uint32_t)w->ptrs.size(),
                      clock_ ? clock_() : SystemNow(), w->verdict.data());
            } catch (...) {
                w->error = std::current_exception();
            }
            lk.lock();
            w->done = true;
            w->cv.notify_all();
        } else {
            w->cv.wait(lk, [&] { return w->done; });
        }
        if (w->error) std::rethrow_exception(w->error);
        if (verdict && !note)
            for (uint32_t i = 0; i < n; i++) verdict[i] = w->verdict[first + i];
    }

    CoalesceStats Stats()
    {
        std::lock_guard<std::mutex> lk(mu_);
        return stats_;
    }

    static int64_t SystemNow()
    {
        return std::chrono::duration_cast<std::chrono::nanoseconds>(
                   std::chrono::system_clock::now().time_since_epoch())
            .count();
    }

private:
    struct Window {
        std::vector<const uint8_t *> ptrs;
        std::vector<uint32_t> lens;
        std::vector<uint8_t> note, verdict;
        uint32_t callers = 0;
        bool full = false, done = false;
        std::exception_ptr error;
        std::condition_variable cv;
    };

    Executor exec_;
    const size_t max_packets_;
    const std::chrono::microseconds max_wait_;
    std::chrono::microseconds solo_wait_;
    uint32_t last_callers_ = 2; // the first window waits in full
    Clock clock_;
    std::mutex mu_;
    std::shared_ptr<Window> open_;
    CoalesceStats stats_;
};

} // namespace bnk_host
