// Merging of small host calls into GPU-sized batches, inside the library.
//
// wireguard-go hands over at most 128 packets per call and calls from one
// goroutine per peer: filteredTUN.Write once per peer batch
// (internal/filter/filter.go:171-186), Bind.Send "concurrently by per-peer
// goroutines" (internal/magicsock/bind.go:326-328, batch size bind.go:372-377).
// One context has one stream and one lock, so such calls would run one after
// the other, each paying a launch and a wait for a few hundred kilobytes.  With
// merging switched on (bnk_set_coalesce) the calls that carry packet bytes --
// seal, open, encapsulate, decapsulate, with or without the filter -- join a
// window per kind of call: the first caller of a window leads it, the others
// append their packets and wait; the leader runs one batch for everyone and
// every caller takes its own results.  No background thread.
//
// What a window is made of: callers whose arenas lie in pinned rings of the
// context (bnk_ring_alloc).  The merged batch addresses the ring itself, every
// packet by its offset from the ring's start, so nothing is copied on the host
// but the per-packet arrays.  Calls are appended in arrival order and each
// call's packets stay in their order, so whatever depends on the order of one
// peer's packets (send counters, anti-replay windows) sees them as some
// serial execution of the calls would: one peer's calls come from one thread
// and never overlap.  Calls of a window that carry a `now` share the latest of
// theirs (the callers overlap in time, so the reference could have served all
// of them at that instant).
//
// How long a leader waits: for company, until its window holds its share of the
// callers that are inside these entry points at that moment or max_wait_us have
// passed.  The share: half of all of them, so that two windows are in the
// pipeline and one is enqueued while the other runs, but no more than are making
// this kind of call (with senders and receivers calling at the same time, the
// senders' window and the receivers' window are the two).  A caller alone is
// its own share and waits for nobody.  Then for one of two places in the
// pipeline: at most two windows are enqueued or running, one on the GPU and one
// behind it, so that the GPU does not wait for the host, and a window that
// waits for its turn stays open and fills up.  The leader holds the context
// lock only to stage and launch the batch; it waits for the results outside
// the lock, with staging of its own, while the next window is enqueued.
#pragma once

#include <stdint.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/bnkhip.h"

namespace bnk {

enum CoKind : int { CO_SEAL = 0, CO_OPEN, CO_ENCAP, CO_NOTE_ENCAP, CO_DECAP, CO_DECAP_FILTER, CO_KINDS };

// One call as it arrives at an entry point.
struct CoRequest {
    CoKind kind;
    const bnk_batch *a = nullptr; // in / slots / wire
    const bnk_batch *b = nullptr; // out (null for encapsulation: in place)
    uint32_t mtu = 0;
    int64_t now = 0;
    uint8_t *r8 = nullptr;    // verdict / result
    uint32_t *r32a = nullptr; // wire_len / out_len
    uint32_t *r32b = nullptr; // peer
    uint64_t *r64 = nullptr;  // counter
};

struct CoWindow {
    CoKind kind = CO_SEAL;
    uint32_t mtu = 0;
    uintptr_t ring_a_host = 0, ring_b_host = 0; // the rings the arenas lie in: host address and size
    uint64_t ring_a_bytes = 0, ring_b_bytes = 0;
    int64_t now = INT64_MIN;
    bool in_place = true;   // every call so far reads and writes the same places
    bool any_peer = false;  // some call named peers (else every packet is peer 0)
    bool same_len = true;   // every packet so far has length len0
    uint32_t len0 = 0;
    std::vector<uint64_t> off_a, off_b, counters;
    std::vector<uint32_t> lens, peer;
    std::vector<uint8_t> r8;
    std::vector<uint32_t> r32a, r32b;
    std::vector<uint64_t> r64;
    std::atomic<uint32_t> n{0}, callers{0};
    std::atomic<int> done{0};
    std::atomic<bool> closed{false}; // no one joins any more (written under Coalescer::mu)
    int rc = 0;          // BNK_OK, an error every caller returns, or CO_RETRY
    std::mutex mu;       // with cv: for callers that have spun long enough
    std::condition_variable cv;
};

// rc of a window whose merged call was refused before it did anything for a reason one of
// its callers can be told apart by (layout, peer index, state): every caller then makes its
// own call, and the one at fault gets its own error.
constexpr int CO_RETRY = 1;

struct Coalescer {
    std::atomic<uint32_t> max_packets{0}; // 0: off
    std::atomic<uint32_t> max_wait_us{0};
    std::atomic<uint32_t> in_flight{0}; // windows enqueued or running, not yet done
    // callers inside a window right now (gathering, enqueued or running), per kind of call
    std::atomic<uint32_t> active[CO_KINDS] = {};
    std::mutex mu; // open[], expected[], stats
    std::shared_ptr<CoWindow> open[CO_KINDS];
    uint32_t expected[CO_KINDS] = {1, 1, 1, 1, 1, 1};
    bnk_coalesce_stats stats{};
};

// True when the call was served as part of a window (*rc is its result); false when it
// does not qualify or its window asked for a retry, and the caller goes on by itself.
bool coalesce_submit(bnk_ctx *ctx, const CoRequest &rq, int *rc);

} // namespace bnk
