// Device-side views of the filter's tables, shared by kernels and host code.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bnk {

constexpr uint32_t FLOW_REGIONS = 6;     // protocol class (3) x top address bit (2)
constexpr int64_t FLOW_TOMB = INT64_MIN; // expiry of a deleted (or never used) slot
enum : uint32_t { FLOW_LIVE = 0, FLOW_CLAIMED = 1, FLOW_SWEEP = 2, FLOW_COUNTERS = 4 };

// One 16-byte slot, so a probe is a single memory transaction.
struct FlowSlotMem {
    uint64_t key; // 0 = empty
    int64_t exp;  // expiry in Unix ns, FLOW_TOMB = not in the map
};

struct FlowTableDev {
    FlowSlotMem *slots; // [FLOW_REGIONS * cap]
    uint32_t *counters; // [FLOW_COUNTERS]: entries in the map, slots ever claimed, sweep flag
    uint32_t *present;  // [present_bits / 32] one hashed bit per key ever stored in this table:
                        // small enough to stay in L2, it answers most misses without a probe
    uint32_t cap;       // slots per region, a power of two
    uint32_t present_mask; // present_bits - 1 (a power of two)
};

// A key is class << 16 | port with class < 3, so key_lo 0x3FFFF never occurs.
constexpr uint32_t RANGE_PAD = 0x3FFFFu << 14;
constexpr uint32_t RANGE_MAX_SPAN = (1u << 14) - 1u; // largest key_hi - key_lo one entry holds
constexpr uint32_t RANGE_BLOCK = 16;                 // entries per 64-byte block

struct RuleIndexDev {
    const uint32_t *bounds; // [n_bounds] ascending starts of the elementary source intervals
    const uint32_t *meta;   // [n_bounds + 1] (first 64-byte block of the interval's list) << 8 |
                            // min(entries, 255); the last element only carries the block count
    const uint32_t *ranges; // per interval: sorted disjoint key ranges, one word each
                            // (key_lo << 14 | key_hi - key_lo; wider ranges are cut into
                            // pieces), padded to a multiple of 16 entries (one 64-byte block)
                            // with RANGE_PAD, which contains no key
    const uint4 *wide;      // [n_wide] (net, mask, key_lo, key_hi) scanned by every packet
    uint32_t n_bounds;
    uint32_t top_step;      // largest power of two < n_bounds (0 when n_bounds == 1)
    uint32_t n_wide;
};

struct FilterArgs {
    const uint8_t *pkts;
    const uint64_t *off;  // or nullptr: i * stride
    const uint32_t *lens; // or nullptr: len
    const uint8_t *gate;  // or nullptr; gate[i] == 0 skips packet i (verdict 0)
    uint8_t *verdict;     // check only
    uint32_t *status;
    int64_t now;
    uint32_t n, stride, len;
    uint32_t trim;        // bytes at the end of each packet that are not payload
    RuleIndexDev rules;
    FlowTableDev flows;
};

hipError_t launch_fill_u64(uint64_t *p, uint32_t n, uint64_t v, hipStream_t s);
hipError_t launch_flow_clear(FlowSlotMem *p, uint32_t n, hipStream_t s);
hipError_t launch_fill_u8(uint8_t *p, uint32_t n, uint8_t v, hipStream_t s);
hipError_t launch_filter_check(const FilterArgs &a, uint32_t max_blocks, hipStream_t s);
// inserts, then the reference's conditional expiry sweep
hipError_t launch_filter_note(const FilterArgs &a, uint32_t max_blocks, hipStream_t s);
hipError_t launch_flow_rehash(const FlowTableDev &from, const FlowTableDev &to, uint32_t *status,
                              uint32_t max_blocks, hipStream_t s);

} // namespace bnk
