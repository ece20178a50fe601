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
    uint32_t *present_small; // [SMALL_BITS / 32] two hashed bits per key (a Bloom filter) in a
                             // size a workgroup can hold in LDS beside the cut points: with
                             // few enough keys the check kernel asks this one and never
                             // leaves the CU for a packet without a flow
    uint32_t cap;       // slots per region, a power of two
    uint32_t present_mask; // present_bits - 1 (a power of two)
    uint32_t small_ok;  // host's call: few enough keys for present_small to be worth reading
};

constexpr uint32_t SMALL_BITS = 44u * 1024u * 8u; // 44 KiB: leaves 36 KiB of a workgroup's 80 for cut points
constexpr uint32_t SMALL_KEYS_MAX = 3u << 16;     // beyond this a clear answer gets too rare (false
                                                  // positives pass 43 %) and the large bitmap is asked

// A key is class << 16 | port with class < 3, so key_lo 0x3FFFF and 0x3FFFE never occur.
constexpr uint32_t RANGE_PAD = 0x3FFFFu << 14;
constexpr uint32_t RANGE_LONG = 0x3FFFEu << 14;      // first word of a block that only points on
constexpr uint32_t RANGE_MAX_SPAN = (1u << 14) - 1u; // largest key_hi - key_lo one entry holds
constexpr uint32_t RANGE_BLOCK = 16;
constexpr uint32_t JUMP_BUCKETS = 1024;                 // entries per 64-byte block

struct RuleIndexDev {
    const uint32_t *bounds; // [n_bounds] ascending starts of the elementary source intervals
    const uint32_t *ranges; // 64-byte blocks of RANGE_BLOCK one-word key ranges
                            // (key_lo << 14 | key_hi - key_lo; wider ranges are cut into
                            // pieces), sorted, disjoint, padded with RANGE_PAD.  Block j is
                            // interval j's list, so finding the interval finds the list.  A
                            // list of more than RANGE_BLOCK pieces lives in blocks past the
                            // first n_bounds, and block j is {RANGE_LONG, first block, blocks}
    const uint4 *wide;      // [n_wide] (net, mask, key_lo, key_hi) scanned by every packet
    const uint16_t *jump;   // [JUMP_BUCKETS + 1] when n_bounds fits 16 bits, else null: the cut
                            // points from bounds[1] up are spread over equal address buckets
                            // and jump[b] is the last cut point at or below bucket b's start,
                            // so a search only has to look between jump[b] and jump[b + 1]
    uint32_t jump_lo;       // bounds[1]
    uint32_t jump_shift;    // bucket of src = (src - jump_lo) >> jump_shift
    uint32_t n_bounds;
    uint32_t top_step;      // largest power of two < n_bounds (0 when n_bounds == 1)
    uint32_t n_wide;
};

struct FilterArgs {
    const uint8_t *pkts;
    const uint64_t *off;  // or nullptr: i * stride
    const uint32_t *lens; // or nullptr: len
    const uint8_t *gate;  // or nullptr; gate[i] == 0 skips packet i (verdict 0)
    const uint8_t *heads; // check only, or nullptr: the records AeadArgs::heads describes.  With
                          // them the kernel goes through the records (record t is packet
                          // order[t], or t), takes length and authenticity from them (lens
                          // and gate are not read) and looks at the packet itself only for
                          // an IP header with options
    const uint32_t *order; // with heads, or nullptr
    uint8_t *verdict;     // check only
    uint8_t *wg_result;   // check only, or nullptr: the BNK_WG_* results of the decapsulation that
                          // delivered these packets; a denied packet's BNK_WG_OK becomes BNK_WG_FILTERED
    unsigned long long *tally; // check only, or nullptr: the launch counts its verdicts here
                          // (TALLY_ALLOWED / TALLY_DENIED, see tally_bump)
    uint32_t *status;
    int64_t now;
    uint32_t n, stride, len;
    uint64_t limit;       // arena size for device-resident batches with per-packet arrays: a
                          // packet reaching beyond it is not read, fails the parse and
                          // raises STATUS_BOUNDS.  0: the host has checked the layout
    uint32_t trim;        // bytes at the end of each packet that are not payload
    uint32_t small_in_lds; // set by the launcher: presence questions go to the folded bitmap in LDS
    RuleIndexDev rules;
    FlowTableDev flows;
};

hipError_t launch_fill_u64(uint64_t *p, uint32_t n, uint64_t v, hipStream_t s);
hipError_t launch_flow_clear(FlowSlotMem *p, uint32_t n, hipStream_t s);
hipError_t launch_fill_u8(uint8_t *p, uint32_t n, uint8_t v, hipStream_t s);
hipError_t launch_filter_check(const FilterArgs &a, uint32_t max_blocks, hipStream_t s);
// inserts, then the reference's conditional expiry sweep
// may_sweep: the table may hold more than 4096 entries after this batch (the
// host's upper bound on claimed slots says so); otherwise the expiry sweep
// cannot fire and its two launches are left out.
hipError_t launch_filter_note(const FilterArgs &a, uint32_t max_blocks, bool may_sweep, hipStream_t s);
hipError_t launch_flow_rehash(const FlowTableDev &from, const FlowTableDev &to, uint32_t *status,
                              uint32_t max_blocks, hipStream_t s);

} // namespace bnk
