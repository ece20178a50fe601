// Packet filter kernels for gfx950: IPv4 5-tuple parse, rule lookup, flow
// (conntrack) table.  One lane per packet.
//
// Restates internal/filter/filter.go (parse :62-106, CheckInbound :121-147,
// NoteOutbound :189-209) and acl.CompiledRule.Match (internal/acl/acl.go:149-172)
// of the reference, batched with one `now` per batch as filteredTUN.Read/Write
// do (filter.go:160-186).
//
// Rule lookup.  Every rule tuple allows a source interval [net, net|~mask] and
// a key interval [class<<16 | first, class<<16 | last] (class 0 icmp, 1 tcp,
// 2 udp; icmp packets carry key 0 and icmp rules cover the whole class).  The
// host cuts the 32-bit source space at every interval end into elementary
// intervals and stores, per elementary interval, the sorted disjoint union of
// the key intervals of all rules covering it, in 64-byte blocks.  A packet does
// one binary search over the cut points (staged in LDS together with each
// interval's block number and length) and then reads its interval's list: one
// memory transaction when the list fits a block, a binary search otherwise.
// "Any rule matches" is all the reference asks (filter.go:131-135), so this is
// exact.  Rules too wide to expand go to a short list every packet scans.
//
// Flow table.  Open addressing in HBM, one 16-byte slot (64-bit key word,
// 64-bit expiry) so a probe is one memory transaction.  The reference's flowKey (remote addr, remote port, local
// port, proto) is 66 bits with the protocol class; the class and the top
// address bit select one of six equal regions and the other 63 bits plus a
// marker bit form the key word, so 0 can mean "empty" and a slot is claimed
// with one 64-bit compare-and-swap.  Deleted entries keep their key and carry
// expiry FLOW_TOMB.
#include "../../include/bnkhip.h"
#include "filter_dev.hpp"
#include "kernels.hpp"

namespace bnk {

#define BNK_DEV __device__ __forceinline__

BNK_DEV uint32_t ld32u(const uint8_t *p)
{
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}

struct Parsed {
    uint32_t src, dst;
    uint32_t sport, dport;
    uint32_t proto;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 __attribute__((aligned(1))) u32x4_unaligned;
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef u32x2 __attribute__((aligned(1))) u32x2_unaligned;

// filter.go:71-106.  Bytes 0-15 come in one load and bytes 16-23 (destination
// and, without IP options, the ports) in a second when the packet has them:
// every load instruction here reads 64 different lines, so their number is
// what the kernel pays for.
// Where packet i lies in its arena, worked out only when somebody asks.
struct PacketAt {
    const uint8_t *pkts;
    const uint64_t *off;
    uint32_t stride, i;
    BNK_DEV const uint8_t *get() const { return pkts + (off ? off[i] : (uint64_t)i * stride); }
};

// `p`: the packet's first 24 bytes (as many as it has); `full`: the packet
// where it lies, looked at only for a header with options.
BNK_DEV bool parse_words(const u32x4 a, uint32_t dst_w, uint32_t l4_w, bool wide, uint32_t len, Parsed &o,
                         const PacketAt &full)
{
    const uint32_t w0 = a.x;
    if (((w0 >> 4) & 0xFu) != 4u) return false;
    const uint32_t ihl = (w0 & 0xFu) * 4u;
    if (ihl < 20u || len < ihl) return false;
    o.proto = (a.z >> 8) & 0xFFu;
    o.src = __builtin_bswap32(a.w);
    o.dst = __builtin_bswap32(dst_w);
    const uint32_t body = len - ihl;
    if (o.proto == 6u || o.proto == 17u) {
        if (body < 4u) return false;
        const uint32_t w = __builtin_bswap32(wide && ihl == 20u ? l4_w : ld32u(full.get() + ihl));
        o.sport = w >> 16;
        o.dport = w & 0xFFFFu;
        return true;
    }
    if (o.proto == 1u) {
        if (body < 1u) return false;
        o.sport = 0;
        o.dport = 0;
        return true;
    }
    return false;
}

BNK_DEV bool parse_packet(const uint8_t *p, uint32_t len, Parsed &o, const PacketAt &full)
{
    if (len < 20u) return false;
    const u32x4 a = *reinterpret_cast<const u32x4_unaligned *>(p);
    uint32_t dst_w, l4_w = 0;
    const bool wide = len >= 24u;
    if (wide) {
        const u32x2 b = *reinterpret_cast<const u32x2_unaligned *>(p + 16);
        dst_w = b.x;
        l4_w = b.y;
    } else {
        dst_w = ld32u(p + 16);
    }
    return parse_words(a, dst_w, l4_w, wide, len, o, full);
}

BNK_DEV uint32_t proto_class(uint32_t proto) { return proto == 1u ? 0u : proto == 6u ? 1u : 2u; }

// filter.go:108-117
BNK_DEV int64_t flow_ttl_ns(uint32_t proto)
{
    return proto == 6u ? 120000000000LL : 30000000000LL;
}

BNK_DEV uint64_t mix64(uint64_t x)
{
    x ^= x >> 33;
    x *= 0xff51afd7ed558ccdULL;
    x ^= x >> 33;
    x *= 0xc4ceb9fe1a85ec53ULL;
    x ^= x >> 33;
    return x;
}

// The two positions of a key in the small presence bitmap (a Bloom filter with
// two hash functions over SMALL_BITS bits, which is not a power of two).
BNK_DEV uint32_t small_bit0(uint64_t hsh) { return __umulhi((uint32_t)(hsh >> 32), SMALL_BITS); }
BNK_DEV uint32_t small_bit1(uint64_t hsh) { return __umulhi((uint32_t)hsh * 0x9E3779B1u, SMALL_BITS); }

struct FlowSlot {
    uint64_t word;   // stored key word (never 0)
    uint32_t base;   // first slot of the region
    uint32_t start;  // probe start within the region
    uint32_t bit;    // this key's bit in the presence bitmap
    uint32_t sbit0, sbit1; // and its two bits in the small one
};

BNK_DEV FlowSlot flow_slot(const FlowTableDev &ft, uint32_t remote, uint32_t rport, uint32_t lport,
                           uint32_t proto)
{
    FlowSlot s;
    const uint32_t region = proto_class(proto) * 2u + (remote >> 31);
    s.word = (1ULL << 63) | ((uint64_t)(remote & 0x7FFFFFFFu) << 32) | ((uint64_t)rport << 16) | lport;
    s.base = region * ft.cap;
    const uint64_t hsh = mix64(s.word ^ ((uint64_t)region << 59));
    s.start = (uint32_t)hsh & (ft.cap - 1u);
    s.bit = (uint32_t)(hsh >> 32) & ft.present_mask;
    s.sbit0 = small_bit0(hsh);
    s.sbit1 = small_bit1(hsh);
    return s;
}

// ---- rule lookup ----------------------------------------------------------

// Largest j with bounds[j] <= src; bounds[0] is 0 so j always exists.
template <class Ptr>
BNK_DEV uint32_t interval_of(Ptr bounds, uint32_t n, uint32_t top_step, uint32_t src)
{
    uint32_t pos = 0;
    for (uint32_t step = top_step; step; step >>= 1) {
        const uint32_t q = pos + step;
        if (q < n && bounds[q] <= src) pos = q;
    }
    return pos;
}

// The same with the jump table: only the cut points of src's address bucket
// are searched (a handful instead of thirteen halvings for 8192 cut points).
BNK_DEV uint32_t interval_of_jump(const uint32_t *bounds, const uint16_t *jump, uint32_t jump_lo,
                                  uint32_t jump_shift, uint32_t src)
{
    if (src < jump_lo) return 0; // below bounds[1]
    uint32_t b = (src - jump_lo) >> jump_shift;
    b = b < JUMP_BUCKETS ? b : JUMP_BUCKETS - 1u;
    uint32_t lo = jump[b], hi = jump[b + 1u] + 1u; // the answer lies in [lo, hi)
    if (b == JUMP_BUCKETS - 1u) {
        // the last bucket also takes everything above the last cut point
        hi = jump[JUMP_BUCKETS] + 1u;
    }
    while (hi - lo > 1u) {
        const uint32_t mid = (lo + hi) >> 1;
        if (bounds[mid] <= src) lo = mid;
        else hi = mid;
    }
    return lo;
}

// One word holds a range: key_lo << 14 | key_hi - key_lo.
BNK_DEV bool in_range(uint32_t e, uint32_t key) { return key - (e >> 14) <= (e & RANGE_MAX_SPAN); }

BNK_DEV bool quad_hit(uint4 v, uint32_t key)
{
    return in_range(v.x, key) || in_range(v.y, key) || in_range(v.z, key) || in_range(v.w, key);
}

// Value of x in lane J of this lane's quad (lanes 4k .. 4k+3).
template <int J>
BNK_DEV uint32_t quad_bcast(uint32_t x)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, J | J << 2 | J << 4 | J << 6, 0xF, 0xF, true);
}

// A list of more than 16 pieces: head is the first quad of the interval's own
// block, {RANGE_LONG, first block, blocks}.  Finds the block by its first key
// (the ranges are sorted and disjoint, so only that block can hold the key).
BNK_DEV bool long_list_hit(const RuleIndexDev &ri, uint32_t first, uint32_t nblk, uint32_t key)
{
    const uint4 *ob = reinterpret_cast<const uint4 *>(ri.ranges + (size_t)first * RANGE_BLOCK);
    uint32_t lo = 0, hi = nblk;
    while (hi - lo > 1u) {
        const uint32_t mid = (lo + hi) >> 1;
        if ((ob[4u * mid].x >> 14) <= key) lo = mid;
        else hi = mid;
    }
    const uint4 *b = ob + 4u * lo;
    const uint4 w0 = b[0], w1 = b[1], w2 = b[2], w3 = b[3];
    return quad_hit(w0, key) || quad_hit(w1, key) || quad_hit(w2, key) || quad_hit(w3, key);
}

// Rule lookup for the four packets of a quad of lanes at once; every lane of the
// wave must call it (lanes without a packet pass iv 0 and ignore the answer).
// The kernel is bound by the cache lookups its scattered loads cause, one per
// distinct line per load instruction.  A lane fetching its own 64-byte block
// with four 16-byte loads causes four; here the four lanes of a quad fetch one
// packet's block together, 16 bytes each, which the memory pipeline sees as a
// single 64-byte access, and do that for each of their four packets in turn.
// Each lane tests its 16 bytes against the key of the packet they belong to and
// the verdicts are gathered per quad with a wave-wide vote.
BNK_DEV bool rules_match_quad(const RuleIndexDev &ri, uint32_t lane, uint32_t iv, uint32_t src, uint32_t key)
{
    const uint32_t part = lane & 3u, qshift = lane & ~3u;
    const uint32_t *mine = ri.ranges + part * 4u;
    const uint32_t iv0 = quad_bcast<0>(iv), iv1 = quad_bcast<1>(iv), iv2 = quad_bcast<2>(iv), iv3 = quad_bcast<3>(iv);
    const uint4 p0 = *reinterpret_cast<const uint4 *>(mine + (size_t)iv0 * RANGE_BLOCK);
    const uint4 p1 = *reinterpret_cast<const uint4 *>(mine + (size_t)iv1 * RANGE_BLOCK);
    const uint4 p2 = *reinterpret_cast<const uint4 *>(mine + (size_t)iv2 * RANGE_BLOCK);
    const uint4 p3 = *reinterpret_cast<const uint4 *>(mine + (size_t)iv3 * RANGE_BLOCK);
    const unsigned long long h0 = __ballot(quad_hit(p0, quad_bcast<0>(key)));
    const unsigned long long h1 = __ballot(quad_hit(p1, quad_bcast<1>(key)));
    const unsigned long long h2 = __ballot(quad_hit(p2, quad_bcast<2>(key)));
    const unsigned long long h3 = __ballot(quad_hit(p3, quad_bcast<3>(key)));
    const unsigned long long hm = part == 0u ? h0 : part == 1u ? h1 : part == 2u ? h2 : h3;
    bool hit = ((hm >> qshift) & 0xFull) != 0ull;
    // a long list shows in the first word of its block, which the quad's first
    // lane holds for round j as p<j>; the votes are taken by all lanes together
    const unsigned long long l0 = __ballot(part == 0u && p0.x == RANGE_LONG);
    const unsigned long long l1 = __ballot(part == 0u && p1.x == RANGE_LONG);
    const unsigned long long l2 = __ballot(part == 0u && p2.x == RANGE_LONG);
    const unsigned long long l3 = __ballot(part == 0u && p3.x == RANGE_LONG);
    const unsigned long long lm = part == 0u ? l0 : part == 1u ? l1 : part == 2u ? l2 : l3;
    if ((lm >> qshift) & 1ull) {
        // rare: fetch the pointer words myself (the line is in L1 by now)
        const uint4 head = *reinterpret_cast<const uint4 *>(ri.ranges + (size_t)iv * RANGE_BLOCK);
        hit = long_list_hit(ri, head.y, head.z, key);
    }
    if (!hit)
        for (uint32_t w = 0; w < ri.n_wide; w++) {
            const uint4 r = ri.wide[w];
            if ((src & r.y) == r.x && key >= r.z && key <= r.w) hit = true;
        }
    return hit;
}

constexpr uint32_t LDS_BOUNDS_MAX = 24576; // 96 KiB of cut points
constexpr uint32_t FILTER_THREADS = 1024; // one copy of the index serves 16 waves

// filter.go:121-147 for a batch; enforcement is on (the host short-circuits
// allow-all mode).
__global__ __launch_bounds__(FILTER_THREADS, 8) void filter_check_kernel(FilterArgs a)
{
    extern __shared__ uint32_t lds[]; // the cut points when they fit, then the small presence bitmap
    const RuleIndexDev ri = a.rules;
    const bool in_lds = ri.n_bounds <= LDS_BOUNDS_MAX;
    const bool small = a.small_in_lds != 0u;
    const bool jumps = in_lds && ri.jump != nullptr;
    constexpr uint32_t JUMP_WORDS = (JUMP_BUCKETS + 2u) / 2u;
    uint32_t *lb = lds, *ljw = lds + ri.n_bounds;
    uint32_t *lsmall = lds + (in_lds ? ri.n_bounds + (jumps ? JUMP_WORDS : 0u) : 0u);
    const uint16_t *lj = reinterpret_cast<const uint16_t *>(ljw);
    if (in_lds)
        for (uint32_t q = threadIdx.x; q < ri.n_bounds; q += FILTER_THREADS) lb[q] = ri.bounds[q];
    if (jumps)
        for (uint32_t q = threadIdx.x; q < JUMP_WORDS; q += FILTER_THREADS)
            ljw[q] = reinterpret_cast<const uint32_t *>(ri.jump)[q];
    if (small)
        for (uint32_t q = threadIdx.x; q < SMALL_BITS / 32u; q += FILTER_THREADS)
            lsmall[q] = a.flows.present_small[q];
    __syncthreads();
    const uint32_t stride = gridDim.x * FILTER_THREADS;
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t n_pass = 0, n_drop = 0; // this wave's verdicts (the same in every lane)
    // whole waves stay in the loop together: the rule lookup is a joint effort
    for (uint32_t i0 = blockIdx.x * FILTER_THREADS + (threadIdx.x & ~63u); i0 < a.n; i0 += stride) {
        // t: this lane's place in the sweep; i: the packet it answers for
        const uint32_t t = i0 + lane;
        uint32_t i = t;
        bool valid;
        Parsed h{};
        if (a.heads) {
            valid = t < a.n;
            const uint32_t tt = valid ? t : 0u;
            const u32x4 r0 = *reinterpret_cast<const u32x4 *>(a.heads + 32ull * tt);
            const u32x4 r1 = *reinterpret_cast<const u32x4 *>(a.heads + 32ull * tt + 16);
            if (a.order) i = a.order[tt];
            // whoever wrote the records has checked the packets against the arena
            const uint32_t plen = r1.z;
            valid = valid && r1.w != 0u && plen >= 20u &&
                    parse_words(r0, r1.x, r1.y, plen >= 24u, plen, h, PacketAt{a.pkts, a.off, a.stride, i});
        } else {
            valid = t < a.n && !(a.gate && a.gate[t] == 0);
            if (valid) {
                const uint32_t len = a.lens ? a.lens[t] : a.len;
                const uint32_t plen = len - (len >= a.trim ? a.trim : len);
                const uint64_t at = a.off ? a.off[t] : (uint64_t)t * a.stride;
                if (beyond_arena(at, len, a.limit)) {
                    status_raise(a.status, STATUS_BOUNDS);
                    valid = false;
                } else {
                    valid = parse_packet(a.pkts + at, plen, h, PacketAt{a.pkts, a.off, a.stride, t});
                }
            }
        }
        uint32_t key = 0, iv = 0;
        bool maybe = false;
        FlowSlot s{};
        if (valid) {
            key = proto_class(h.proto) << 16 | h.dport;
            iv = jumps    ? interval_of_jump(lb, lj, ri.jump_lo, ri.jump_shift, h.src)
                 : in_lds ? interval_of(lb, ri.n_bounds, ri.top_step, h.src)
                          : interval_of(ri.bounds, ri.n_bounds, ri.top_step, h.src);
            // return traffic: remote = src, remotePort = srcPort, localPort = dstPort.
            // A clear presence bit means the key was never stored: no probe
            // needed.  The bits come from LDS when the small bitmap is in use;
            // otherwise the word is fetched alongside the rule list, not after it.
            s = flow_slot(a.flows, h.src, h.sport, h.dport, h.proto);
            if (small) {
                maybe = ((lsmall[s.sbit0 >> 5] >> (s.sbit0 & 31u)) & (lsmall[s.sbit1 >> 5] >> (s.sbit1 & 31u)) & 1u) != 0u;
                // one in eleven keys that were never stored passes the small
                // filter; the large one (a word from L2) turns nine in ten of
                // those away before they cost a 128-byte line of the table
                if (maybe) maybe = ((a.flows.present[s.bit >> 5] >> (s.bit & 31u)) & 1u) != 0u;
            } else {
                maybe = ((a.flows.present[s.bit >> 5] >> (s.bit & 31u)) & 1u) != 0u;
            }
        }
        uint8_t pass = 0;
        if (rules_match_quad(ri, lane, iv, h.src, key)) {
            pass = valid ? 1 : 0;
        } else if (valid) {
            for (uint32_t probe = 0; maybe && probe < a.flows.cap; probe++) {
                FlowSlotMem *slot = a.flows.slots + s.base + ((s.start + probe) & (a.flows.cap - 1u));
                // Keys only change in NoteOutbound batches, never during this
                // kernel.  An expiry that another lane is refreshing may be seen
                // old or new: both are values this batch's single `now` allows.
                const ulonglong2 cur = *reinterpret_cast<const ulonglong2 *>(slot);
                if (cur.x == 0) break; // miss
                if (cur.x != s.word) continue;
                unsigned long long *ep = reinterpret_cast<unsigned long long *>(&slot->exp);
                const int64_t e = (int64_t)cur.y;
                if (e == FLOW_TOMB) break; // deleted earlier
                if (a.now < e) {
                    // keep-alive on traffic (filter.go:141)
                    // A plain store on purpose.  Every lane that refreshes this
                    // flow in this batch writes the same value, a reader may see
                    // the old expiry or the new one (both lie after `now`, so the
                    // verdict is the same), and deletion cannot race with it: all
                    // lanes see the same side of `now < e`.  An atomic store would
                    // have to be visible across the eight L2s at once and is
                    // pushed out to memory for it; this one waits for the end of
                    // the kernel like any other store.
                    // (`volatile` gets the same treatment as an atomic, hence not even that.)
                    *ep = (unsigned long long)(a.now + flow_ttl_ns(h.proto));
                    pass = 1;
                } else {
                    // expired: delete (filter.go:144); only the lane that
                    // turns it into a tombstone adjusts the entry count
                    const int64_t prev = (int64_t)atomicExch(ep, (unsigned long long)FLOW_TOMB);
                    if (prev != FLOW_TOMB) atomicSub(&a.flows.counters[FLOW_LIVE], 1u);
                }
                break;
            }
        }
        if (t < a.n) {
            a.verdict[i] = pass;
            // a packet WireGuard delivered and this filter denied (BNK_WG_OK is 0)
            if (a.wg_result && !pass && a.wg_result[i] == 0) a.wg_result[i] = BNK_WG_FILTERED;
        }
        if (a.tally) {
            const unsigned long long in = __ballot(t < a.n), ok = __ballot(t < a.n && pass != 0);
            n_pass += (uint32_t)__popcll(ok);
            n_drop += (uint32_t)__popcll(in & ~ok);
        }
    }
    if (a.tally && lane == 0u) {
        tally_bump(a.tally, TALLY_ALLOWED, n_pass);
        tally_bump(a.tally, TALLY_DENIED, n_drop);
    }
}

// filter.go:189-201 for a batch (the sweep of :202-208 follows as its own
// kernels because it depends on the entry count after every insert).
__global__ __launch_bounds__(256) void filter_note_kernel(FilterArgs a)
{
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < a.n; i += stride) {
        const uint64_t at = a.off ? a.off[i] : (uint64_t)i * a.stride;
        const uint32_t len = a.lens ? a.lens[i] : a.len;
        if (beyond_arena(at, len, a.limit)) {
            status_raise(a.status, STATUS_BOUNDS);
            continue;
        }
        const uint8_t *p = a.pkts + at;
        Parsed h;
        if (!parse_packet(p, len, h, PacketAt{a.pkts, a.off, a.stride, i})) continue;
        // remote = dst, remotePort = dstPort, localPort = srcPort
        const FlowSlot s = flow_slot(a.flows, h.dst, h.dport, h.sport, h.proto);
        const unsigned long long expiry = (unsigned long long)(a.now + flow_ttl_ns(h.proto));
        bool placed = false;
        for (uint32_t probe = 0; probe < a.flows.cap; probe++) {
            FlowSlotMem *slot = a.flows.slots + s.base + ((s.start + probe) & (a.flows.cap - 1u));
            unsigned long long *kp = reinterpret_cast<unsigned long long *>(&slot->key);
            const unsigned long long old = atomicCAS(kp, 0ULL, (unsigned long long)s.word);
            if (old == 0ULL) {
                atomicAdd(&a.flows.counters[FLOW_CLAIMED], 1u);
                atomicOr(&a.flows.present[s.bit >> 5], 1u << (s.bit & 31u));
                atomicOr(&a.flows.present_small[s.sbit0 >> 5], 1u << (s.sbit0 & 31u));
                atomicOr(&a.flows.present_small[s.sbit1 >> 5], 1u << (s.sbit1 & 31u));
            }
            if (old == 0ULL || old == s.word) {
                unsigned long long *ep = reinterpret_cast<unsigned long long *>(&slot->exp);
                // every lane of this batch writes the same expiry for this key;
                // the one that replaces a tombstone (fresh slots start as
                // tombstones) brings the entry into the map
                const int64_t prev = (int64_t)atomicExch(ep, expiry);
                if (prev == FLOW_TOMB) atomicAdd(&a.flows.counters[FLOW_LIVE], 1u);
                placed = true;
                break;
            }
        }
        if (!placed) status_raise(a.status, STATUS_FLOWS_FULL);
    }
}

// filter.go:202: the sweep runs only when the map holds more than 4096
// entries; decided once so every thread of the sweep sees the same answer.
__global__ void flow_sweep_flag_kernel(FlowTableDev ft)
{
    if (threadIdx.x == 0 && blockIdx.x == 0)
        ft.counters[FLOW_SWEEP] = ft.counters[FLOW_LIVE] > 4096u ? 1u : 0u;
}

// filter.go:203-207: delete entries with now.After(exp).
__global__ __launch_bounds__(256) void flow_sweep_kernel(FlowTableDev ft, int64_t now)
{
    if (ft.counters[FLOW_SWEEP] == 0u) return;
    const uint32_t total = ft.cap * FLOW_REGIONS;
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t idx = blockIdx.x * 256u + threadIdx.x; idx < total; idx += stride) {
        if (ft.slots[idx].key == 0) continue;
        const int64_t e = ft.slots[idx].exp;
        if (e != FLOW_TOMB && now > e) {
            ft.slots[idx].exp = FLOW_TOMB;
            atomicSub(&ft.counters[FLOW_LIVE], 1u);
        }
    }
}

// Moves every entry of the map into a larger table (tombstones are dropped).
__global__ __launch_bounds__(256) void flow_rehash_kernel(FlowTableDev from, FlowTableDev to,
                                                          uint32_t *status)
{
    const uint32_t total = from.cap * FLOW_REGIONS;
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t idx = blockIdx.x * 256u + threadIdx.x; idx < total; idx += stride) {
        const uint64_t word = from.slots[idx].key;
        const int64_t e = from.slots[idx].exp;
        if (word == 0 || e == FLOW_TOMB) continue;
        const uint32_t region = idx / from.cap;
        const uint64_t hsh = mix64(word ^ ((uint64_t)region << 59));
        const uint32_t start = (uint32_t)hsh & (to.cap - 1u);
        const uint32_t bit = (uint32_t)(hsh >> 32) & to.present_mask;
        bool placed = false;
        for (uint32_t probe = 0; probe < to.cap; probe++) {
            const uint32_t t = region * to.cap + ((start + probe) & (to.cap - 1u));
            unsigned long long *kp = reinterpret_cast<unsigned long long *>(&to.slots[t].key);
            if (atomicCAS(kp, 0ULL, (unsigned long long)word) == 0ULL) {
                to.slots[t].exp = e;
                atomicOr(&to.present[bit >> 5], 1u << (bit & 31u));
                const uint32_t b0 = small_bit0(hsh), b1 = small_bit1(hsh);
                atomicOr(&to.present_small[b0 >> 5], 1u << (b0 & 31u));
                atomicOr(&to.present_small[b1 >> 5], 1u << (b1 & 31u));
                atomicAdd(&to.counters[FLOW_CLAIMED], 1u);
                atomicAdd(&to.counters[FLOW_LIVE], 1u);
                placed = true;
                break;
            }
        }
        if (!placed) status_raise(status, STATUS_FLOWS_FULL);
    }
}

__global__ __launch_bounds__(256) void fill_u64_kernel(uint64_t *p, uint32_t n, uint64_t v)
{
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += stride) p[i] = v;
}

__global__ __launch_bounds__(256) void flow_clear_kernel(FlowSlotMem *p, uint32_t n)
{
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += stride) {
        p[i].key = 0;
        p[i].exp = FLOW_TOMB;
    }
}

__global__ __launch_bounds__(256) void fill_u8_kernel(uint8_t *p, uint32_t n, uint8_t v)
{
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += stride) p[i] = v;
}

static uint32_t grid_for(uint32_t n, uint32_t max_blocks)
{
    uint32_t b = (n + 255u) / 256u;
    return b < 1u ? 1u : (b > max_blocks ? max_blocks : b);
}

hipError_t launch_fill_u64(uint64_t *p, uint32_t n, uint64_t v, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(fill_u64_kernel, dim3(grid_for(n, 4096)), dim3(256), 0, s, p, n, v);
    return hipGetLastError();
}

hipError_t launch_flow_clear(FlowSlotMem *p, uint32_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(flow_clear_kernel, dim3(grid_for(n, 4096)), dim3(256), 0, s, p, n);
    return hipGetLastError();
}

hipError_t launch_fill_u8(uint8_t *p, uint32_t n, uint8_t v, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(fill_u8_kernel, dim3(grid_for(n, 4096)), dim3(256), 0, s, p, n, v);
    return hipGetLastError();
}

hipError_t launch_filter_check(const FilterArgs &args, uint32_t max_blocks, hipStream_t s)
{
    if (args.n == 0) return hipSuccess;
    FilterArgs a = args;
    uint32_t lds = a.rules.n_bounds <= LDS_BOUNDS_MAX
                       ? a.rules.n_bounds * 4u + (a.rules.jump ? (JUMP_BUCKETS + 2u) * 2u : 0u)
                       : 0u;
    // the small bitmap rides along while two workgroups still fit a CU's 160 KiB
    a.small_in_lds = a.flows.small_ok && lds + SMALL_BITS / 8u <= 80u * 1024u ? 1u : 0u;
    if (a.small_in_lds) lds += SMALL_BITS / 8u;
    if (lds > 48u * 1024u) {
        // more dynamic LDS than the default limit: opt in (gfx950 has 160 KiB per CU)
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(filter_check_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)(LDS_BOUNDS_MAX * 4u + (JUMP_BUCKETS + 2u) * 2u));
        if (e != hipSuccess) return e;
    }
    // one index copy per workgroup: as many workgroups per CU as their LDS allows, two at most
    const uint32_t per_cu = lds > 80u * 1024u ? 1u : 2u;
    uint32_t blocks = (a.n + FILTER_THREADS - 1u) / FILTER_THREADS;
    const uint32_t cap = (max_blocks / 8u) * per_cu; // max_blocks is 8 per CU
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(filter_check_kernel, dim3(blocks), dim3(FILTER_THREADS), lds, s, a);
    return hipGetLastError();
}

hipError_t launch_filter_note(const FilterArgs &a, uint32_t max_blocks, bool may_sweep, hipStream_t s)
{
    if (a.n == 0) return hipSuccess;
    hipLaunchKernelGGL(filter_note_kernel, dim3(grid_for(a.n, max_blocks)), dim3(256), 0, s, a);
    // filter.go:202: no sweep while the map holds at most 4096 entries
    if (!may_sweep) return hipGetLastError();
    hipLaunchKernelGGL(flow_sweep_flag_kernel, dim3(1), dim3(64), 0, s, a.flows);
    hipLaunchKernelGGL(flow_sweep_kernel, dim3(grid_for(a.flows.cap * FLOW_REGIONS, max_blocks)),
                       dim3(256), 0, s, a.flows, a.now);
    return hipGetLastError();
}

hipError_t launch_flow_rehash(const FlowTableDev &from, const FlowTableDev &to, uint32_t *status,
                              uint32_t max_blocks, hipStream_t s)
{
    hipLaunchKernelGGL(flow_rehash_kernel, dim3(grid_for(from.cap * FLOW_REGIONS, max_blocks)),
                       dim3(256), 0, s, from, to, status);
    return hipGetLastError();
}

} // namespace bnk
