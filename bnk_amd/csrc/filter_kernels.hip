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
// the key intervals of all rules covering it.  A packet does one binary search
// over the cut points (staged in LDS) and one over its interval's key list.
// "Any rule matches" is all the reference asks (filter.go:131-135), so this is
// exact.  Rules too wide to expand go to a short list every packet scans.
//
// Flow table.  Open addressing in HBM, one 64-bit key word and one 64-bit
// expiry per slot.  The reference's flowKey (remote addr, remote port, local
// port, proto) is 66 bits with the protocol class; the class and the top
// address bit select one of six equal regions and the other 63 bits plus a
// marker bit form the key word, so 0 can mean "empty" and a slot is claimed
// with one 64-bit compare-and-swap.  Deleted entries keep their key and carry
// expiry FLOW_TOMB.
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

// filter.go:71-106
BNK_DEV bool parse_packet(const uint8_t *p, uint32_t len, Parsed &o)
{
    if (len < 20u) return false;
    const uint32_t w0 = ld32u(p);
    if (((w0 >> 4) & 0xFu) != 4u) return false;
    const uint32_t ihl = (w0 & 0xFu) * 4u;
    if (ihl < 20u || len < ihl) return false;
    o.proto = (ld32u(p + 8) >> 8) & 0xFFu;
    o.src = __builtin_bswap32(ld32u(p + 12));
    o.dst = __builtin_bswap32(ld32u(p + 16));
    const uint32_t body = len - ihl;
    if (o.proto == 6u || o.proto == 17u) {
        if (body < 4u) return false;
        const uint32_t w = __builtin_bswap32(ld32u(p + ihl));
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

struct FlowSlot {
    uint64_t word;   // stored key word (never 0)
    uint32_t base;   // first slot of the region
    uint32_t start;  // probe start within the region
};

BNK_DEV FlowSlot flow_slot(const FlowTableDev &ft, uint32_t remote, uint32_t rport, uint32_t lport,
                           uint32_t proto)
{
    FlowSlot s;
    const uint32_t region = proto_class(proto) * 2u + (remote >> 31);
    s.word = (1ULL << 63) | ((uint64_t)(remote & 0x7FFFFFFFu) << 32) | ((uint64_t)rport << 16) | lport;
    s.base = region * ft.cap;
    s.start = (uint32_t)mix64(s.word ^ ((uint64_t)region << 59)) & (ft.cap - 1u);
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

BNK_DEV bool rules_match(const RuleIndexDev &ri, uint32_t interval, uint32_t src, uint32_t key)
{
    uint32_t lo = ri.starts[interval], hi = ri.starts[interval + 1];
    // last range with klo <= key
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        const uint2 r = ri.ranges[mid];
        if (r.x <= key) {
            if (key <= r.y) return true;
            lo = mid + 1;
        } else {
            hi = mid;
        }
    }
    for (uint32_t w = 0; w < ri.n_wide; w++) {
        const uint4 r = ri.wide[w];
        if ((src & r.y) == r.x && key >= r.z && key <= r.w) return true;
    }
    return false;
}

constexpr uint32_t LDS_BOUNDS_MAX = 12288; // 48 KiB of cut points

// filter.go:121-147 for a batch; enforcement is on (the host short-circuits
// allow-all mode).
__global__ __launch_bounds__(256) void filter_check_kernel(FilterArgs a)
{
    extern __shared__ uint32_t lb[]; // n_bounds words when they fit, else unused
    const RuleIndexDev ri = a.rules;
    const bool in_lds = ri.n_bounds <= LDS_BOUNDS_MAX;
    if (in_lds) {
        for (uint32_t q = threadIdx.x; q < ri.n_bounds; q += 256u) lb[q] = ri.bounds[q];
        __syncthreads();
    }
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < a.n; i += stride) {
        if (a.gate && a.gate[i] == 0) {
            a.verdict[i] = 0;
            continue;
        }
        const uint8_t *p = a.pkts + (a.off ? a.off[i] : (uint64_t)i * a.stride);
        const uint32_t len = a.lens ? a.lens[i] : a.len;
        Parsed h;
        uint8_t pass = 0;
        if (parse_packet(p, len - (len >= a.trim ? a.trim : len), h)) {
            const uint32_t key = proto_class(h.proto) << 16 | h.dport;
            const uint32_t iv = in_lds ? interval_of(lb, ri.n_bounds, ri.top_step, h.src)
                                       : interval_of(ri.bounds, ri.n_bounds, ri.top_step, h.src);
            if (rules_match(ri, iv, h.src, key)) {
                pass = 1;
            } else {
                // return traffic: remote = src, remotePort = srcPort, localPort = dstPort
                const FlowSlot s = flow_slot(a.flows, h.src, h.sport, h.dport, h.proto);
                for (uint32_t probe = 0; probe < a.flows.cap; probe++) {
                    const uint32_t idx = s.base + ((s.start + probe) & (a.flows.cap - 1u));
                    const uint64_t kw = __atomic_load_n(&a.flows.keys[idx], __ATOMIC_RELAXED);
                    if (kw == 0) break; // miss
                    if (kw != s.word) continue;
                    unsigned long long *ep = reinterpret_cast<unsigned long long *>(&a.flows.exp[idx]);
                    const int64_t e = (int64_t)__atomic_load_n(ep, __ATOMIC_RELAXED);
                    if (e == FLOW_TOMB) break; // deleted earlier
                    if (a.now < e) {
                        // keep-alive on traffic (filter.go:141)
                        __atomic_store_n(ep, (unsigned long long)(a.now + flow_ttl_ns(h.proto)),
                                         __ATOMIC_RELAXED);
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
        }
        a.verdict[i] = pass;
    }
}

// filter.go:189-201 for a batch (the sweep of :202-208 follows as its own
// kernels because it depends on the entry count after every insert).
__global__ __launch_bounds__(256) void filter_note_kernel(FilterArgs a)
{
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < a.n; i += stride) {
        const uint8_t *p = a.pkts + (a.off ? a.off[i] : (uint64_t)i * a.stride);
        const uint32_t len = a.lens ? a.lens[i] : a.len;
        Parsed h;
        if (!parse_packet(p, len, h)) continue;
        // remote = dst, remotePort = dstPort, localPort = srcPort
        const FlowSlot s = flow_slot(a.flows, h.dst, h.dport, h.sport, h.proto);
        const unsigned long long expiry = (unsigned long long)(a.now + flow_ttl_ns(h.proto));
        bool placed = false;
        for (uint32_t probe = 0; probe < a.flows.cap; probe++) {
            const uint32_t idx = s.base + ((s.start + probe) & (a.flows.cap - 1u));
            unsigned long long *kp = reinterpret_cast<unsigned long long *>(&a.flows.keys[idx]);
            const unsigned long long old = atomicCAS(kp, 0ULL, (unsigned long long)s.word);
            if (old == 0ULL) atomicAdd(&a.flows.counters[FLOW_CLAIMED], 1u);
            if (old == 0ULL || old == s.word) {
                unsigned long long *ep = reinterpret_cast<unsigned long long *>(&a.flows.exp[idx]);
                // every lane of this batch writes the same expiry for this key;
                // the one that replaces a tombstone (fresh slots start as
                // tombstones) brings the entry into the map
                const int64_t prev = (int64_t)atomicExch(ep, expiry);
                if (prev == FLOW_TOMB) atomicAdd(&a.flows.counters[FLOW_LIVE], 1u);
                placed = true;
                break;
            }
        }
        if (!placed) atomicOr(a.status, STATUS_FLOWS_FULL);
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
        if (ft.keys[idx] == 0) continue;
        const int64_t e = ft.exp[idx];
        if (e != FLOW_TOMB && now > e) {
            ft.exp[idx] = FLOW_TOMB;
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
        const uint64_t word = from.keys[idx];
        const int64_t e = from.exp[idx];
        if (word == 0 || e == FLOW_TOMB) continue;
        const uint32_t region = idx / from.cap;
        const uint32_t start = (uint32_t)mix64(word ^ ((uint64_t)region << 59)) & (to.cap - 1u);
        bool placed = false;
        for (uint32_t probe = 0; probe < to.cap; probe++) {
            const uint32_t t = region * to.cap + ((start + probe) & (to.cap - 1u));
            unsigned long long *kp = reinterpret_cast<unsigned long long *>(&to.keys[t]);
            if (atomicCAS(kp, 0ULL, (unsigned long long)word) == 0ULL) {
                to.exp[t] = e;
                atomicAdd(&to.counters[FLOW_CLAIMED], 1u);
                atomicAdd(&to.counters[FLOW_LIVE], 1u);
                placed = true;
                break;
            }
        }
        if (!placed) atomicOr(status, STATUS_FLOWS_FULL);
    }
}

__global__ __launch_bounds__(256) void fill_u64_kernel(uint64_t *p, uint32_t n, uint64_t v)
{
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += stride) p[i] = v;
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

hipError_t launch_fill_u8(uint8_t *p, uint32_t n, uint8_t v, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(fill_u8_kernel, dim3(grid_for(n, 4096)), dim3(256), 0, s, p, n, v);
    return hipGetLastError();
}

hipError_t launch_filter_check(const FilterArgs &a, uint32_t max_blocks, hipStream_t s)
{
    if (a.n == 0) return hipSuccess;
    const uint32_t lds = a.rules.n_bounds <= LDS_BOUNDS_MAX ? a.rules.n_bounds * 4u : 0u;
    hipLaunchKernelGGL(filter_check_kernel, dim3(grid_for(a.n, max_blocks)), dim3(256), lds, s, a);
    return hipGetLastError();
}

hipError_t launch_filter_note(const FilterArgs &a, uint32_t max_blocks, hipStream_t s)
{
    if (a.n == 0) return hipSuccess;
    hipLaunchKernelGGL(filter_note_kernel, dim3(grid_for(a.n, max_blocks)), dim3(256), 0, s, a);
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
