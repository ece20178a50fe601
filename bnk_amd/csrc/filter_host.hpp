// Host-side state of the packet filter: the compiled rule index and the flow
// table's capacity management.  The per-packet work is in filter_kernels.hip.
#pragma once

#include <algorithm>
#include <string>
#include <vector>

#include "ctx.hpp"
#include "filter_dev.hpp"

namespace bnk {

struct HostRuleIndex {
    std::vector<uint32_t> bounds;
    std::vector<uint16_t> jump; // see RuleIndexDev::jump; empty when not applicable
    uint32_t jump_lo = 0, jump_shift = 0;
    std::vector<uint32_t> ranges;
    std::vector<uint4> wide;
};

// Upper limit on expanded (interval, key range) entries; rules that would push
// the total beyond it are kept in the wide list instead.
constexpr size_t RULE_EXPANSION_BUDGET = size_t(1) << 22;

// Compiles bnk_rule tuples (each one prefix x one port range of an
// acl.CompiledRule, internal/acl/acl.go:33-42) into the interval index the
// check kernel searches.  Returns false with a message for a mask that is not
// a prefix mask.
inline bool build_rule_index(const bnk_rule *rules, uint32_t n, HostRuleIndex &out,
                             std::string &err, size_t budget = RULE_EXPANSION_BUDGET)
{
    struct Tuple {
        uint32_t lo, hi, klo, khi, net, mask;
        uint32_t a = 0, b = 0;
        bool wide = false;
    };
    std::vector<Tuple> ts;
    ts.reserve(n);
    for (uint32_t i = 0; i < n; i++) {
        const bnk_rule &r = rules[i];
        uint32_t cls;
        if (r.proto == 1) cls = 0;
        else if (r.proto == 6) cls = 1;
        else if (r.proto == 17) cls = 2;
        else continue; // acl.go:150: no parsed packet carries another protocol name
        const uint32_t inv = ~r.src_mask;
        if ((inv & (inv + 1u)) != 0u) {
            err = "rule " + std::to_string(i) + ": src_mask is not a prefix mask";
            return false;
        }
        Tuple t;
        if (cls == 0) {
            t.klo = 0;
            t.khi = 0xFFFFu; // acl.go:163-165: icmp ignores ports
        } else {
            if (r.port_first > r.port_last) continue; // empty range never matches
            t.klo = cls << 16 | r.port_first;
            t.khi = cls << 16 | r.port_last;
        }
        t.mask = r.src_mask;
        t.net = r.src_net & r.src_mask; // Contains ignores host bits
        t.lo = t.net;
        t.hi = t.net | inv;
        ts.push_back(t);
    }
    std::vector<uint32_t> &B = out.bounds;
    B.clear();
    B.push_back(0);
    for (const Tuple &t : ts) {
        B.push_back(t.lo);
        if (t.hi != 0xFFFFFFFFu) B.push_back(t.hi + 1u);
    }
    std::sort(B.begin(), B.end());
    B.erase(std::unique(B.begin(), B.end()), B.end());
    const uint32_t nb = (uint32_t)B.size();
    size_t total = 0;
    for (Tuple &t : ts) {
        t.a = (uint32_t)(std::lower_bound(B.begin(), B.end(), t.lo) - B.begin());
        t.b = t.hi == 0xFFFFFFFFu
                  ? nb
                  : (uint32_t)(std::lower_bound(B.begin(), B.end(), t.hi + 1u) - B.begin());
        total += t.b - t.a;
    }
    out.wide.clear();
    if (total > budget) {
        std::vector<uint32_t> by_cover(ts.size());
        for (uint32_t i = 0; i < ts.size(); i++) by_cover[i] = i;
        std::sort(by_cover.begin(), by_cover.end(), [&](uint32_t x, uint32_t y) {
            return ts[x].b - ts[x].a > ts[y].b - ts[y].a;
        });
        for (uint32_t idx : by_cover) {
            if (total <= budget) break;
            Tuple &t = ts[idx];
            t.wide = true;
            total -= t.b - t.a;
            out.wide.push_back(make_uint4(t.net, t.mask, t.klo, t.khi));
        }
    }
    std::vector<uint32_t> cnt(nb + 1, 0);
    for (const Tuple &t : ts)
        if (!t.wide)
            for (uint32_t j = t.a; j < t.b; j++) cnt[j]++;
    std::vector<uint32_t> raw_start(nb + 1, 0);
    for (uint32_t j = 0; j < nb; j++) raw_start[j + 1] = raw_start[j] + cnt[j];
    std::vector<uint2> raw(raw_start[nb]);
    std::vector<uint32_t> fill(raw_start.begin(), raw_start.end() - 1);
    for (const Tuple &t : ts)
        if (!t.wide)
            for (uint32_t j = t.a; j < t.b; j++) raw[fill[j]++] = make_uint2(t.klo, t.khi);
    // per interval: sort by key_lo, merge overlapping or adjacent key ranges,
    // cut what is left into one-word pieces; block j takes interval j's pieces,
    // or points at blocks appended behind the first nb when there are too many
    // jump table over the populated part of the address space
    out.jump.clear();
    if (nb >= 2 && nb <= 0xFFFFu) {
        out.jump_lo = B[1];
        const uint32_t span = B[nb - 1] - B[1];
        out.jump_shift = 0;
        while ((span >> out.jump_shift) >= JUMP_BUCKETS) out.jump_shift++;
        out.jump.resize(JUMP_BUCKETS + 1);
        uint32_t j = 1;
        for (uint32_t b = 0; b <= JUMP_BUCKETS; b++) {
            const uint64_t start = (uint64_t)B[1] + ((uint64_t)b << out.jump_shift);
            while (j + 1 < nb && (uint64_t)B[j + 1] <= start) j++;
            out.jump[b] = (uint16_t)j;
        }
    }
    out.ranges.assign((size_t)nb * RANGE_BLOCK, RANGE_PAD);
    std::vector<uint2> merged;
    std::vector<uint32_t> pieces;
    for (uint32_t j = 0; j < nb; j++) {
        auto lo = raw.begin() + raw_start[j], hi = raw.begin() + raw_start[j + 1];
        std::sort(lo, hi, [](const uint2 &x, const uint2 &y) { return x.x < y.x; });
        merged.clear();
        for (auto it = lo; it != hi; ++it) {
            if (!merged.empty() && it->x <= merged.back().y + 1u) {
                if (it->y > merged.back().y) merged.back().y = it->y;
            } else {
                merged.push_back(*it);
            }
        }
        pieces.clear();
        for (const uint2 &r : merged)
            for (uint32_t at = r.x;; at += RANGE_MAX_SPAN + 1u) {
                const uint32_t span = std::min(r.y - at, RANGE_MAX_SPAN);
                pieces.push_back(at << 14 | span);
                if (at + span == r.y) break;
            }
        uint32_t *blk = out.ranges.data() + (size_t)j * RANGE_BLOCK;
        if (pieces.size() <= RANGE_BLOCK) {
            std::copy(pieces.begin(), pieces.end(), blk);
        } else {
            const size_t first = out.ranges.size() / RANGE_BLOCK;
            out.ranges.insert(out.ranges.end(), pieces.begin(), pieces.end());
            while (out.ranges.size() % RANGE_BLOCK) out.ranges.push_back(RANGE_PAD);
            blk = out.ranges.data() + (size_t)j * RANGE_BLOCK; // the vector may have moved
            blk[0] = RANGE_LONG;
            blk[1] = (uint32_t)first;
            blk[2] = (uint32_t)(out.ranges.size() / RANGE_BLOCK - first);
        }
    }
    return true;
}

struct FilterState {
    bool enforce = false; // filter.New: allow-all until a policy arrives (filter.go:41-43)
    DevBuf bounds, jump, ranges, wide;
    RuleIndexDev ridx{};
    DevBuf slots, counters, present, present_small;
    FlowTableDev flows{};
    uint64_t claimed_upper = 0; // host bound on slots ever claimed in the current table
    uint32_t max_blocks = 2048;
    void release()
    {
        for (DevBuf *b : {&bounds, &jump, &ranges, &wide, &slots, &counters, &present, &present_small}) b->release();
    }
};

constexpr uint32_t FLOW_CAP_INITIAL = 8192;      // slots per region
constexpr uint32_t FLOW_CAP_MAX = 1u << 26;

FilterState *filter_create(hipStream_t s, int cu_count);
// Makes room for n_new more distinct flows before a NoteOutbound launch (may
// rehash the table, which waits for the context's stream).
int flows_reserve(bnk_ctx *ctx, uint32_t n_new);
void filter_destroy(FilterState *f);

} // namespace bnk
