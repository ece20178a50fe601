// Host-side mirror of the reference's filter interface over libbnkhip.so.
//
// The reference is Go; this image has no Go toolchain, so the adapter a cgo
// build would provide is written in C++ above the same C ABI
// (include/bnkhip.h) with the reference's names, argument meaning and error
// behaviour:
//   filter.New / SetRules / SetAllowAll / CheckInbound / NoteOutbound
//       internal/filter/filter.go:41-59, 121-147, 189-209
//   filter.WrapTUN and filteredTUN.Read / Write
//       internal/filter/filter.go:151-186
//   acl.CompiledRule / PortRange
//       internal/acl/acl.go:33-42
//   tun.Device method set as the reference's fake implements it
//       internal/filter/tun_test.go:19-41
// Go's []byte is a (pointer, length) view; ByteSlice is the same thing.
#pragma once

#include <stdint.h>

#include <chrono>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/bnkhip.h"
#include "bnk_coalesce.hpp"

namespace bnk_host {

struct ByteSlice {
    uint8_t *data = nullptr;
    size_t len = 0;
    ByteSlice() = default;
    ByteSlice(uint8_t *d, size_t n) : data(d), len(n) {}
    explicit ByteSlice(std::vector<uint8_t> &v) : data(v.data()), len(v.size()) {}
    // b[from:]
    ByteSlice from(size_t off) const { return off <= len ? ByteSlice(data + off, len - off) : ByteSlice(); }
    // b[from:to]
    ByteSlice sub(size_t a, size_t b) const { return (a <= b && b <= len) ? ByteSlice(data + a, b - a) : ByteSlice(); }
};

// Go's error: empty string is nil.
using Error = std::string;

// netip.Prefix, as far as Contains on an IPv4 address looks at it.
struct Prefix {
    uint32_t addr = 0; // a<<24 | b<<16 | c<<8 | d
    int bits = -1;     // -1 is the invalid prefix
    bool is4 = true;
};

inline Prefix MustParsePrefix(const std::string &s)
{
    unsigned a, b, c, d;
    int bits;
    if (sscanf(s.c_str(), "%u.%u.%u.%u/%d", &a, &b, &c, &d, &bits) != 5 || a > 255 || b > 255 ||
        c > 255 || d > 255 || bits < 0 || bits > 32)
        throw std::invalid_argument("MustParsePrefix: " + s);
    return Prefix{a << 24 | b << 16 | c << 8 | d, bits, true};
}

struct PortRange {
    uint16_t First = 0, Last = 0;
};

struct CompiledRule {
    std::vector<Prefix> Srcs;
    std::string Proto; // "tcp" | "udp" | "icmp"
    std::vector<PortRange> Ports;
};

// The (prefix, range) pairs of a rule set, as the C ABI takes them.
inline std::vector<bnk_rule> FlattenRules(const std::vector<CompiledRule> &rules)
{
    std::vector<bnk_rule> out;
    for (const CompiledRule &r : rules) {
        uint8_t proto;
        if (r.Proto == "tcp") proto = 6;
        else if (r.Proto == "udp") proto = 17;
        else if (r.Proto == "icmp") proto = 1;
        else continue; // acl.go:150: never equal to a parsed packet's protoName
        std::vector<PortRange> ports = r.Ports;
        if (proto == 1) ports = {PortRange{0, 0}}; // acl.go:163-165
        for (const Prefix &p : r.Srcs) {
            if (p.bits < 0 || p.bits > 32 || !p.is4) continue; // Contains is false
            const uint32_t mask = p.bits == 0 ? 0u : 0xFFFFFFFFu << (32 - p.bits);
            for (const PortRange &pr : ports) {
                bnk_rule t{};
                t.src_net = p.addr & mask;
                t.src_mask = mask;
                t.port_first = pr.First;
                t.port_last = pr.Last;
                t.proto = proto;
                out.push_back(t);
            }
        }
    }
    return out;
}

inline int64_t UnixNano(std::chrono::system_clock::time_point t)
{
    return std::chrono::duration_cast<std::chrono::nanoseconds>(t.time_since_epoch()).count();
}

// What the TUN wrapper needs from a filter: one verdict per packet of a batch,
// and the outbound packets of a batch recorded.
struct PacketFilter {
    virtual ~PacketFilter() = default;
    virtual std::vector<uint8_t> CheckInboundBatch(const std::vector<ByteSlice> &pkts, int64_t now_ns) = 0;
    virtual void NoteOutboundBatch(const std::vector<ByteSlice> &pkts, int64_t now_ns) = 0;
};

// filter.Filter.  One GPU context per filter; calls are serialised inside the
// library as the reference serialises them with its mutex (filter.go:34).
class Filter : public PacketFilter {
public:
    // filter.New: allow-all until a policy arrives.
    explicit Filter(int device = 0)
    {
        if (int rc = bnk_init(device, &ctx_))
            throw std::runtime_error(std::string("bnk_init: ") + bnk_last_error(nullptr) + " (" +
                                     std::to_string(rc) + ")");
    }
    ~Filter() { bnk_shutdown(ctx_); }
    Filter(const Filter &) = delete;
    Filter &operator=(const Filter &) = delete;

    void SetRules(const std::vector<CompiledRule> &rules)
    {
        const std::vector<bnk_rule> flat = FlattenRules(rules);
        check(bnk_filter_set_rules(ctx_, flat.data(), (uint32_t)flat.size()));
    }
    void SetAllowAll() { check(bnk_filter_set_allow_all(ctx_)); }

    bool CheckInbound(ByteSlice pkt, int64_t now_ns)
    {
        const uint8_t *p = pkt.data;
        const uint32_t len = (uint32_t)pkt.len;
        uint8_t v = 0;
        check(bnk_filter_check_inbound_ptrs(ctx_, &p, &len, 1, now_ns, &v));
        return v != 0;
    }
    void NoteOutbound(ByteSlice pkt, int64_t now_ns)
    {
        const uint8_t *p = pkt.data;
        const uint32_t len = (uint32_t)pkt.len;
        check(bnk_filter_note_outbound_ptrs(ctx_, &p, &len, 1, now_ns));
    }
    // One verdict per packet with one `now`, as filteredTUN.Write needs.
    std::vector<uint8_t> CheckInboundBatch(const std::vector<ByteSlice> &pkts, int64_t now_ns) override
    {
        std::vector<const uint8_t *> ptrs(pkts.size());
        std::vector<uint32_t> lens(pkts.size());
        for (size_t i = 0; i < pkts.size(); i++) {
            ptrs[i] = pkts[i].data;
            lens[i] = (uint32_t)pkts[i].len;
        }
        std::vector<uint8_t> v(pkts.size());
        check(bnk_filter_check_inbound_ptrs(ctx_, ptrs.data(), lens.data(), (uint32_t)pkts.size(),
                                            now_ns, v.data()));
        return v;
    }
    void NoteOutboundBatch(const std::vector<ByteSlice> &pkts, int64_t now_ns) override
    {
        std::vector<const uint8_t *> ptrs(pkts.size());
        std::vector<uint32_t> lens(pkts.size());
        for (size_t i = 0; i < pkts.size(); i++) {
            ptrs[i] = pkts[i].data;
            lens[i] = (uint32_t)pkts[i].len;
        }
        check(bnk_filter_note_outbound_ptrs(ctx_, ptrs.data(), lens.data(), (uint32_t)pkts.size(),
                                            now_ns));
    }
    uint32_t FlowCount()
    {
        uint32_t c = 0;
        check(bnk_filter_flow_count(ctx_, &c));
        return c;
    }
    bnk_ctx *ctx() { return ctx_; }

private:
    void check(int rc)
    {
        if (rc) throw std::runtime_error(std::string("libbnkhip: ") + bnk_last_error(ctx_));
    }
    bnk_ctx *ctx_ = nullptr;
};

// A Filter behind a BatchCoalescer: calls from many threads (one per peer in
// wireguard-go) that arrive within max_wait of each other become one GPU
// batch.  The `now_ns` arguments are ignored: a merged batch takes the clock
// when it is flushed.  A caller that was alone in the previous window waits
// only solo_wait for company (a call by itself costs about 20 us, so a lone
// peer should not pay a 200 us window on every write).
class CoalescedFilter : public PacketFilter {
public:
    CoalescedFilter(Filter *f, size_t max_packets = 8192,
                    std::chrono::microseconds max_wait = std::chrono::microseconds(200),
                    std::chrono::microseconds solo_wait = std::chrono::microseconds(10))
        : f_(f), co_([this](const uint8_t *const *ptrs, const uint32_t *lens, const uint8_t *note,
                            uint32_t n, int64_t now, uint8_t *verdict) { Run(ptrs, lens, note, n, now, verdict); },
                     max_packets, max_wait)
    {
        co_.SetSoloWait(solo_wait);
    }
    bool CheckInbound(ByteSlice pkt)
    {
        const uint8_t *p = pkt.data;
        const uint32_t len = (uint32_t)pkt.len;
        uint8_t v = 0;
        co_.Submit(&p, &len, 1, false, &v);
        return v != 0;
    }
    void NoteOutbound(ByteSlice pkt)
    {
        const uint8_t *p = pkt.data;
        const uint32_t len = (uint32_t)pkt.len;
        co_.Submit(&p, &len, 1, true, nullptr);
    }
    std::vector<uint8_t> CheckInboundBatch(const std::vector<ByteSlice> &pkts, int64_t) override
    {
        std::vector<const uint8_t *> ptrs(pkts.size());
        std::vector<uint32_t> lens(pkts.size());
        for (size_t i = 0; i < pkts.size(); i++) {
            ptrs[i] = pkts[i].data;
            lens[i] = (uint32_t)pkts[i].len;
        }
        std::vector<uint8_t> v(pkts.size());
        co_.Submit(ptrs.data(), lens.data(), (uint32_t)pkts.size(), false, v.data());
        return v;
    }
    void NoteOutboundBatch(const std::vector<ByteSlice> &pkts, int64_t) override
    {
        std::vector<const uint8_t *> ptrs(pkts.size());
        std::vector<uint32_t> lens(pkts.size());
        for (size_t i = 0; i < pkts.size(); i++) {
            ptrs[i] = pkts[i].data;
            lens[i] = (uint32_t)pkts[i].len;
        }
        co_.Submit(ptrs.data(), lens.data(), (uint32_t)pkts.size(), true, nullptr);
    }
    CoalesceStats Stats() { return co_.Stats(); }

private:
    // notes first, then checks, each as one call
    void Run(const uint8_t *const *ptrs, const uint32_t *lens, const uint8_t *note, uint32_t n,
             int64_t now, uint8_t *verdict)
    {
        std::vector<const uint8_t *> p[2];
        std::vector<uint32_t> l[2], where;
        for (uint32_t i = 0; i < n; i++) {
            p[note[i] ? 1 : 0].push_back(ptrs[i]);
            l[note[i] ? 1 : 0].push_back(lens[i]);
            if (!note[i]) where.push_back(i);
        }
        bnk_ctx *ctx = f_->ctx();
        if (!p[1].empty() &&
            bnk_filter_note_outbound_ptrs(ctx, p[1].data(), l[1].data(), (uint32_t)p[1].size(), now))
            throw std::runtime_error(std::string("libbnkhip: ") + bnk_last_error(ctx));
        if (p[0].empty()) return;
        std::vector<uint8_t> v(p[0].size());
        if (bnk_filter_check_inbound_ptrs(ctx, p[0].data(), l[0].data(), (uint32_t)p[0].size(), now, v.data()))
            throw std::runtime_error(std::string("libbnkhip: ") + bnk_last_error(ctx));
        for (size_t k = 0; k < where.size(); k++) verdict[where[k]] = v[k];
    }
    Filter *f_;
    BatchCoalescer co_;
};

namespace tun {

enum Event { EventUp = 1, EventDown = 2, EventMTUUpdate = 4 };

// wireguard-go's tun.Device, with Go's (n int, err error) returns as
// std::pair<int, Error>.
struct Device {
    virtual ~Device() = default;
    virtual int File() { return -1; }
    virtual std::pair<int, Error> Read(std::vector<ByteSlice> &bufs, std::vector<int> &sizes, int offset) = 0;
    virtual std::pair<int, Error> Write(std::vector<ByteSlice> &bufs, int offset) = 0;
    virtual std::pair<int, Error> MTU() = 0;
    virtual std::pair<std::string, Error> Name() = 0;
    virtual std::vector<Event> *Events() { return nullptr; }
    virtual int BatchSize() = 0;
    virtual Error Close() = 0;
};

} // namespace tun

// filteredTUN (filter.go:155-186).
class FilteredTUN : public tun::Device {
public:
    FilteredTUN(tun::Device *inner, PacketFilter *f) : inner_(inner), f_(f) {}

    // filter.go:160-167
    std::pair<int, Error> Read(std::vector<ByteSlice> &bufs, std::vector<int> &sizes, int offset) override
    {
        auto r = inner_->Read(bufs, sizes, offset);
        const int64_t now = UnixNano(std::chrono::system_clock::now());
        std::vector<ByteSlice> pkts;
        for (int i = 0; i < r.first; i++)
            pkts.push_back(bufs[i].sub((size_t)offset, (size_t)offset + (size_t)sizes[i]));
        if (!pkts.empty()) f_->NoteOutboundBatch(pkts, now);
        return r;
    }

    // filter.go:171-186: denied packets are dropped in place but still
    // reported written; survivors move to the front of the caller's slice in
    // order.
    std::pair<int, Error> Write(std::vector<ByteSlice> &bufs, int offset) override
    {
        const int64_t now = UnixNano(std::chrono::system_clock::now());
        std::vector<ByteSlice> pkts;
        for (const ByteSlice &b : bufs) pkts.push_back(b.from((size_t)offset));
        const std::vector<uint8_t> verdict = f_->CheckInboundBatch(pkts, now);
        size_t kept = 0;
        for (size_t i = 0; i < bufs.size(); i++)
            if (verdict[i]) bufs[kept++] = bufs[i]; // kept := bufs[:0]; append(kept, b)
        if (kept == 0) return {(int)bufs.size(), Error()};
        std::vector<ByteSlice> keep(bufs.begin(), bufs.begin() + (long)kept);
        auto r = inner_->Write(keep, offset);
        if (!r.second.empty()) return {0, r.second};
        return {(int)bufs.size(), Error()};
    }

    int File() override { return inner_->File(); }
    std::pair<int, Error> MTU() override { return inner_->MTU(); }
    std::pair<std::string, Error> Name() override { return inner_->Name(); }
    std::vector<tun::Event> *Events() override { return inner_->Events(); }
    int BatchSize() override { return inner_->BatchSize(); }
    Error Close() override { return inner_->Close(); }

private:
    tun::Device *inner_;
    PacketFilter *f_;
};

// filter.WrapTUN (filter.go:151-153)
inline std::unique_ptr<tun::Device> WrapTUN(tun::Device *inner, PacketFilter *f)
{
    return std::unique_ptr<tun::Device>(new FilteredTUN(inner, f));
}

// Anti-replay window for received transport counters (RFC 6479), with the
// geometry wireguard-go's replay.Filter uses: a ring of 128 64-bit blocks,
// so a counter is still acceptable while it trails the newest one by at most
// (128 - 1) * 64 = 8128.  The reference gets this from
// golang.zx2c4.com/wireguard/replay through device.NewDevice
// (internal/dataplane/engine.go:51).  bnk_wg_decap_batch keeps these windows
// on the device by default; this sequential form is for a caller that has
// switched them off there (bnk_wg_set_replay(ctx, 0)) and keeps them itself:
// one filter per peer keypair, fed the (peer, counter) pairs the call reports
// for authentic packets, in arrival order.
class ReplayFilter {
public:
    static constexpr uint64_t kBlocks = 128;
    static constexpr uint64_t kWindow = (kBlocks - 1) * 64;
    // wireguard-go's RejectAfterMessages: 2^64 - 2^13 - 1
    static constexpr uint64_t kRejectAfterMessages = ~uint64_t(0) - (uint64_t(1) << 13);

    ReplayFilter() { Reset(); }
    void Reset()
    {
        newest_ = 0;
        for (uint64_t &w : seen_) w = 0;
    }
    // true = first sighting inside the window (accept and remember);
    // false = duplicate, too old, or at/after `limit`.
    bool ValidateCounter(uint64_t counter, uint64_t limit = kRejectAfterMessages)
    {
        if (counter >= limit) return false;
        const uint64_t blk = counter / 64;
        if (counter > newest_) {
            // blocks between the old head and the new one start empty
            const uint64_t head = newest_ / 64;
            uint64_t fresh = blk - head;
            if (fresh > kBlocks) fresh = kBlocks;
            for (uint64_t k = 1; k <= fresh; k++) seen_[(head + k) % kBlocks] = 0;
            newest_ = counter;
        } else if (newest_ - counter > kWindow) {
            return false;
        }
        uint64_t &word = seen_[blk % kBlocks];
        const uint64_t bit = uint64_t(1) << (counter % 64);
        const bool fresh = (word & bit) == 0;
        word |= bit;
        return fresh;
    }

private:
    uint64_t newest_;
    uint64_t seen_[kBlocks];
};

} // namespace bnk_host
