// The reference's filter and TUN-wrapper tests restated against the C++ host
// mirror over libbnkhip.so (runs on the GPU).  Sources:
// internal/filter/filter_test.go:13-170, internal/filter/tun_test.go:13-94.
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <thread>

#include "../../bnk_amd/host/bnk_host.hpp"

using namespace bnk_host;
using Bytes = std::vector<uint8_t>;

static int failures = 0;
#define EXPECT(cond, msg)                                              \
    do {                                                               \
        if (!(cond)) {                                                 \
            printf("FAIL %s:%d %s\n", __FILE__, __LINE__, msg);        \
            failures++;                                                \
        }                                                              \
    } while (0)

static uint32_t addr(const char *s)
{
    unsigned a, b, c, d;
    sscanf(s, "%u.%u.%u.%u", &a, &b, &c, &d);
    return a << 24 | b << 16 | c << 8 | d;
}
static void be16(uint8_t *p, uint16_t v) { p[0] = (uint8_t)(v >> 8); p[1] = (uint8_t)v; }
static void be32(uint8_t *p, uint32_t v) { be16(p, (uint16_t)(v >> 16)); be16(p + 2, (uint16_t)v); }

// filter_test.go:13-24
static Bytes ipv4(uint8_t proto, const char *src, const char *dst, const Bytes &payload)
{
    Bytes pkt(20 + payload.size());
    pkt[0] = 0x45;
    be16(&pkt[2], (uint16_t)pkt.size());
    pkt[8] = 64;
    pkt[9] = proto;
    be32(&pkt[12], addr(src));
    be32(&pkt[16], addr(dst));
    memcpy(pkt.data() + 20, payload.data(), payload.size());
    return pkt;
}
static Bytes tcp(const char *src, const char *dst, uint16_t sport, uint16_t dport, bool syn)
{
    Bytes hdr(20);
    be16(&hdr[0], sport);
    be16(&hdr[2], dport);
    hdr[12] = 5 << 4;
    hdr[13] = syn ? 0x02 : 0x10;
    return ipv4(6, src, dst, hdr);
}
static Bytes udp(const char *src, const char *dst, uint16_t sport, uint16_t dport)
{
    Bytes hdr(8);
    be16(&hdr[0], sport);
    be16(&hdr[2], dport);
    be16(&hdr[4], 8);
    return ipv4(17, src, dst, hdr);
}
static Bytes icmpEcho(const char *src, const char *dst, bool reply)
{
    Bytes hdr(8);
    hdr[0] = reply ? 0 : 8;
    return ipv4(1, src, dst, hdr);
}

static const char *peer = "100.64.0.9", *other = "100.64.0.7", *self = "100.64.0.1";
static const int64_t SEC = 1000000000LL, MIN = 60 * SEC;
static const int64_t t0 = 1700000000LL * SEC;

static bool check(Filter &f, Bytes pkt, int64_t now) { return f.CheckInbound(ByteSlice(pkt), now); }
static void note(Filter &f, Bytes pkt, int64_t now) { f.NoteOutbound(ByteSlice(pkt), now); }

static void sshOnly(Filter &f)
{
    f.SetRules({CompiledRule{{MustParsePrefix(std::string(peer) + "/32")}, "tcp", {PortRange{22, 22}}}});
}

static void TestAllowAllModePassesEverything()
{
    Filter f;
    EXPECT(check(f, tcp(peer, self, 5555, 23, true), t0), "allow-all dropped a packet");
}
static void TestRuleAllowsMatchingInbound()
{
    Filter f; sshOnly(f);
    EXPECT(check(f, tcp(peer, self, 5555, 22, true), t0), "rule-allowed tcp/22 dropped");
}
static void TestDefaultDenyDropsNonMatching()
{
    Filter f; sshOnly(f);
    EXPECT(!check(f, tcp(peer, self, 5555, 23, true), t0), "tcp/23 passed despite ssh-only policy");
    EXPECT(!check(f, tcp(other, self, 5555, 22, true), t0), "tcp/22 from disallowed source passed");
    EXPECT(!check(f, udp(peer, self, 53, 22), t0), "udp passed a tcp-only rule");
}
static void TestReturnTrafficAllowedViaFlowTable()
{
    Filter f; sshOnly(f);
    note(f, udp(self, peer, 40000, 9999), t0);
    EXPECT(check(f, udp(peer, self, 9999, 40000), t0 + 2 * SEC), "UDP reply to our own flow dropped");
    EXPECT(!check(f, udp(peer, self, 9999, 40000), t0 + 5 * MIN), "UDP reply passed after expiry");
    EXPECT(!check(f, udp(peer, self, 9998, 40000), t0 + SEC), "different source port matched the flow");
}
static void TestTCPReturnFlowAllowed()
{
    Filter f; sshOnly(f);
    note(f, tcp(self, peer, 40000, 8080, true), t0);
    EXPECT(check(f, tcp(peer, self, 8080, 40000, false), t0 + SEC), "TCP reply dropped");
    EXPECT(!check(f, tcp(peer, self, 8081, 40000, false), t0 + SEC), "TCP from wrong port matched");
}
static void TestICMPEchoReplyViaFlow()
{
    Filter f; sshOnly(f);
    note(f, icmpEcho(self, peer, false), t0);
    EXPECT(check(f, icmpEcho(peer, self, true), t0 + SEC), "ICMP echo reply dropped");
    EXPECT(!check(f, icmpEcho(other, self, true), t0 + SEC), "ICMP reply from unpinged host passed");
}
static void TestICMPRuleAllowsInboundPing()
{
    Filter f;
    f.SetRules({CompiledRule{{MustParsePrefix(std::string(peer) + "/32")}, "icmp", {}}});
    EXPECT(check(f, icmpEcho(peer, self, false), t0), "icmp rule did not allow inbound ping");
}
static void TestMalformedAndNonIPv4Dropped()
{
    Filter f; sshOnly(f);
    EXPECT(!check(f, Bytes{0x60, 0x00, 0x00}, t0), "IPv6/short packet passed while enforcing");
    EXPECT(!f.CheckInbound(ByteSlice(), t0), "nil packet passed");
    Bytes truncated = tcp(peer, self, 1, 22, true);
    truncated.resize(22);
    EXPECT(!check(f, truncated, t0), "truncated transport header passed");
}
static void TestSetAllowAllDisablesEnforcement()
{
    Filter f; sshOnly(f);
    f.SetAllowAll();
    EXPECT(check(f, tcp(other, self, 5555, 23, true), t0), "allow-all after rules still dropped");
}

// tun_test.go:13-41
struct fakeTUN : tun::Device {
    std::vector<Bytes> written, pending;
    bool fail_write = false;
    std::pair<int, Error> Read(std::vector<ByteSlice> &bufs, std::vector<int> &sizes, int offset) override
    {
        int n = 0;
        while (n < (int)bufs.size() && !pending.empty()) {
            Bytes pkt = pending.front();
            pending.erase(pending.begin());
            memcpy(bufs[n].data + offset, pkt.data(), pkt.size());
            sizes[n] = (int)pkt.size();
            n++;
        }
        return {n, Error()};
    }
    std::pair<int, Error> Write(std::vector<ByteSlice> &bufs, int offset) override
    {
        if (fail_write) return {0, "write failed"};
        for (const ByteSlice &b : bufs) written.emplace_back(b.data + offset, b.data + b.len);
        return {(int)bufs.size(), Error()};
    }
    std::pair<int, Error> MTU() override { return {1280, Error()}; }
    std::pair<std::string, Error> Name() override { return {"fake0", Error()}; }
    int BatchSize() override { return 4; }
    Error Close() override { return Error(); }
};

static Bytes pad(const Bytes &p, int offset)
{
    Bytes b(offset);
    b.insert(b.end(), p.begin(), p.end());
    return b;
}

static void TestWrapTUNDropsDeniedInboundWrites()
{
    fakeTUN inner;
    Filter f; sshOnly(f);
    auto wrapped = WrapTUN(&inner, &f);
    Bytes allowed = tcp(peer, self, 5555, 22, true), denied = tcp(peer, self, 5555, 23, true);
    const int offset = 16;
    Bytes a = pad(allowed, offset), d = pad(denied, offset);
    std::vector<ByteSlice> bufs{ByteSlice(d), ByteSlice(a)};
    auto r = wrapped->Write(bufs, offset);
    EXPECT(r.second.empty(), "Write returned an error");
    EXPECT(r.first == 2, "Write must report both packets written");
    EXPECT(inner.written.size() == 1, "inner TUN must get only the allowed packet");
    EXPECT(inner.written.size() == 1 && inner.written[0] == allowed, "survivor is not the allowed one");
    EXPECT(bufs[0].data == a.data(), "survivor must move to the front of the caller's slice");
    // everything dropped: still reports all written, inner never called
    inner.written.clear();
    Bytes d2 = pad(denied, offset);
    std::vector<ByteSlice> all_denied{ByteSlice(d2)};
    r = wrapped->Write(all_denied, offset);
    EXPECT(r.first == 1 && r.second.empty() && inner.written.empty(), "all-denied batch");
    // inner error surfaces as (0, err)
    inner.fail_write = true;
    Bytes a2 = pad(allowed, offset);
    std::vector<ByteSlice> one{ByteSlice(a2)};
    r = wrapped->Write(one, offset);
    EXPECT(r.first == 0 && !r.second.empty(), "inner write error must surface");
}

static void TestWrapTUNReadRecordsOutboundFlows()
{
    fakeTUN inner;
    Filter f;
    f.SetRules({}); // deny-all policy: only flows admit traffic
    auto wrapped = WrapTUN(&inner, &f);
    inner.pending.push_back(udp(self, peer, 40000, 9999));
    Bytes buf(2048);
    std::vector<ByteSlice> bufs{ByteSlice(buf)};
    std::vector<int> sizes(1);
    auto r = wrapped->Read(bufs, sizes, 16);
    EXPECT(r.second.empty() && r.first == 1, "Read failed");
    EXPECT(f.FlowCount() == 1, "Read must record the outbound flow");
    const int offset = 16;
    Bytes reply = udp(peer, self, 9999, 40000), unrelated = udp(peer, self, 9999, 40001);
    Bytes pr = pad(reply, offset), pu = pad(unrelated, offset);
    std::vector<ByteSlice> w{ByteSlice(pr), ByteSlice(pu)};
    r = wrapped->Write(w, offset);
    EXPECT(r.second.empty(), "Write failed");
    EXPECT(inner.written.size() == 1 && inner.written[0] == reply, "inner must get just the reply");
    EXPECT(wrapped->BatchSize() == 4 && wrapped->MTU().first == 1280 &&
               wrapped->Name().first == "fake0",
           "other Device methods pass through");
}

// Per-peer writers in parallel, as wireguard-go calls filteredTUN.Write: each
// thread's own packets get their own verdicts, the same as a direct filter
// gives, while the GPU sees merged batches.
static void TestCoalescedWritesFromManyThreads()
{
    Filter f; sshOnly(f);
    note(f, udp(self, peer, 40000, 9999), UnixNano(std::chrono::system_clock::now()));
    CoalescedFilter cf(&f, 4096, std::chrono::microseconds(500));
    constexpr int T = 16, ROUNDS = 25;
    std::atomic<int> wrong{0}, delivered{0};
    std::vector<std::thread> th;
    for (int t = 0; t < T; t++)
        th.emplace_back([&, t] {
            fakeTUN inner;
            auto wrapped = WrapTUN(&inner, &cf);
            for (int r = 0; r < ROUNDS; r++) {
                // ssh (rule), a reply to the noted flow, and two packets nothing admits
                std::vector<Bytes> pk{pad(tcp(peer, self, (uint16_t)(1000 + t), 22, true), 16),
                                      pad(tcp(peer, self, (uint16_t)(1000 + t), 23, true), 16),
                                      pad(udp(peer, self, 9999, 40000), 16),
                                      pad(udp(peer, self, 9999, (uint16_t)(40001 + r)), 16)};
                std::vector<ByteSlice> bufs;
                for (Bytes &b : pk) bufs.push_back(ByteSlice(b));
                const size_t before = inner.written.size();
                auto res = wrapped->Write(bufs, 16);
                if (res.first != 4 || !res.second.empty()) wrong++;
                if (inner.written.size() != before + 2) wrong++;
                else {
                    if (inner.written[before][9] != 6 || inner.written[before + 1][9] != 17) wrong++;
                    delivered += 2;
                }
            }
        });
    for (auto &x : th) x.join();
    EXPECT(wrong == 0, "coalesced verdicts differ from the direct filter's");
    EXPECT(delivered == T * ROUNDS * 2, "two of four packets pass in every write");
    const CoalesceStats st = cf.Stats();
    EXPECT(st.calls == (uint64_t)T * ROUNDS && st.batches < st.calls, "writes were merged into fewer launches");
    printf("coalescer: %llu writes -> %llu batches, largest %llu packets\n", (unsigned long long)st.calls,
           (unsigned long long)st.batches, (unsigned long long)st.largest_batch);
    // outbound notes go through the same window and are seen by later checks
    Bytes query = udp(self, peer, 41000, 53);
    cf.NoteOutbound(ByteSlice(query));
    Bytes reply = udp(peer, self, 53, 41000);
    EXPECT(cf.CheckInbound(ByteSlice(reply)), "reply to a coalesced note must pass");
}

int main()
{
    try {
        TestAllowAllModePassesEverything();
        TestRuleAllowsMatchingInbound();
        TestDefaultDenyDropsNonMatching();
        TestReturnTrafficAllowedViaFlowTable();
        TestTCPReturnFlowAllowed();
        TestICMPEchoReplyViaFlow();
        TestICMPRuleAllowsInboundPing();
        TestMalformedAndNonIPv4Dropped();
        TestSetAllowAllDisablesEnforcement();
        TestWrapTUNDropsDeniedInboundWrites();
        TestWrapTUNReadRecordsOutboundFlows();
        TestCoalescedWritesFromManyThreads();
    } catch (const std::exception &e) {
        printf("FAIL exception: %s\n", e.what());
        return 2;
    }
    printf(failures ? "FAILED %d\n" : "PASS all host-mirror tests (%d failures)\n", failures);
    return failures ? 1 : 0;
}
