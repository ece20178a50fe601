// CPU-only: the ring-based Bind mirror over loopback UDP, restating the
// reference's own Bind tests:
//   internal/magicsock/bind_batch_test.go:16-20, 62-140
//   internal/magicsock/bind_transport_test.go:68-130
//   internal/magicsock/disco_demux_test.go:43-120
// The ring here is ordinary memory; on a GPU box it comes from bnk_ring_alloc.
#include <stdio.h>
#include <stdlib.h>

#include <set>
#include <string>
#include <thread>

#include "../../bnk_amd/host/bnk_bind.hpp"

using namespace bnk_host;

static int failures = 0;
#define EXPECT(cond, msg)                                              \
    do {                                                               \
        if (!(cond)) {                                                 \
            printf("FAIL %s:%d %s\n", __FILE__, __LINE__, msg);        \
            failures++;                                                \
        }                                                              \
    } while (0)

static NodeKey key_of(uint8_t seed)
{
    NodeKey k;
    for (size_t i = 0; i < k.size(); i++) k[i] = (uint8_t)(seed * 31 + i);
    return k;
}

struct Arena {
    Ring ring;
    std::vector<uint8_t> mem;
    Arena(uint32_t slots, uint32_t stride, uint32_t headroom) : mem((size_t)slots * stride, 0xEE)
    {
        ring.base = mem.data();
        ring.bytes = mem.size();
        ring.stride = stride;
        ring.headroom = headroom;
    }
};

// a plain UDP socket that no table knows
struct Stranger {
    int fd;
    sockaddr_in to{};
    explicit Stranger(uint16_t port)
    {
        fd = socket(AF_INET, SOCK_DGRAM, 0);
        to.sin_family = AF_INET;
        to.sin_port = htons(port);
        to.sin_addr.s_addr = htonl(0x7F000001u);
    }
    ~Stranger() { close(fd); }
    void write(const std::string &s)
    {
        if (sendto(fd, s.data(), s.size(), 0, reinterpret_cast<sockaddr *>(&to), sizeof to) < 0) perror("sendto");
    }
};

static void send_strings(RingBind &b, const std::vector<std::string> &msgs, const NodeKey &to)
{
    std::vector<uint8_t> arena;
    std::vector<uint64_t> off;
    std::vector<uint32_t> len;
    for (const std::string &m : msgs) {
        off.push_back(arena.size());
        len.push_back((uint32_t)m.size());
        arena.insert(arena.end(), m.begin(), m.end());
    }
    b.Send(arena.data(), off.data(), len.data(), (uint32_t)msgs.size(), to);
}

static std::string disco_pkt(const std::string &body) { return std::string(kDiscoMagic, kDiscoMagicLen) + body; }

static void batch_size_is_ideal()
{
    RingBind b;
    EXPECT(b.BatchSize() == 128, "BatchSize is conn.IdealBatchSize");
}

static void batched_send_delivers_all_packets_tagged_with_sender()
{
    const NodeKey keyA = key_of(1), keyB = key_of(2);
    RingBind A, B;
    const uint16_t portA = A.Open(0), portB = B.Open(0);
    A.SetPeerAddr(keyB, 7, AddrPort::Loopback(portB));
    B.SetPeerAddr(keyA, 42, AddrPort::Loopback(portA));
    const int n = 300; // more than two sendmmsg chunks
    std::vector<std::string> msgs;
    for (int i = 0; i < n; i++) {
        char buf[32];
        snprintf(buf, sizeof buf, "packet-%03d", i);
        msgs.push_back(buf);
    }
    send_strings(A, msgs, keyB);
    Arena ar(128, 1536, 16);
    std::set<std::string> got;
    std::vector<uint32_t> sizes(128), peer(128);
    std::vector<NodeKey> keys(128);
    while ((int)got.size() < n) {
        const uint32_t k = B.Receive(ar.ring, 128, sizes.data(), peer.data(), keys.data(), 5000);
        if (k == 0) break;
        for (uint32_t i = 0; i < k; i++) {
            got.insert(std::string((const char *)ar.ring.slot(i), sizes[i]));
            EXPECT(peer[i] == 42, "tagged with the sender's index");
            EXPECT(keys[i] == keyA, "tagged with the sender's identity");
        }
    }
    EXPECT((int)got.size() == n, "all payloads arrived");
    EXPECT(got.count("packet-000") && got.count("packet-299"), "first and last payload present");
    // headroom and the bytes between slots are untouched
    EXPECT(ar.mem[0] == 0xEE && ar.mem[15] == 0xEE, "headroom untouched");
}

static void receive_peels_disco_and_stun_and_drops_strangers()
{
    const NodeKey keyA = key_of(3), keyB = key_of(4);
    RingBind A, B;
    const uint16_t portA = A.Open(0), portB = B.Open(0);
    A.SetPeerAddr(keyB, 0, AddrPort::Loopback(portB));
    B.SetPeerAddr(keyA, 5, AddrPort::Loopback(portA));
    std::vector<std::vector<uint8_t>> disco, stun;
    std::vector<AddrPort> disco_src;
    B.SetDiscoHandler([&](const AddrPort &src, std::vector<uint8_t> p) {
        disco.push_back(std::move(p));
        disco_src.push_back(src);
    });
    B.SetSTUNHandler([&](std::vector<uint8_t> p) { stun.push_back(std::move(p)); });
    Stranger s(portB);
    s.write("intruder-junk");
    s.write(disco_pkt("punch"));                   // disco from an unknown source still reaches the handler
    std::string stunp(20, '\0');
    stunp[0] = 0x01; stunp[1] = 0x01;              // binding success response
    stunp[4] = 0x21; stunp[5] = 0x12; stunp[6] = (char)0xA4; stunp[7] = 0x42;
    s.write(stunp);
    send_strings(A, {disco_pkt("probe"), "legit"}, keyB); // disco from a known peer is peeled too
    Arena ar(16, 256, 0);
    uint32_t sizes[16], peer[16];
    std::set<std::string> got;
    const uint32_t k = B.Receive(ar.ring, 16, sizes, peer, nullptr, 5000);
    for (uint32_t i = 0; i < k; i++) got.insert(std::string((const char *)ar.ring.slot(i), sizes[i]));
    EXPECT(k == 1 && got.count("legit") == 1, "exactly the legitimate packet surfaces");
    EXPECT(k == 1 && peer[0] == 5, "with its peer index");
    EXPECT(disco.size() == 2, "both disco packets reached the handler");
    EXPECT(stun.size() == 1 && stun[0].size() == 20, "STUN reached its handler");
    bool from_a = false;
    for (const AddrPort &a : disco_src) from_a |= a.port == portA && a.is4;
    EXPECT(from_a, "disco handler sees the normalised IPv4 source");
    // nothing else is waiting
    EXPECT(B.Receive(ar.ring, 16, sizes, peer, nullptr, 100) == 0, "no stray packet afterwards");
}

static void send_without_known_path_fails_and_closed_bind_errors()
{
    RingBind A;
    A.Open(0);
    bool no_path = false;
    try {
        send_strings(A, {"hello"}, key_of(9));
    } catch (const ErrNoPath &) {
        no_path = true;
    }
    EXPECT(no_path, "Send to a peer with no known path is ErrNoPath");
    A.Close();
    bool closed = false;
    try {
        send_strings(A, {"hello"}, key_of(9));
    } catch (const ErrClosed &) {
        closed = true;
    }
    EXPECT(closed, "Send on a closed bind is ErrClosed");
    Arena ar(4, 64, 0);
    uint32_t sizes[4], peer[4];
    closed = false;
    try {
        A.Receive(ar.ring, 4, sizes, peer, nullptr, 10);
    } catch (const ErrClosed &) {
        closed = true;
    }
    EXPECT(closed, "Receive on a closed bind is ErrClosed");
}

static void removed_and_moved_peers()
{
    const NodeKey keyA = key_of(5), keyB = key_of(6);
    RingBind A, A2, B;
    const uint16_t portA = A.Open(0), portA2 = A2.Open(0), portB = B.Open(0);
    A.SetPeerAddr(keyB, 0, AddrPort::Loopback(portB));
    A2.SetPeerAddr(keyB, 0, AddrPort::Loopback(portB));
    B.SetPeerAddr(keyA, 1, AddrPort::Loopback(portA));
    B.SetPeerAddr(keyA, 1, AddrPort::Loopback(portA2)); // the peer moved: the old address no longer attributes
    send_strings(A, {"old-address"}, keyB);
    send_strings(A2, {"new-address"}, keyB);
    Arena ar(8, 128, 0);
    uint32_t sizes[8], peer[8];
    std::set<std::string> got;
    for (int round = 0; round < 2 && got.empty(); round++) {
        const uint32_t k = B.Receive(ar.ring, 8, sizes, peer, nullptr, 2000);
        for (uint32_t i = 0; i < k; i++) got.insert(std::string((const char *)ar.ring.slot(i), sizes[i]));
    }
    EXPECT(got.size() == 1 && got.count("new-address"), "only the current address attributes");
    B.RemovePeer(keyA);
    send_strings(A2, {"after-removal"}, keyB);
    EXPECT(B.Receive(ar.ring, 8, sizes, peer, nullptr, 200) == 0, "a removed peer's packets are dropped");
}

// internal/magicsock/relay_path_test.go:15-127, clear_addr_test.go:8-46
static void relay_fallback_and_relay_receive()
{
    const NodeKey keyA = key_of(21), keyB = key_of(22);
    RingBind A, B;
    A.Open(0);
    const uint16_t portB = B.Open(0);
    Arena ar(8, 256, 16);
    std::vector<std::pair<uint32_t, std::string>> relayed;
    A.SetRelaySender([&](uint32_t dst, const uint8_t *p, uint32_t len) {
        relayed.emplace_back(dst, std::string((const char *)p, len));
    });
    A.SetPeerRelay(keyB, 2, 7);
    // TestSendPrefersRelayWhenNoDirectPath
    const std::string pay = "payload", second = "second";
    std::vector<uint8_t> buf(pay.begin(), pay.end());
    buf.insert(buf.end(), second.begin(), second.end());
    const uint64_t offs[2] = {0, pay.size()};
    const uint32_t lens[2] = {(uint32_t)pay.size(), (uint32_t)second.size()};
    A.Send(buf.data(), offs, lens, 2, keyB);
    EXPECT(relayed.size() == 2 && relayed[0].first == 2 && relayed[0].second == "payload" &&
               relayed[1].second == "second", "no direct path: every packet goes through the relay sender");
    uint64_t tx = 0, rx = 0;
    A.RelayStats(&tx, &rx);
    EXPECT(tx == 2 && rx == 0, "relay tx counts packets");
    A.SetPeerRelay(keyA, 1);
    A.DeliverRelay(1, (const uint8_t *)"inbound", 7);
    A.RelayStats(&tx, &rx);
    EXPECT(rx == 1, "relay rx counts delivered packets");
    // TestDirectPathStillWinsOverRelay + TestClearPeerAddrFallsBackToRelay
    relayed.clear();
    A.SetPeerAddr(keyB, 7, AddrPort::Loopback(portB));
    B.SetPeerAddr(keyA, 3, AddrPort::Loopback(A.LocalPort()));
    A.Send(buf.data(), offs, lens, 1, keyB);
    uint32_t sizes[8], peer[8];
    NodeKey keys[8];
    uint32_t k = B.Receive(ar.ring, 8, sizes, peer, keys, 2000);
    EXPECT(k == 1 && std::string((const char *)ar.ring.slot(0), sizes[0]) == "payload" && relayed.empty(),
           "a known direct path wins over the relay");
    A.ClearPeerAddr(keyB);
    A.Send(buf.data(), offs + 1, lens + 1, 1, keyB);
    EXPECT(relayed.size() == 1 && relayed[0].second == "second", "after ClearPeerAddr Send uses the relay");
    // a failing relay sender stops the batch and surfaces
    int calls = 0;
    A.SetRelaySender([&](uint32_t, const uint8_t *, uint32_t) {
        calls++;
        throw BindError("relay down");
    });
    bool threw = false;
    try {
        A.Send(buf.data(), offs, lens, 2, keyB);
    } catch (const BindError &) {
        threw = true;
    }
    EXPECT(threw && calls == 1, "the first relay failure stops the batch");
    // no relay ID, no address: ErrNoPath as before
    threw = false;
    try {
        A.Send(buf.data(), offs, lens, 1, key_of(99));
    } catch (const ErrNoPath &) {
        threw = true;
    }
    EXPECT(threw, "no path at all");
    // TestDeliverRelaySurfacesIdentityEndpoint + TestDeliverRelayFromUnknownIDIsDropped
    B.SetPeerRelay(keyA, 1, 3);
    B.DeliverRelay(99, (const uint8_t *)"stranger", 8);
    B.DeliverRelay(1, (const uint8_t *)"known", 5);
    B.DeliverRelay(1, (const uint8_t *)"again", 5);
    k = B.ReceiveRelay(ar.ring, 8, sizes, peer, keys, 1000);
    EXPECT(k == 2 && std::string((const char *)ar.ring.slot(0), sizes[0]) == "known" &&
               std::string((const char *)ar.ring.slot(1), sizes[1]) == "again" && peer[0] == 3 && keys[0] == keyA,
           "relay packets surface in order, tagged with the registered identity");
    EXPECT(B.ReceiveRelay(ar.ring, 8, sizes, peer, keys, 50) == 0, "nothing queued: the wait times out");
    // the queue holds 64; the rest are dropped
    for (int i = 0; i < 80; i++) B.DeliverRelay(1, (const uint8_t *)"x", 1);
    uint32_t total = 0;
    while ((k = B.ReceiveRelay(ar.ring, 8, sizes, peer, keys, 20)) != 0) total += k;
    EXPECT(total == 64, "the relay queue drops beyond 64 waiting packets");
    // a closed bind ends a waiting relay receiver
    std::thread closer([&] {
        usleep(50 * 1000);
        B.Close();
    });
    threw = false;
    try {
        (void)B.ReceiveRelay(ar.ring, 8, sizes, peer, keys, -1);
    } catch (const ErrClosed &) {
        threw = true;
    }
    closer.join();
    EXPECT(threw, "ReceiveRelay on a closed bind");
}

int main()
{
    batch_size_is_ideal();
    batched_send_delivers_all_packets_tagged_with_sender();
    receive_peels_disco_and_stun_and_drops_strangers();
    send_without_known_path_fails_and_closed_bind_errors();
    removed_and_moved_peers();
    relay_fallback_and_relay_receive();
    if (failures) {
        printf("%d failure(s)\n", failures);
        return 1;
    }
    printf("ok\n");
    return 0;
}
