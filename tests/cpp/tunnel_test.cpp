// End to end on the GPU box: four spokes encapsulate IPv4 packets into a
// pinned ring (bnk_wg_encap_batch), send them over loopback UDP with
// sendmmsg straight from the ring; the hub receives with recvmmsg straight
// into its pinned ring (RingBind), decapsulates the ring as one batch
// (bnk_wg_decap_batch), runs the replay window and gets every packet back
// once, attributed to the right peer both by source address (the Bind's
// table, internal/magicsock/bind.go:263-268) and by receiver index.
#include <stdio.h>
#include <string.h>

#include <map>
#include <set>

#include "../../bnk_amd/host/bnk_bind.hpp"
#include "../../bnk_amd/host/bnk_host.hpp"

using namespace bnk_host;

static int failures = 0;
#define EXPECT(cond, msg)                                              \
    do {                                                               \
        if (!(cond)) {                                                 \
            printf("FAIL %s:%d %s\n", __FILE__, __LINE__, msg);        \
            failures++;                                                \
        }                                                              \
    } while (0)
#define MUST(call)                                                                         \
    do {                                                                                   \
        const int rc_ = (call);                                                            \
        if (rc_ != 0) {                                                                    \
            printf("FAIL %s:%d %s -> %d\n", __FILE__, __LINE__, #call, rc_);               \
            return 1;                                                                      \
        }                                                                                  \
    } while (0)

constexpr uint32_t SPOKES = 4, PER_SPOKE = 500, N = SPOKES * PER_SPOKE;
constexpr uint32_t STRIDE = 1536, MTU = 1420;

static uint64_t mix(uint64_t &s)
{
    s += 0x9E3779B97F4A7C15ull;
    uint64_t z = s;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

int main()
{
    bnk_ctx *tx = nullptr, *rx = nullptr;
    MUST(bnk_init(0, &tx));
    MUST(bnk_init(0, &rx));
    uint64_t seed = 0x626E6B;
    uint8_t keys[SPOKES][32];
    for (auto &k : keys)
        for (uint8_t &b : k) b = (uint8_t)mix(seed);
    bnk_wg_peer spoke_side[SPOKES], hub_side[SPOKES];
    for (uint32_t i = 0; i < SPOKES; i++) {
        const uint32_t hub_index = 0x1000u + 17u * i, spoke_index = 0x9000u + 5u * i;
        const uint32_t addr = 0x64400001u + i; // 100.64.0.1+i: the spoke's tunnel address
        spoke_side[i] = bnk_wg_peer{spoke_index, hub_index, addr, 0xFFFFFFFFu};
        hub_side[i] = bnk_wg_peer{hub_index, spoke_index, addr, 0xFFFFFFFFu};
    }
    // one context stands for the four spokes' sending halves (row i = spoke i's session)
    MUST(bnk_keys_set(tx, BNK_KEYS_SEND, &keys[0][0], SPOKES));
    MUST(bnk_wg_peers_set(tx, spoke_side, SPOKES));
    MUST(bnk_keys_set(rx, BNK_KEYS_RECV, &keys[0][0], SPOKES));
    MUST(bnk_wg_peers_set(rx, hub_side, SPOKES));

    void *p = nullptr;
    MUST(bnk_ring_alloc(tx, (size_t)N * STRIDE, &p));
    uint8_t *send_ring = static_cast<uint8_t *>(p);
    MUST(bnk_ring_alloc(rx, (size_t)N * STRIDE, &p));
    uint8_t *recv_ring = static_cast<uint8_t *>(p);
    MUST(bnk_ring_alloc(rx, (size_t)N * STRIDE, &p));
    uint8_t *plain_ring = static_cast<uint8_t *>(p);
    memset(send_ring, 0, (size_t)N * STRIDE);

    // inner packets: IPv4/UDP from the spoke's tunnel address, (spoke, seq) in the payload
    std::vector<uint32_t> lens(N), peer(N), wire_len(N);
    std::vector<std::vector<uint8_t>> sent(N);
    for (uint32_t i = 0; i < N; i++) {
        const uint32_t sp = i % SPOKES, seq = i / SPOKES;
        const uint32_t len = 28 + 8 + (uint32_t)(mix(seed) % 1300);
        uint8_t *pkt = send_ring + (size_t)i * STRIDE + 16;
        for (uint32_t k = 0; k < len; k++) pkt[k] = (uint8_t)mix(seed);
        pkt[0] = 0x45;
        pkt[2] = (uint8_t)(len >> 8);
        pkt[3] = (uint8_t)len;
        pkt[9] = 17;
        const uint32_t src = 0x64400001u + sp;
        pkt[12] = (uint8_t)(src >> 24); pkt[13] = (uint8_t)(src >> 16);
        pkt[14] = (uint8_t)(src >> 8);  pkt[15] = (uint8_t)src;
        memcpy(pkt + 28, &sp, 4);
        memcpy(pkt + 32, &seq, 4);
        lens[i] = len;
        peer[i] = sp;
        sent[i].assign(pkt, pkt + len);
    }
    bnk_batch slots{};
    slots.base = send_ring;
    slots.bytes = (uint64_t)N * STRIDE;
    slots.n = N;
    slots.mem = BNK_MEM_HOST;
    slots.stride = STRIDE;
    slots.lens = lens.data();
    slots.peer = peer.data();
    MUST(bnk_wg_encap_batch(tx, &slots, MTU, wire_len.data()));

    // sockets: one per spoke, one hub
    RingBind hub;
    const uint16_t hub_port = hub.Open(0);
    NodeKey hub_key{};
    hub_key[0] = 0xAA;
    RingBind spokes[SPOKES];
    for (uint32_t sp = 0; sp < SPOKES; sp++) {
        const uint16_t port = spokes[sp].Open(0);
        NodeKey k{};
        k[0] = (uint8_t)(sp + 1);
        hub.SetPeerAddr(k, sp, AddrPort::Loopback(port));
        spokes[sp].SetPeerAddr(hub_key, 0, AddrPort::Loopback(hub_port));
    }
    Ring ring;
    ring.base = recv_ring;
    ring.bytes = (size_t)N * STRIDE;
    ring.stride = STRIDE;
    ring.headroom = 0;
    std::vector<ReplayFilter> replay(SPOKES);
    std::set<std::pair<uint32_t, uint32_t>> delivered;
    std::vector<uint32_t> sizes(N), by_addr(N), out_len(N), by_index(N);
    std::vector<uint8_t> result(N);
    std::vector<uint64_t> counter(N);
    // A socket buffer holds a few hundred datagrams at most: send in rounds and
    // drain each round before the next.
    constexpr uint32_t ROUND = 25; // datagrams per spoke per round
    uint32_t total = 0, batches = 0, sent_so_far = 0, next_seq = 0, last_batch = 0;
    while (total < N) {
        if (total == sent_so_far && next_seq < PER_SPOKE) {
            const uint32_t upto = next_seq + ROUND < PER_SPOKE ? next_seq + ROUND : PER_SPOKE;
            for (uint32_t sp = 0; sp < SPOKES; sp++) {
                std::vector<uint64_t> off;
                std::vector<uint32_t> wl;
                for (uint32_t seq = next_seq; seq < upto; seq++) {
                    const uint32_t i = seq * SPOKES + sp;
                    off.push_back((uint64_t)i * STRIDE);
                    wl.push_back(wire_len[i]);
                }
                spokes[sp].Send(send_ring, off.data(), wl.data(), (uint32_t)off.size(), hub_key);
            }
            sent_so_far += (upto - next_seq) * SPOKES;
            next_seq = upto;
        }
        const uint32_t k = hub.Receive(ring, N, sizes.data(), by_addr.data(), nullptr, 3000);
        if (k == 0) break;
        batches++;
        bnk_batch wire{}, out{};
        wire.base = recv_ring;
        wire.bytes = ring.bytes;
        wire.n = k;
        wire.mem = BNK_MEM_HOST;
        wire.stride = STRIDE;
        wire.lens = sizes.data();
        out.base = plain_ring + 16; // plaintext in line with the ciphertext
        out.bytes = ring.bytes - 16;
        out.n = k;
        out.mem = BNK_MEM_HOST;
        out.stride = STRIDE;
        MUST(bnk_wg_decap_batch(rx, &wire, &out, result.data(), out_len.data(), by_index.data(),
                                counter.data()));
        for (uint32_t i = 0; i < k; i++) {
            EXPECT(result[i] == BNK_WG_OK, "every datagram decapsulates");
            if (result[i] != BNK_WG_OK) continue;
            EXPECT(by_index[i] == by_addr[i], "receiver index and source address name the same peer");
            EXPECT(replay[by_index[i]].ValidateCounter(counter[i]), "fresh counter");
            const uint8_t *pkt = plain_ring + 16 + (size_t)i * STRIDE;
            uint32_t sp, seq;
            memcpy(&sp, pkt + 28, 4);
            memcpy(&seq, pkt + 32, 4);
            EXPECT(sp == by_index[i] && seq < PER_SPOKE, "payload names its spoke");
            if (sp >= SPOKES || seq >= PER_SPOKE) continue;
            EXPECT(counter[i] == seq, "counters follow each spoke's send order");
            const std::vector<uint8_t> &want = sent[seq * SPOKES + sp];
            EXPECT(out_len[i] == want.size() && memcmp(pkt, want.data(), want.size()) == 0,
                   "plaintext round trip");
            delivered.insert({sp, seq});
        }
        total += k;
        last_batch = k;
    }
    EXPECT(total == N && delivered.size() == N, "every packet delivered exactly once");
    // a replayed datagram still authenticates and is then refused by the window
    {
        bnk_batch wire{}, out{};
        wire.base = recv_ring;
        wire.bytes = ring.bytes;
        wire.n = 1;
        wire.mem = BNK_MEM_HOST;
        wire.stride = STRIDE;
        wire.lens = sizes.data();
        out.base = plain_ring + 16;
        out.bytes = ring.bytes - 16;
        out.n = 1;
        out.mem = BNK_MEM_HOST;
        out.stride = STRIDE;
        MUST(bnk_wg_decap_batch(rx, &wire, &out, result.data(), out_len.data(), by_index.data(),
                                counter.data()));
        EXPECT(result[0] == BNK_WG_REPLAY && out_len[0] == 0,
               "the replayed datagram is authentic and the peer's window on the device refuses it");
        EXPECT(!replay[by_index[0]].ValidateCounter(counter[0]), "as the host-side window does");
    }
    // the receive path with the inbound filter in the same call: the hub admits
    // UDP from the even spokes only; the last batch is still in the ring
    {
        std::vector<bnk_rule> rules;
        for (uint32_t sp = 0; sp < SPOKES; sp += 2) {
            bnk_rule r{};
            r.src_net = 0x64400001u + sp;
            r.src_mask = 0xFFFFFFFFu;
            r.port_first = 0;
            r.port_last = 65535;
            r.proto = 17;
            rules.push_back(r);
        }
        MUST(bnk_filter_set_rules(rx, rules.data(), (uint32_t)rules.size()));
        // (the datagrams in the ring have been through the windows once: this
        // part is about the filter, so the windows are left out of it)
        MUST(bnk_wg_set_replay(rx, 0));
        const uint32_t k = last_batch;
        bnk_batch wire{}, out{};
        wire.base = recv_ring;
        wire.bytes = ring.bytes;
        wire.n = k;
        wire.mem = BNK_MEM_HOST;
        wire.stride = STRIDE;
        wire.lens = sizes.data();
        out.base = plain_ring + 16;
        out.bytes = ring.bytes - 16;
        out.n = k;
        out.mem = BNK_MEM_HOST;
        out.stride = STRIDE;
        MUST(bnk_wg_decap_filter_batch(rx, &wire, &out, 1700000000000000000LL, result.data(), out_len.data(),
                                       by_index.data(), counter.data()));
        uint32_t passed = 0, filtered = 0;
        for (uint32_t i = 0; i < k; i++) {
            const bool even = (by_index[i] & 1u) == 0;
            EXPECT(result[i] == (even ? BNK_WG_OK : BNK_WG_FILTERED), "the filter admits the even spokes only");
            passed += result[i] == BNK_WG_OK;
            filtered += result[i] == BNK_WG_FILTERED;
        }
        EXPECT(k > 0 && passed > 0 && filtered > 0, "both kinds occurred");
        // with the windows back on, the same datagrams are all replays, and a
        // replay never reaches the filter
        MUST(bnk_wg_set_replay(rx, 1));
        MUST(bnk_wg_decap_filter_batch(rx, &wire, &out, 1700000000000000000LL, result.data(), out_len.data(),
                                       by_index.data(), counter.data()));
        for (uint32_t i = 0; i < k; i++) EXPECT(result[i] == BNK_WG_REPLAY, "replays stop at the window");
        MUST(bnk_filter_set_allow_all(rx));
    }
    printf("%u datagrams in %u receive batches\n", total, batches);
    bnk_ring_free(tx, send_ring);
    bnk_ring_free(rx, recv_ring);
    bnk_ring_free(rx, plain_ring);
    bnk_shutdown(tx);
    bnk_shutdown(rx);
    if (failures) {
        printf("%d failure(s)\n", failures);
        return 1;
    }
    printf("PASS tunnel over loopback\n");
    return 0;
}
