// Host-side mirror of the reference's UDP Bind for batches that live in one
// arena: datagrams are received with recvmmsg straight into equally spaced
// slots of a caller-provided ring (a pinned ring from bnk_ring_alloc makes the
// later upload a single DMA) and sent with sendmmsg straight out of it, so the
// result of Receive is already a bnk_batch.  The demultiplexing stays on the
// CPU exactly as in the reference:
//   Bind.Open / receive / classify / isSTUN / lookupAddr / normalize
//       internal/magicsock/bind.go:85-107, 153-228, 250-274
//   Bind.Send / sendBatch / BatchSize / SetPeerAddr / ErrNoPath
//       internal/magicsock/bind.go:296-377
//   disco.IsDisco, disco.Magic
//       internal/disco/disco.go:20, 177-179
//   Bind.receiveRelay / Send's relay fallback / SetRelaySender / SetPeerRelay /
//   DeliverRelay / RelayStats / ClearPeerAddr
//       internal/magicsock/bind.go:108-139, 313-320, 431-473, 489-493
// Not mirrored: the path manager, which carries no batch of packets.  Linux
// only (recvmmsg / sendmmsg).
#pragma once

#ifndef _GNU_SOURCE
#define _GNU_SOURCE
#endif
#include <arpa/inet.h>
#include <errno.h>
#include <netinet/in.h>
#include <poll.h>
#include <stdint.h>
#include <string.h>
#include <sys/socket.h>
#include <unistd.h>

#include <array>
#include <atomic>
#include <condition_variable>
#include <deque>
#include <functional>
#include <map>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

namespace bnk_host {

// magicsock.NodeKey: a peer's 32-byte public key.
using NodeKey = std::array<uint8_t, 32>;

// netip.AddrPort after normalize(): IPv4 kept as IPv4 whatever the socket
// reported (bind.go:270-274).
struct AddrPort {
    bool is4 = true;
    std::array<uint8_t, 16> ip{}; // IPv4 in the first four bytes when is4
    uint16_t port = 0;
    bool operator<(const AddrPort &o) const
    {
        if (is4 != o.is4) return is4 < o.is4;
        if (ip != o.ip) return ip < o.ip;
        return port < o.port;
    }
    bool operator==(const AddrPort &o) const { return is4 == o.is4 && ip == o.ip && port == o.port; }
    static AddrPort V4(uint32_t host_order_addr, uint16_t port)
    {
        AddrPort a;
        a.ip[0] = (uint8_t)(host_order_addr >> 24);
        a.ip[1] = (uint8_t)(host_order_addr >> 16);
        a.ip[2] = (uint8_t)(host_order_addr >> 8);
        a.ip[3] = (uint8_t)host_order_addr;
        a.port = port;
        return a;
    }
    static AddrPort Loopback(uint16_t port) { return V4(0x7F000001u, port); }
};

inline AddrPort FromSockaddr(const sockaddr_storage &ss)
{
    AddrPort a;
    if (ss.ss_family == AF_INET) {
        const sockaddr_in *s4 = reinterpret_cast<const sockaddr_in *>(&ss);
        memcpy(a.ip.data(), &s4->sin_addr, 4);
        a.port = ntohs(s4->sin_port);
        return a;
    }
    const sockaddr_in6 *s6 = reinterpret_cast<const sockaddr_in6 *>(&ss);
    a.port = ntohs(s6->sin6_port);
    if (IN6_IS_ADDR_V4MAPPED(&s6->sin6_addr)) { // Unmap
        memcpy(a.ip.data(), s6->sin6_addr.s6_addr + 12, 4);
        return a;
    }
    a.is4 = false;
    memcpy(a.ip.data(), s6->sin6_addr.s6_addr, 16);
    return a;
}

// The dual-stack socket takes IPv6 destinations; IPv4 goes out v4-mapped.
inline sockaddr_in6 ToSockaddr(const AddrPort &a)
{
    sockaddr_in6 s{};
    s.sin6_family = AF_INET6;
    s.sin6_port = htons(a.port);
    if (a.is4) {
        s.sin6_addr.s6_addr[10] = 0xFF;
        s.sin6_addr.s6_addr[11] = 0xFF;
        memcpy(s.sin6_addr.s6_addr + 12, a.ip.data(), 4);
    } else {
        memcpy(s.sin6_addr.s6_addr, a.ip.data(), 16);
    }
    return s;
}

constexpr char kDiscoMagic[] = "bnk\0disco"; // 10 bytes with the trailing NUL: "bnk\x00disco\x00"
constexpr size_t kDiscoMagicLen = 10;

inline bool IsDisco(const uint8_t *pkt, size_t len)
{
    return len >= kDiscoMagicLen && memcmp(pkt, kDiscoMagic, kDiscoMagicLen) == 0;
}

// RFC 5389 shape: top two bits zero and the magic cookie at bytes 4-8.
inline bool IsSTUN(const uint8_t *pkt, size_t len)
{
    return len >= 20 && (pkt[0] >> 6) == 0 && pkt[4] == 0x21 && pkt[5] == 0x12 && pkt[6] == 0xA4 &&
           pkt[7] == 0x42;
}

struct BindError : std::runtime_error {
    using std::runtime_error::runtime_error;
};
struct ErrNoPath : BindError {
    ErrNoPath() : BindError("magicsock: no known path to peer") {}
};
struct ErrClosed : BindError {
    ErrClosed() : BindError("use of closed network connection") {}
};

// Equally spaced slots in one arena: slot i is [base + i*stride, +stride),
// datagrams are placed `headroom` bytes into their slot.
struct Ring {
    uint8_t *base = nullptr;
    size_t bytes = 0;
    uint32_t stride = 0;
    uint32_t headroom = 0;
    uint32_t slots() const { return stride ? (uint32_t)(bytes / stride) : 0; }
    uint8_t *slot(uint32_t i) const { return base + (size_t)i * stride + headroom; }
    uint32_t room() const { return stride - headroom; }
};

class RingBind {
public:
    static constexpr int kIdealBatchSize = 128; // conn.IdealBatchSize

    RingBind() = default;
    ~RingBind() { Close(); }
    RingBind(const RingBind &) = delete;
    RingBind &operator=(const RingBind &) = delete;

    // Bind.Open: one dual-stack UDP socket; port 0 picks a free one.
    uint16_t Open(uint16_t port)
    {
        std::lock_guard<std::mutex> lk(mu_);
        if (fd_ >= 0) throw BindError("bind already open");
        const int fd = socket(AF_INET6, SOCK_DGRAM | SOCK_CLOEXEC, 0);
        if (fd < 0) throw BindError(std::string("socket: ") + strerror(errno));
        int off = 0;
        (void)setsockopt(fd, IPPROTO_IPV6, IPV6_V6ONLY, &off, sizeof off);
        int buf = 8 << 20; // room for a burst of batches between receive calls
        (void)setsockopt(fd, SOL_SOCKET, SO_RCVBUF, &buf, sizeof buf);
        (void)setsockopt(fd, SOL_SOCKET, SO_SNDBUF, &buf, sizeof buf);
        sockaddr_in6 sa{};
        sa.sin6_family = AF_INET6;
        sa.sin6_port = htons(port);
        if (bind(fd, reinterpret_cast<sockaddr *>(&sa), sizeof sa) != 0) {
            const std::string e = strerror(errno);
            close(fd);
            throw BindError("bind: " + e);
        }
        socklen_t sl = sizeof sa;
        getsockname(fd, reinterpret_cast<sockaddr *>(&sa), &sl);
        fd_ = fd;
        port_ = ntohs(sa.sin6_port);
        return port_;
    }

    void Close()
    {
        {
            std::lock_guard<std::mutex> lk(mu_);
            if (fd_ >= 0) close(fd_);
            fd_ = -1;
            port_ = 0;
        }
        relay_cv_.notify_all(); // a receiver waiting on the relay queue sees the bind closed
    }

    int BatchSize() const { return kIdealBatchSize; }
    uint16_t LocalPort()
    {
        std::lock_guard<std::mutex> lk(mu_);
        return port_;
    }

    // SetPeerAddr / RemovePeer: identity <-> current direct address, and the
    // dense index the GPU tables use for that peer.
    void SetPeerAddr(const NodeKey &key, uint32_t peer_index, const AddrPort &addr)
    {
        std::lock_guard<std::mutex> lk(mu_);
        auto it = peers_.find(key);
        if (it != peers_.end()) by_addr_.erase(it->second.addr);
        peers_[key] = Peer{addr, peer_index};
        by_addr_[addr] = key;
    }
    // Bind.ClearPeerAddr: forgets the direct address; Send falls back to the
    // relay.  (The reverse map keeps the address, as in the reference.)
    void ClearPeerAddr(const NodeKey &key)
    {
        std::lock_guard<std::mutex> lk(mu_);
        peers_.erase(key);
    }
    // Bind.SetRelaySender: the transport for peers with no direct path.  The
    // function reports failure by throwing; Send passes that on.
    void SetRelaySender(std::function<void(uint32_t dst, const uint8_t *pkt, uint32_t len)> send)
    {
        std::lock_guard<std::mutex> lk(mu_);
        relay_send_ = std::move(send);
    }
    // Bind.SetPeerRelay: the peer's relay ID, and the dense index the GPU
    // tables use for it (ReceiveRelay reports that index).
    void SetPeerRelay(const NodeKey &key, uint32_t id, uint32_t peer_index = 0)
    {
        std::lock_guard<std::mutex> lk(mu_);
        auto it = relay_ids_.find(key);
        if (it != relay_ids_.end()) by_relay_id_.erase(it->second.id);
        relay_ids_[key] = RelayPeer{id, peer_index};
        by_relay_id_[id] = key;
    }
    // Bind.DeliverRelay: one WireGuard packet that arrived through the relay
    // from the peer registered under src.  Unknown IDs are dropped, and so is
    // the packet when 64 are already waiting (UDP semantics).
    void DeliverRelay(uint32_t src, const uint8_t *pkt, uint32_t len)
    {
        {
            std::lock_guard<std::mutex> lk(mu_);
            auto it = by_relay_id_.find(src);
            if (it == by_relay_id_.end()) return;
            if (relay_q_.size() >= kRelayQueue) return;
            relay_q_.push_back(RelayPacket{it->second, relay_ids_[it->second].index,
                                           std::vector<uint8_t>(pkt, pkt + len)});
        }
        relay_rx_.fetch_add(1);
        relay_cv_.notify_one();
    }
    // Bind.RelayStats
    void RelayStats(uint64_t *tx, uint64_t *rx) const
    {
        *tx = relay_tx_.load();
        *rx = relay_rx_.load();
    }
    // Bind.receiveRelay into ring slots [0, max): waits for the first queued
    // packet (or timeout_ms; < 0 waits until the bind closes), then drains what
    // else has queued up to max.  Same outputs as Receive.
    uint32_t ReceiveRelay(const Ring &ring, uint32_t max, uint32_t *sizes, uint32_t *peer,
                          NodeKey *keys = nullptr, int timeout_ms = -1)
    {
        std::unique_lock<std::mutex> lk(mu_);
        if (fd_ < 0) throw ErrClosed();
        if (max > ring.slots()) max = ring.slots();
        if (max == 0) return 0;
        const auto ready = [this] { return fd_ < 0 || !relay_q_.empty(); };
        if (timeout_ms < 0) relay_cv_.wait(lk, ready);
        else if (!relay_cv_.wait_for(lk, std::chrono::milliseconds(timeout_ms), ready)) return 0;
        if (fd_ < 0) throw ErrClosed();
        uint32_t n = 0;
        while (n < max && !relay_q_.empty()) {
            RelayPacket &rp = relay_q_.front();
            const uint32_t len = (uint32_t)std::min<size_t>(rp.pkt.size(), ring.room()); // copy() truncates
            memcpy(ring.slot(n), rp.pkt.data(), len);
            sizes[n] = len;
            peer[n] = rp.index;
            if (keys) keys[n] = rp.key;
            relay_q_.pop_front();
            n++;
        }
        return n;
    }
    void RemovePeer(const NodeKey &key)
    {
        std::lock_guard<std::mutex> lk(mu_);
        auto it = peers_.find(key);
        if (it == peers_.end()) return;
        by_addr_.erase(it->second.addr);
        peers_.erase(it);
    }
    void SetDiscoHandler(std::function<void(const AddrPort &, std::vector<uint8_t>)> h)
    {
        std::lock_guard<std::mutex> lk(mu_);
        on_disco_ = std::move(h);
    }
    void SetSTUNHandler(std::function<void(std::vector<uint8_t>)> h)
    {
        std::lock_guard<std::mutex> lk(mu_);
        on_stun_ = std::move(h);
    }

    // Bind.receive into ring slots [0, max): reads batches until at least one
    // datagram comes from a known peer (or timeout_ms passes; < 0 waits
    // forever).  Kept datagrams are compacted to slots 0..n-1 in arrival
    // order; sizes[i] is the datagram length, peer[i] the sender's index,
    // keys (optional) its identity.  Disco and STUN go to their handlers,
    // unknown sources are dropped.  One receiver at a time, as in the
    // reference.
    uint32_t Receive(const Ring &ring, uint32_t max, uint32_t *sizes, uint32_t *peer,
                     NodeKey *keys = nullptr, int timeout_ms = -1)
    {
        int fd;
        {
            std::lock_guard<std::mutex> lk(mu_);
            fd = fd_;
        }
        if (fd < 0) throw ErrClosed();
        if (max > ring.slots()) max = ring.slots();
        if (max == 0) return 0;
        if (rmsgs_.size() < max) {
            rmsgs_.resize(max);
            riov_.resize(max);
            raddr_.resize(max);
        }
        for (;;) {
            for (uint32_t i = 0; i < max; i++) {
                riov_[i].iov_base = ring.slot(i);
                riov_[i].iov_len = ring.room();
                memset(&rmsgs_[i], 0, sizeof rmsgs_[i]);
                rmsgs_[i].msg_hdr.msg_iov = &riov_[i];
                rmsgs_[i].msg_hdr.msg_iovlen = 1;
                rmsgs_[i].msg_hdr.msg_name = &raddr_[i];
                rmsgs_[i].msg_hdr.msg_namelen = sizeof raddr_[i];
            }
            pollfd pfd{fd, POLLIN, 0};
            const int pr = poll(&pfd, 1, timeout_ms);
            if (pr == 0) return 0;
            if (pr < 0) {
                if (errno == EINTR) continue;
                throw BindError(std::string("poll: ") + strerror(errno));
            }
            const int n = recvmmsg(fd, rmsgs_.data(), max, MSG_DONTWAIT, nullptr);
            if (n < 0) {
                if (errno == EINTR || errno == EAGAIN) continue;
                if (errno == EBADF) throw ErrClosed();
                throw BindError(std::string("recvmmsg: ") + strerror(errno));
            }
            uint32_t out = 0;
            for (int i = 0; i < n; i++) {
                const uint8_t *pkt = ring.slot((uint32_t)i);
                const uint32_t len = rmsgs_[i].msg_len;
                Peer who;
                NodeKey key;
                if (!Classify(pkt, len, FromSockaddr(raddr_[i]), &key, &who)) continue;
                if (out != (uint32_t)i) memcpy(ring.slot(out), pkt, len);
                sizes[out] = len;
                peer[out] = who.index;
                if (keys) keys[out] = key;
                out++;
            }
            if (out > 0) return out;
        }
    }

    // Bind.Send: datagram i is lens[i] bytes at ring.base + offsets[i].  With
    // a direct address known all go there in sendmmsg chunks of at most
    // BatchSize(); else, when the peer has a relay ID and a relay sender is
    // set, one by one through the relay (the first failure stops the batch);
    // else ErrNoPath.  Safe to call from several threads.
    void Send(const uint8_t *base, const uint64_t *offsets, const uint32_t *lens, uint32_t n,
              const NodeKey &to)
    {
        int fd;
        AddrPort addr;
        bool direct = false, has_relay = false;
        uint32_t relay_id = 0;
        std::function<void(uint32_t, const uint8_t *, uint32_t)> relay_send;
        {
            std::lock_guard<std::mutex> lk(mu_);
            fd = fd_;
            auto it = peers_.find(to);
            if (it != peers_.end()) {
                addr = it->second.addr;
                direct = true;
            }
            auto rt = relay_ids_.find(to);
            if (rt != relay_ids_.end()) {
                relay_id = rt->second.id;
                has_relay = true;
            }
            relay_send = relay_send_;
        }
        if (fd < 0) throw ErrClosed();
        if (!direct) {
            if (!(has_relay && relay_send)) throw ErrNoPath();
            for (uint32_t i = 0; i < n; i++) {
                relay_send(relay_id, base + offsets[i], lens[i]);
                relay_tx_.fetch_add(1);
            }
            return;
        }
        sockaddr_in6 sa = ToSockaddr(addr);
        mmsghdr msgs[kIdealBatchSize];
        iovec iov[kIdealBatchSize];
        for (uint32_t done = 0; done < n;) {
            const uint32_t chunk = n - done < (uint32_t)kIdealBatchSize ? n - done : (uint32_t)kIdealBatchSize;
            for (uint32_t i = 0; i < chunk; i++) {
                iov[i].iov_base = const_cast<uint8_t *>(base + offsets[done + i]);
                iov[i].iov_len = lens[done + i];
                memset(&msgs[i], 0, sizeof msgs[i]);
                msgs[i].msg_hdr.msg_iov = &iov[i];
                msgs[i].msg_hdr.msg_iovlen = 1;
                msgs[i].msg_hdr.msg_name = &sa;
                msgs[i].msg_hdr.msg_namelen = sizeof sa;
            }
            for (uint32_t sent = 0; sent < chunk;) {
                const int k = sendmmsg(fd, msgs + sent, chunk - sent, 0);
                if (k < 0) {
                    if (errno == EINTR) continue;
                    if (errno == EAGAIN || errno == ENOBUFS) {
                        pollfd pfd{fd, POLLOUT, 0};
                        (void)poll(&pfd, 1, 10);
                        continue;
                    }
                    throw BindError(std::string("sendmmsg: ") + strerror(errno));
                }
                sent += (uint32_t)k;
            }
            done += chunk;
        }
    }

private:
    struct Peer {
        AddrPort addr;
        uint32_t index = 0;
    };

    // Bind.classify: disco peels off before any peer check.
    bool Classify(const uint8_t *pkt, uint32_t len, const AddrPort &src, NodeKey *key, Peer *who)
    {
        if (IsDisco(pkt, len)) {
            std::function<void(const AddrPort &, std::vector<uint8_t>)> h;
            {
                std::lock_guard<std::mutex> lk(mu_);
                h = on_disco_;
            }
            if (h) h(src, std::vector<uint8_t>(pkt, pkt + len));
            return false;
        }
        if (IsSTUN(pkt, len)) {
            std::function<void(std::vector<uint8_t>)> h;
            {
                std::lock_guard<std::mutex> lk(mu_);
                h = on_stun_;
            }
            if (h) h(std::vector<uint8_t>(pkt, pkt + len));
            return false;
        }
        std::lock_guard<std::mutex> lk(mu_);
        auto it = by_addr_.find(src);
        if (it == by_addr_.end()) return false;
        *key = it->second;
        *who = peers_[it->second];
        return true;
    }

    struct RelayPeer {
        uint32_t id = 0, index = 0;
    };
    struct RelayPacket {
        NodeKey key;
        uint32_t index;
        std::vector<uint8_t> pkt;
    };
    static constexpr size_t kRelayQueue = 64; // the reference's channel capacity

    std::mutex mu_;
    int fd_ = -1;
    uint16_t port_ = 0;
    std::map<NodeKey, Peer> peers_;
    std::map<NodeKey, RelayPeer> relay_ids_;
    std::map<uint32_t, NodeKey> by_relay_id_;
    std::function<void(uint32_t, const uint8_t *, uint32_t)> relay_send_;
    std::deque<RelayPacket> relay_q_;
    std::condition_variable relay_cv_;
    std::atomic<uint64_t> relay_tx_{0}, relay_rx_{0};
    std::map<AddrPort, NodeKey> by_addr_;
    std::function<void(const AddrPort &, std::vector<uint8_t>)> on_disco_;
    std::function<void(std::vector<uint8_t>)> on_stun_;
    // receive staging; owned by the single receiver
    std::vector<mmsghdr> rmsgs_;
    std::vector<iovec> riov_;
    std::vector<sockaddr_storage> raddr_;
};

} // namespace bnk_host
