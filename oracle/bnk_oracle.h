/*
 * bnk_oracle.h -- CPU restatement of the bnk packet hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, the smoke
 * check and the cpu_baseline leg of bench.py may link or call it, and only
 * as the checker.  The shipped library (libbnkhip.so) never routes through
 * anything declared here.
 *
 * What it restates, and what pins each piece:
 *
 *  - ChaCha20 block / stream, Poly1305, AEAD_CHACHA20_POLY1305 (RFC 8439),
 *    which is what golang.org/x/crypto v0.55.0 chacha20poly1305 computes for
 *    wireguard-go's transport seal/open (reference go.mod:8,10; the only
 *    reference call site is device.NewDevice at
 *    internal/dataplane/engine.go:51).  That module is not vendored in the
 *    reference tree, so the published algorithm is restated here.
 *    Pinned by: RFC 8439 sections 2.3.2, 2.4.2, 2.5.2, 2.6.2, 2.8.2 and the
 *    appendix A.3 Poly1305 edge-case vectors; a literal big-integer
 *    transcription of the RFC pseudocode in tests/; OpenSSL
 *    EVP_chacha20_poly1305 on the benchmark shapes.
 *  - WireGuard transport nonce: 4 zero bytes then the 64-bit little-endian
 *    per-peer counter, empty AAD (WireGuard protocol, section 5.4.6).
 *  - internal/filter (filter.go:62-209) and acl.CompiledRule.Match
 *    (acl.go:149-172), restated line by line.  Pinned by the reference's own
 *    filter_test.go, tun_test.go and acl_test.go cases, transcribed as tests.
 *  - The fused relay open -> filter -> re-seal has no reference function;
 *    its semantics are defined here: "parity unpinned" beyond the pieces
 *    above that it composes.
 */
#ifndef BNK_ORACLE_H
#define BNK_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------- RFC 8439 primitives ---------------- */

/* RFC 8439 section 2.3: one 64-byte keystream block. */
void bnko_chacha20_block(const uint8_t key[32], uint32_t counter,
                         const uint8_t nonce[12], uint8_t out[64]);

/* RFC 8439 section 2.4: out = in XOR keystream(counter, counter+1, ...). */
void bnko_chacha20_xor(const uint8_t key[32], uint32_t counter,
                       const uint8_t nonce[12], const uint8_t *in,
                       uint8_t *out, size_t len);

/* RFC 8439 section 2.5: tag = ((sum of blocks * r^k) mod 2^130-5) + s. */
void bnko_poly1305(const uint8_t key[32], const uint8_t *msg, size_t len,
                   uint8_t tag[16]);

/* RFC 8439 section 2.6: Poly1305 one-time key = first 32 bytes of block 0. */
void bnko_poly1305_keygen(const uint8_t key[32], const uint8_t nonce[12],
                          uint8_t otk[32]);

/* RFC 8439 section 2.8.  out receives len bytes of ciphertext then 16 bytes
 * of tag.  in and out may alias exactly. */
void bnko_aead_seal(const uint8_t key[32], const uint8_t nonce[12],
                    const uint8_t *pt, size_t len, const uint8_t *aad,
                    size_t aad_len, uint8_t *out);

/* ct_len includes the 16-byte tag.  Returns 1 and writes ct_len-16 bytes of
 * plaintext on success; returns 0 and zero-fills those bytes on failure
 * (x/crypto's Open clears its output before returning the error). */
int bnko_aead_open(const uint8_t key[32], const uint8_t nonce[12],
                   const uint8_t *ct, size_t ct_len, const uint8_t *aad,
                   size_t aad_len, uint8_t *out);

/* WireGuard transport nonce: 00 00 00 00 || LE64(counter). */
void bnko_wg_nonce(uint64_t counter, uint8_t nonce[12]);

/* ---------------- batched WireGuard transport AEAD ---------------- */

/* Packet i: input at in + in_off[i], in_len[i] bytes; output at
 * out + out_off[i]; key = keys + 32*peer[i] (peer NULL: key 0); counter
 * counters[i].  Seal: in_len = plaintext length, output in_len+16 bytes.
 * Open: in_len = ciphertext length including the tag; output in_len-16
 * bytes; verdict[i] = 1 authentic, 0 rejected (in_len < 16 rejects and
 * writes nothing).  nthreads > 1 splits the batch over pthreads. */
void bnko_seal_batch(const uint8_t *keys, const uint32_t *peer,
                     const uint64_t *counters, const uint8_t *in,
                     const uint64_t *in_off, const uint32_t *in_len,
                     uint8_t *out, const uint64_t *out_off, uint32_t n,
                     int nthreads);
void bnko_open_batch(const uint8_t *keys, const uint32_t *peer,
                     const uint64_t *counters, const uint8_t *in,
                     const uint64_t *in_off, const uint32_t *in_len,
                     uint8_t *out, const uint64_t *out_off, uint8_t *verdict,
                     uint32_t n, int nthreads);

/* ---------------- internal/filter + acl.Match ---------------- */

/* acl.PortRange (acl.go:39-42). */
typedef struct {
    uint16_t first, last;
} bnko_port_range;

/* netip.Prefix restricted to what Contains() looks at.  bits < 0 is the
 * invalid prefix (never contains anything); is4 == 0 is an IPv6 prefix
 * (never contains an IPv4 address). */
typedef struct {
    uint32_t addr; /* host byte order: a.b.c.d = a<<24|b<<16|c<<8|d */
    int32_t bits;
    int32_t is4;
} bnko_prefix;

/* acl.CompiledRule (acl.go:33-37). */
typedef struct {
    const bnko_prefix *srcs;
    uint32_t n_srcs;
    const char *proto; /* "tcp" | "udp" | "icmp" | anything else */
    const bnko_port_range *ports;
    uint32_t n_ports;
} bnko_rule;

/* acl.go:149-172.  src is IPv4, host byte order. */
int bnko_rule_match(const bnko_rule *r, uint32_t src, const char *proto,
                    uint16_t dst_port);

/* filter.go:62-106.  Returns 1 and fills the fields on success. */
typedef struct {
    uint8_t proto;
    uint32_t src, dst;
    uint16_t src_port, dst_port;
    const char *proto_name;
    uint8_t icmp_type;
} bnko_parsed;
int bnko_parse(const uint8_t *pkt, size_t len, bnko_parsed *out);

/* filter.go:108-117, nanoseconds. */
int64_t bnko_flow_ttl_ns(uint8_t proto);

typedef struct bnko_filter bnko_filter;
bnko_filter *bnko_filter_new(void);                      /* filter.go:41 */
void bnko_filter_free(bnko_filter *f);
/* filter.go:46; the rules are deep-copied. */
void bnko_filter_set_rules(bnko_filter *f, const bnko_rule *rules, uint32_t n);
void bnko_filter_set_allow_all(bnko_filter *f);          /* filter.go:54 */
/* filter.go:121-147; now_ns is the time.Time as Unix nanoseconds. */
int bnko_filter_check_inbound(bnko_filter *f, const uint8_t *pkt, size_t len,
                              int64_t now_ns);
/* filter.go:189-209 including the len(flows) > 4096 expiry sweep. */
void bnko_filter_note_outbound(bnko_filter *f, const uint8_t *pkt, size_t len,
                               int64_t now_ns);
/* len(f.flows) */
uint32_t bnko_filter_flow_count(const bnko_filter *f);
/* Dump the flow map: for entry k, key[k] = remote<<32 | remotePort<<16 |
 * localPort, proto[k], expiry_ns[k].  Arrays must hold flow_count entries;
 * order is unspecified.  Returns the number written. */
uint32_t bnko_filter_flow_dump(const bnko_filter *f, uint64_t *key,
                               uint8_t *proto, int64_t *expiry_ns);

/* filter.go:160-186 applied to a flat batch: packet i is pkts + off[i],
 * len[i] bytes; one `now` for the whole batch. */
void bnko_filter_check_inbound_batch(bnko_filter *f, const uint8_t *pkts,
                                     const uint64_t *off, const uint32_t *len,
                                     uint32_t n, int64_t now_ns,
                                     uint8_t *verdict);
void bnko_filter_note_outbound_batch(bnko_filter *f, const uint8_t *pkts,
                                     const uint64_t *off, const uint32_t *len,
                                     uint32_t n, int64_t now_ns);

/* ---------------- fused relay (no reference function) ---------------- */

enum { BNKO_RELAY_OK = 0, BNKO_RELAY_FORGED = 1, BNKO_RELAY_DENIED = 2 };

/* For packet i in batch order: open in+in_off[i] (in_len[i] bytes incl. tag)
 * under keys_in[peer_in[i]] with counter ctr_in[i]; failure -> FORGED.
 * Else CheckInbound on the plaintext at now_ns; false -> DENIED.  Else seal
 * the plaintext under keys_out[peer_out[i]] with counter
 * ctr_base_out[peer_out[i]] + (number of earlier OK packets with the same
 * peer_out), writing in_len[i] bytes at out+out_off[i] and that counter to
 * ctr_out[i].  FORGED/DENIED packets leave their output bytes untouched and
 * set ctr_out[i] = 0.  A dropped packet never consumes a nonce, as in
 * wireguard-go where the counter is assigned only to packets that are sent. */
void bnko_relay_fused_batch(bnko_filter *f, const uint8_t *keys_in,
                            const uint32_t *peer_in, const uint64_t *ctr_in,
                            const uint8_t *keys_out, const uint32_t *peer_out,
                            const uint64_t *ctr_base_out, uint32_t n_peers_out,
                            const uint8_t *in, const uint64_t *in_off,
                            const uint32_t *in_len, uint8_t *out,
                            const uint64_t *out_off, int64_t now_ns,
                            uint8_t *verdict, uint64_t *ctr_out, uint32_t n);

/* ---------------- WireGuard transport framing (wireguard-go, not vendored) ----------------
 *
 * PARITY UNPINNED: the reference reaches this code only through
 * device.NewDevice (internal/dataplane/engine.go:51) and wireguard-go's source
 * is not in the reference tree.  What follows restates the WireGuard protocol
 * paper (section 5.4.6: type 4, receiver index, 64-bit counter, zero padding of
 * the plaintext to a multiple of 16) and wireguard-go's documented behaviour
 * (padding capped at the MTU, IPv4 total-length trim, source must be an
 * allowed IP of the sending peer, RFC 6479 replay window of 8128 counters).
 * In-repo corroboration: offset 16 (internal/filter/tun_test.go:50), type byte 4
 * (internal/magicsock/bind_bench_test.go:29), one /32 allowed IP per peer
 * (internal/dataplane/engine.go:292-299). */

enum {
    BNKO_WG_OK = 0,            /* deliver out_len bytes of plaintext */
    BNKO_WG_KEEPALIVE = 1,     /* authentic, empty */
    BNKO_WG_BAD_HEADER = 2,    /* shorter than 32 bytes or type != 4 */
    BNKO_WG_UNKNOWN_INDEX = 3, /* receiver index names no keypair */
    BNKO_WG_AUTH_FAIL = 4,
    BNKO_WG_BAD_IP = 5,        /* not IPv4/IPv6, or its length field is inconsistent */
    BNKO_WG_NOT_ALLOWED = 6    /* source address is not the peer's allowed IP */
};

typedef struct {
    uint32_t local_index;  /* index this side handed out; arrives in the header */
    uint32_t remote_index; /* index the peer handed out; goes into the header */
    uint32_t allowed_net, allowed_mask; /* the peer's allowed IPv4 prefix */
} bnko_wg_peer;

/* Bytes of zero padding wireguard-go appends before sealing. */
uint32_t bnko_wg_padding(uint32_t packet_len, uint32_t mtu);

/* slot: 16 bytes of headroom, then `len` plaintext bytes, then room for the
 * padding and the tag.  Writes the header, pads, seals in place with `counter`
 * under key; returns the wire length (16 + padded + 16). */
uint32_t bnko_wg_encap(uint8_t *slot, uint32_t len, uint32_t mtu, const uint8_t key[32],
                       uint32_t remote_index, uint64_t counter);

/* wire: a received datagram.  peers/keys_recv: n_peers entries.  On OK writes
 * the trimmed plaintext to out (may be wire + 16) and its length to *out_len;
 * *peer and *counter are set whenever the index resolves. */
int bnko_wg_decap(const uint8_t *wire, uint32_t wire_len, const bnko_wg_peer *peers,
                  const uint8_t *keys_recv, uint32_t n_peers, uint8_t *out, uint32_t *out_len,
                  uint32_t *peer, uint64_t *counter);

/* RFC 6479 sliding window as wireguard-go's replay.Filter keeps it. */
typedef struct {
    uint64_t last;
    uint64_t ring[128];
} bnko_replay;
void bnko_replay_reset(bnko_replay *f);
/* 1 = fresh (accept), 0 = replayed, too old, or counter >= limit */
int bnko_replay_validate(bnko_replay *f, uint64_t counter, uint64_t limit);

/* ---- OpenSSL as a second CPU baseline (openssl_batch.c) ------------------ */

/* 1 when libcrypto could be loaded at run time. */
int bnko_ossl_available(void);
/* EVP_chacha20_poly1305 seal into `sealed` then open into `opened`, split over
 * nthreads; returns the number of packets whose round trip verified. */
uint32_t bnko_ossl_seal_open_batch(const uint8_t *keys, const uint32_t *peer, const uint64_t *counters,
                                   const uint8_t *in, const uint64_t *off, const uint32_t *len,
                                   uint8_t *sealed, uint8_t *opened, uint32_t n, int nthreads);

#ifdef __cplusplus
}
#endif
#endif
