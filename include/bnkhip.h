/*
 * bnkhip.h -- C ABI of libbnkhip.so: the MI355X (gfx950) implementation of
 * the bnk packet hot path, batched.
 *
 *   WireGuard transport seal/open   ChaCha20-Poly1305 (RFC 8439), nonce =
 *                                   00 00 00 00 || LE64(counter), empty AAD
 *   internal/filter verdicts        5-tuple ACL + conntrack flow table
 *   fused relay                     open -> filter -> re-seal
 *
 * This is what a cgo shim in the reference would bind.  Each entry point
 * names the reference interface it stands behind (paths relative to the
 * reference tree).  Conventions:
 *   - plain C types only; every buffer is caller-owned and is not retained
 *     after the call returns (BNK_MEM_HOST) or after the stream reaches the
 *     call (BNK_MEM_DEVICE);
 *   - return value 0 on success, a negative BNK_E_* code on failure; nothing
 *     aborts or throws across the boundary; bnk_last_error() has the text;
 *   - calls on one context are serialised by an internal mutex, so Go may
 *     call from many goroutines (the reference serialises its filter the same
 *     way, internal/filter/filter.go:34,122,190);
 *   - there is no CPU fallback: without a gfx950 device bnk_init fails;
 *   - a BNK_MEM_HOST call that ends with a kernel waits for it by watching a
 *     word in pinned memory that a last one-thread launch writes, spinning on
 *     the calling core for up to 100 us before it falls back to
 *     hipStreamSynchronize (BNK_WAIT_SYNC=1 in the environment at bnk_init:
 *     always the latter).  A launch that fails is reported by the call that
 *     made it; BNK_MEM_DEVICE calls only enqueue, so what goes wrong while
 *     their work runs is reported by the next call that waits (bnk_sync).
 */
#ifndef BNKHIP_H
#define BNKHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct bnk_ctx bnk_ctx;

enum {
    BNK_OK = 0,
    BNK_E_INVAL = -1, /* null pointer, bad size, layout outside the arena */
    BNK_E_NODEV = -2, /* no gfx950 device with that ordinal */
    BNK_E_HIP = -3,   /* HIP runtime failure */
    BNK_E_NOMEM = -4, /* host or device allocation failed */
    BNK_E_RANGE = -5, /* peer index beyond the key table */
    BNK_E_STATE = -6  /* keys not loaded, context shut down */
};

/* Where the pointers of a bnk_batch live. */
enum {
    BNK_MEM_HOST = 0,  /* host memory; the call stages, runs and copies back
                          before it returns.  Arenas inside pinned rings from
                          bnk_ring_alloc are fastest: batches of up to 8 MB
                          are read and written in place by the kernels, larger
                          ones are copied in overlapped chunks */
    BNK_MEM_DEVICE = 1 /* device memory of the context's GPU; the call only
                          enqueues work on the context stream (bnk_sync waits) */
};

/* WireGuard keeps a sending and a receiving key per peer keypair. */
enum { BNK_KEYS_SEND = 0, BNK_KEYS_RECV = 1 };

/*
 * A batch of packets in one arena: the flat form of the [][]byte that
 * tun.Device.Read/Write and conn.Bind.Send/ReceiveFunc carry
 * (internal/filter/tun_test.go:19-41, internal/magicsock/bind.go:153,296).
 * Packet i starts at base + (offsets ? offsets[i] : i * stride) and is
 * (lens ? lens[i] : len) bytes long.
 */
typedef struct bnk_batch {
    void *base;              /* arena */
    uint64_t bytes;          /* arena size; every packet must lie inside it.
                                Host batches are checked before anything runs
                                (BNK_E_INVAL).  Device batches whose offsets or
                                lengths are device arrays are checked by the
                                kernels: a packet reaching beyond the arena is
                                neither read nor written (verdict 0, wire_len
                                0, BNK_WG_BAD_HEADER, BNK_RELAY_FORGED), the
                                rest of the batch runs, and the next bnk_sync
                                returns BNK_E_INVAL */
    uint32_t n;              /* packets */
    uint32_t mem;            /* BNK_MEM_HOST or BNK_MEM_DEVICE: applies to base
                                and to every array below */
    const uint64_t *offsets; /* n byte offsets, or NULL for a uniform stride */
    uint32_t stride;         /* used when offsets == NULL */
    uint32_t len;            /* used when lens == NULL */
    const uint32_t *lens;    /* n lengths, or NULL for a uniform length */
    const uint32_t *peer;    /* n indices into the key table, or NULL (peer 0) */
    const uint64_t *counters;/* n 64-bit nonce counters, or NULL for
                                counter0 + i */
    uint64_t counter0;
} bnk_batch;

/* One allowance: the flat form of acl.CompiledRule (internal/acl/acl.go:33-42)
 * for a single source prefix and a single port range.  A rule with several
 * prefixes or ranges is the set of all (prefix, range) pairs, which
 * Match's any-of semantics (acl.go:149-172) make exact; a tcp/udp rule with
 * no ranges, or any other proto string, matches nothing and has no tuples. */
typedef struct bnk_rule {
    uint32_t src_net;    /* host byte order a<<24|b<<16|c<<8|d */
    uint32_t src_mask;   /* prefix mask; 0 for /0.  Host bits of src_net outside
                            the mask are ignored, as netip.Prefix.Contains does */
    uint16_t port_first; /* inclusive; ignored when proto is 1 (icmp) */
    uint16_t port_last;
    uint8_t proto;       /* 1 icmp, 6 tcp, 17 udp; anything else never matches */
    uint8_t pad[3];
} bnk_rule;

/* ---- lifetime ---------------------------------------------------------- */

/* Opens device `device_ordinal` (must be gfx950) and creates the context's
 * stream.  Replaces nothing in the reference: it is the library's init. */
int bnk_init(int device_ordinal, bnk_ctx **out);
void bnk_shutdown(bnk_ctx *ctx);
/* Text of the last failure on this context (or of a failed bnk_init when
 * ctx is NULL).  Valid until the next call on the context. */
const char *bnk_last_error(bnk_ctx *ctx);

/* Pinned host packet ring for wireguard-go style buffer pools.  The GPU can
 * address it: small batches whose arenas lie inside a ring of the same context
 * need no staging copies. */
int bnk_ring_alloc(bnk_ctx *ctx, size_t bytes, void **host_pinned);
int bnk_ring_free(bnk_ctx *ctx, void *host_pinned);
/* Device memory for callers that keep batches resident (BNK_MEM_DEVICE). */
int bnk_dev_alloc(bnk_ctx *ctx, size_t bytes, void **dev);
int bnk_dev_free(bnk_ctx *ctx, void *dev);
int bnk_copy_to_device(bnk_ctx *ctx, void *dev, const void *host, size_t bytes);
int bnk_copy_to_host(bnk_ctx *ctx, void *host, const void *dev, size_t bytes);
/* Waits for everything enqueued on the context stream. */
int bnk_sync(bnk_ctx *ctx);
/* The context's hipStream_t, for callers that time or order work on it. */
void *bnk_stream(bnk_ctx *ctx);

/* Tuning: seal/open batches of at most max_packets packets give each packet
 * a whole wave instead of one lane (a lane needs about 85 us for a 1420-byte
 * packet however small the batch; a wave about a tenth of that).  Default
 * 4096, scaled by the packet length when the batch has one common length; 0
 * always uses a lane per packet.  Results do not depend on it.  No
 * counterpart in the reference. */
int bnk_set_spread_max_packets(bnk_ctx *ctx, uint32_t max_packets);

/* ---- merging of small host calls ----------------------------------------
 *
 * wireguard-go calls with at most 128 packets at a time, from one goroutine
 * per peer: filteredTUN.Write once per peer batch
 * (internal/filter/filter.go:171-186), Bind.Send "concurrently by per-peer
 * goroutines" (internal/magicsock/bind.go:326-328; batch size bind.go:372-377).
 * A context runs one call at a time, so at that calling pattern every call
 * pays a launch and a wait for 180 KB.  With merging on, BNK_MEM_HOST calls of
 * bnk_aead_seal_batch, bnk_aead_open_batch, bnk_wg_encap_batch,
 * bnk_wg_note_encap_batch, bnk_wg_decap_batch and bnk_wg_decap_filter_batch
 * that arrive from different threads while the context is busy (or within
 * max_wait_us of each other once callers have been seen to come in groups)
 * are run as one batch; every caller blocks until that batch is done and gets
 * exactly its own results.  Nothing changes in any signature.
 *
 * A call takes part when its arenas lie inside pinned rings of the context
 * (bnk_ring_alloc; callers of one window must use the same ring or pair of
 * rings, each its own part of it) and it has at most max(128, max_packets/4)
 * packets; any other call runs by itself as before.  Per call the results are
 * those of some serial order of the merged calls: each call's packets stay in
 * order and calls are taken in arrival order, so send counters and anti-replay
 * windows, which depend on the order of one peer's packets, are as if the calls
 * had run one after the other (a peer's calls come from one thread and do not
 * overlap).  Calls of a window that carry a now_ns share the latest of theirs.
 * A call whose arguments a direct call would refuse (BNK_E_INVAL, BNK_E_RANGE,
 * BNK_E_STATE) is refused alone, with its own message.
 *
 * max_packets: size at which a window is run without waiting further (4096
 * keeps a window within what one launch of a wave per packet takes); 0
 * switches merging off (the default).  max_wait_us: how long the first caller
 * of a window waits for company: half of the callers that are inside these
 * entry points at that moment, and never fewer than expect_callers (0 or 1:
 * no such floor; for an application that knows how many threads call and
 * wants them in one launch); a caller that is alone does not wait at all.
 * Added latency per call is at most max_wait_us plus
 * the time the batch before takes, which a direct call would have waited for
 * on the context's lock as well.
 * No counterpart in the reference (wireguard-go fans its AEAD out over CPU
 * cores instead). */
int bnk_set_coalesce(bnk_ctx *ctx, uint32_t max_packets, uint32_t max_wait_us,
                     uint32_t expect_callers);

typedef struct bnk_coalesce_stats {
    uint64_t calls;           /* calls that joined a window */
    uint64_t packets;         /* their packets */
    uint64_t batches;         /* windows run */
    uint64_t largest_batch;   /* packets in the largest window */
    uint64_t largest_callers; /* calls in the window that merged most */
    uint64_t full_windows;    /* closed because max_packets was reached */
    uint64_t timed_out;       /* leader waited max_wait_us and went without the expected company */
    uint64_t retried;         /* windows refused as a whole, whose callers then ran by themselves */
    uint64_t gather_ns;       /* summed over windows: from the first caller's arrival to the window's close */
    uint64_t enqueue_ns;      /* ... the context lock held to stage and launch the merged batch */
    uint64_t wait_ns;         /* ... from there until the batch's results were back */
} bnk_coalesce_stats;
int bnk_coalesce_stats_get(bnk_ctx *ctx, bnk_coalesce_stats *out);

/* ---- hot-path counters -------------------------------------------------- */

/* Packets by outcome since bnk_init (or the last reset), over every entry point
 * of this context.  An addition: the reference keeps no such counts (its
 * filter drops without counting, internal/filter/filter.go:100-145, and
 * wireguard-go counts bytes per peer only).  They are a histogram of the
 * result bytes every call already leaves per packet.  A host batch is counted
 * on the host once the call has succeeded (a call that returns an error counts
 * nothing).  A device-resident batch is counted on the device as it runs: by
 * the opening launch and by the CheckInbound launch themselves, elsewhere by
 * one small launch behind the call's own.
 *   sealed         bnk_aead_seal_batch(_noalloc), packets bnk_wg_(note_)encap_batch
 *                  gave a wire length other than 0
 *   opened         bnk_aead_open_batch, verdict 1
 *   rejected       a tag that did not verify: bnk_aead_open_batch verdict 0,
 *                  BNK_WG_AUTH_FAIL, BNK_RELAY_FORGED
 *   allowed/denied CheckInbound: bnk_filter_check_inbound_* verdict 1 / 0;
 *                  bnk_wg_decap_filter_batch BNK_WG_OK / BNK_WG_FILTERED;
 *                  BNK_RELAY_DENIED
 *   delivered      BNK_WG_OK of the decapsulating calls
 *   keepalive, replayed, bad_header, unknown_index, bad_ip, not_allowed
 *                  the BNK_WG_* results of those names
 *   relayed        BNK_RELAY_OK (opened and re-sealed)
 * bnk_counters_get waits for the context's stream. */
typedef struct bnk_counters {
    uint64_t sealed, opened, rejected, allowed, denied, delivered, keepalive, replayed, bad_header,
        unknown_index, bad_ip, not_allowed, relayed;
} bnk_counters;
int bnk_counters_get(bnk_ctx *ctx, bnk_counters *out);
int bnk_counters_reset(bnk_ctx *ctx);
/* Counting is on from bnk_init.  Where a device-resident batch needs a launch
 * of its own for it (the framing calls and the relay) that costs about 8 us
 * per 2^20 packets; on = 0 leaves the counting out, and calls made meanwhile
 * are not counted. */
int bnk_counters_enable(bnk_ctx *ctx, int on);

/* ---- transport AEAD ---------------------------------------------------- */

/* Loads n_peers 32-byte ChaCha20-Poly1305 keys (host memory) into key table
 * `which`.  Stands where wireguard-go installs a keypair after the Noise
 * handshake; the reference never sees these keys itself
 * (internal/dataplane/engine.go:51 hands everything to device.NewDevice). */
int bnk_keys_set(bnk_ctx *ctx, int which, const uint8_t *keys32,
                 uint32_t n_peers);

/* Seal: for every packet, ciphertext (len bytes) then the 16-byte tag are
 * written at the packet's position in `out` (only base, bytes, mem, offsets,
 * stride of `out` are read).  Keys come from BNK_KEYS_SEND.  in and out may
 * be the same arena at the same offsets (in place), as wireguard-go's
 * AEAD.Seal(header, nonce, plaintext, nil) is. */
int bnk_aead_seal_batch(bnk_ctx *ctx, const bnk_batch *in,
                        const bnk_batch *out);

/* Open: packet lengths in `in` include the 16-byte tag.  verdict[i] = 1 and
 * the plaintext (len-16 bytes) is written when the tag verifies; verdict[i] =
 * 0 and the plaintext region is zero-filled when it does not (what
 * chacha20poly1305.Open leaves behind); a packet shorter than 16 bytes gets
 * verdict 0 and nothing is written.  Keys come from BNK_KEYS_RECV.  `verdict`
 * lives where in->mem says.  wireguard-go drops packets with verdict 0. */
int bnk_aead_open_batch(bnk_ctx *ctx, const bnk_batch *in,
                        const bnk_batch *out, uint8_t *verdict);

/* bnk_aead_seal_batch for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  The call allocates
 * nothing: the scratch the length grouping needs lives in a file-scope device
 * array of BNK_NOALLOC_MAX_PACKETS + 2072 words (4 MiB + 8 KiB per GPU, held
 * until the process ends).  Device-resident batches only (in->mem and out->mem
 * BNK_MEM_DEVICE), at most BNK_NOALLOC_MAX_PACKETS packets, otherwise
 * BNK_E_INVAL.  Results are those of bnk_aead_seal_batch.  Every call on a GPU
 * shares that GPU's array: calls on one context are serialised on its stream,
 * and a call on another context of the same GPU first makes its stream wait
 * (hipStreamWaitEvent, no host wait) for the event the previous user recorded
 * behind its launches, so such calls take turns on the device. */
#define BNK_NOALLOC_MAX_PACKETS (1u << 20)
int bnk_aead_seal_batch_noalloc(bnk_ctx *ctx, const bnk_batch *in,
                                const bnk_batch *out);

/* ---- packet filter ----------------------------------------------------- */

/* filter.SetRules (internal/filter/filter.go:46-51): enforcement on, rule
 * table replaced; n == 0 is deny-all-but-flows (internal/netmap/netmap.go:49-51).
 * The flow table is kept.  A fresh context is in allow-all mode (filter.New,
 * filter.go:41-43). */
int bnk_filter_set_rules(bnk_ctx *ctx, const bnk_rule *rules, uint32_t n);
/* filter.SetAllowAll (filter.go:54-59): enforcement off, rules dropped,
 * flows kept. */
int bnk_filter_set_allow_all(bnk_ctx *ctx);
/* The filter half of Engine.ApplyNetmap (internal/dataplane/engine.go:279-283)
 * fed with the wire format the control server pushes: a netmap JSON document
 * whose "filter_enabled" / "filter" fields carry []acl.CompiledRule
 * (internal/netmap/netmap.go:44-53, internal/acl/acl.go:33-42); a bare JSON array
 * of rules is accepted too and means filter_enabled.  filter_enabled true ->
 * SetRules(filter), false -> SetAllowAll().  A document Go's decoder would
 * reject (malformed JSON, bad prefix text, port outside 0..65535) returns
 * BNK_E_INVAL and leaves the filter as it was. */
int bnk_filter_apply_netmap_json(bnk_ctx *ctx, const char *json, size_t len);
/* The same parse without a context (no GPU needed): writes up to cap tuples,
 * the total number of tuples to *n_tuples (call again with a larger array when
 * it exceeds cap), filter_enabled as 0/1, and on failure a message to err. */
int bnk_rules_from_netmap_json(const char *json, size_t len, bnk_rule *out, uint32_t cap,
                               uint32_t *n_tuples, int *filter_enabled, char *err,
                               size_t err_cap);

/* filter.NoteOutbound over a batch with one `now` (filter.go:160-167,
 * 189-209), including the len(flows) > 4096 expiry sweep.  now_ns is the
 * time.Time as Unix nanoseconds.  peer/counters of the batch are ignored. */
int bnk_filter_note_outbound_batch(bnk_ctx *ctx, const bnk_batch *pkts,
                                   int64_t now_ns);
/* filter.CheckInbound over a batch with one `now` (filter.go:121-147,
 * 171-178): verdict[i] = 1 pass, 0 drop.  `verdict` lives where pkts->mem
 * says. */
int bnk_filter_check_inbound_batch(bnk_ctx *ctx, const bnk_batch *pkts,
                                   int64_t now_ns, uint8_t *verdict);
/* The [][]byte form the tun.Device wrapper receives (filter.go:160-186):
 * n host pointers and lengths.  Only the first 64 bytes of a packet can
 * matter to the filter (IPv4 header of at most 60 bytes plus 4 port bytes),
 * so only those are staged. */
int bnk_filter_note_outbound_ptrs(bnk_ctx *ctx, const uint8_t *const *pkts,
                                  const uint32_t *lens, uint32_t n,
                                  int64_t now_ns);
int bnk_filter_check_inbound_ptrs(bnk_ctx *ctx, const uint8_t *const *pkts,
                                  const uint32_t *lens, uint32_t n,
                                  int64_t now_ns, uint8_t *verdict);
/* len(f.flows): entries currently in the flow table (live or expired but not
 * yet deleted), as the reference's map would hold. */
int bnk_filter_flow_count(bnk_ctx *ctx, uint32_t *count);
/* Copies up to cap flow entries to host arrays: key = remote<<32 |
 * remotePort<<16 | localPort, proto, expiry in Unix ns (the reference's
 * flowKey and map value, filter.go:26-31,37).  *count receives the number
 * written.  Order unspecified. */
int bnk_filter_flow_dump(bnk_ctx *ctx, uint64_t *key, uint8_t *proto,
                         int64_t *expiry_ns, uint32_t cap, uint32_t *count);

/* ---- WireGuard transport framing ----------------------------------------
 *
 * The datagram around the AEAD: type (LE32 = 4) || receiver index (LE32) ||
 * counter (LE64) || ChaCha20-Poly1305(plaintext zero-padded to 16 bytes).
 * The reference delegates this to golang.zx2c4.com/wireguard's device
 * package, which it only instantiates (internal/dataplane/engine.go:51) and
 * configures with one /32 allowed IP per peer (engine.go:292-299); that
 * package is not in the reference tree, so these entry points follow the
 * WireGuard protocol paper (section 5.4.6) and wireguard-go's documented
 * behaviour (device/send.go, device/receive.go, replay/replay.go). */

enum {
    BNK_WG_OK = 0,            /* data packet, delivered */
    BNK_WG_KEEPALIVE = 1,     /* authentic, empty plaintext */
    BNK_WG_BAD_HEADER = 2,    /* shorter than 32 bytes or type != 4 */
    BNK_WG_UNKNOWN_INDEX = 3, /* no peer owns the receiver index */
    BNK_WG_AUTH_FAIL = 4,     /* tag mismatch */
    BNK_WG_BAD_IP = 5,        /* not IPv4/IPv6 or length fields beyond the plaintext */
    BNK_WG_NOT_ALLOWED = 6,   /* inner source outside the peer's allowed IP */
    BNK_WG_FILTERED = 7,      /* bnk_wg_decap_filter_batch only: delivered by
                                 WireGuard, dropped by the inbound filter */
    BNK_WG_REPLAY = 8         /* authentic, but its counter was seen before, lies
                                 more than 8128 behind the peer's newest, or is
                                 at or beyond RejectAfterMessages */
};

typedef struct bnk_wg_peer {
    uint32_t local_index;  /* receiver index we handed out; unique per peer */
    uint32_t remote_index; /* receiver index the peer expects */
    uint32_t allowed_net;  /* IPv4 prefix, host order (engine.go:292-299: a /32) */
    uint32_t allowed_mask;
} bnk_wg_peer;

/* Installs the whole peer table; peer i uses row i of both key tables.  A row
 * whose local_index and remote_index are both unchanged from the table before
 * is the same keypair and keeps its send counter (a handshake hands out fresh
 * indices, so an unchanged pair means an unchanged key, and restarting its
 * counter would reuse nonces); every other row starts at 0.  Use it for a
 * netmap push (peers added or removed); after one peer's handshake use
 * bnk_wg_peer_set. */
int bnk_wg_peers_set(bnk_ctx *ctx, const bnk_wg_peer *peers, uint32_t n);
/* One peer's new keypair, where wireguard-go installs it after that peer's
 * Noise handshake: replaces row `row` of the peer table and of both key tables
 * (a null key pointer leaves that key as it is) and restarts that row's send
 * counter at 0.  No other row changes: WireGuard peers rekey independently. */
int bnk_wg_peer_set(bnk_ctx *ctx, uint32_t row, const bnk_wg_peer *peer,
                    const uint8_t *key_send32, const uint8_t *key_recv32);
/* Sets one row's next send counter (values above RejectAfterMessages are
 * stored as RejectAfterMessages): for restoring state into a fresh context. */
int bnk_wg_send_counter_set(bnk_ctx *ctx, uint32_t row, uint64_t next);
/* Copies the next send counter of peers [0, n) to a host array. */
int bnk_wg_send_counters(bnk_ctx *ctx, uint64_t *out, uint32_t n);
/* Outgoing: slot i starts at slots' offset i with 16 bytes of headroom,
 * lens[i] bytes of plaintext after it, and room for the padding and the
 * tag.  Pads the plaintext with zeros to a multiple of 16 (never beyond
 * mtu; mtu 0 = no cap), gives each packet its peer's next counter in batch
 * order, writes the header into the headroom and seals in place.
 * wire_len[i] = 16 + lens[i] + padding + 16, the datagram to send from the
 * slot's start.  A keypair stops sending when its counter reaches
 * RejectAfterMessages = 2^64 - 2^13 - 1 (wireguard-go device/send.go): such a
 * packet is left as it was, gets wire_len[i] = 0 and uses no counter, and the
 * peer needs a new handshake (bnk_wg_peer_set).  slots->counters and counter0
 * are ignored.  wire_len lives where slots->mem says. */
int bnk_wg_encap_batch(bnk_ctx *ctx, const bnk_batch *slots, uint32_t mtu,
                       uint32_t *wire_len);
/* Incoming: wire->lens[i] bytes at wire's offset i are one datagram.
 * result[i] is BNK_WG_*; for BNK_WG_OK the inner packet, trimmed to its IP
 * total length, is out_len[i] bytes at out's offset i.  For every result but
 * BAD_HEADER/UNKNOWN_INDEX peer[i] and counter[i] name the sender and the
 * nonce counter; otherwise peer[i] = 0xFFFFFFFF.  A failed open leaves zeros in
 * `out`, like the AEAD entry points.
 * Every authentic packet (any result but BAD_HEADER, UNKNOWN_INDEX, AUTH_FAIL)
 * goes through its peer's anti-replay window (RFC 6479, 8128 counters, kept on
 * the device per row of the peer table) in batch order, before the keepalive,
 * IP and allowed-IP checks count, as wireguard-go's sequential receiver does:
 * a packet the window turns away reports BNK_WG_REPLAY (out_len 0, plaintext
 * left in `out`), and an authentic packet with a bad or disallowed inner
 * header still moves the window.  bnk_wg_set_replay(ctx, 0) leaves the windows
 * out (for a caller that keeps its own).  wire->peer/counters are ignored.
 * result, out_len, peer and counter live where wire->mem says. */
int bnk_wg_decap_batch(bnk_ctx *ctx, const bnk_batch *wire, const bnk_batch *out,
                       uint8_t *result, uint32_t *out_len, uint32_t *peer,
                       uint64_t *counter);

/* Anti-replay windows on (default) or off for bnk_wg_decap_batch and
 * bnk_wg_decap_filter_batch.  Off: no packet reports BNK_WG_REPLAY and the
 * windows stand still; the caller then feeds peer[i]/counter[i] of every
 * authentic packet to a window of its own. */
int bnk_wg_set_replay(bnk_ctx *ctx, int on);

/* Where the framing of large batches (a packet per lane) is done: inside the
 * AEAD launch (default), or (on = 0) in kernels of their own around a plain
 * seal or open.  Results are the same; the second form is kept as a
 * cross-check and costs about 80 us per 2^20 packets.  No counterpart in the
 * reference. */
int bnk_wg_set_fused(bnk_ctx *ctx, int on);

/* The receive path of a tunnel in one call: bnk_wg_decap_batch, then
 * CheckInbound (internal/filter/filter.go:121-147) with one now_ns on every
 * packet that came out BNK_WG_OK, as filteredTUN.Write (filter.go:171-186)
 * does with what wireguard-go hands it.  A packet the filter denies reports
 * BNK_WG_FILTERED; everything else about it (plaintext in its slot, out_len,
 * peer, counter) is as for BNK_WG_OK, and its counter has moved the replay
 * window, because wireguard-go runs the window before the write that filters.
 * In allow-all mode nothing is filtered.  Same arguments as
 * bnk_wg_decap_batch otherwise. */
int bnk_wg_decap_filter_batch(bnk_ctx *ctx, const bnk_batch *wire, const bnk_batch *out,
                              int64_t now_ns, uint8_t *result, uint32_t *out_len,
                              uint32_t *peer, uint64_t *counter);
/* The send path in one call: NoteOutbound (filter.go:189-209) with one
 * now_ns on every plaintext, as filteredTUN.Read (filter.go:160-167) does
 * with what the TUN hands it, then bnk_wg_encap_batch. */
int bnk_wg_note_encap_batch(bnk_ctx *ctx, const bnk_batch *slots, uint32_t mtu,
                            int64_t now_ns, uint32_t *wire_len);

/* ---- fused relay ------------------------------------------------------- */

enum { BNK_RELAY_OK = 0, BNK_RELAY_FORGED = 1, BNK_RELAY_DENIED = 2 };

/* open (BNK_KEYS_RECV, in->peer, in->counters) -> CheckInbound at now_ns ->
 * seal under BNK_KEYS_SEND[peer_out[i]] with counter ctr_base_out[peer_out[i]]
 * + (number of earlier packets in the batch with verdict OK and the same
 * peer_out).  verdict[i] is BNK_RELAY_*; for OK packets the re-sealed packet
 * (same length as the input) is written to `out` and its counter to
 * ctr_out[i]; FORGED and DENIED packets leave `out` untouched and get
 * ctr_out[i] = 0.  The reference has no such function (its server relays
 * ciphertext unopened, internal/coord/server/server.go:439-453); this is the
 * composition of the three steps above.  peer_out, ctr_base_out (n_peers_out
 * entries), verdict and ctr_out live where in->mem says. */
int bnk_relay_fused_batch(bnk_ctx *ctx, const bnk_batch *in,
                          const uint32_t *peer_out,
                          const uint64_t *ctr_base_out, uint32_t n_peers_out,
                          int64_t now_ns, const bnk_batch *out,
                          uint8_t *verdict, uint64_t *ctr_out);

#ifdef __cplusplus
}
#endif
#endif
