// Device-side views for the WireGuard transport framing kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bnk {

struct WgPeersDev {
    const uint2 *index_sorted;   // (local receiver index, peer), ascending by index
    const uint2 *index_hash;     // the same pairs in a hash table of 2^hash_bits slots (wg_hash_slot)
    uint32_t hash_bits;
    const uint32_t *remote_index; // [n] index the peer expects in the header
    const uint2 *allowed;         // [n] (net, mask) of the peer's allowed IPv4 prefix
    uint64_t *send_ctr;           // [n] next nonce counter per peer
    uint32_t n;
};

struct WgBatch {
    const uint8_t *base;
    const uint64_t *off;  // or nullptr: i * stride
    const uint32_t *lens; // or nullptr: len
    uint32_t n, stride, len;
    uint32_t first; // the launch covers packets first .. first+n-1 of the arrays
    uint64_t limit; // arena size when the host could not check the layout (device-resident
                    // per-packet arrays), else 0: see AeadArgs::in_limit
};

hipError_t launch_wg_parse(const WgBatch &b, const WgPeersDev &pe, uint32_t *peer, uint64_t *counter,
                           uint32_t *ct_len, uint8_t *result, uint32_t *status, hipStream_t s);
hipError_t launch_wg_finish(const WgBatch &out, uint32_t out_skip, const WgPeersDev &pe,
                            const uint32_t *peer, const uint32_t *ct_len, const uint8_t *auth,
                            uint8_t *result, uint32_t *out_len, hipStream_t s);
hipError_t launch_wg_keys(const uint32_t *peer, uint32_t n_peers, uint32_t n, uint32_t *keys,
                          uint32_t *idx, uint32_t *status, hipStream_t s);
hipError_t launch_wg_encap_prep(const WgBatch &b, uint8_t *hdr_base, const WgPeersDev &pe, const uint32_t *peer,
                                const uint64_t *counter, uint32_t mtu, uint32_t *padded_len,
                                uint32_t *wire_len, uint8_t *skip, uint32_t *status, hipStream_t s);

// Anti-replay windows (wg_replay.hip): per peer WG_REPLAY_WORDS 64-bit words,
// `last` then a ring of WG_REPLAY_BLOCKS blocks of 64 counters (RFC 6479 as
// wireguard-go's replay.Filter: window (128 - 1) * 64 = 8128).
constexpr uint32_t WG_REPLAY_BLOCKS = 128;
constexpr uint32_t WG_REPLAY_WORDS = 1 + WG_REPLAY_BLOCKS;
constexpr uint32_t WG_REPLAY_SMALL_MAX = 1024; // at most this many packets: one launch of one block

struct WgReplayDev {
    uint64_t *state; // [n_peers][WG_REPLAY_WORDS]
    uint32_t n_peers;
};

// Device scratch of one replay pass over n packets (beyond WG_REPLAY_SMALL_MAX).
struct WgReplayScratch {
    uint32_t *keys, *idx, *skeys, *sidx;   // n words each
    uint64_t *sctr, *sval, *pmax;          // n each
    uint8_t *cls;                          // n
    uint32_t *flags;                       // two words, used in turn (parity): "this pass had late
                                           // packets".  Both start out 0; a pass clears the other one
    uint32_t parity;                       // 0 or 1, the other value in the next pass
    uint32_t *table;                       // table_slots words, a power of two >= 2 n, all
                                           // 0xFFFFFFFF between passes (a pass that used it clears it)
    uint32_t table_slots;
    bool keys_ready;                       // keys[] and idx[] have been written by the open launch
    void *tmp;                             // wg_replay_tmp_bytes(n, n_peers)
    size_t tmp_bytes;
};
size_t wg_replay_tmp_bytes(uint32_t n, uint32_t n_peers);
// When a sender and a position within a pass of n packets fit one word together: the bits
// the position takes (the sender sits above them; see wg_replay_pack), else 0.  With it
// WgReplayScratch::keys holds those words (and idx is scratch), without it keys and idx
// hold senders and positions.
unsigned wg_replay_index_bits(uint32_t n, uint32_t n_peers);
uint32_t wg_replay_table_slots(uint32_t n);
// Runs every packet whose result so far says "authentic" (anything but
// BAD_HEADER, UNKNOWN_INDEX, AUTH_FAIL) through its peer's window, in batch
// order per peer; a packet the window turns away gets BNK_WG_REPLAY and
// out_len 0.  The arrays are indexed from the first packet of the pass.
hipError_t launch_wg_replay(uint8_t *result, uint32_t *out_len, const uint32_t *peer, const uint64_t *counter,
                            uint32_t n, const WgReplayDev &rp, const WgReplayScratch &sc, hipStream_t s);
// Clears the windows of the rows whose flag is set.
hipError_t launch_wg_replay_reset(uint64_t *state, const uint8_t *flags, uint32_t n_peers, hipStream_t s);


} // namespace bnk
