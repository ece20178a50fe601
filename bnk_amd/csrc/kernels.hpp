// Launch interfaces between the C ABI (api.hip) and the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bnk {

// WireGuard pads the plaintext with zeros to a multiple of 16, never beyond the
// MTU (a packet longer than the MTU pads its remainder).
__host__ __device__ inline uint32_t wg_padding(uint32_t len, uint32_t mtu)
{
    uint32_t last = len;
    if (mtu == 0) return ((last + 15u) & ~15u) - last;
    if (last > mtu) last %= mtu;
    uint32_t padded = (last + 15u) & ~15u;
    if (padded > mtu) padded = mtu;
    return padded - last;
}

// A keypair whose send counter has reached this value sends nothing more
// (wireguard-go device/constants.go: RejectAfterMessages = 2^64 - 2^13 - 1).
constexpr uint64_t WG_REJECT_AFTER_MESSAGES = ~0ull - (1ull << 13);

// base + rank, stopping at `limit` instead of wrapping (limit 0: plain sum).
__host__ __device__ inline uint64_t ctr_add(uint64_t base, uint64_t rank, uint64_t limit)
{
    const uint64_t c = base + rank;
    if (limit == 0) return c;
    return (c < base || c > limit) ? limit : c;
}

// WireGuard transport framing done by the AEAD launch itself.  A wave-per-packet
// launch (small batches): in/out offsets address the slot or datagram
// (in_skip = out_skip = 0) and every packet must be at most WG_FUSE_MAX_LEN
// bytes long, padding included.  A lane-per-packet launch: in_skip and
// out_skip say where the AEAD data starts within the slot or datagram (16 past
// the header), any length.
// Receiver index -> peer row as an open-addressing table of (index, row) pairs
// with linear probing; an empty slot has row WG_HASH_EMPTY.
constexpr uint32_t WG_HASH_EMPTY = 0xFFFFFFFFu;
__host__ __device__ inline uint32_t wg_hash_slot(uint32_t index, uint32_t bits)
{
    return (index * 0x9E3779B1u) >> (32u - bits);
}

// Sender (0xFFFFFFFF: none) and position of a packet in one word: the position in the low
// index_bits bits, the sender's low bits above them ("none" is then all ones, above every
// sender, as long as the field is wider than the largest sender).
__host__ __device__ inline uint32_t wg_replay_pack(uint32_t sender, uint32_t position, unsigned index_bits)
{
    return sender << index_bits | position;
}

struct WgFuse {
    uint32_t mode;               // WG_FUSE_*
    uint32_t n_peers;            // rows of the peer tables
    uint32_t mtu;                // encapsulate: padding cap
    const uint2 *index_sorted;   // decapsulate, a wave per packet: (receiver index, peer), ascending
    const uint2 *index_hash;     // decapsulate, a lane per packet: the same as a hash table of
    uint32_t hash_bits;          // 2^hash_bits slots (wg_hash_slot)
    const uint2 *allowed;        // decapsulate: (net, mask) per peer
    const uint32_t *remote_index; // encapsulate: index the peer expects
    uint8_t *result;             // decapsulate: BNK_WG_* per packet
    uint32_t *out_len;           // decapsulate: inner packet length
    uint32_t *peer_out;          // decapsulate: sender
    uint64_t *counter_out;       // decapsulate: its counter
    uint32_t *replay_keys;       // decapsulate, a lane per packet, or nullptr: [i - first] = the sender
    uint32_t *replay_idx;        // when the tag verified, else 0xFFFFFFFF; and i - first itself.  With
    uint32_t replay_index_bits;  // replay_index_bits != 0 both in one word of replay_keys
                                 // (wg_replay_pack) and replay_idx is not written
    uint32_t *wire_len;          // encapsulate: datagram length
};
enum : uint32_t { WG_FUSE_OFF = 0, WG_FUSE_ENCAP = 1, WG_FUSE_DECAP = 2 };
constexpr uint32_t WG_FUSE_MAX_LEN = 63u * 64u;
// No packet is longer than this: a length word above it (only a device-resident
// batch can carry one unseen) is treated as reaching beyond the arena, so that
// length + tag and length + padding never wrap 32 bits.
constexpr uint32_t MAX_PACKET_BYTES = 0x7FFFFFFFu;

// Device-side view of one AEAD launch.  All pointers are device pointers.
struct AeadArgs {
    const uint8_t *in;
    uint8_t *out;
    const uint32_t *keys;      // n_peers * 8 little-endian words
    const uint64_t *in_off;    // or nullptr: i * in_stride
    const uint64_t *out_off;   // or nullptr: i * out_stride
    const uint32_t *lens;      // or nullptr: len
    const uint32_t *peer;      // or nullptr: 0
    const uint64_t *counters;  // or nullptr: counter0 + i
    const uint32_t *order;     // or nullptr: lane t handles packet t
    uint8_t *verdict;          // open only
    uint8_t *heads;            // open by aead_wave_kernel only, or nullptr: one 32-byte record per
                               // lane of the launch, in launch order (record t belongs to packet
                               // first + order[t], or first + t without order[]): bytes 0-23 of the
                               // plaintext, then its length and 1 if it is authentic (two words)
    const uint8_t *skip;       // or nullptr; skip[i] != 0 leaves packet i alone
    uint32_t *status;          // device status word, bit 0 = peer out of range
    uint64_t counter0;
    uint32_t n;
    uint32_t in_stride, out_stride;
    uint32_t len;
    uint32_t n_peers;
    uint32_t trim;             // seal only: lens[i] - trim is the plaintext length
    uint32_t in_skip, out_skip; // bytes between a packet's offset and its AEAD data
    uint64_t in_limit, out_limit; // arena sizes for batches whose per-packet arrays the host cannot
                               // read (device resident): a packet reaching beyond them is left
                               // alone, gets verdict 0 and raises STATUS_BOUNDS.  0: the host
                               // has checked the layout
    uint32_t first;            // the launch covers packets first .. first+n-1; order[] is relative to first
    uint32_t spread_max;       // launches of at most this many packets run one wave per packet
    unsigned long long *tally; // open, a lane per packet, or nullptr: the launch counts its own verdicts
                               // here (TALLY_OPENED / TALLY_REJECTED, see tally_bump)
    WgFuse wg;                 // only with aead_runs_spread(); mode 0: plain AEAD
};

// Below this many packets a wave per packet finishes sooner than a lane per
// packet (which needs 64 packets per wave and about 130 000 to fill the chip).
constexpr uint32_t SPREAD_MAX_PACKETS = 4096;

// What kernels report besides their results.  The status words live in pinned
// host memory that the GPU can write: one word per condition, raised with a
// plain store of 1 (the same store from every lane that has the news, so no
// atomic is needed), and read by the host after it has waited for the stream,
// with no copy.
// Hot-path counters (tally.hip): TALLY_LANES words per counter, summed when they
// are read, so that the waves of a launch that counts for itself spread their
// additions.
enum TallySlot {
    TALLY_SEALED, TALLY_OPENED, TALLY_REJECTED, TALLY_ALLOWED, TALLY_DENIED, TALLY_DELIVERED, TALLY_KEEPALIVE,
    TALLY_REPLAYED, TALLY_BAD_HEADER, TALLY_UNKNOWN_INDEX, TALLY_BAD_IP, TALLY_NOT_ALLOWED, TALLY_RELAYED
};
constexpr int TALLY_SLOTS = 16;
constexpr uint32_t TALLY_LANES = 64;
static_assert(TALLY_RELAYED < TALLY_SLOTS, "slots");
#if defined(__HIPCC__)
__device__ inline void tally_bump(unsigned long long *tally, uint32_t slot, uint32_t k)
{
    if (k != 0u) atomicAdd(&tally[slot * TALLY_LANES + (blockIdx.x & (TALLY_LANES - 1u))], (unsigned long long)k);
}
#endif

enum : uint32_t { STATUS_PEER_RANGE = 1u, STATUS_FLOWS_FULL = 2u, STATUS_BOUNDS = 4u, STATUS_INTERNAL = 8u };
constexpr uint32_t STATUS_WORDS = 8; // word [bit value] holds that condition
// Word 7 of the same block is no condition: a one-thread launch writes the number of the
// wait it ends there, for the host to watch (wait_stream in api.hip).
constexpr uint32_t STATUS_DONE_WORD = 7;

// True when [off, off + len) does not fit an arena of `limit` bytes (limit 0: not checked).
__host__ __device__ inline bool beyond_arena(uint64_t off, uint64_t len, uint64_t limit)
{
    return limit != 0 && (off > limit || len > limit - off);
}
#if defined(__HIPCC__)
__device__ inline void status_raise(uint32_t *status, uint32_t condition)
{
    __hip_atomic_store(&status[condition], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
#endif

// True when the launch will run one wave per packet (then order[] is not used
// and callers need not build it).
bool aead_runs_spread(const AeadArgs &a);
hipError_t launch_aead_seal(const AeadArgs &a, hipStream_t s);
hipError_t launch_aead_open(const AeadArgs &a, hipStream_t s);

// order[] = packet indices grouped by ChaCha20 block count, longest first, so
// the lanes of a wave run the same number of rounds.  hist and cursor are
// device scratch of LEN_BINS and LEN_CURSOR_WORDS words; hist must be all zeros on entry and
// is all zeros again when the grouping has run.
constexpr uint32_t LEN_BINS = 1032;
constexpr uint32_t LEN_CURSOR_WORDS = LEN_BINS + 8;
hipError_t launch_length_sort(const uint32_t *lens, uint32_t n, uint32_t tag_bytes,
                              uint32_t *order, uint32_t *hist, uint32_t *cursor,
                              hipStream_t s);

// p[0..n) = v on the stream (a kernel, so it is safe under graph capture).
hipError_t launch_fill_u32(uint32_t *p, uint32_t n, uint32_t v, hipStream_t s);
// One thread behind everything queued so far: fence, then store v to *word at system scope.
hipError_t launch_done_word(uint32_t *word, uint32_t v, hipStream_t s);

// Fused relay bookkeeping (relay_kernels.hip).  After open (auth[i]) and the
// filter (pass[i]): verdicts, then per-peer batch-order counters for the
// survivors.  sort_tmp holds sort_tmp_bytes of scratch (relay_sort_tmp_bytes).
// With advance set, ctr_base_out (then writable) moves past the counters
// handed out, so that the next part of the same batch continues them.
size_t relay_sort_tmp_bytes(uint32_t n, uint32_t n_keys);
hipError_t launch_relay_assign(const uint8_t *auth, const uint8_t *pass, const uint32_t *peer_out,
                               const uint64_t *ctr_base_out, uint32_t n_peers_out, uint32_t n,
                               uint32_t *keys, uint32_t *idx, uint32_t *skeys, uint32_t *sidx,
                               void *sort_tmp, size_t sort_tmp_bytes, uint8_t *verdict,
                               uint64_t *ctr_out, uint32_t *status, bool advance, hipStream_t s);

// Batch-order counters per peer: ctr_out[i] = ctr_base[keys[i]] + (number of
// earlier i' with the same key), for keys[i] < n_keys; other keys must be
// 0xFFFFFFFF.  keys/idx are
// inputs (idx[i] = i), skeys/sidx and sort_tmp scratch.  With advance set,
// ctr_base[key] moves past the counters handed out.
// ctr_limit: 0, or the value counters saturate at (handed-out counters never wrap
// past it and an advanced base stops there): WG_REJECT_AFTER_MESSAGES for a
// keypair's send counter.
hipError_t launch_peer_rank(uint32_t *keys, uint32_t *idx, uint32_t *skeys, uint32_t *sidx,
                            void *sort_tmp, size_t sort_tmp_bytes, uint64_t *ctr_base, uint32_t n_keys,
                            uint32_t n, uint64_t *ctr_out, bool advance, uint64_t ctr_limit, hipStream_t s);

// The same straight from a caller's peer array, without a sort, where the peer
// table is small enough for the counting form (peer_rank_counts says whether;
// tmp as for launch_peer_rank): a peer index beyond the table raises
// STATUS_PEER_RANGE in *status and gets counter 0.
bool peer_rank_counts(uint32_t n, uint32_t n_keys, size_t tmp_bytes);
hipError_t launch_peer_rank_counting(const uint32_t *peer, void *tmp, uint64_t *ctr_base, uint32_t n_keys, uint32_t n,
                                     uint64_t *ctr_out, bool advance, uint64_t ctr_limit, uint32_t *status,
                                     hipStream_t s);

// Copy of a byte span whose two ends share their alignment within 16 bytes,
// one aligned 16-byte piece per lane (used to fetch small spans of pinned
// host memory).
hipError_t launch_pull(const void *src, void *dst, uint64_t bytes, hipStream_t s);

// launch_wg_keys + launch_peer_rank for at most PEER_RANK_SMALL_MAX packets in
// one launch, straight from the peer array (null: every packet is peer 0).  A
// peer index beyond the table sets STATUS_PEER_RANGE and gets no counter.
constexpr uint32_t PEER_RANK_SMALL_MAX = 1024;
hipError_t launch_peer_rank_small(const uint32_t *peer, uint32_t n_keys, uint32_t n, uint64_t *ctr_base,
                                  uint64_t *ctr_out, bool advance, uint64_t ctr_limit, uint32_t *status,
                                  hipStream_t s);

} // namespace bnk
