// Anti-replay window of the WireGuard receive path (RFC 6479 as wireguard-go's
// replay.Filter keeps it: a ring of 128 64-bit blocks, window 8128 counters),
// one window per peer, device resident, applied to a whole batch at once with
// the result the sequential receiver would reach packet by packet.
//
// wireguard-go validates the counter of every authentic packet, in arrival
// order per peer, before it looks at the plaintext (device/receive.go,
// RoutineSequentialReceiver; the reference only instantiates that device,
// internal/dataplane/engine.go:51).  Sequentially the filter does, per packet:
// reject counter >= limit; if counter > last, clear the blocks passed over and
// move last; else reject when last - counter > window; then test-and-set the
// counter's bit.  For a batch this unrolls without walking it in order:
//
//   last before packet j  = max(last before the batch, counters of earlier
//                           packets of the same peer)   -- a running maximum,
//                           whether those packets were accepted or not, because
//                           a packet that does not move last is not above it;
//   packet j reaches the bit test iff counter < limit and it is not more than
//                           the window behind that last;
//   its bit is already set iff the counter was seen before: in the window the
//                           batch started with, or by an earlier packet of the
//                           batch with the same counter (which reached the bit
//                           test too, the window having only moved forward
//                           since).  Inside the window a bit is never stale:
//                           a slot is cleared the moment last enters or passes
//                           its block.
//
// So: a stable sort of (peer, position) brings each peer's packets together in
// batch order, a segmented running maximum gives every packet its `last`, a
// hash table keyed by (peer, counter) finds the first of equal counters (only
// packets at or below an earlier counter can be repeats, so a batch whose
// counters rise within every peer never touches the table), and the windows
// are brought up to date afterwards (clear what last passed over, then set the
// bits of everything that reached the bit test and still lies in the final
// window).
#include <string.h>

#include <algorithm>

#include <rocprim/rocprim.hpp>

#include "../../include/bnkhip.h"
#include "kernels.hpp"
#include "wg_dev.hpp"

namespace bnk {

namespace {

constexpr uint32_t NO_PEER = 0xFFFFFFFFu;
constexpr uint32_t HASH_EMPTY = 0xFFFFFFFFu;
constexpr uint64_t WINDOW = (WG_REPLAY_BLOCKS - 1u) * 64u; // 8128

__device__ __forceinline__ bool replay_subject(uint8_t result)
{
    // everything that was authentic: the tag verified
    return result != BNK_WG_BAD_HEADER && result != BNK_WG_UNKNOWN_INDEX && result != BNK_WG_AUTH_FAIL;
}

__device__ __forceinline__ uint64_t mix(uint64_t x)
{
    x ^= x >> 33;
    x *= 0xff51afd7ed558ccdULL;
    x ^= x >> 33;
    x *= 0xc4ceb9fe1a85ec53ULL;
    x ^= x >> 33;
    return x;
}

// Does the packet reach the filter's bit test, given `last` just before it?
__device__ __forceinline__ bool reaches_bit_test(uint64_t c, uint64_t last)
{
    return c < WG_REJECT_AFTER_MESSAGES && (c > last || last - c <= WINDOW);
}

// Was counter c (at or below last0, inside the window) seen before the batch?
__device__ __forceinline__ bool seen_before(const uint64_t *st, uint64_t c)
{
    return (st[1u + ((c >> 6) & (WG_REPLAY_BLOCKS - 1u))] >> (c & 63u)) & 1ull;
}

// Brings one peer's window to `new_last`: clears the blocks passed over.
__device__ __forceinline__ void advance_window(uint64_t *st, uint64_t new_last)
{
    const uint64_t last0 = st[0];
    if (new_last <= last0) return;
    const uint64_t cur = last0 >> 6;
    uint64_t diff = (new_last >> 6) - cur;
    if (diff > WG_REPLAY_BLOCKS) diff = WG_REPLAY_BLOCKS;
    for (uint64_t b = cur + 1; b <= cur + diff; b++) st[1u + (b & (WG_REPLAY_BLOCKS - 1u))] = 0;
    st[0] = new_last;
}

// ---- large batches ---------------------------------------------------------

__global__ __launch_bounds__(256) void replay_keys_kernel(const uint8_t *result, const uint32_t *peer,
                                                          uint32_t n_peers, uint32_t n, uint32_t *keys,
                                                          uint32_t *idx)
{
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n) return;
    const uint32_t p = peer[i];
    keys[i] = (replay_subject(result[i]) && p < n_peers) ? p : NO_PEER;
    idx[i] = i;
}

// The same as one word per packet, sender above position (wg_replay_index_bits):
// a stable sort on the sender's bits alone then moves half the bytes.
__global__ __launch_bounds__(256) void replay_keys_packed_kernel(const uint8_t *result, const uint32_t *peer,
                                                                 uint32_t n_peers, uint32_t n, unsigned index_bits,
                                                                 uint32_t *packed)
{
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n) return;
    const uint32_t p = peer[i];
    packed[i] = wg_replay_pack((replay_subject(result[i]) && p < n_peers) ? p : NO_PEER, i, index_bits);
}

// ---------------------------------------------------------------------------
// Running maximum per peer in sorted order: pmax[p] = the largest sval of the
// earlier positions with p's key, 0 when there is none.  A segmented exclusive
// max-scan, the segments being the peers' runs.  Two steps: every block of
// SEG_BLOCK positions reduces to what it hands on (in the launch that puts the
// counters into sorted order), and every block scans itself again, together
// with the carries of the blocks before it back to the nearest head (seg_handed;
// inside replay_classify_kernel, which needs the values).
// ---------------------------------------------------------------------------
constexpr uint32_t SEG_BLOCK = 1024;

__device__ __forceinline__ uint64_t shfl_up64(uint64_t v, unsigned off)
{
    const uint32_t lo = (uint32_t)__shfl_up((int)(uint32_t)v, off, 64);
    const uint32_t hi = (uint32_t)__shfl_up((int)(uint32_t)(v >> 32), off, 64);
    return (uint64_t)hi << 32 | lo;
}

struct SegScan {
    uint64_t excl;    // maximum over my run's earlier positions within the block
    bool open;        // my run began before the block (and I am not its head)
    uint64_t prev;    // what the position before me ends with (0 for the block's first)
    uint64_t total;   // the block's last run, maximum over its positions in the block
    bool total_open;  // the block holds no head at all
};

// For a block of SEG_BLOCK threads in position order; head: my key differs from
// the position before me.
__device__ __forceinline__ SegScan seg_block_scan(uint64_t v, bool head)
{
    __shared__ uint64_t wave_x[SEG_BLOCK / 64];
    __shared__ uint32_t wave_f[SEG_BLOCK / 64];
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;
    // inclusive within the wave: x = maximum back to my run's head or the wave's
    // first lane, f = a head lies in that span
    uint64_t x = v;
    uint32_t f = head ? 1u : 0u;
#pragma unroll
    for (unsigned off = 1; off < 64; off <<= 1) {
        const uint64_t xo = shfl_up64(x, off);
        const uint32_t fo = (uint32_t)__shfl_up((int)f, off, 64);
        if (lane >= off && !f) {
            x = xo > x ? xo : x;
            f = fo;
        }
    }
    if (lane == 63u) {
        wave_x[wv] = x;
        wave_f[wv] = f;
    }
    __syncthreads();
    // the same over the waves' last lanes, by the first wave
    if (wv == 0) {
        uint64_t ax = lane < SEG_BLOCK / 64 ? wave_x[lane] : 0;
        uint32_t af = lane < SEG_BLOCK / 64 ? wave_f[lane] : 1u;
#pragma unroll
        for (unsigned off = 1; off < SEG_BLOCK / 64; off <<= 1) {
            const uint64_t xo = shfl_up64(ax, off);
            const uint32_t fo = (uint32_t)__shfl_up((int)af, off, 64);
            if (lane >= off && !af) {
                ax = xo > ax ? xo : ax;
                af = fo;
            }
        }
        if (lane < SEG_BLOCK / 64) {
            wave_x[lane] = ax;
            wave_f[lane] = af;
        }
    }
    __syncthreads();
    const uint64_t before_x = wv ? wave_x[wv - 1] : 0; // up to the last lane of the wave before mine
    const uint32_t before_f = wv ? wave_f[wv - 1] : 0u;
    if (!f) {
        x = before_x > x ? before_x : x;
        f = before_f;
    }
    // exclusive: what the position before me holds
    uint64_t px = shfl_up64(x, 1);
    uint32_t pf = (uint32_t)__shfl_up((int)f, 1, 64);
    if (lane == 0) {
        px = before_x;
        pf = before_f;
    }
    SegScan r;
    r.excl = head ? 0 : px;
    r.open = !head && !pf;
    r.prev = px;
    r.total = wave_x[SEG_BLOCK / 64 - 1];
    r.total_open = wave_f[SEG_BLOCK / 64 - 1] == 0u;
    return r;
}

__device__ __forceinline__ bool seg_head(const uint32_t *skeys, uint32_t p, uint32_t n, uint32_t key)
{
    return p >= n || p == 0u || skeys[p - 1u] != key;
}

// Sender, position and counter of the packets in sorted order, from the sorted
// words, and what each block of positions hands on to the running maximum
// (carry_x: the maximum over the block's last run; carry_open: the block holds no head).
__global__ __launch_bounds__(SEG_BLOCK) void replay_unpack_kernel(const uint32_t *sorted, const uint64_t *counter,
                                                                  uint32_t n, unsigned index_bits, unsigned peer_bits,
                                                                  uint32_t *skeys, uint32_t *sidx, uint64_t *sctr,
                                                                  uint64_t *sval, uint64_t *carry_x,
                                                                  uint32_t *carry_open)
{
    const uint32_t p = blockIdx.x * SEG_BLOCK + threadIdx.x;
    const uint32_t none = (1u << peer_bits) - 1u;
    uint32_t field = none, before = none;
    uint64_t v = 0;
    if (p < n) {
        const uint32_t w = sorted[p];
        field = (w >> index_bits) & none;
        if (p) before = (sorted[p - 1u] >> index_bits) & none;
        const uint32_t i = w & ((1u << index_bits) - 1u);
        const uint64_t c = field != none ? counter[i] : 0;
        v = c < WG_REJECT_AFTER_MESSAGES ? c : 0;
        skeys[p] = field != none ? field : NO_PEER;
        sidx[p] = i;
        sctr[p] = c;
        sval[p] = v;
    }
    const SegScan r = seg_block_scan(v, p >= n || p == 0u || before != field);
    if (threadIdx.x == 0) {
        carry_x[blockIdx.x] = r.total;
        carry_open[blockIdx.x] = r.total_open ? 1u : 0u;
    }
}

// Counters in sorted order (a counter the filter turns away outright counts as
// 0 for the running maximum: it never moves last), and the blocks' carries.
__global__ __launch_bounds__(SEG_BLOCK) void replay_gather_kernel(const uint32_t *skeys, const uint32_t *sidx,
                                                                  const uint64_t *counter, uint32_t n,
                                                                  uint64_t *sctr, uint64_t *sval, uint64_t *carry_x,
                                                                  uint32_t *carry_open)
{
    const uint32_t p = blockIdx.x * SEG_BLOCK + threadIdx.x;
    const uint32_t key = p < n ? skeys[p] : NO_PEER;
    uint64_t v = 0;
    if (p < n) {
        const uint64_t c = key != NO_PEER ? counter[sidx[p]] : 0;
        v = c < WG_REJECT_AFTER_MESSAGES ? c : 0;
        sctr[p] = c;
        sval[p] = v;
    }
    const SegScan r = seg_block_scan(v, seg_head(skeys, p, n, key));
    if (threadIdx.x == 0) {
        carry_x[blockIdx.x] = r.total;
        carry_open[blockIdx.x] = r.total_open ? 1u : 0u;
    }
}

// What block b is handed: the maximum of the run that runs into it, over the
// blocks before it -- the blocks' carries from the nearest one that holds a
// head onwards.  Every thread of the block takes part; the carries are read
// SEG_BLOCK at a time, going back (a run seldom spans more than a few blocks).
__device__ __forceinline__ uint64_t seg_handed(const uint64_t *carry_x, const uint32_t *carry_open, uint32_t b)
{
    uint64_t acc = 0;
    for (uint32_t hi = b; hi > 0u;) {
        // blocks hi - SEG_BLOCK .. hi - 1, right-aligned: what falls before block 0 is neutral
        const int64_t at = (int64_t)hi - (int64_t)SEG_BLOCK + (int64_t)threadIdx.x;
        const uint64_t v = at >= 0 ? carry_x[at] : 0;
        const bool head = at >= 0 && carry_open[at] == 0u;
        __syncthreads(); // the scan before this one has been read out of its LDS words
        const SegScan r = seg_block_scan(v, head);
        acc = r.total > acc ? r.total : acc;
        if (!r.total_open) break;
        hi = hi > SEG_BLOCK ? hi - SEG_BLOCK : 0u;
    }
    return acc;
}

// What the window decides about a packet without looking at other packets'
// counters: turned away outright, ahead of everything before it (fresh for
// certain), inside the window with its bit set before the batch (a repeat for
// certain), or inside the window at or below an earlier counter with the bit
// clear ("late": fresh unless an earlier packet of the batch carried the
// counter too).
enum : uint8_t { RP_NONE = 0, RP_AHEAD = 1, RP_LATE = 2, RP_SEEN = 3 };

__device__ __forceinline__ uint32_t table_home(uint32_t key, uint64_t c, uint32_t mask)
{
    return (uint32_t)mix(c ^ ((uint64_t)key << 40) ^ key) & mask;
}

// The running maximum of every packet's peer (a segmented scan within the block
// plus what the block is handed), the packet's class, REPLAY for what never
// reaches the bit test and for what the window had seen before the batch; late
// packets enter the table (slot = earliest sorted position among the late
// packets carrying that peer and counter) and raise flags[0].
__global__ __launch_bounds__(SEG_BLOCK) void replay_classify_kernel(const uint32_t *skeys, const uint32_t *sidx,
                                                                    const uint64_t *sctr, const uint64_t *sval,
                                                                    const uint64_t *carry_x,
                                                                    const uint32_t *carry_open, uint64_t *pmax,
                                                                    const uint64_t *state, uint32_t n, uint8_t *cls,
                                                                    uint32_t *table, uint32_t mask, uint32_t *flags,
                                                                    uint8_t *result, uint32_t *out_len)
{
    const uint32_t p = blockIdx.x * SEG_BLOCK + threadIdx.x;
    const uint32_t key = p < n ? skeys[p] : NO_PEER;
    const SegScan seg = seg_block_scan(p < n ? sval[p] : 0, seg_head(skeys, p, n, key));
    const uint64_t handed = seg_handed(carry_x, carry_open, blockIdx.x);
    if (p >= n) return;
    uint64_t before = seg.excl;
    if (seg.open && handed > before) before = handed;
    pmax[p] = before;
    uint8_t k = RP_NONE;
    if (key != NO_PEER) {
        const uint64_t c = sctr[p];
        const uint64_t *st = state + (size_t)key * WG_REPLAY_WORDS;
        const uint64_t last0 = st[0];
        const uint64_t last = last0 > before ? last0 : before;
        if (reaches_bit_test(c, last)) k = c > last ? RP_AHEAD : RP_LATE;
        if (k == RP_LATE && c <= last0 && seen_before(st, c)) k = RP_SEEN;
        if (k == RP_NONE || k == RP_SEEN) {
            const uint32_t i = sidx[p];
            result[i] = BNK_WG_REPLAY;
            out_len[i] = 0;
        } else if (k == RP_LATE) {
            flags[0] = 1u; // the same value from every lane that has the news
            uint32_t h = table_home(key, c, mask);
            for (;;) {
                const uint32_t old = atomicCAS(&table[h], HASH_EMPTY, p);
                if (old == HASH_EMPTY) break;
                if (skeys[old] == key && sctr[old] == c) {
                    atomicMin(&table[h], p);
                    break;
                }
                h = (h + 1u) & mask; // the table has at least twice as many slots as packets
            }
        }
    }
    cls[p] = k;
}

// Did an earlier packet of p's run raise the run's maximum to exactly c (c > 0)?
// Such a packet carried c and reached the bit test.  The running maximum before
// each position does not fall along a run, so the first position whose value
// reaches c is found by doubling steps back from p and halving in between;
// position q's packet carried c iff the value before q + 1 is c.
__device__ __forceinline__ bool raised_to(const uint32_t *skeys, const uint64_t *pmax, uint32_t p, uint32_t key,
                                          uint64_t c)
{
    if (pmax[p] < c) return false;
    // invariant: below lo the value is under c or the run has not begun; at hi it is at least c
    uint32_t hi = p, lo = 0;
    for (uint32_t step = 1;; step <<= 1) {
        if (step > hi) break;
        const uint32_t q = hi - step;
        if (skeys[q] != key || pmax[q] < c) {
            lo = q + 1u;
            break;
        }
        hi = q;
        if (step >= 0x80000000u) break;
    }
    while (lo < hi) {
        const uint32_t mid = lo + (hi - lo) / 2u;
        if (skeys[mid] == key && pmax[mid] >= c) hi = mid;
        else lo = mid + 1u;
    }
    return pmax[hi] == c;
}

// Two things no packet of the other needs: a late packet is fresh when no
// earlier packet of the batch carried its counter -- neither a late one (the
// table holds the first of those) nor one that was ahead when it came (those
// raised the running maximum to their counter) -- and the last packet of each
// peer's run brings that peer's window to where `last` ends up (clearing the
// blocks it passed over; the class of every packet was settled against the
// windows as the batch found them by the launch before this one).
__global__ __launch_bounds__(256) void replay_late_advance_kernel(const uint32_t *skeys, const uint32_t *sidx,
                                                                  const uint64_t *sctr, const uint64_t *pmax,
                                                                  const uint8_t *cls, uint64_t *state, uint32_t n,
                                                                  const uint32_t *table, uint32_t mask,
                                                                  const uint32_t *flags, uint8_t *result,
                                                                  uint32_t *out_len)
{
    const uint32_t p = blockIdx.x * 256u + threadIdx.x;
    if (p >= n) return;
    const uint32_t key = skeys[p];
    if (key == NO_PEER) return;
    const uint64_t c = sctr[p];
    if (flags[0] != 0u && cls[p] == RP_LATE) {
        bool fresh = true;
        uint32_t h = table_home(key, c, mask);
        for (;;) {
            const uint32_t at = table[h];
            if (at == HASH_EMPTY) break; // cannot happen: it was entered
            if (skeys[at] == key && sctr[at] == c) {
                fresh = at == p;
                break;
            }
            h = (h + 1u) & mask;
        }
        // (counter 0 is never ahead of anything: every packet carrying it is in the table)
        if (fresh && c != 0u && raised_to(skeys, pmax, p, key, c)) fresh = false;
        if (!fresh) {
            const uint32_t i = sidx[p];
            result[i] = BNK_WG_REPLAY;
            out_len[i] = 0;
        }
    }
    if (p + 1u < n && skeys[p + 1u] == key) return;
    uint64_t last = pmax[p];
    if (c < WG_REJECT_AFTER_MESSAGES && c > last) last = c;
    advance_window(state + (size_t)key * WG_REPLAY_WORDS, last);
}

// Sets the bit of every packet that reached the bit test and still lies in the
// window its peer ends the batch with.  Neighbours in sorted order mostly
// share their peer and their block of 64 counters: a lane whose left neighbour
// differs gathers the bits of the lanes behind it that agree with it and
// issues one atomic for all of them.
//
// The same launch leaves the first-occurrence table empty for the next pass
// (nothing to do when this pass had no late packet, the usual case) and clears
// the flag word the next pass will use (nobody reads that one now).
__global__ __launch_bounds__(256) void replay_mark_kernel(const uint32_t *skeys, const uint64_t *sctr,
                                                          const uint8_t *cls, uint64_t *state, uint32_t n,
                                                          uint32_t *table, uint32_t slots, uint32_t *flags,
                                                          uint32_t parity)
{
    if (blockIdx.x == 0 && threadIdx.x == 0) flags[parity ^ 1u] = 0u;
    if (flags[parity] != 0u)
        for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < slots; i += gridDim.x * 256u) table[i] = HASH_EMPTY;
    const uint32_t p = blockIdx.x * 256u + threadIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t key = NO_PEER;
    uint64_t block = ~0ull, bit = 0;
    if (p < n && cls[p] != RP_NONE) {
        key = skeys[p];
        const uint64_t c = sctr[p];
        const uint64_t final_last = state[(size_t)key * WG_REPLAY_WORDS];
        if ((final_last >> 6) - (c >> 6) < WG_REPLAY_BLOCKS) { // else its slot now belongs to a later block
            block = c >> 6;
            bit = 1ull << (c & 63u);
        } else {
            key = NO_PEER;
        }
    }
    // runs of equal (peer, block) among neighbouring lanes
    const uint32_t pkey = (uint32_t)__shfl_up((int)key, 1, 64);
    const uint32_t pblo = (uint32_t)__shfl_up((int)(uint32_t)block, 1, 64);
    const uint32_t pbhi = (uint32_t)__shfl_up((int)(uint32_t)(block >> 32), 1, 64);
    const bool head = lane == 0 || pkey != key || pblo != (uint32_t)block || pbhi != (uint32_t)(block >> 32);
    const unsigned long long heads = __ballot(head);
    // my run ends before the next head after me
    const unsigned long long after = lane == 63u ? 0ull : heads & ~((2ull << lane) - 1ull);
    const uint32_t end = after ? (uint32_t)__ffsll((long long)after) - 1u : 64u;
    uint64_t acc = bit;
    // suffix OR within the run: six doubling steps cover 64 lanes
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t lo = (uint32_t)__shfl_down((int)(uint32_t)acc, off, 64);
        const uint32_t hi = (uint32_t)__shfl_down((int)(uint32_t)(acc >> 32), off, 64);
        if (lane + (uint32_t)off < end) acc |= (uint64_t)hi << 32 | lo;
    }
    if (head && key != NO_PEER && acc != 0)
        atomicOr(reinterpret_cast<unsigned long long *>(
                     &state[(size_t)key * WG_REPLAY_WORDS + 1u + (block & (WG_REPLAY_BLOCKS - 1u))]),
                 (unsigned long long)acc);
}

unsigned key_bits(uint32_t n_keys)
{
    unsigned bits = 1;
    while (bits < 32 && (n_keys >> bits) != 0) bits++;
    return bits;
}

using SortConfig = rocprim::radix_sort_config<rocprim::default_config, rocprim::default_config,
                                              rocprim::default_config, 32768>;

// ---- small batches: one block, everything in LDS ----------------------------

// Segmented running maximum: the value restarts where the key changes.
struct RunMax {
    uint32_t k;
    uint64_t v;
};
struct RunMaxOp {
    __device__ RunMax operator()(const RunMax &a, const RunMax &b) const
    {
        return RunMax{b.k, (a.k == b.k && a.v > b.v) ? a.v : b.v};
    }
};

// (SMALL threads: 256 for the batches wireguard-go itself hands over, 1024 up to
// the limit of the one-block form)
template <uint32_t SMALL>
__global__ __launch_bounds__(SMALL) void replay_small_kernel(uint8_t *result, uint32_t *out_len,
                                                             const uint32_t *peer, const uint64_t *counter,
                                                             uint32_t n_peers, uint32_t n, uint64_t *state,
                                                             unsigned bits)
{
    using Sort = rocprim::block_radix_sort<uint32_t, SMALL, 1, uint32_t>;
    using Scan = rocprim::block_scan<uint32_t, SMALL>;
    using ScanMax = rocprim::block_scan<RunMax, SMALL>;
    __shared__ union {
        typename Sort::storage_type sort;
        typename Scan::storage_type scan;
        typename ScanMax::storage_type scan_max;
    } tmp;
    __shared__ uint32_t sk[SMALL + 1];
    __shared__ uint64_t sc[SMALL];
    __shared__ uint64_t smax[SMALL];
    const uint32_t t = threadIdx.x;
    uint32_t key[1] = {NO_PEER}, pos[1] = {t};
    if (t < n) {
        const uint32_t p = peer[t];
        if (replay_subject(result[t]) && p < n_peers) key[0] = p;
    }
    // stable: a peer's packets stay in batch order
    Sort().sort(key, pos, tmp.sort, 0, bits);
    const bool valid = key[0] != NO_PEER;
    const uint64_t c = valid ? counter[pos[0]] : 0;
    sk[t] = key[0];
    sc[t] = c;
    if (t == 0) sk[SMALL] = NO_PEER;
    __syncthreads();
    const bool head = t == 0 || sk[t - 1] != key[0];
    uint32_t start = 0;
    Scan().inclusive_scan(head ? t : 0u, start, tmp.scan, rocprim::maximum<uint32_t>());
    __syncthreads();
    // running maximum of the counters within each peer's run
    RunMax mine{key[0], c < WG_REJECT_AFTER_MESSAGES ? c : 0}, upto;
    ScanMax().inclusive_scan(mine, upto, tmp.scan_max, RunMaxOp());
    smax[t] = upto.v;
    __syncthreads();
    uint64_t *st = valid ? state + (size_t)key[0] * WG_REPLAY_WORDS : nullptr;
    const uint64_t last0 = valid ? st[0] : 0;
    uint64_t last = last0;
    if (valid && !head && smax[t - 1] > last) last = smax[t - 1];
    // only a packet at or below an earlier counter can repeat one: it looks
    // through the packets of its peer ahead of it
    bool dup = false;
    if (valid && c <= last)
        for (uint32_t u = start; u < t; u++) dup |= sc[u] == c;
    const bool reached = valid && reaches_bit_test(c, last);
    bool fresh = reached && !dup;
    if (fresh && c <= last0 && seen_before(st, c)) fresh = false;
    if (valid && !fresh) {
        result[pos[0]] = BNK_WG_REPLAY;
        out_len[pos[0]] = 0;
    }
    __syncthreads(); // every window has been read as the batch found it
    const bool tail = valid && sk[t + 1] != key[0];
    if (tail) {
        uint64_t nl = last;
        if (c < WG_REJECT_AFTER_MESSAGES && c > nl) nl = c;
        advance_window(st, nl);
    }
    // (one workgroup does all of this: waiting for its stores to be acknowledged is
    // enough; a device-wide fence would write the whole L2 back)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads(); // the cleared blocks are in place before bits go in
    if (reached) {
        const uint64_t final_last = *reinterpret_cast<volatile uint64_t *>(st);
        if ((final_last >> 6) - (c >> 6) < WG_REPLAY_BLOCKS)
            atomicOr(reinterpret_cast<unsigned long long *>(&st[1u + ((c >> 6) & (WG_REPLAY_BLOCKS - 1u))]),
                     1ull << (c & 63u));
    }
}

__global__ __launch_bounds__(256) void replay_reset_kernel(uint64_t *state, const uint8_t *flags, uint32_t n_peers)
{
    const uint32_t total = n_peers * WG_REPLAY_WORDS;
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t w = blockIdx.x * 256u + threadIdx.x; w < total; w += stride)
        if (flags[w / WG_REPLAY_WORDS]) state[w] = 0;
}

} // namespace

hipError_t launch_wg_replay_reset(uint64_t *state, const uint8_t *flags, uint32_t n_peers, hipStream_t s)
{
    if (n_peers == 0) return hipSuccess;
    const uint32_t blocks = std::min<uint32_t>((n_peers * WG_REPLAY_WORDS + 255u) / 256u, 2048u);
    hipLaunchKernelGGL(replay_reset_kernel, dim3(blocks), dim3(256), 0, s, state, flags, n_peers);
    return hipGetLastError();
}

unsigned wg_replay_index_bits(uint32_t n, uint32_t n_peers)
{
    unsigned bits = 1;
    while (bits < 32 && ((uint64_t)1 << bits) < n) bits++;
    return bits + key_bits(n_peers) <= 32 ? bits : 0;
}

size_t wg_replay_tmp_bytes(uint32_t n, uint32_t n_peers)
{
    size_t a = 0, b = 0, c = 0;
    (void)rocprim::radix_sort_keys<SortConfig>(nullptr, c, (const uint32_t *)nullptr, (uint32_t *)nullptr, (size_t)n,
                                               0, 32);
    (void)rocprim::radix_sort_pairs<SortConfig>(nullptr, a, (const uint32_t *)nullptr, (uint32_t *)nullptr,
                                                (const uint32_t *)nullptr, (uint32_t *)nullptr, (size_t)n, 0,
                                                key_bits(n_peers));
    b = ((size_t)(n + SEG_BLOCK - 1u) / SEG_BLOCK) * 12u + 16u; // the scan's block carries
    return std::max(std::max(a, b), c);
}

uint32_t wg_replay_table_slots(uint32_t n)
{
    uint32_t s = 1024;
    while (s < 2u * n && s < (1u << 31)) s <<= 1;
    return s;
}

hipError_t launch_wg_replay(uint8_t *result, uint32_t *out_len, const uint32_t *peer, const uint64_t *counter,
                            uint32_t n, const WgReplayDev &rp, const WgReplayScratch &sc, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    if (n <= 256u) {
        hipLaunchKernelGGL(replay_small_kernel<256>, dim3(1), dim3(256), 0, s, result, out_len, peer, counter,
                           rp.n_peers, n, rp.state, key_bits(rp.n_peers));
        return hipGetLastError();
    }
    if (n <= WG_REPLAY_SMALL_MAX) {
        hipLaunchKernelGGL(replay_small_kernel<WG_REPLAY_SMALL_MAX>, dim3(1), dim3(WG_REPLAY_SMALL_MAX), 0, s,
                           result, out_len, peer, counter, rp.n_peers, n, rp.state, key_bits(rp.n_peers));
        return hipGetLastError();
    }
    const dim3 grid((n + 255u) / 256u);
    size_t bytes = sc.tmp_bytes;
    hipError_t e = hipSuccess;
    const unsigned peer_bits = key_bits(rp.n_peers);
    // (what the blocks hand on to the running maximum goes into the sort's scratch, free by then)
    const uint32_t seg_blocks = (n + SEG_BLOCK - 1u) / SEG_BLOCK;
    uint64_t *carry_x = static_cast<uint64_t *>(sc.tmp);
    uint32_t *carry_open = reinterpret_cast<uint32_t *>(carry_x + seg_blocks);
    if (const unsigned index_bits = wg_replay_index_bits(n, rp.n_peers)) {
        // one word per packet: keys[] in, idx[] out
        if (!sc.keys_ready)
            hipLaunchKernelGGL(replay_keys_packed_kernel, grid, dim3(256), 0, s, result, peer, rp.n_peers, n,
                               index_bits, sc.keys);
        e = rocprim::radix_sort_keys<SortConfig>(sc.tmp, bytes, sc.keys, sc.idx, (size_t)n, index_bits,
                                                 index_bits + peer_bits, s);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(replay_unpack_kernel, dim3(seg_blocks), dim3(SEG_BLOCK), 0, s, sc.idx, counter, n,
                           index_bits, peer_bits, sc.skeys, sc.sidx, sc.sctr, sc.sval, carry_x, carry_open);
    } else {
        if (!sc.keys_ready)
            hipLaunchKernelGGL(replay_keys_kernel, grid, dim3(256), 0, s, result, peer, rp.n_peers, n, sc.keys,
                               sc.idx);
        e = rocprim::radix_sort_pairs<SortConfig>(sc.tmp, bytes, sc.keys, sc.skeys, sc.idx, sc.sidx, (size_t)n, 0,
                                                  peer_bits, s);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(replay_gather_kernel, dim3(seg_blocks), dim3(SEG_BLOCK), 0, s, sc.skeys, sc.sidx, counter,
                           n, sc.sctr, sc.sval, carry_x, carry_open);
    }
    // the running maximum per peer is finished inside the classifying launch
    const uint32_t mask = sc.table_slots - 1u;
    uint32_t *late_flag = sc.flags + sc.parity;
    hipLaunchKernelGGL(replay_classify_kernel, dim3(seg_blocks), dim3(SEG_BLOCK), 0, s, sc.skeys, sc.sidx, sc.sctr,
                       sc.sval, carry_x, carry_open, sc.pmax, rp.state, n, sc.cls, sc.table, mask, late_flag, result,
                       out_len);
    hipLaunchKernelGGL(replay_late_advance_kernel, grid, dim3(256), 0, s, sc.skeys, sc.sidx, sc.sctr, sc.pmax, sc.cls,
                       rp.state, n, sc.table, mask, late_flag, result, out_len);
    hipLaunchKernelGGL(replay_mark_kernel, grid, dim3(256), 0, s, sc.skeys, sc.sctr, sc.cls, rp.state, n, sc.table,
                       sc.table_slots, sc.flags, sc.parity);
    return hipGetLastError();
}

} // namespace bnk
