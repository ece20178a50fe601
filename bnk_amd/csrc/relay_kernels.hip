// Bookkeeping of the fused relay step open -> filter -> re-seal: verdicts and
// the outbound nonce counters.  A packet that survives takes the next counter
// of its outbound peer in batch order; dropped packets consume none (as in
// wireguard-go, where the nonce is assigned when a packet is queued for
// sending).  That is a segmented exclusive count over the survivors keyed by
// peer: a stable radix sort of (peer, index) pairs puts each peer's survivors
// together in batch order, and a survivor's rank is its distance from the
// first element of its segment.
#include <string.h>

#include <algorithm>

#include <rocprim/rocprim.hpp>

#include "../../include/bnkhip.h"
#include "kernels.hpp"

namespace bnk {

constexpr uint32_t NO_PEER = 0xFFFFFFFFu;

__global__ __launch_bounds__(256) void relay_verdict_kernel(
    const uint8_t *auth, const uint8_t *pass, const uint32_t *peer_out, uint32_t n_peers_out,
    uint32_t n, uint32_t *keys, uint32_t *idx, uint8_t *verdict, uint64_t *ctr_out, uint32_t *status)
{
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n) return;
    uint8_t v = !auth[i] ? BNK_RELAY_FORGED : !pass[i] ? BNK_RELAY_DENIED : BNK_RELAY_OK;
    uint32_t key = NO_PEER;
    if (v == BNK_RELAY_OK) {
        key = peer_out[i];
        if (key >= n_peers_out) {
            status_raise(status, STATUS_PEER_RANGE);
            v = BNK_RELAY_DENIED;
            key = NO_PEER;
        }
    }
    verdict[i] = v;
    keys[i] = key;
    // (the counting kernels need no positions and write every packet's counter themselves)
    if (idx) {
        idx[i] = i;
        ctr_out[i] = 0;
    }
}

// Where each peer's run starts in the sorted sequence.
__global__ __launch_bounds__(256) void peer_heads_kernel(const uint32_t *skeys, uint32_t n,
                                                         uint32_t *seg_start)
{
    const uint32_t p = blockIdx.x * 256u + threadIdx.x;
    if (p >= n) return;
    const uint32_t key = skeys[p];
    if (key == NO_PEER) return;
    if (p == 0u || skeys[p - 1u] != key) seg_start[key] = p;
}

__global__ __launch_bounds__(256) void relay_rank_kernel(const uint32_t *skeys, const uint32_t *sidx,
                                                         const uint32_t *seg_start,
                                                         const uint64_t *ctr_base_out, uint32_t n,
                                                         uint64_t *ctr_out, uint64_t ctr_limit)
{
    const uint32_t p = blockIdx.x * 256u + threadIdx.x;
    if (p >= n) return;
    const uint32_t key = skeys[p];
    if (key == NO_PEER) return;
    ctr_out[sidx[p]] = ctr_add(ctr_base_out[key], (uint64_t)(p - seg_start[key]), ctr_limit);
}

// The last element of each peer's segment holds the largest counter handed out.
__global__ __launch_bounds__(256) void peer_advance_kernel(const uint32_t *skeys, const uint32_t *sidx,
                                                           const uint64_t *ctr_out, uint32_t n,
                                                           uint64_t *ctr_base, uint64_t ctr_limit)
{
    const uint32_t p = blockIdx.x * 256u + threadIdx.x;
    if (p >= n) return;
    const uint32_t key = skeys[p];
    if (key == NO_PEER) return;
    if (p + 1u < n && skeys[p + 1u] == key) return;
    ctr_base[key] = ctr_add(ctr_out[sidx[p]], 1u, ctr_limit);
}

// Peer keys are below n_keys and the "no peer" key is all ones, so the low
// bit_width(n_keys) bits order them the same way the full word does.
static unsigned key_bits(uint32_t n_keys)
{
    unsigned bits = 1;
    while (bits < 32 && (n_keys >> bits) != 0) bits++;
    return bits;
}

// A few key bits sort faster in one or two Onesweep passes than in the merge
// sort rocPRIM picks by default for up to 2^20 items.
using SortConfig = rocprim::radix_sort_config<rocprim::default_config, rocprim::default_config,
                                              rocprim::default_config, 32768>;

constexpr uint32_t RANK_TABLE_MAX_KEYS = 4096;
constexpr uint32_t RANK_ROW_STEP = 256; // 64 lanes x 16 bytes
constexpr uint32_t RANK_ROW_STEPS = RANK_TABLE_MAX_KEYS / RANK_ROW_STEP;
constexpr uint32_t TILE_RUNS_MAX = 32;
constexpr size_t RANK_TABLE_MAX_BYTES = 64u << 20;

struct RankPlan {
    uint32_t runs;  // runs of 64 packets per tile
    uint32_t tiles;
    uint32_t cols;  // entries per row of the table: the keys, rounded up to what a wave moves at once
    size_t bytes;   // the table, then one total per peer, then every peer's counter as the batch found it
    bool fits;
};

static RankPlan rank_plan(uint32_t n, uint32_t n_keys)
{
    RankPlan p{};
    // about 2048 tiles (a wave each: enough to keep every CU busy), as long as a wave
    // can hold its tile's keys in registers
    p.runs = std::min<uint32_t>(TILE_RUNS_MAX, std::max<uint32_t>(1u, (n + 64u * 2048u - 1u) / (64u * 2048u)));
    p.tiles = (n + 64u * p.runs - 1u) / (64u * p.runs);
    p.cols = (n_keys + RANK_ROW_STEP - 1u) / RANK_ROW_STEP * RANK_ROW_STEP;
    p.bytes = ((size_t)p.tiles + 1u) * p.cols * 4u + (size_t)p.cols * 8u;
    p.fits = n_keys <= RANK_TABLE_MAX_KEYS && p.bytes <= RANK_TABLE_MAX_BYTES;
    return p;
}

size_t relay_sort_tmp_bytes(uint32_t n, uint32_t n_keys)
{
    size_t bytes = 0;
    (void)rocprim::radix_sort_pairs<SortConfig>(nullptr, bytes, (const uint32_t *)nullptr, (uint32_t *)nullptr,
                                    (const uint32_t *)nullptr, (uint32_t *)nullptr, (size_t)n, 0,
                                    key_bits(n_keys));
    // once the sort is done the same scratch holds one run start per key
    bytes = std::max(bytes, (size_t)n_keys * 4);
    // the sort-free form's table, for this batch or any part of it (a part is cut
    // into up to 2048 tiles however small it is)
    const RankPlan plan = rank_plan(n, n_keys);
    if (!plan.fits) return bytes;
    const size_t rows = std::max<size_t>(plan.tiles, std::min<size_t>(n / 64u + 1u, 2048u)) + 1u;
    return std::max(bytes, rows * plan.cols * 4u + (size_t)plan.cols * 8u);
}

__global__ void peer_rank_small_kernel(const uint32_t *peer, uint32_t n_keys, uint32_t n, uint64_t *ctr_base,
                                       uint64_t *ctr_out, int advance, int no_peer_ok, unsigned bits,
                                       uint64_t ctr_limit, uint32_t *status);

static hipError_t launch_peer_rank_table(const uint32_t *keys, const RankPlan &plan, void *tmp,
                                         uint64_t *ctr_base, uint32_t n_keys, uint32_t n, uint64_t *ctr_out,
                                         bool advance, uint64_t ctr_limit, bool zero_others, uint32_t *status,
                                         hipStream_t s);

hipError_t launch_relay_assign(const uint8_t *auth, const uint8_t *pass, const uint32_t *peer_out,
                               const uint64_t *ctr_base_out, uint32_t n_peers_out, uint32_t n,
                               uint32_t *keys, uint32_t *idx, uint32_t *skeys, uint32_t *sidx,
                               void *sort_tmp, size_t sort_tmp_bytes, uint8_t *verdict,
                               uint64_t *ctr_out, uint32_t *status, bool advance, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    const dim3 grid((n + 255u) / 256u);
    const RankPlan plan = rank_plan(n, n_peers_out);
    const bool counting = n > PEER_RANK_SMALL_MAX && plan.fits && plan.bytes <= sort_tmp_bytes;
    hipLaunchKernelGGL(relay_verdict_kernel, grid, dim3(256), 0, s, auth, pass, peer_out, n_peers_out,
                       n, keys, counting ? (uint32_t *)nullptr : idx, verdict, ctr_out, status);
    if (n <= PEER_RANK_SMALL_MAX) {
        // keys[] is the peer of each survivor and all ones for the rest
        hipLaunchKernelGGL(peer_rank_small_kernel, dim3(1), dim3(PEER_RANK_SMALL_MAX), 0, s, keys, n_peers_out,
                           n, const_cast<uint64_t *>(ctr_base_out), ctr_out, advance ? 1 : 0, 1,
                           key_bits(n_peers_out), 0ull, status);
        return hipGetLastError();
    }
    if (counting)
        return launch_peer_rank_table(keys, plan, sort_tmp, const_cast<uint64_t *>(ctr_base_out), n_peers_out, n,
                                      ctr_out, advance, 0ull, true, nullptr, s);
    return launch_peer_rank(keys, idx, skeys, sidx, sort_tmp, sort_tmp_bytes,
                            const_cast<uint64_t *>(ctr_base_out), n_peers_out, n, ctr_out, advance, 0ull, s);
}

// Batch-order counters for a small batch in one launch of one block, straight
// from the peer array: a stable block-wide radix sort of (peer, position)
// brings each peer's packets together in batch order; a packet's rank is its
// distance from the head of its run, and the last packet of a run moves the
// peer's base.
__global__ __launch_bounds__(PEER_RANK_SMALL_MAX) void peer_rank_small_kernel(
    const uint32_t *peer, uint32_t n_keys, uint32_t n, uint64_t *ctr_base, uint64_t *ctr_out,
    int advance, int no_peer_ok, unsigned bits, uint64_t ctr_limit, uint32_t *status)
{
    using Sort = rocprim::block_radix_sort<uint32_t, PEER_RANK_SMALL_MAX, 1, uint32_t>;
    using Scan = rocprim::block_scan<uint32_t, PEER_RANK_SMALL_MAX>;
    __shared__ union {
        typename Sort::storage_type sort;
        typename Scan::storage_type scan;
    } tmp;
    __shared__ uint32_t sk[PEER_RANK_SMALL_MAX + 1];
    const uint32_t t = threadIdx.x;
    uint32_t key[1] = {NO_PEER}, pos[1] = {t};
    if (t < n) {
        key[0] = peer ? peer[t] : 0u;
        if (key[0] >= n_keys) {
            if (!(no_peer_ok && key[0] == NO_PEER)) status_raise(status, STATUS_PEER_RANGE);
            key[0] = NO_PEER;
        }
    }
    // valid keys are below n_keys < 2^bits and "no peer" is all ones, so the low
    // bits order them the way the full word does, "no peer" last
    Sort().sort(key, pos, tmp.sort, 0, bits);
    sk[t] = key[0];
    if (t == 0) sk[PEER_RANK_SMALL_MAX] = NO_PEER;
    __syncthreads();
    const bool valid = key[0] != NO_PEER;
    const bool head = t == 0 || sk[t - 1] != key[0];
    const bool last = sk[t + 1] != key[0];
    uint32_t start = 0;
    Scan().inclusive_scan(head ? t : 0u, start, tmp.scan, rocprim::maximum<uint32_t>());
    uint64_t mine = 0;
    if (valid) {
        mine = ctr_add(ctr_base[key[0]], t - start, ctr_limit);
        ctr_out[pos[0]] = mine;
    }
    __syncthreads(); // every base has been read
    if (advance && valid && last) ctr_base[key[0]] = ctr_add(mine, 1u, ctr_limit);
}

hipError_t launch_peer_rank_small(const uint32_t *peer, uint32_t n_keys, uint32_t n, uint64_t *ctr_base,
                                  uint64_t *ctr_out, bool advance, uint64_t ctr_limit, uint32_t *status,
                                  hipStream_t s)
{
    if (n == 0) return hipSuccess;
    if (n > PEER_RANK_SMALL_MAX) return hipErrorInvalidValue;
    hipLaunchKernelGGL(peer_rank_small_kernel, dim3(1), dim3(PEER_RANK_SMALL_MAX), 0, s, peer, n_keys, n,
                       ctr_base, ctr_out, advance ? 1 : 0, 0, key_bits(n_keys), ctr_limit, status);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// The same counters without a sort, for peer tables of at most
// RANK_TABLE_MAX_KEYS rows.  The batch is cut into tiles of TILE_RUNS runs of
// 64 packets, one wave per tile.  rank_count_kernel counts each tile's packets
// per peer into a row of a table; rank_scan_kernel turns every column (a
// peer's counts, tile after tile) into exclusive prefixes and keeps the
// totals; rank_assign_kernel loads its tile's row into LDS and walks the tile
// run by run in batch order: a packet's rank is its peer's entry plus the
// number of lower lanes of the run with the same peer, and one lane per peer
// then moves the entry past the run.  The scan also moves the peers' counters
// past the batch, leaving the values it found for the assigning launch.
// Three launches over the keys, against eight (two of them passes over
// key-index pairs) for the sort.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(64) void rank_count_kernel(const uint32_t *keys, uint32_t n, uint32_t n_keys,
                                                        uint32_t cols, uint32_t runs, uint32_t *table,
                                                        uint32_t *status)
{
    __shared__ __attribute__((aligned(16))) uint32_t cnt[RANK_TABLE_MAX_KEYS];
    const uint32_t lane = threadIdx.x;
    uint4 *cnt4 = reinterpret_cast<uint4 *>(cnt);
    for (uint32_t q = lane; q < cols / 4u; q += 64u) cnt4[q] = make_uint4(0, 0, 0, 0);
    const uint32_t first = blockIdx.x * runs * 64u;
    uint32_t key[TILE_RUNS_MAX];
    // all of the tile's keys are on their way before the first one is counted
#pragma unroll
    for (uint32_t r = 0; r < TILE_RUNS_MAX; r++) {
        const uint32_t i = first + r * 64u + lane;
        key[r] = r < runs && i < n ? keys[i] : NO_PEER;
    }
    __syncthreads();
#pragma unroll
    for (uint32_t r = 0; r < TILE_RUNS_MAX; r++) {
        if (key[r] < n_keys) atomicAdd(&cnt[key[r]], 1u);
        // (keys straight from a caller's peer array: one beyond the table gets no counter and is reported)
        else if (status && r < runs && first + r * 64u + lane < n) status_raise(status, STATUS_PEER_RANGE);
    }
    __syncthreads();
    uint4 *row = reinterpret_cast<uint4 *>(table + (size_t)blockIdx.x * cols);
    for (uint32_t q = lane; q < cols / 4u; q += 64u) row[q] = cnt4[q];
}

// One block per 16 peers: 64 groups of threads share the tiles between them.
constexpr uint32_t SCAN_PEERS = 16, SCAN_PARTS = 64;
constexpr uint32_t SCAN_KEEP = 32; // tiles of a part held in registers between the two passes
__global__ __launch_bounds__(SCAN_PEERS * SCAN_PARTS) void rank_scan_kernel(uint32_t *table, uint32_t tiles,
                                                                             uint32_t n_keys, uint32_t cols,
                                                                             uint32_t *total, uint64_t *ctr_base,
                                                                             uint64_t *base_was, int advance,
                                                                             uint64_t ctr_limit)
{
    __shared__ uint32_t part_sum[SCAN_PARTS][SCAN_PEERS];
    const uint32_t x = threadIdx.x % SCAN_PEERS, y = threadIdx.x / SCAN_PEERS;
    const uint32_t key = blockIdx.x * SCAN_PEERS + x;
    const uint32_t per = (tiles + SCAN_PARTS - 1u) / SCAN_PARTS;
    const uint32_t lo = min(y * per, tiles), hi = min(lo + per, tiles);
    const bool mine = key < n_keys;
    const bool keep = per <= SCAN_KEEP; // (the same for every thread)
    uint32_t c[SCAN_KEEP];
    uint32_t sum = 0;
    if (keep) {
        // every load of the part in flight at once
#pragma unroll
        for (uint32_t j = 0; j < SCAN_KEEP; j++) c[j] = mine && lo + j < hi ? table[(size_t)(lo + j) * cols + key] : 0u;
#pragma unroll
        for (uint32_t j = 0; j < SCAN_KEEP; j++) sum += c[j];
    } else if (mine) {
#pragma unroll 8
        for (uint32_t t = lo; t < hi; t++) sum += table[(size_t)t * cols + key];
    }
    part_sum[y][x] = sum;
    __syncthreads();
    uint32_t run = 0;
    for (uint32_t q = 0; q < y; q++) run += part_sum[q][x];
    if (!mine) return;
    if (keep) {
#pragma unroll
        for (uint32_t j = 0; j < SCAN_KEEP; j++) {
            if (lo + j < hi) table[(size_t)(lo + j) * cols + key] = run;
            run += c[j];
        }
    } else {
        for (uint32_t t = lo; t < hi; t++) {
            uint32_t *e = table + (size_t)t * cols + key;
            const uint32_t v = *e;
            *e = run;
            run += v;
        }
    }
    if (y == SCAN_PARTS - 1u) {
        // the peer's counter as the batch found it stays behind for the assigning launch;
        // the counter itself moves past what the batch takes
        total[key] = run;
        const uint64_t was = ctr_base[key];
        base_was[key] = was;
        if (advance && run != 0u) ctr_base[key] = ctr_add(was, run, ctr_limit);
    }
}

__global__ __launch_bounds__(64) void rank_assign_kernel(const uint32_t *keys, uint32_t n, uint32_t n_keys,
                                                         uint32_t cols, uint32_t runs, const uint32_t *table,
                                                         unsigned bits,
                                                         const uint64_t *ctr_base, uint64_t *ctr_out,
                                                         uint64_t ctr_limit, int zero_others)
{
    // packets of each peer ahead of the run at hand
    __shared__ __attribute__((aligned(16))) uint32_t before[RANK_TABLE_MAX_KEYS];
    const uint32_t lane = threadIdx.x;
    {
        // the tile's row, every load in flight before the first is used
        const uint4 *row = reinterpret_cast<const uint4 *>(table + (size_t)blockIdx.x * cols);
        uint4 v[RANK_ROW_STEPS];
#pragma unroll
        for (uint32_t q = 0; q < RANK_ROW_STEPS; q++)
            v[q] = q * RANK_ROW_STEP < cols ? row[q * 64u + lane] : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (uint32_t q = 0; q < RANK_ROW_STEPS; q++)
            if (q * RANK_ROW_STEP < cols) reinterpret_cast<uint4 *>(before)[q * 64u + lane] = v[q];
    }
    const uint32_t first = blockIdx.x * runs * 64u;
    uint32_t key[TILE_RUNS_MAX];
    uint64_t base[TILE_RUNS_MAX];
    // keys and the peers' bases are fetched up front: nothing inside the walk
    // below waits for memory
#pragma unroll
    for (uint32_t r = 0; r < TILE_RUNS_MAX; r++) {
        const uint32_t i = first + r * 64u + lane;
        key[r] = r < runs && i < n ? keys[i] : NO_PEER;
    }
#pragma unroll
    for (uint32_t r = 0; r < TILE_RUNS_MAX; r++) base[r] = key[r] < n_keys ? ctr_base[key[r]] : 0ull;
    __syncthreads();
#pragma unroll
    for (uint32_t r = 0; r < TILE_RUNS_MAX; r++) {
        if (r < runs) { // uniform
        const uint32_t kk = key[r];
        const bool valid = kk < n_keys;
        // the lanes of this run with my peer
        unsigned long long same = __ballot(valid);
        for (unsigned b = 0; b < bits; b++) {
            const unsigned long long m = __ballot((kk >> b) & 1u);
            same &= ((kk >> b) & 1u) ? m : ~m;
        }
        if (valid) {
            const uint32_t lower = (uint32_t)__popcll(same & ((1ull << lane) - 1ull));
            const uint32_t rank = before[kk] + lower;
            ctr_out[first + r * 64u + lane] = ctr_add(base[r], rank, ctr_limit);
            // every lane has read the entry before any lane writes one: the lanes of a
            // wave run in lockstep and LDS serves their accesses in order
            if (lower == 0u) before[kk] += (uint32_t)__popcll(same);
        } else if (zero_others && first + r * 64u + lane < n) {
            ctr_out[first + r * 64u + lane] = 0; // a packet without a peer gets no counter
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        }
    }
}

static hipError_t launch_peer_rank_table(const uint32_t *keys, const RankPlan &plan, void *tmp,
                                         uint64_t *ctr_base, uint32_t n_keys, uint32_t n, uint64_t *ctr_out,
                                         bool advance, uint64_t ctr_limit, bool zero_others, uint32_t *status,
                                         hipStream_t s)
{
    uint32_t *table = static_cast<uint32_t *>(tmp);
    uint32_t *total = table + (size_t)plan.tiles * plan.cols;
    uint64_t *base_was = reinterpret_cast<uint64_t *>(total + plan.cols);
    hipLaunchKernelGGL(rank_count_kernel, dim3(plan.tiles), dim3(64), 0, s, keys, n, n_keys, plan.cols, plan.runs,
                       table, status);
    hipLaunchKernelGGL(rank_scan_kernel, dim3((n_keys + SCAN_PEERS - 1u) / SCAN_PEERS),
                       dim3(SCAN_PEERS * SCAN_PARTS), 0, s, table, plan.tiles, n_keys, plan.cols, total, ctr_base,
                       base_was, advance ? 1 : 0, ctr_limit);
    hipLaunchKernelGGL(rank_assign_kernel, dim3(plan.tiles), dim3(64), 0, s, keys, n, n_keys, plan.cols, plan.runs,
                       table, key_bits(n_keys), base_was, ctr_out, ctr_limit, zero_others ? 1 : 0);
    return hipGetLastError();
}

bool peer_rank_counts(uint32_t n, uint32_t n_keys, size_t tmp_bytes)
{
    const RankPlan plan = rank_plan(n, n_keys);
    return n > PEER_RANK_SMALL_MAX && plan.fits && plan.bytes <= tmp_bytes;
}

hipError_t launch_peer_rank_counting(const uint32_t *peer, void *tmp, uint64_t *ctr_base, uint32_t n_keys, uint32_t n,
                                     uint64_t *ctr_out, bool advance, uint64_t ctr_limit, uint32_t *status,
                                     hipStream_t s)
{
    if (n == 0) return hipSuccess;
    // (a packet whose peer lies beyond the table gets counter 0, as one without a peer does)
    return launch_peer_rank_table(peer, rank_plan(n, n_keys), tmp, ctr_base, n_keys, n, ctr_out, advance, ctr_limit,
                                  true, status, s);
}

hipError_t launch_peer_rank(uint32_t *keys, uint32_t *idx, uint32_t *skeys, uint32_t *sidx,
                            void *sort_tmp, size_t sort_tmp_bytes, uint64_t *ctr_base, uint32_t n_keys,
                            uint32_t n, uint64_t *ctr_out, bool advance, uint64_t ctr_limit, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    const RankPlan plan = rank_plan(n, n_keys);
    if (plan.fits && plan.bytes <= sort_tmp_bytes)
        return launch_peer_rank_table(keys, plan, sort_tmp, ctr_base, n_keys, n, ctr_out, advance, ctr_limit, false,
                                      nullptr, s);
    const dim3 grid((n + 255u) / 256u);
    hipError_t e = rocprim::radix_sort_pairs<SortConfig>(sort_tmp, sort_tmp_bytes, keys, skeys, idx, sidx, (size_t)n,
                                             0, key_bits(n_keys), s);
    if (e != hipSuccess) return e;
    uint32_t *seg_start = static_cast<uint32_t *>(sort_tmp);
    hipLaunchKernelGGL(peer_heads_kernel, grid, dim3(256), 0, s, skeys, n, seg_start);
    hipLaunchKernelGGL(relay_rank_kernel, grid, dim3(256), 0, s, skeys, sidx, seg_start, ctr_base, n, ctr_out,
                       ctr_limit);
    if (advance)
        hipLaunchKernelGGL(peer_advance_kernel, grid, dim3(256), 0, s, skeys, sidx, ctr_out, n, ctr_base,
                           ctr_limit);
    return hipGetLastError();
}

} // namespace bnk
