// C ABI entry points of the WireGuard transport framing (see
// include/bnkhip.h): peer table, encapsulation, decapsulation.
#include <vector>

#include "api_common.hpp"
#include "filter_host.hpp"
#include "wg_dev.hpp"

using namespace bnk;

namespace {

WgPeersDev peers_view(bnk_ctx *ctx)
{
    WgPeersDev pe{};
    pe.index_sorted = ctx->wg_index.as<uint2>();
    pe.index_hash = ctx->wg_hash.as<uint2>();
    pe.hash_bits = ctx->wg_hash_bits;
    pe.remote_index = ctx->wg_remote.as<uint32_t>();
    pe.allowed = ctx->wg_allowed.as<uint2>();
    pe.send_ctr = ctx->wg_send_ctr.as<uint64_t>();
    pe.n = ctx->n_wg_peers;
    return pe;
}

int upload(bnk_ctx *ctx, DevBuf *dst, const void *src, size_t bytes)
{
    HIPCHK(ctx, dst->reserve(bytes));
    HIPCHK(ctx, hipMemcpyAsync(dst->p, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    return BNK_OK;
}

} // namespace

// The anti-replay windows follow the peer table: n rows, those flagged in
// `fresh` (n bytes, host) start empty, the others keep what they hold.
static int wg_replay_rows(bnk_ctx *ctx, uint32_t n, const std::vector<uint8_t> &fresh)
{
    if (n > ctx->wg_replay_rows) {
        uint64_t *grown = nullptr;
        const size_t row = (size_t)WG_REPLAY_WORDS * 8;
        HIPCHK(ctx, hipMalloc((void **)&grown, (size_t)n * row));
        hipError_t e = hipMemsetAsync(grown, 0, (size_t)n * row, ctx->stream);
        if (e == hipSuccess && ctx->wg_replay_rows)
            e = hipMemcpyAsync(grown, ctx->wg_replay, (size_t)ctx->wg_replay_rows * row, hipMemcpyDeviceToDevice,
                               ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) {
            (void)hipFree(grown);
            return fail_hip(ctx, "replay windows", e);
        }
        if (ctx->wg_replay) (void)hipFree(ctx->wg_replay);
        ctx->wg_replay = grown;
        ctx->wg_replay_rows = n;
    }
    int rc = upload(ctx, &ctx->wg_rflags, fresh.data(), n);
    if (rc) return rc;
    HIPCHK(ctx, launch_wg_replay_reset(ctx->wg_replay, ctx->wg_rflags.as<uint8_t>(), n, ctx->stream));
    return BNK_OK;
}

// Checks the rows and builds the sorted (local index, row) table.
static int wg_build_index(bnk_ctx *ctx, const bnk_wg_peer *peers, uint32_t n, std::vector<uint2> *index)
{
    index->resize(n);
    for (uint32_t i = 0; i < n; i++) {
        const uint32_t inv = ~peers[i].allowed_mask;
        if ((inv & (inv + 1u)) != 0u)
            return fail(ctx, BNK_E_INVAL, "peer " + std::to_string(i) + ": allowed_mask is not a prefix mask");
        (*index)[i] = make_uint2(peers[i].local_index, i);
    }
    std::sort(index->begin(), index->end(), [](const uint2 &a, const uint2 &b) { return a.x < b.x; });
    for (uint32_t i = 1; i < n; i++)
        if ((*index)[i].x == (*index)[i - 1].x)
            return fail(ctx, BNK_E_INVAL, "local_index " + std::to_string((*index)[i].x) + " is used by two peers");
    return BNK_OK;
}

// The same map as an open-addressing hash table (see wg_hash_slot): at least
// four slots per peer, so a lookup is one probe nine times in ten.
static void wg_build_hash(const std::vector<uint2> &index, std::vector<uint2> *table, uint32_t *bits)
{
    uint32_t b = 6;
    while (b < 31 && (1ull << b) < 4ull * index.size()) b++;
    table->assign((size_t)1 << b, make_uint2(0, WG_HASH_EMPTY));
    const uint32_t mask = (1u << b) - 1u;
    for (const uint2 &e : index) {
        uint32_t at = wg_hash_slot(e.x, b);
        while ((*table)[at].y != WG_HASH_EMPTY) at = (at + 1u) & mask;
        (*table)[at] = e;
    }
    *bits = b;
}

// Installs both forms of the receiver-index map.
static int wg_upload_index(bnk_ctx *ctx, const std::vector<uint2> &index)
{
    std::vector<uint2> table;
    uint32_t bits = 0;
    wg_build_hash(index, &table, &bits);
    int rc = upload(ctx, &ctx->wg_index, index.data(), index.size() * 8);
    if (!rc) rc = upload(ctx, &ctx->wg_hash, table.data(), table.size() * 8);
    if (rc) return rc;
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream)); // `table` goes away
    ctx->wg_hash_bits = bits;
    return BNK_OK;
}

extern "C" int bnk_wg_peers_set(bnk_ctx *ctx, const bnk_wg_peer *peers, uint32_t n)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!peers || n == 0) return fail(ctx, BNK_E_INVAL, "empty peer table");
    std::vector<uint2> index, allowed(n);
    std::vector<uint32_t> remote(n);
    int rc = wg_build_index(ctx, peers, n, &index);
    if (rc) return rc;
    for (uint32_t i = 0; i < n; i++) {
        remote[i] = peers[i].remote_index;
        allowed[i] = make_uint2(peers[i].allowed_net, peers[i].allowed_mask);
    }
    // in-flight batches may still read the old tables
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    // A row whose index pair is unchanged is the same keypair (a handshake
    // hands out fresh indices on both sides): it keeps its send counter, or its
    // next packet would reuse a nonce under an unchanged key.  Any other row is
    // a fresh keypair and starts at 0.
    const uint32_t n_old = ctx->n_wg_peers;
    std::vector<uint64_t> ctr(std::max(n, n_old), 0);
    std::vector<uint8_t> fresh(n, 1);
    if (n_old)
        HIPCHK(ctx, hipMemcpy(ctr.data(), ctx->wg_send_ctr.p, (size_t)n_old * 8, hipMemcpyDeviceToHost));
    for (uint32_t i = 0; i < n; i++) {
        const bool same = i < n_old && ctx->wg_rows[i].local_index == peers[i].local_index &&
                          ctx->wg_rows[i].remote_index == peers[i].remote_index;
        if (!same) ctr[i] = 0;
        fresh[i] = same ? 0 : 1; // the anti-replay window belongs to the keypair as well
    }
    rc = wg_upload_index(ctx, index);
    if (!rc) rc = upload(ctx, &ctx->wg_remote, remote.data(), (size_t)n * 4);
    if (!rc) rc = upload(ctx, &ctx->wg_allowed, allowed.data(), (size_t)n * 8);
    if (!rc) rc = upload(ctx, &ctx->wg_send_ctr, ctr.data(), (size_t)n * 8);
    if (!rc) rc = wg_replay_rows(ctx, n, fresh);
    if (rc) {
        ctx->n_wg_peers = 0; // a half-installed table is no table
        ctx->wg_rows.clear();
        return rc;
    }
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream)); // the vectors above go away
    ctx->wg_rows.assign(peers, peers + n);
    ctx->n_wg_peers = n;
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

extern "C" int bnk_wg_peer_set(bnk_ctx *ctx, uint32_t row, const bnk_wg_peer *peer, const uint8_t *key_send32,
                               const uint8_t *key_recv32)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!peer) return fail(ctx, BNK_E_INVAL, "null peer");
    if (row >= ctx->n_wg_peers) return fail(ctx, BNK_E_RANGE, "row beyond the peer table");
    if ((key_send32 && row >= ctx->n_keys[BNK_KEYS_SEND]) || (key_recv32 && row >= ctx->n_keys[BNK_KEYS_RECV]))
        return fail(ctx, BNK_E_RANGE, "row beyond the key table");
    std::vector<bnk_wg_peer> rows = ctx->wg_rows;
    rows[row] = *peer;
    std::vector<uint2> index;
    int rc = wg_build_index(ctx, rows.data(), (uint32_t)rows.size(), &index);
    if (rc) return rc;
    // in-flight batches may still read the old row
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    const uint2 allowed = make_uint2(peer->allowed_net, peer->allowed_mask);
    const uint64_t zero = 0;
    hipStream_t s = ctx->stream;
    // Everything about the row goes up before the index that makes it findable;
    // a failure part-way leaves tables that disagree, and a half-installed table
    // is no table (as in bnk_wg_peers_set).
    auto install = [&]() -> int {
        HIPCHK(ctx, hipMemcpyAsync(ctx->wg_remote.as<uint32_t>() + row, &peer->remote_index, 4, hipMemcpyHostToDevice, s));
        HIPCHK(ctx, hipMemcpyAsync(ctx->wg_allowed.as<uint2>() + row, &allowed, 8, hipMemcpyHostToDevice, s));
        // this row's keypair is new: its nonces and its anti-replay window start
        // over; every other row goes on
        HIPCHK(ctx, hipMemcpyAsync(ctx->wg_send_ctr.as<uint64_t>() + row, &zero, 8, hipMemcpyHostToDevice, s));
        HIPCHK(ctx, hipMemsetAsync(ctx->wg_replay + (size_t)row * WG_REPLAY_WORDS, 0, (size_t)WG_REPLAY_WORDS * 8, s));
        if (key_send32)
            HIPCHK(ctx, hipMemcpyAsync(ctx->d_keys[BNK_KEYS_SEND] + 8u * row, key_send32, 32, hipMemcpyHostToDevice, s));
        if (key_recv32)
            HIPCHK(ctx, hipMemcpyAsync(ctx->d_keys[BNK_KEYS_RECV] + 8u * row, key_recv32, 32, hipMemcpyHostToDevice, s));
        if (int irc = wg_upload_index(ctx, index)) return irc;
        HIPCHK(ctx, hipStreamSynchronize(s));
        return BNK_OK;
    };
    rc = install();
    if (rc) {
        ctx->n_wg_peers = 0;
        ctx->wg_rows.clear();
        return rc;
    }
    ctx->wg_rows.swap(rows);
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

extern "C" int bnk_wg_send_counter_set(bnk_ctx *ctx, uint32_t row, uint64_t next)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (row >= ctx->n_wg_peers) return fail(ctx, BNK_E_RANGE, "row beyond the peer table");
    if (next > WG_REJECT_AFTER_MESSAGES) next = WG_REJECT_AFTER_MESSAGES;
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipMemcpy(ctx->wg_send_ctr.as<uint64_t>() + row, &next, 8, hipMemcpyHostToDevice));
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

extern "C" int bnk_wg_set_replay(bnk_ctx *ctx, int on)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    ctx->wg_replay_on = on != 0;
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

extern "C" int bnk_wg_set_fused(bnk_ctx *ctx, int on)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    ctx->wg_unfused = on == 0;
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

extern "C" int bnk_wg_send_counters(bnk_ctx *ctx, uint64_t *out, uint32_t n)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!out) return fail(ctx, BNK_E_INVAL, "null out pointer");
    if (n > ctx->n_wg_peers) return fail(ctx, BNK_E_RANGE, "more counters asked for than peers");
    if (n == 0) return BNK_OK;
    HIPCHK(ctx, hipMemcpyAsync(out, ctx->wg_send_ctr.p, (size_t)n * 8, hipMemcpyDeviceToHost, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

// bnk_wg_encap_batch, with NoteOutbound at *note_now on the plaintexts first
// when note_now is given.
int bnk::wg_encap_impl(bnk_ctx *ctx, const bnk_batch *slots, uint32_t mtu, uint32_t *wire_len,
                       const int64_t *note_now)
{
    int rc = check_batch_common(ctx, slots, "slots");
    if (rc) return rc;
    const uint32_t n = slots->n;
    if (n == 0) return BNK_OK;
    if (!wire_len) return fail(ctx, BNK_E_INVAL, "null wire_len array");
    if (ctx->n_wg_peers == 0) return fail(ctx, BNK_E_STATE, "no peer table loaded");
    if (!ctx->d_keys[BNK_KEYS_SEND] || ctx->n_keys[BNK_KEYS_SEND] < ctx->n_wg_peers)
        return fail(ctx, BNK_E_STATE, "send key table is smaller than the peer table");
    const bool host = slots->mem == BNK_MEM_HOST;
    const auto slot_ext = [slots, mtu](uint32_t i) {
        const uint32_t len = slots->lens ? slots->lens[i] : slots->len;
        return 16ull + len + wg_padding(len, mtu) + 16ull;
    };

    WgBatch b{};
    b.n = n;
    b.stride = slots->stride;
    b.len = slots->len;
    const uint32_t *d_peer = nullptr;
    uint32_t *d_wire_len = nullptr;
    Span span;
    HostPipe hp;
    bool chunked = false;
    // A wave-per-packet launch does the framing itself; it needs every packet to
    // fit 63 ChaCha20 blocks, which only a host batch can promise.
    bool fits = host;
    if (host) {
        if (slots->lens) {
            for (uint32_t i = 0; i < n && fits; i++) fits = slots->lens[i] + 15u <= WG_FUSE_MAX_LEN;
        } else {
            fits = slots->len + 15u <= WG_FUSE_MAX_LEN;
        }
    }
    // Which kernel will read the packets: the framing launch when the batch
    // qualifies for it, else a plain launch over per-packet padded lengths.
    AeadArgs probe{};
    probe.spread_max = ctx->spread_max;
    probe.n = n;
    probe.len = slots->len;
    probe.lens = slots->lens; // only whether there is one matters here
    const bool wave_per_packet = (fits && aead_runs_spread(probe)) || n <= ctx->spread_max;

    // direct route (small batches in a pinned ring): the plaintexts are fetched
    // by a copy kernel, headers and sealed packets go straight into the ring
    uint8_t *ring_out = nullptr;
    uint32_t *h_wire_len = nullptr;
    if (host) {
        rc = check_index_range(ctx, slots->peer, n, ctx->n_wg_peers, "peer index", "the peer table");
        if (rc) return rc;
        uint8_t *d_ring = n <= DIRECT_MAX_PACKETS ? ring_device_ptr(ctx, slots->base, slots->bytes) : nullptr;
        if (d_ring) {
            Span sp;
            for (uint32_t i = 0; i < n; i++) {
                const uint64_t off = pkt_off(slots, i), need = slot_ext(i);
                if (off > slots->bytes || need > slots->bytes - off)
                    return fail(ctx, BNK_E_INVAL, "slots: packet " + std::to_string(i) + " lies outside the arena");
                sp.add(off, off + need);
            }
            // (a wave per packet reads each slot where it lies; a lane per packet
            // first fetches the whole span)
            if ((wave_per_packet ? host_payload_bytes(slots) : sp.size()) <= DIRECT_MAX_BYTES) {
                span = sp;
                ring_out = d_ring + span.lo;
            }
        }
    }
    if (ring_out) {
        PinBuf &stage = *ctx->pin_cur;
        HIPCHK(ctx, stage.reserve((size_t)n * 20 + 64));
        uint64_t *p_off = stage.as<uint64_t>();
        uint32_t *p_lens = (uint32_t *)(p_off + n), *p_peer = p_lens + n;
        h_wire_len = p_peer + n;
        if (wave_per_packet) {
            // a wave per packet reads the ring itself (see aead_batch_host_direct)
            b.base = ring_out;
        } else {
            const uint32_t mis = (uint32_t)((uintptr_t)ring_out & 127u);
            HIPCHK(ctx, ctx->in_arena.reserve(span.size() + 160));
            HIPCHK(ctx, launch_pull(ring_out, ctx->in_arena.as<uint8_t>() + mis, span.size(), ctx->stream));
            b.base = ctx->in_arena.as<uint8_t>() + mis;
        }
        if (slots->offsets) {
            for (uint32_t i = 0; i < n; i++) p_off[i] = slots->offsets[i] - span.lo;
            b.off = stage.dev(p_off);
        }
        if (slots->lens) { memcpy(p_lens, slots->lens, (size_t)n * 4); b.lens = stage.dev(p_lens); }
        if (slots->peer) { memcpy(p_peer, slots->peer, (size_t)n * 4); d_peer = stage.dev(p_peer); }
        d_wire_len = stage.dev(h_wire_len);
    } else if (host) {
        HIPCHK(ctx, ctx->wg_wirelen.reserve((size_t)n * 4));
        d_wire_len = ctx->wg_wirelen.as<uint32_t>();
        hp.ctx = ctx;
        hp.in = hp.out = slots;
        hp.in_ext = hp.out_ext = slot_ext;
        rc = hp.plan(0);
        if (rc != BNK_OK && rc != 1) return rc;
        chunked = rc == BNK_OK;
        if (chunked) {
            hp.add_result(wire_len, d_wire_len, 4);
            rc = hp.begin();
            if (rc) return rc;
            b.base = hp.d_in;
            b.off = hp.d_in_off;
        } else {
            for (uint32_t i = 0; i < n; i++) {
                const uint64_t off = pkt_off(slots, i), need = slot_ext(i);
                if (off > slots->bytes || need > slots->bytes - off)
                    return fail(ctx, BNK_E_INVAL, "slots: packet " + std::to_string(i) + " lies outside the arena");
                span.add(off, off + need);
            }
            HIPCHK(ctx, ctx->pin.reserve((size_t)n * 16 + 64));
            HIPCHK(ctx, ctx->in_arena.reserve(span.size() + 16));
            HIPCHK(ctx, hipMemcpyAsync(ctx->in_arena.p, (const uint8_t *)slots->base + span.lo, span.size(),
                                       hipMemcpyHostToDevice, ctx->stream));
            b.base = ctx->in_arena.as<uint8_t>();
            rc = upload_offsets(ctx, slots, n, span.lo, &ctx->off_in, 0, &b.off);
            if (rc) return rc;
        }
        if (slots->lens) {
            rc = upload(ctx, &ctx->lens, slots->lens, (size_t)n * 4);
            if (rc) return rc;
            b.lens = ctx->lens.as<uint32_t>();
        }
        if (slots->peer) {
            rc = upload(ctx, &ctx->peer, slots->peer, (size_t)n * 4);
            if (rc) return rc;
            d_peer = ctx->peer.as<uint32_t>();
        }
    } else {
        if (!slots->offsets && !slots->lens &&
            (uint64_t)(n - 1) * slots->stride + slot_ext(0) > slots->bytes)
            return fail(ctx, BNK_E_INVAL, "slots: uniform layout exceeds the arena");
        if (slots->bytes == 0) return fail(ctx, BNK_E_INVAL, "slots: arena size 0");
        b.base = (const uint8_t *)slots->base;
        b.off = slots->offsets;
        b.lens = slots->lens;
        if (slots->offsets || slots->lens) b.limit = slots->bytes; // the lanes check what the host cannot read
        d_peer = slots->peer;
        d_wire_len = wire_len;
    }

    for (DevBuf *buf : {&ctx->r_keys, &ctx->r_idx, &ctx->r_skeys, &ctx->r_sidx, &ctx->wg_padded})
        HIPCHK(ctx, buf->reserve((size_t)n * 4));
    HIPCHK(ctx, ctx->r_ctr_out.reserve((size_t)n * 8));
    HIPCHK(ctx, ctx->wg_skip.reserve(n));
    const size_t tmp_bytes = relay_sort_tmp_bytes(n, ctx->n_wg_peers);
    HIPCHK(ctx, ctx->r_tmp.reserve(tmp_bytes + 16));
    if (slots->lens) {
        HIPCHK(ctx, ctx->order.reserve((size_t)n * 4));
        HIPCHK(ctx, ctx->hist.reserve(LEN_BINS * 4));
        HIPCHK(ctx, ctx->cursor.reserve(LEN_CURSOR_WORDS * 4));
    }
    const WgPeersDev pe = peers_view(ctx);
    uint64_t *d_ctr = ctx->r_ctr_out.as<uint64_t>();
    uint32_t *d_padded = ctx->wg_padded.as<uint32_t>();
    uint8_t *d_skip = ctx->wg_skip.as<uint8_t>();

    // counters in batch order per peer, advancing the peers' send counters:
    // needs the peer array only, so it runs ahead of the packet bytes
    if (n <= PEER_RANK_SMALL_MAX) {
        HIPCHK(ctx, launch_peer_rank_small(d_peer, pe.n, n, pe.send_ctr, d_ctr, true, WG_REJECT_AFTER_MESSAGES,
                                           ctx->d_status, ctx->stream));
    } else if (d_peer && peer_rank_counts(n, pe.n, tmp_bytes)) {
        HIPCHK(ctx, launch_peer_rank_counting(d_peer, ctx->r_tmp.p, pe.send_ctr, pe.n, n, d_ctr, true,
                                              WG_REJECT_AFTER_MESSAGES, ctx->d_status, ctx->stream));
    } else {
        HIPCHK(ctx, launch_wg_keys(d_peer, pe.n, n, ctx->r_keys.as<uint32_t>(), ctx->r_idx.as<uint32_t>(),
                                   ctx->d_status, ctx->stream));
        HIPCHK(ctx, launch_peer_rank(ctx->r_keys.as<uint32_t>(), ctx->r_idx.as<uint32_t>(),
                                     ctx->r_skeys.as<uint32_t>(), ctx->r_sidx.as<uint32_t>(), ctx->r_tmp.p,
                                     tmp_bytes, pe.send_ctr, pe.n, n, d_ctr, true, WG_REJECT_AFTER_MESSAGES,
                                     ctx->stream));
    }

    // filter.go:192-194: NoteOutbound does nothing in allow-all mode
    const bool note = note_now != nullptr && ctx->filter->enforce;
    if (note) {
        rc = flows_reserve(ctx, n);
        if (rc) return rc;
    }

    // NoteOutbound, then header, padding and seal of packets [lo, hi)
    auto run = [&](uint32_t lo, uint32_t hi) -> int {
        WgBatch c = b;
        c.first = lo;
        c.n = hi - lo;
        uint8_t *sealed = ring_out ? ring_out : const_cast<uint8_t *>(b.base);
        if (note) {
            FilterState *f = ctx->filter;
            FilterArgs fa{};
            fa.pkts = b.base + 16 + (b.off ? 0 : (uint64_t)lo * slots->stride);
            fa.off = b.off ? b.off + lo : nullptr;
            fa.lens = b.lens ? b.lens + lo : nullptr;
            fa.stride = slots->stride;
            fa.len = slots->len;
            fa.status = ctx->d_status;
            fa.now = *note_now;
            fa.n = hi - lo;
            fa.rules = f->ridx;
            fa.flows = f->flows;
            HIPCHK(ctx, launch_filter_note(fa, f->max_blocks, f->claimed_upper > 4096, ctx->stream));
        }
        if (fits) {
            AeadArgs se{};
            se.spread_max = ctx->spread_max;
            se.keys = ctx->d_keys[BNK_KEYS_SEND];
            se.n_peers = pe.n;
            se.status = ctx->d_status;
            se.first = lo;
            se.n = hi - lo;
            se.in = b.base;
            se.out = sealed;
            se.in_off = se.out_off = b.off;
            se.in_stride = se.out_stride = slots->stride;
            se.lens = b.lens;
            se.len = slots->len;
            se.peer = d_peer;
            se.counters = d_ctr;
            if (aead_runs_spread(se)) {
                se.wg.mode = WG_FUSE_ENCAP;
                se.wg.n_peers = pe.n;
                se.wg.mtu = mtu;
                se.wg.remote_index = pe.remote_index;
                se.wg.wire_len = d_wire_len;
                HIPCHK(ctx, launch_aead_seal(se, ctx->stream));
                return BNK_OK;
            }
        }
        AeadArgs se{};
        se.spread_max = ctx->spread_max;
        se.keys = ctx->d_keys[BNK_KEYS_SEND];
        se.n_peers = pe.n;
        se.status = ctx->d_status;
        se.first = lo;
        se.n = hi - lo;
        se.in = b.base;
        se.out = sealed;
        se.in_off = se.out_off = b.off;
        se.in_stride = se.out_stride = slots->stride;
        se.in_skip = se.out_skip = 16;
        se.lens = d_padded;
        se.peer = d_peer;
        se.counters = d_ctr;
        if (!ctx->wg_unfused && !aead_runs_spread(se)) {
            // a lane per packet: header, padding (as implied zeros) and lengths are
            // the launch's own work too
            se.lens = b.lens;
            se.len = slots->len;
            // the slot from its first byte to the end of the tag, as the separate kernel checks it
            se.in_limit = se.out_limit = b.limit;
            se.wg.mode = WG_FUSE_ENCAP;
            se.wg.n_peers = pe.n;
            se.wg.mtu = mtu;
            se.wg.remote_index = pe.remote_index;
            se.wg.wire_len = d_wire_len;
        } else {
            // the framing in a kernel of its own, then a plain seal of the padded packets
            se.skip = d_skip;
            HIPCHK(ctx, launch_wg_encap_prep(c, sealed, pe, d_peer, d_ctr, mtu, d_padded, d_wire_len, d_skip,
                                             ctx->d_status, ctx->stream));
        }
        // (padding never changes a packet's number of 64-byte blocks, so the plaintext
        // lengths group the packets as the padded ones would)
        if (slots->lens && se.n > 64 && !aead_runs_spread(se)) {
            HIPCHK(ctx, launch_length_sort(se.lens + lo, se.n, 0, ctx->order.as<uint32_t>() + lo,
                                           ctx->hist.as<uint32_t>(), ctx->cursor.as<uint32_t>(), ctx->stream));
            se.order = ctx->order.as<uint32_t>() + lo;
        }
        HIPCHK(ctx, launch_aead_seal(se, ctx->stream));
        return BNK_OK;
    };

    if (chunked) {
        rc = hp.open_gate();
        if (rc) return rc;
        for (uint32_t k = 0; k < hp.chunks; k++) {
            uint32_t lo, hi;
            if (!hp.range(k, &lo, &hi)) break;
            if ((rc = hp.upload(k)) || (rc = run(lo, hi)) || (rc = hp.download(k))) return rc;
        }
        rc = hp.finish();
        if (rc) return rc;
    } else {
        rc = run(0, n);
        if (rc) return rc;
        if (!host) return BNK_OK;
        if (ring_out) {
            // peer indices were checked above: only a flow table overflow could come
            // back through the status word
            return finish_direct(ctx, note, {{wire_len, h_wire_len, (size_t)n * 4}});
        }
        HIPCHK(ctx, hipMemcpyAsync((uint8_t *)slots->base + span.lo, ctx->in_arena.p, span.size(),
                                   hipMemcpyDeviceToHost, ctx->stream));
        HIPCHK(ctx, hipMemcpyAsync(wire_len, d_wire_len, (size_t)n * 4, hipMemcpyDeviceToHost, ctx->stream));
    }
    uint32_t status = 0;
    rc = take_status(ctx, &status);
    if (rc) return rc;
    return status_to_rc(ctx, status);
}

extern "C" int bnk_wg_encap_batch(bnk_ctx *ctx, const bnk_batch *slots, uint32_t mtu, uint32_t *wire_len)
{
    BNK_API_TRY
    {
        CoRequest rq{CO_ENCAP, slots, nullptr, mtu, 0, nullptr, wire_len, nullptr, nullptr};
        int crc;
        if (coalesce_submit(ctx, rq, &crc)) {
            if (crc == BNK_OK) (void)tally_nonzero(ctx, TALLY_SEALED, wire_len, slots->n, BNK_MEM_HOST);
            return crc;
        }
    }
    Guard g(ctx);
    if (g.rc) return g.rc;
    const int rc = wg_encap_impl(ctx, slots, mtu, wire_len, nullptr);
    if (rc == BNK_OK) return tally_nonzero(ctx, TALLY_SEALED, wire_len, slots->n, slots->mem);
    return rc;
    BNK_API_CATCH(ctx)
}

extern "C" int bnk_wg_note_encap_batch(bnk_ctx *ctx, const bnk_batch *slots, uint32_t mtu, int64_t now_ns,
                                       uint32_t *wire_len)
{
    BNK_API_TRY
    {
        CoRequest rq{CO_NOTE_ENCAP, slots, nullptr, mtu, now_ns, nullptr, wire_len, nullptr, nullptr};
        int crc;
        if (coalesce_submit(ctx, rq, &crc)) {
            if (crc == BNK_OK) (void)tally_nonzero(ctx, TALLY_SEALED, wire_len, slots->n, BNK_MEM_HOST);
            return crc;
        }
    }
    Guard g(ctx);
    if (g.rc) return g.rc;
    const int rc = wg_encap_impl(ctx, slots, mtu, wire_len, &now_ns);
    if (rc == BNK_OK) return tally_nonzero(ctx, TALLY_SEALED, wire_len, slots->n, slots->mem);
    return rc;
    BNK_API_CATCH(ctx)
}

// bnk_wg_decap_batch, with CheckInbound at *check_now on the delivered
// packets afterwards when check_now is given.
int bnk::wg_decap_impl(bnk_ctx *ctx, const bnk_batch *wire, const bnk_batch *out, uint8_t *result,
                       uint32_t *out_len, uint32_t *peer, uint64_t *counter, const int64_t *check_now)
{
    int rc = check_batch_common(ctx, wire, "wire");
    if (rc) return rc;
    rc = check_batch_common(ctx, out, "out");
    if (rc) return rc;
    if (wire->mem != out->mem) return fail(ctx, BNK_E_INVAL, "wire and out must use the same mem kind");
    const uint32_t n = wire->n;
    if (n == 0) return BNK_OK;
    if (!result || !out_len || !peer || !counter) return fail(ctx, BNK_E_INVAL, "null result array");
    if (ctx->n_wg_peers == 0) return fail(ctx, BNK_E_STATE, "no peer table loaded");
    if (!ctx->d_keys[BNK_KEYS_RECV] || ctx->n_keys[BNK_KEYS_RECV] < ctx->n_wg_peers)
        return fail(ctx, BNK_E_STATE, "receive key table is smaller than the peer table");
    const bool host = wire->mem == BNK_MEM_HOST;

    WgBatch wb{}, ob{};
    wb.n = ob.n = n;
    wb.stride = wire->stride;
    wb.len = wire->len;
    ob.stride = out->stride;
    uint8_t *d_result = nullptr;
    uint32_t *d_out_len = nullptr, *d_peer = nullptr;
    uint64_t *d_counter = nullptr;
    Staged st;
    HostPipe hp;
    bool chunked = false;
    bnk_batch w2 = *wire; // the sender's identity comes out of the datagrams, not in with them
    w2.peer = nullptr;
    w2.counters = nullptr;
    // the pipeline keeps these until the call returns: they live at function scope
    // and hold copies of what they need
    const auto wire_ext = [wire](uint32_t i) { return (uint64_t)(wire->lens ? wire->lens[i] : wire->len); };
    const auto plain_ext = [wire](uint32_t i) {
        const uint64_t l = wire->lens ? wire->lens[i] : wire->len;
        return l >= 32u ? l - 32u : (uint64_t)0;
    };
    // A wave-per-packet launch does the framing itself; it needs every packet to
    // fit 63 ChaCha20 blocks, which only a host batch can promise.
    bool fits = host;
    if (host) {
        if (wire->lens) {
            for (uint32_t i = 0; i < n && fits; i++) fits = wire->lens[i] <= WG_FUSE_MAX_LEN + 32u;
        } else {
            fits = wire->len <= WG_FUSE_MAX_LEN + 32u;
        }
    }
    // Which kernel will read the datagrams: the framing launch when the batch
    // qualifies for it, else a plain launch over per-packet ciphertext lengths.
    AeadArgs probe{};
    probe.spread_max = ctx->spread_max;
    probe.n = n;
    probe.len = wire->len;
    probe.lens = wire->lens; // only whether there is one matters here
    const bool wave_per_packet = (fits && aead_runs_spread(probe)) || n <= ctx->spread_max;

    // direct route (small batches in pinned rings): datagrams fetched by a copy
    // kernel, plaintexts written straight into the out ring, per-packet results
    // into pinned staging
    bool direct = false;
    uint8_t *h_result = nullptr;
    uint32_t *h_out_len = nullptr, *h_peer = nullptr;
    uint64_t *h_counter = nullptr;
    if (host && n <= DIRECT_MAX_PACKETS) {
        uint8_t *d_wire = ring_device_ptr(ctx, wire->base, wire->bytes);
        uint8_t *d_outr = ring_device_ptr(ctx, out->base, out->bytes);
        if (d_wire && d_outr) {
            Span sin, sout;
            rc = scan_host_layout(ctx, &w2, &w2, 0, &sin, "in");
            if (rc) return rc;
            rc = scan_host_layout(ctx, out, &w2, -32, &sout, "out");
            if (rc) return rc;
            if ((wave_per_packet ? host_payload_bytes(&w2) : sin.size()) <= DIRECT_MAX_BYTES) {
                direct = true;
                PinBuf &stage = *ctx->pin_cur;
                HIPCHK(ctx, stage.reserve((size_t)n * 37 + 64));
                uint64_t *p_in_off = stage.as<uint64_t>(), *p_out_off = p_in_off + n;
                h_counter = p_out_off + n;
                uint32_t *p_lens = (uint32_t *)(h_counter + n);
                h_out_len = p_lens + n;
                h_peer = h_out_len + n;
                h_result = (uint8_t *)(h_peer + n);
                if (wave_per_packet) {
                    // a wave per packet reads the ring itself (see aead_batch_host_direct)
                    wb.base = d_wire + sin.lo;
                } else {
                    const uint32_t mis = (uint32_t)((uintptr_t)(d_wire + sin.lo) & 127u);
                    HIPCHK(ctx, ctx->in_arena.reserve(sin.size() + 160));
                    HIPCHK(ctx, launch_pull(d_wire + sin.lo, ctx->in_arena.as<uint8_t>() + mis, sin.size(), ctx->stream));
                    wb.base = ctx->in_arena.as<uint8_t>() + mis;
                }
                if (wire->offsets) {
                    for (uint32_t i = 0; i < n; i++) p_in_off[i] = wire->offsets[i] - sin.lo;
                    wb.off = stage.dev(p_in_off);
                }
                if (wire->lens) { memcpy(p_lens, wire->lens, (size_t)n * 4); wb.lens = stage.dev(p_lens); }
                ob.base = d_outr;
                if (out->offsets) { memcpy(p_out_off, out->offsets, (size_t)n * 8); ob.off = stage.dev(p_out_off); }
                d_result = stage.dev(h_result);
                d_out_len = stage.dev(h_out_len);
                d_peer = stage.dev(h_peer);
                d_counter = stage.dev(h_counter);
            }
        }
    }
    if (host && !direct) {
        HIPCHK(ctx, ctx->wg_result.reserve(n));
        HIPCHK(ctx, ctx->wg_outlen.reserve((size_t)n * 4));
        HIPCHK(ctx, ctx->wg_peer.reserve((size_t)n * 4));
        HIPCHK(ctx, ctx->wg_counter.reserve((size_t)n * 8));
        d_result = ctx->wg_result.as<uint8_t>();
        d_out_len = ctx->wg_outlen.as<uint32_t>();
        d_peer = ctx->wg_peer.as<uint32_t>();
        d_counter = ctx->wg_counter.as<uint64_t>();
        hp.ctx = ctx;
        hp.in = &w2;
        hp.out = out;
        hp.in_ext = wire_ext;
        hp.out_ext = plain_ext;
        rc = hp.plan(wire->lens ? 0 : plain_ext(0));
        if (rc != BNK_OK && rc != 1) return rc;
        chunked = rc == BNK_OK;
        if (chunked) {
            hp.add_result(result, d_result, 1);
            hp.add_result(out_len, d_out_len, 4);
            hp.add_result(peer, d_peer, 4);
            hp.add_result(counter, d_counter, 8);
            rc = hp.begin();
            if (rc) return rc;
            wb.base = hp.d_in;
            wb.off = hp.d_in_off;
            ob.base = hp.d_out;
            ob.off = hp.d_out_off;
            if (wire->lens) {
                rc = upload(ctx, &ctx->lens, wire->lens, (size_t)n * 4);
                if (rc) return rc;
                wb.lens = ctx->lens.as<uint32_t>();
            }
        } else {
            rc = stage_host(ctx, &w2, out, -32, 0, &st);
            if (rc) return rc;
            wb.base = st.d_in;
            wb.off = st.d_in_off;
            wb.lens = st.d_lens;
            ob.base = st.d_out;
            ob.off = st.d_out_off;
        }
    } else if (!host) {
        if (!wire->offsets && !wire->lens && (uint64_t)(n - 1) * wire->stride + wire->len > wire->bytes)
            return fail(ctx, BNK_E_INVAL, "wire: uniform layout exceeds the arena");
        if (!out->offsets && !wire->lens &&
            (uint64_t)(n - 1) * out->stride + (wire->len >= 32u ? wire->len - 32u : 0u) > out->bytes)
            return fail(ctx, BNK_E_INVAL, "out: uniform layout exceeds the arena");
        if (wire->bytes == 0 || out->bytes == 0) return fail(ctx, BNK_E_INVAL, "arena size 0");
        wb.base = (const uint8_t *)wire->base;
        wb.off = wire->offsets;
        wb.lens = wire->lens;
        ob.base = (const uint8_t *)out->base;
        ob.off = out->offsets;
        if (wire->offsets || wire->lens || out->offsets) {
            // the lanes check what the host cannot read: the datagram where it is
            // parsed, the plaintext where it is written
            wb.limit = wire->bytes;
            ob.limit = out->bytes;
        }
        d_result = result;
        d_out_len = out_len;
        d_peer = peer;
        d_counter = counter;
    }
    HIPCHK(ctx, ctx->wg_ctlen.reserve((size_t)n * 4));
    HIPCHK(ctx, ctx->r_auth.reserve(n));
    if (wire->lens) {
        HIPCHK(ctx, ctx->order.reserve((size_t)n * 4));
        HIPCHK(ctx, ctx->hist.reserve(LEN_BINS * 4));
        HIPCHK(ctx, ctx->cursor.reserve(LEN_CURSOR_WORDS * 4));
    }
    uint32_t *d_ctlen = ctx->wg_ctlen.as<uint32_t>();
    uint8_t *d_auth = ctx->r_auth.as<uint8_t>();
    const WgPeersDev pe = peers_view(ctx);

    // filter.go:124-126: CheckInbound passes everything in allow-all mode
    const bool check = check_now != nullptr && ctx->filter->enforce;
    if (check) HIPCHK(ctx, ctx->r_pass.reserve(n));

    // the anti-replay windows, walked per chunk in batch order
    const bool replay = ctx->wg_replay_on;
    WgReplayDev rpd{ctx->wg_replay, pe.n};
    WgReplayScratch rsc{};
    if (replay && n > WG_REPLAY_SMALL_MAX) {
        const uint32_t biggest = chunked ? hp.per : n;
        for (DevBuf *buf : {&ctx->r_keys, &ctx->r_idx, &ctx->r_skeys, &ctx->r_sidx})
            HIPCHK(ctx, buf->reserve((size_t)biggest * 4));
        for (DevBuf *buf : {&ctx->wg_sctr, &ctx->wg_sval, &ctx->wg_pmax}) HIPCHK(ctx, buf->reserve((size_t)biggest * 8));
        // the flag words and the first-occurrence table keep their resting state from pass
        // to pass: set it when they are first allocated or grow
        const void *had = ctx->wg_lastb.p;
        HIPCHK(ctx, ctx->wg_lastb.reserve((size_t)biggest + 64));
        if (ctx->wg_lastb.p != had) HIPCHK(ctx, hipMemsetAsync(ctx->wg_lastb.p, 0, 64, ctx->stream));
        rsc.table_slots = wg_replay_table_slots(biggest);
        had = ctx->wg_rtable.p;
        HIPCHK(ctx, ctx->wg_rtable.reserve((size_t)rsc.table_slots * 4));
        if (ctx->wg_rtable.p != had)
            HIPCHK(ctx, hipMemsetAsync(ctx->wg_rtable.p, 0xFF, ctx->wg_rtable.cap, ctx->stream));
        rsc.tmp_bytes = wg_replay_tmp_bytes(biggest, pe.n);
        HIPCHK(ctx, ctx->r_tmp.reserve(rsc.tmp_bytes + 16));
        rsc.keys = ctx->r_keys.as<uint32_t>();
        rsc.idx = ctx->r_idx.as<uint32_t>();
        rsc.skeys = ctx->r_skeys.as<uint32_t>();
        rsc.sidx = ctx->r_sidx.as<uint32_t>();
        rsc.sctr = ctx->wg_sctr.as<uint64_t>();
        rsc.sval = ctx->wg_sval.as<uint64_t>();
        rsc.pmax = ctx->wg_pmax.as<uint64_t>();
        rsc.cls = ctx->wg_lastb.as<uint8_t>() + 64;
        rsc.flags = ctx->wg_lastb.as<uint32_t>();
        rsc.table = ctx->wg_rtable.as<uint32_t>();
        rsc.tmp = ctx->r_tmp.p;
    }
    // wireguard-go's sequential receiver validates the counter of every
    // authentic packet before it looks inside: ahead of the inbound filter
    auto replay_range = [&](uint32_t lo, uint32_t hi, bool keys_from_open = false) -> int {
        if (!replay) return BNK_OK;
        WgReplayScratch c = rsc;
        c.table_slots = hi - lo > WG_REPLAY_SMALL_MAX ? wg_replay_table_slots(hi - lo) : 0;
        if (c.table_slots) c.parity = ctx->wg_replay_parity++ & 1u;
        c.keys_ready = keys_from_open;
        HIPCHK(ctx, launch_wg_replay(d_result + lo, d_out_len + lo, d_peer + lo, d_counter + lo, hi - lo, rpd, c,
                                     ctx->stream));
        return BNK_OK;
    };

    // CheckInbound of what packets [lo, hi) delivered: a packet that was not
    // delivered has length 0 here, which the filter refuses without a side effect
    auto filter_range = [&](uint32_t lo, uint32_t hi) -> int {
        if (!check) return BNK_OK;
        FilterState *f = ctx->filter;
        uint8_t *d_pass = ctx->r_pass.as<uint8_t>();
        FilterArgs fa{};
        fa.pkts = ob.base + (ob.off ? 0 : (uint64_t)lo * out->stride);
        fa.off = ob.off ? ob.off + lo : nullptr;
        fa.lens = d_out_len + lo;
        fa.stride = out->stride;
        fa.verdict = d_pass + lo;
        fa.status = ctx->d_status;
        fa.now = *check_now;
        fa.n = hi - lo;
        fa.rules = f->ridx;
        fa.flows = f->flows;
        fa.wg_result = d_result + lo;
        HIPCHK(ctx, launch_filter_check(fa, f->max_blocks, ctx->stream));
        return BNK_OK;
    };

    // parse, open and check packets [lo, hi)
    auto run = [&](uint32_t lo, uint32_t hi) -> int {
        WgBatch cw = wb, co = ob;
        cw.first = co.first = lo;
        cw.n = co.n = hi - lo;
        if (fits) {
            AeadArgs op{};
            op.spread_max = ctx->spread_max;
            op.keys = ctx->d_keys[BNK_KEYS_RECV];
            op.n_peers = pe.n;
            op.status = ctx->d_status;
            op.first = lo;
            op.n = hi - lo;
            op.in = wb.base;
            op.in_off = wb.off;
            op.in_stride = wire->stride;
            op.out = const_cast<uint8_t *>(ob.base);
            op.out_off = ob.off;
            op.out_stride = out->stride;
            op.lens = wb.lens;
            op.len = wire->len;
            if (aead_runs_spread(op)) {
                op.wg.mode = WG_FUSE_DECAP;
                op.wg.n_peers = pe.n;
                op.wg.index_sorted = pe.index_sorted;
                op.wg.allowed = pe.allowed;
                op.wg.result = d_result;
                op.wg.out_len = d_out_len;
                op.wg.peer_out = d_peer;
                op.wg.counter_out = d_counter;
                HIPCHK(ctx, launch_aead_open(op, ctx->stream));
                if (int rr = replay_range(lo, hi)) return rr;
                return filter_range(lo, hi);
            }
        }
        AeadArgs op{};
        op.spread_max = ctx->spread_max;
        op.keys = ctx->d_keys[BNK_KEYS_RECV];
        op.n_peers = pe.n;
        op.status = ctx->d_status;
        op.first = lo;
        op.n = hi - lo;
        op.in = wb.base;
        op.in_off = wb.off;
        op.in_stride = wire->stride;
        op.in_skip = 16;
        op.out = const_cast<uint8_t *>(ob.base);
        op.out_off = ob.off;
        op.out_stride = out->stride;
        op.lens = d_ctlen;
        op.out_limit = ob.limit;
        if (!ctx->wg_unfused && !aead_runs_spread(op)) {
            // a lane per packet: header checks, index lookup and what follows the
            // open are the launch's own work too
            op.lens = wb.lens;
            op.len = wire->len;
            op.in_limit = wb.limit;
            op.wg.mode = WG_FUSE_DECAP;
            op.wg.n_peers = pe.n;
            op.wg.index_hash = pe.index_hash;
            op.wg.hash_bits = pe.hash_bits;
            op.wg.allowed = pe.allowed;
            op.wg.result = d_result;
            op.wg.out_len = d_out_len;
            op.wg.peer_out = d_peer;
            op.wg.counter_out = d_counter;
            // the window pass sorts the authentic packets by peer: its keys come from here
            const bool keys_here = replay && op.n > WG_REPLAY_SMALL_MAX;
            if (keys_here) {
                op.wg.replay_keys = rsc.keys;
                op.wg.replay_idx = rsc.idx;
                op.wg.replay_index_bits = wg_replay_index_bits(op.n, pe.n);
            }
            if (wire->lens && op.n > 64) {
                // (32 bytes of every datagram are header and tag)
                HIPCHK(ctx, launch_length_sort(wb.lens + lo, op.n, 32, ctx->order.as<uint32_t>() + lo,
                                               ctx->hist.as<uint32_t>(), ctx->cursor.as<uint32_t>(), ctx->stream));
                op.order = ctx->order.as<uint32_t>() + lo;
            }
            HIPCHK(ctx, launch_aead_open(op, ctx->stream));
            if (int rr = replay_range(lo, hi, keys_here)) return rr;
            return filter_range(lo, hi);
        }
        // the framing in kernels of its own around a plain open
        HIPCHK(ctx, launch_wg_parse(cw, pe, d_peer, d_counter, d_ctlen, d_result, ctx->d_status, ctx->stream));
        op.peer = d_peer;
        op.counters = d_counter;
        op.verdict = d_auth;
        // (the datagram's own bounds were checked by the parse)
        op.skip = d_result; // BNK_WG_OK is 0: header failures are not opened
        if (wire->lens && op.n > 64 && !aead_runs_spread(op)) {
            HIPCHK(ctx, launch_length_sort(d_ctlen + lo, op.n, 16, ctx->order.as<uint32_t>() + lo,
                                           ctx->hist.as<uint32_t>(), ctx->cursor.as<uint32_t>(), ctx->stream));
            op.order = ctx->order.as<uint32_t>() + lo;
        }
        HIPCHK(ctx, launch_aead_open(op, ctx->stream));
        HIPCHK(ctx, launch_wg_finish(co, 0, pe, d_peer, d_ctlen, d_auth, d_result, d_out_len, ctx->stream));
        if (int rr = replay_range(lo, hi)) return rr;
        return filter_range(lo, hi);
    };

    if (chunked) {
        rc = hp.open_gate();
        if (rc) return rc;
        for (uint32_t k = 0; k < hp.chunks; k++) {
            uint32_t lo, hi;
            if (!hp.range(k, &lo, &hi)) break;
            if ((rc = hp.upload(k)) || (rc = run(lo, hi)) || (rc = hp.download(k))) return rc;
        }
        rc = hp.finish();
        if (rc) return rc;
    } else {
        rc = run(0, n);
        if (rc) return rc;
        if (!host) return BNK_OK;
        if (direct) {
            // the peer index of every opened packet comes from the table lookup:
            // nothing comes back through the status word
            return finish_direct(ctx, false, {{result, h_result, (size_t)n},
                                              {out_len, h_out_len, (size_t)n * 4},
                                              {peer, h_peer, (size_t)n * 4},
                                              {counter, h_counter, (size_t)n * 8}});
        }
        HIPCHK(ctx, hipMemcpyAsync((uint8_t *)out->base + st.sout.lo, st.d_out, st.sout.size(),
                                   hipMemcpyDeviceToHost, ctx->stream));
        HIPCHK(ctx, hipMemcpyAsync(result, d_result, n, hipMemcpyDeviceToHost, ctx->stream));
        HIPCHK(ctx, hipMemcpyAsync(out_len, d_out_len, (size_t)n * 4, hipMemcpyDeviceToHost, ctx->stream));
        HIPCHK(ctx, hipMemcpyAsync(peer, d_peer, (size_t)n * 4, hipMemcpyDeviceToHost, ctx->stream));
        HIPCHK(ctx, hipMemcpyAsync(counter, d_counter, (size_t)n * 8, hipMemcpyDeviceToHost, ctx->stream));
    }
    uint32_t status = 0;
    rc = take_status(ctx, &status);
    if (rc) return rc;
    return status_to_rc(ctx, status);
}

extern "C" int bnk_wg_decap_batch(bnk_ctx *ctx, const bnk_batch *wire, const bnk_batch *out,
                                  uint8_t *result, uint32_t *out_len, uint32_t *peer, uint64_t *counter)
{
    BNK_API_TRY
    {
        CoRequest rq{CO_DECAP, wire, out, 0, 0, result, out_len, peer, counter};
        int crc;
        if (coalesce_submit(ctx, rq, &crc)) {
            if (crc == BNK_OK) (void)tally_results(ctx, TALLY_DECAP, result, wire->n, BNK_MEM_HOST);
            return crc;
        }
    }
    Guard g(ctx);
    if (g.rc) return g.rc;
    const int rc = wg_decap_impl(ctx, wire, out, result, out_len, peer, counter, nullptr);
    if (rc == BNK_OK) return tally_results(ctx, TALLY_DECAP, result, wire->n, wire->mem);
    return rc;
    BNK_API_CATCH(ctx)
}

extern "C" int bnk_wg_decap_filter_batch(bnk_ctx *ctx, const bnk_batch *wire, const bnk_batch *out,
                                         int64_t now_ns, uint8_t *result, uint32_t *out_len,
                                         uint32_t *peer, uint64_t *counter)
{
    BNK_API_TRY
    {
        CoRequest rq{CO_DECAP_FILTER, wire, out, 0, now_ns, result, out_len, peer, counter};
        int crc;
        if (coalesce_submit(ctx, rq, &crc)) {
            if (crc == BNK_OK) (void)tally_results(ctx, TALLY_DECAP_CHECK, result, wire->n, BNK_MEM_HOST);
            return crc;
        }
    }
    Guard g(ctx);
    if (g.rc) return g.rc;
    const int rc = wg_decap_impl(ctx, wire, out, result, out_len, peer, counter, &now_ns);
    if (rc == BNK_OK) return tally_results(ctx, TALLY_DECAP_CHECK, result, wire->n, wire->mem);
    return rc;
    BNK_API_CATCH(ctx)
}
