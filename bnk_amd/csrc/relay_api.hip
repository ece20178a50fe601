// C ABI entry point of the fused relay step (see include/bnkhip.h):
// open -> filter -> re-seal, composed from the AEAD and filter kernels plus
// the counter assignment of relay_kernels.hip.
#include "api_common.hpp"
#include "filter_host.hpp"

using namespace bnk;

// The chunked host route cuts a batch into at most this many parts.  Every part
// runs a dozen kernels that each need a full batch to fill the chip, so fewer,
// larger parts than the AEAD routes use: measured on 2^18 IMIX packets, 8 parts
// 5.6 ms, 16 parts 7.1 ms, one 6.2 ms (the link carries the input and, to keep
// the bytes between packets, the output arena up, and the output down).
constexpr uint32_t RELAY_CHUNKS = 8;

static int relay_impl(bnk_ctx *ctx, const bnk_batch *in, const uint32_t *peer_out, const uint64_t *ctr_base_out,
                      uint32_t n_peers_out, int64_t now_ns, const bnk_batch *out, uint8_t *verdict,
                      uint64_t *ctr_out)
{
    int rc = check_batch_common(ctx, in, "in");
    if (rc) return rc;
    rc = check_batch_common(ctx, out, "out");
    if (rc) return rc;
    if (in->mem != out->mem) return fail(ctx, BNK_E_INVAL, "in and out must use the same mem kind");
    const uint32_t n = in->n;
    if (n == 0) return BNK_OK;
    if (!peer_out || !ctr_base_out || !verdict || !ctr_out || n_peers_out == 0)
        return fail(ctx, BNK_E_INVAL, "null relay array");
    if (!ctx->d_keys[BNK_KEYS_RECV] || !ctx->d_keys[BNK_KEYS_SEND])
        return fail(ctx, BNK_E_STATE, "relay needs both key tables loaded");
    if (n_peers_out > ctx->n_keys[BNK_KEYS_SEND])
        return fail(ctx, BNK_E_RANGE, "n_peers_out exceeds the send key table");
    const bool host = in->mem == BNK_MEM_HOST;

    // ---- where everything lives on the device ----
    AeadArgs op{};
    op.spread_max = ctx->spread_max;
    op.keys = ctx->d_keys[BNK_KEYS_RECV];
    op.n_peers = ctx->n_keys[BNK_KEYS_RECV];
    op.status = ctx->d_status;
    op.counter0 = in->counter0;
    op.n = n;
    op.in_stride = in->stride;
    op.len = in->len;
    uint8_t *d_out = nullptr;
    const uint64_t *d_out_off = nullptr;
    const uint32_t *d_peer_out = nullptr;
    const uint64_t *d_ctr_base = nullptr;
    uint8_t *d_verdict = nullptr;
    uint64_t *d_ctr_out = nullptr;
    uint64_t plain_bytes = 0;
    uint64_t seal_out_limit = 0;
    Staged st;
    // direct route (small batches in pinned rings): the datagrams are fetched by
    // a copy kernel, the re-sealed ones written straight into the out ring, the
    // per-packet arrays sit in pinned staging
    bool direct = false;
    uint32_t plain_shift = 0; // keeps the plaintext scratch aligned with the fetched datagrams
    uint8_t *h_verdict = nullptr;
    uint64_t *h_ctr_out = nullptr;
    if (host && n <= DIRECT_MAX_PACKETS && n_peers_out <= DIRECT_MAX_PACKETS) {
        uint8_t *d_ring_in = ring_device_ptr(ctx, in->base, in->bytes);
        uint8_t *d_ring_out = ring_device_ptr(ctx, out->base, out->bytes);
        if (d_ring_in && d_ring_out) {
            Span sin, sout;
            rc = scan_host_layout(ctx, in, in, 0, &sin, "in");
            if (rc) return rc;
            rc = scan_host_layout(ctx, out, in, 0, &sout, "out");
            if (rc) return rc;
            rc = check_index_range(ctx, in->peer, n, ctx->n_keys[BNK_KEYS_RECV], "peer index", "the key table");
            if (rc) return rc;
            rc = check_index_range(ctx, peer_out, n, n_peers_out, "peer_out index", "n_peers_out");
            if (rc) return rc;
            if (sin.size() <= DIRECT_MAX_BYTES) {
                direct = true;
                HIPCHK(ctx, ctx->pin.reserve((size_t)n * 45 + (size_t)n_peers_out * 8 + 64));
                uint64_t *p_in_off = ctx->pin.as<uint64_t>(), *p_out_off = p_in_off + n, *p_ctr = p_out_off + n;
                h_ctr_out = p_ctr + n;
                uint64_t *p_base = h_ctr_out + n;
                uint32_t *p_lens = (uint32_t *)(p_base + n_peers_out), *p_peer = p_lens + n, *p_peer_out = p_peer + n;
                h_verdict = (uint8_t *)(p_peer_out + n);
                if (in->lens) { memcpy(p_lens, in->lens, (size_t)n * 4); op.lens = ctx->pin.dev(p_lens); }
                const uint32_t mis = (uint32_t)((uintptr_t)(d_ring_in + sin.lo) & 127u);
                if (aead_runs_spread(op)) {
                    // a wave per packet reads the ring itself (see aead_batch_host_direct)
                    op.in = d_ring_in + sin.lo;
                } else {
                    HIPCHK(ctx, ctx->in_arena.reserve(sin.size() + 160));
                    HIPCHK(ctx, launch_pull(d_ring_in + sin.lo, ctx->in_arena.as<uint8_t>() + mis, sin.size(), ctx->stream));
                    op.in = ctx->in_arena.as<uint8_t>() + mis;
                }
                if (in->offsets) {
                    for (uint32_t i = 0; i < n; i++) p_in_off[i] = in->offsets[i] - sin.lo;
                    op.in_off = ctx->pin.dev(p_in_off);
                }
                if (in->peer) { memcpy(p_peer, in->peer, (size_t)n * 4); op.peer = ctx->pin.dev(p_peer); }
                if (in->counters) { memcpy(p_ctr, in->counters, (size_t)n * 8); op.counters = ctx->pin.dev(p_ctr); }
                d_out = d_ring_out;
                if (out->offsets) { memcpy(p_out_off, out->offsets, (size_t)n * 8); d_out_off = ctx->pin.dev(p_out_off); }
                memcpy(p_peer_out, peer_out, (size_t)n * 4);
                memcpy(p_base, ctr_base_out, (size_t)n_peers_out * 8);
                d_peer_out = ctx->pin.dev(p_peer_out);
                d_ctr_base = ctx->pin.dev(p_base);
                d_verdict = ctx->pin.dev(h_verdict);
                d_ctr_out = ctx->pin.dev(h_ctr_out);
                plain_bytes = sin.size() + 128;
                plain_shift = mis;
            }
        }
    }
    // chunked route (large batches whose packets ascend through both arenas):
    // chunk k+1 goes up and chunk k-1 comes down while chunk k is opened,
    // filtered and re-sealed.  A packet's counter depends only on the packets
    // before it, so each chunk continues a running copy of the counter bases.
    HostPipe hp;
    bool chunked = false;
    const auto ct_ext = [in](uint32_t i) { return (uint64_t)(in->lens ? in->lens[i] : in->len); };
    if (host && !direct) {
        hp.ctx = ctx;
        hp.in = in;
        hp.out = out;
        hp.in_ext = hp.out_ext = ct_ext;
        hp.max_chunks = RELAY_CHUNKS;
        rc = hp.plan(in->lens ? 0 : in->len);
        if (rc != BNK_OK && rc != 1) return rc;
        chunked = rc == BNK_OK;
    }
    if (chunked) {
        rc = check_index_range(ctx, in->peer, n, ctx->n_keys[BNK_KEYS_RECV], "peer index", "the key table");
        if (rc) return rc;
        rc = check_index_range(ctx, peer_out, n, n_peers_out, "peer_out index", "n_peers_out");
        if (rc) return rc;
        HIPCHK(ctx, ctx->r_peer_out.reserve((size_t)n * 4));
        HIPCHK(ctx, ctx->r_ctr_base.reserve((size_t)n_peers_out * 8));
        HIPCHK(ctx, ctx->r_ctr_out.reserve((size_t)n * 8));
        HIPCHK(ctx, ctx->r_verdict.reserve(n));
        d_peer_out = ctx->r_peer_out.as<uint32_t>();
        d_ctr_base = ctx->r_ctr_base.as<uint64_t>();
        d_verdict = ctx->r_verdict.as<uint8_t>();
        d_ctr_out = ctx->r_ctr_out.as<uint64_t>();
        hp.add_result(verdict, d_verdict, 1);
        hp.add_result(ctr_out, d_ctr_out, 8);
        rc = hp.begin();
        if (rc) return rc;
        // the per-packet arrays go up whole, ahead of everything, on the compute stream
        auto up = [&](DevBuf *dst, const void *src, size_t bytes) -> hipError_t {
            hipError_t e = dst->reserve(bytes);
            if (e != hipSuccess) return e;
            return hipMemcpyAsync(dst->p, src, bytes, hipMemcpyHostToDevice, ctx->stream);
        };
        HIPCHK(ctx, up(&ctx->r_peer_out, peer_out, (size_t)n * 4));
        HIPCHK(ctx, up(&ctx->r_ctr_base, ctr_base_out, (size_t)n_peers_out * 8));
        if (in->lens) { HIPCHK(ctx, up(&ctx->lens, in->lens, (size_t)n * 4)); op.lens = ctx->lens.as<uint32_t>(); }
        if (in->peer) { HIPCHK(ctx, up(&ctx->peer, in->peer, (size_t)n * 4)); op.peer = ctx->peer.as<uint32_t>(); }
        if (in->counters) {
            HIPCHK(ctx, up(&ctx->counters, in->counters, (size_t)n * 8));
            op.counters = ctx->counters.as<uint64_t>();
        }
        op.in = hp.d_in;
        op.in_off = hp.d_in_off;
        d_out = hp.d_out;
        d_out_off = hp.d_out_off;
        plain_bytes = hp.sin.size();
    } else if (host && !direct) {
        // the re-sealed packet has the input's length: out_delta 0
        rc = stage_host(ctx, in, out, 0, ctx->n_keys[BNK_KEYS_RECV], &st);
        if (rc) return rc;
        rc = check_index_range(ctx, peer_out, n, n_peers_out, "peer_out index", "n_peers_out");
        if (rc) return rc;
        op.in = st.d_in;
        op.in_off = st.d_in_off;
        op.lens = st.d_lens;
        op.peer = st.d_peer;
        op.counters = st.d_counters;
        d_out = st.d_out;
        d_out_off = st.d_out_off;
        plain_bytes = st.sin.size();
        HIPCHK(ctx, ctx->r_peer_out.reserve((size_t)n * 4));
        HIPCHK(ctx, ctx->r_ctr_base.reserve((size_t)n_peers_out * 8));
        HIPCHK(ctx, ctx->r_ctr_out.reserve((size_t)n * 8));
        HIPCHK(ctx, ctx->r_verdict.reserve(n));
        HIPCHK(ctx, hipMemcpyAsync(ctx->r_peer_out.p, peer_out, (size_t)n * 4, hipMemcpyHostToDevice,
                                   ctx->stream));
        HIPCHK(ctx, hipMemcpyAsync(ctx->r_ctr_base.p, ctr_base_out, (size_t)n_peers_out * 8,
                                   hipMemcpyHostToDevice, ctx->stream));
        d_peer_out = ctx->r_peer_out.as<uint32_t>();
        d_ctr_base = ctx->r_ctr_base.as<uint64_t>();
        d_verdict = ctx->r_verdict.as<uint8_t>();
        d_ctr_out = ctx->r_ctr_out.as<uint64_t>();
    } else if (!host) {
        if (!in->offsets && !in->lens && (uint64_t)(n - 1) * in->stride + in->len > in->bytes)
            return fail(ctx, BNK_E_INVAL, "in: uniform layout exceeds the arena");
        if (!out->offsets && !in->lens && (uint64_t)(n - 1) * out->stride + in->len > out->bytes)
            return fail(ctx, BNK_E_INVAL, "out: uniform layout exceeds the arena");
        op.in = (const uint8_t *)in->base;
        op.in_off = in->offsets;
        op.lens = in->lens;
        op.peer = in->peer;
        op.counters = in->counters;
        d_out = (uint8_t *)out->base;
        d_out_off = out->offsets;
        plain_bytes = in->bytes;
        if (in->bytes == 0 || out->bytes == 0) return fail(ctx, BNK_E_INVAL, "arena size 0");
        if (in->offsets || in->lens || out->offsets) {
            // what the host cannot read the lanes check; the plaintext scratch mirrors the input arena
            op.in_limit = op.out_limit = in->bytes;
            seal_out_limit = out->bytes;
        }
        d_peer_out = peer_out;
        d_ctr_base = ctr_base_out;
        d_verdict = verdict;
        d_ctr_out = ctr_out;
    }
    HIPCHK(ctx, ctx->r_plain.reserve(plain_bytes + 16));
    HIPCHK(ctx, ctx->r_heads.reserve((size_t)n * 32));
    HIPCHK(ctx, ctx->r_auth.reserve(n));
    HIPCHK(ctx, ctx->r_pass.reserve(n));
    for (DevBuf *b : {&ctx->r_keys, &ctx->r_idx, &ctx->r_skeys, &ctx->r_sidx})
        HIPCHK(ctx, b->reserve((size_t)n * 4));
    const size_t tmp_bytes = relay_sort_tmp_bytes(n, n_peers_out);
    HIPCHK(ctx, ctx->r_tmp.reserve(tmp_bytes + 16));

    if (in->lens) {
        HIPCHK(ctx, ctx->order.reserve((size_t)n * 4));
        HIPCHK(ctx, ctx->hist.reserve(LEN_BINS * 4));
        HIPCHK(ctx, ctx->cursor.reserve(LEN_CURSOR_WORDS * 4));
    }
    FilterState *f = ctx->filter;
    uint8_t *d_pass = ctx->r_pass.as<uint8_t>();

    // packets [lo, hi): open -> filter -> verdicts and counters -> re-seal
    auto run = [&](uint32_t lo, uint32_t hi, bool advance) -> int {
        const uint32_t m = hi - lo;
        // ---- 1. open into the plaintext scratch (same offsets as the input) ----
        AeadArgs o = op;
        o.first = lo;
        o.n = m;
        o.out = ctx->r_plain.as<uint8_t>() + plain_shift;
        o.out_off = o.in_off;
        o.out_stride = in->stride;
        o.verdict = ctx->r_auth.as<uint8_t>();
        o.order = nullptr;
        if (o.lens && m > 64 && !aead_runs_spread(o)) {
            HIPCHK(ctx, launch_length_sort(o.lens + lo, m, 16, ctx->order.as<uint32_t>() + lo,
                                           ctx->hist.as<uint32_t>(), ctx->cursor.as<uint32_t>(), ctx->stream));
            o.order = ctx->order.as<uint32_t>() + lo;
        }
        // a lane-per-packet open leaves each plaintext's first 32 bytes in a record of
        // its own for the filter, which then need not touch the arena again
        const bool heads = f->enforce && !aead_runs_spread(o);
        if (heads) o.heads = ctx->r_heads.as<uint8_t>() + 32ull * lo;
        HIPCHK(ctx, launch_aead_open(o, ctx->stream));

        // ---- 2. CheckInbound on the authentic plaintexts ----
        if (!f->enforce) {
            HIPCHK(ctx, launch_fill_u8(d_pass + lo, m, 1, ctx->stream)); // filter.go:124-126
        } else {
            FilterArgs fa{};
            fa.pkts = o.out + (o.in_off ? 0 : (uint64_t)lo * in->stride);
            fa.off = o.in_off ? o.in_off + lo : nullptr;
            fa.lens = o.lens ? o.lens + lo : nullptr;
            fa.stride = in->stride;
            fa.len = in->len;
            fa.trim = 16; // lens count the tag
            fa.gate = o.verdict + lo;
            fa.heads = heads ? o.heads : nullptr;
            fa.order = heads ? o.order : nullptr;
            fa.verdict = d_pass + lo;
            fa.status = ctx->d_status;
            fa.now = now_ns;
            fa.n = m;
            fa.rules = f->ridx;
            fa.flows = f->flows;
            HIPCHK(ctx, launch_filter_check(fa, f->max_blocks, ctx->stream));
        }

        // ---- 3. verdicts and outbound counters ----
        HIPCHK(ctx, launch_relay_assign(o.verdict + lo, d_pass + lo, d_peer_out + lo, d_ctr_base, n_peers_out, m,
                                        ctx->r_keys.as<uint32_t>(), ctx->r_idx.as<uint32_t>(),
                                        ctx->r_skeys.as<uint32_t>(), ctx->r_sidx.as<uint32_t>(),
                                        ctx->r_tmp.p, tmp_bytes, d_verdict + lo, d_ctr_out + lo, ctx->d_status,
                                        advance, ctx->stream));

        // ---- 4. re-seal the survivors under the outbound keys ----
        AeadArgs se{};
        se.spread_max = ctx->spread_max;
        se.keys = ctx->d_keys[BNK_KEYS_SEND];
        se.n_peers = n_peers_out;
        se.status = ctx->d_status;
        se.first = lo;
        se.n = m;
        se.in = o.out;
        se.in_off = o.in_off;
        se.in_stride = in->stride;
        se.out = d_out;
        se.out_off = d_out_off;
        se.out_stride = out->stride;
        se.lens = o.lens;
        se.len = in->len;
        se.trim = 16;
        se.peer = d_peer_out;
        se.counters = d_ctr_out;
        se.in_limit = op.in_limit;
        se.out_limit = seal_out_limit;
        se.skip = d_verdict; // BNK_RELAY_OK is 0
        se.order = o.order;
        HIPCHK(ctx, launch_aead_seal(se, ctx->stream));
        return BNK_OK;
    };

    if (chunked) {
        rc = hp.open_gate();
        if (rc) return rc;
        for (uint32_t k = 0; k < hp.chunks; k++) {
            uint32_t lo, hi;
            if (!hp.range(k, &lo, &hi)) break;
            if ((rc = hp.upload(k)) || (rc = run(lo, hi, true)) || (rc = hp.download(k))) return rc;
        }
        rc = hp.finish();
        if (rc) return rc;
        uint32_t status = 0;
        rc = take_status(ctx, &status);
        if (rc) return rc;
        return status_to_rc(ctx, status);
    }
    rc = run(0, n, false);
    if (rc) return rc;
    if (!host) return BNK_OK;
    if (direct) {
        // both peer arrays were checked above: nothing comes back through the status word
        rc = wait_stream(ctx);
        if (rc) return rc;
        memcpy(verdict, h_verdict, n);
        memcpy(ctr_out, h_ctr_out, (size_t)n * 8);
        return BNK_OK;
    }

    HIPCHK(ctx, hipMemcpyAsync((uint8_t *)out->base + st.sout.lo, d_out, st.sout.size(),
                               hipMemcpyDeviceToHost, ctx->stream));
    HIPCHK(ctx, hipMemcpyAsync(verdict, d_verdict, n, hipMemcpyDeviceToHost, ctx->stream));
    HIPCHK(ctx, hipMemcpyAsync(ctr_out, d_ctr_out, (size_t)n * 8, hipMemcpyDeviceToHost, ctx->stream));
    uint32_t status = 0;
    rc = take_status(ctx, &status);
    if (rc) return rc;
    return status_to_rc(ctx, status);
}

extern "C" int bnk_relay_fused_batch(bnk_ctx *ctx, const bnk_batch *in, const uint32_t *peer_out,
                                     const uint64_t *ctr_base_out, uint32_t n_peers_out,
                                     int64_t now_ns, const bnk_batch *out, uint8_t *verdict,
                                     uint64_t *ctr_out)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    const int rc = relay_impl(ctx, in, peer_out, ctr_base_out, n_peers_out, now_ns, out, verdict, ctr_out);
    // (every packet relayed was opened and re-sealed on the way)
    if (rc == BNK_OK) return tally_results(ctx, TALLY_RELAY, verdict, in->n, in->mem);
    return rc;
    BNK_API_CATCH(ctx)
}
