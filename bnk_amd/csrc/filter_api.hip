// C ABI entry points of the packet filter (see include/bnkhip.h).
#include <stdio.h>

#include "api_common.hpp"
#include "filter_host.hpp"
#include "netmap_json.hpp"

using namespace bnk;

namespace bnk {

static hipError_t flow_table_alloc(uint32_t cap, DevBuf &slots, DevBuf &counters, DevBuf &present,
                                   DevBuf &present_small, FlowTableDev &ft, hipStream_t s)
{
    const size_t n = (size_t)cap * FLOW_REGIONS;
    // the table is kept under half full, so 8 * cap bits see at most one key per 16 bits
    const uint32_t bits = cap * 8u;
    hipError_t e;
    if ((e = slots.reserve(n * sizeof(FlowSlotMem))) != hipSuccess) return e;
    if ((e = counters.reserve(FLOW_COUNTERS * 4)) != hipSuccess) return e;
    if ((e = present.reserve(bits / 8)) != hipSuccess) return e;
    if ((e = present_small.reserve(SMALL_BITS / 8)) != hipSuccess) return e;
    ft.present_small = present_small.as<uint32_t>();
    ft.small_ok = 1;
    ft.slots = slots.as<FlowSlotMem>();
    ft.counters = counters.as<uint32_t>();
    ft.present = present.as<uint32_t>();
    ft.cap = cap;
    ft.present_mask = bits - 1u;
    if ((e = launch_flow_clear(ft.slots, (uint32_t)n, s)) != hipSuccess) return e;
    if ((e = launch_fill_u32(ft.present, bits / 32, 0, s)) != hipSuccess) return e;
    if ((e = launch_fill_u32(ft.present_small, SMALL_BITS / 32, 0, s)) != hipSuccess) return e;
    return launch_fill_u32(ft.counters, FLOW_COUNTERS, 0, s);
}

static hipError_t upload_rule_index(FilterState *f, const HostRuleIndex &h, hipStream_t s)
{
    hipError_t e;
    const size_t nb = h.bounds.size();
    if ((e = f->bounds.reserve(std::max<size_t>(nb, 1) * 4)) != hipSuccess) return e;
    if ((e = f->jump.reserve((JUMP_BUCKETS + 2) * 2)) != hipSuccess) return e;
    if ((e = f->ranges.reserve(std::max<size_t>(h.ranges.size(), 1) * 4)) != hipSuccess) return e;
    if ((e = f->wide.reserve(std::max<size_t>(h.wide.size(), 1) * 16)) != hipSuccess) return e;
    if ((e = hipMemcpyAsync(f->bounds.p, h.bounds.data(), nb * 4, hipMemcpyHostToDevice, s)) != hipSuccess)
        return e;
    if (!h.jump.empty() &&
        (e = hipMemcpyAsync(f->jump.p, h.jump.data(), h.jump.size() * 2, hipMemcpyHostToDevice, s)) !=
            hipSuccess)
        return e;
    if (!h.ranges.empty() &&
        (e = hipMemcpyAsync(f->ranges.p, h.ranges.data(), h.ranges.size() * 4, hipMemcpyHostToDevice,
                            s)) != hipSuccess)
        return e;
    if (!h.wide.empty() &&
        (e = hipMemcpyAsync(f->wide.p, h.wide.data(), h.wide.size() * 16, hipMemcpyHostToDevice, s)) !=
            hipSuccess)
        return e;
    // the host vectors die with the caller's frame
    if ((e = hipStreamSynchronize(s)) != hipSuccess) return e;
    f->ridx.bounds = f->bounds.as<uint32_t>();
    f->ridx.jump = h.jump.empty() ? nullptr : f->jump.as<uint16_t>();
    f->ridx.jump_lo = h.jump_lo;
    f->ridx.jump_shift = h.jump_shift;
    f->ridx.ranges = f->ranges.as<uint32_t>();
    f->ridx.wide = f->wide.as<uint4>();
    f->ridx.n_bounds = (uint32_t)nb;
    f->ridx.n_wide = (uint32_t)h.wide.size();
    uint32_t step = 0;
    if (nb >= 2) {
        step = 1;
        while ((size_t)step * 2 <= nb - 1) step *= 2;
    }
    f->ridx.top_step = step;
    return hipSuccess;
}

FilterState *filter_create(hipStream_t s, int cu_count)
{
    FilterState *f = new (std::nothrow) FilterState;
    if (!f) return nullptr;
    f->max_blocks = (uint32_t)std::max(cu_count, 1) * 8u;
    HostRuleIndex h;
    std::string err;
    build_rule_index(nullptr, 0, h, err);
    if (flow_table_alloc(FLOW_CAP_INITIAL, f->slots, f->counters, f->present, f->present_small, f->flows, s) != hipSuccess ||
        upload_rule_index(f, h, s) != hipSuccess) {
        filter_destroy(f);
        return nullptr;
    }
    return f;
}

void filter_destroy(FilterState *f)
{
    if (!f) return;
    f->release();
    delete f;
}

} // namespace bnk

namespace bnk {

// Makes room for n_new more distinct flows: open addressing stays below half
// full per region, growing (and dropping tombstones) when it would not.
int flows_reserve(bnk_ctx *ctx, uint32_t n_new)
{
    FilterState *f = ctx->filter;
    const uint64_t half = f->flows.cap / 2;
    if (f->claimed_upper + n_new <= half) {
        f->claimed_upper += n_new;
        f->flows.small_ok = f->claimed_upper <= SMALL_KEYS_MAX;
        return BNK_OK;
    }
    uint32_t c[FLOW_COUNTERS];
    HIPCHK(ctx, hipMemcpyAsync(c, f->flows.counters, sizeof c, hipMemcpyDeviceToHost, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    f->claimed_upper = c[FLOW_CLAIMED];
    if (f->claimed_upper + n_new <= half) {
        f->claimed_upper += n_new;
        f->flows.small_ok = f->claimed_upper <= SMALL_KEYS_MAX;
        return BNK_OK;
    }
    uint64_t need = 4ull * ((uint64_t)c[FLOW_LIVE] + n_new); // at most a quarter full afterwards
    uint64_t cap = FLOW_CAP_INITIAL;
    while (cap < need) cap *= 2;
    if (cap > FLOW_CAP_MAX) return fail(ctx, BNK_E_NOMEM, "flow table would exceed its maximum size");
    DevBuf ns, nc, np, nps;
    FlowTableDev nt{};
    hipError_t e = flow_table_alloc((uint32_t)cap, ns, nc, np, nps, nt, ctx->stream);
    if (e == hipSuccess)
        e = launch_flow_rehash(f->flows, nt, ctx->d_status, f->max_blocks, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        ns.release(); nc.release(); np.release(); nps.release();
        return fail_hip(ctx, "flow table growth", e);
    }
    f->slots.release(); f->counters.release(); f->present.release(); f->present_small.release();
    f->slots = ns; f->counters = nc; f->present = np; f->present_small = nps;
    f->flows = nt;
    f->claimed_upper = (uint64_t)c[FLOW_LIVE] + n_new;
    f->flows.small_ok = f->claimed_upper <= SMALL_KEYS_MAX;
    return BNK_OK;
}

} // namespace bnk

namespace {

// The filter reads at most the first 64 bytes of a packet (IPv4 header of up
// to 60 bytes, then 4 port bytes): host packets are gathered at a 64-byte
// stride into pinned staging and only that is uploaded.
constexpr uint32_t HDR_BYTES = 64;

// Small batches skip the upload: the kernel reads the pinned staging in place
// and writes its verdicts there (*h_verdict, null when the batch was uploaded).
template <class GetPtr, class GetLen>
int stage_headers(bnk_ctx *ctx, uint32_t n, GetPtr ptr_of, GetLen len_of, FilterArgs *a,
                  uint8_t **h_verdict)
{
    const size_t hdr_bytes = (size_t)n * HDR_BYTES, len_bytes = (size_t)n * 4;
    HIPCHK(ctx, ctx->pin.reserve(hdr_bytes + len_bytes + n));
    uint8_t *hp = ctx->pin.as<uint8_t>();
    uint32_t *hl = reinterpret_cast<uint32_t *>(hp + hdr_bytes);
    for (uint32_t i = 0; i < n; i++) {
        const uint32_t len = len_of(i);
        hl[i] = len;
        const uint32_t c = len < HDR_BYTES ? len : HDR_BYTES;
        if (c) memcpy(hp + (size_t)i * HDR_BYTES, ptr_of(i), c);
    }
    a->off = nullptr;
    a->stride = HDR_BYTES;
    if (n <= DIRECT_MAX_PACKETS) {
        a->pkts = ctx->pin.dev(hp);
        a->lens = ctx->pin.dev(hl);
        *h_verdict = hp + hdr_bytes + len_bytes;
        return BNK_OK;
    }
    *h_verdict = nullptr;
    HIPCHK(ctx, ctx->in_arena.reserve(hdr_bytes));
    HIPCHK(ctx, ctx->lens.reserve(len_bytes));
    HIPCHK(ctx, hipMemcpyAsync(ctx->in_arena.p, hp, hdr_bytes, hipMemcpyHostToDevice, ctx->stream));
    HIPCHK(ctx, hipMemcpyAsync(ctx->lens.p, hl, len_bytes, hipMemcpyHostToDevice, ctx->stream));
    a->pkts = ctx->in_arena.as<uint8_t>();
    a->lens = ctx->lens.as<uint32_t>();
    return BNK_OK;
}

// Runs a staged host batch and brings the verdicts (check) or the overflow
// flag (note) back.
int run_staged(bnk_ctx *ctx, bool check, FilterArgs &a, uint8_t *h_verdict, uint8_t *verdict)
{
    FilterState *f = ctx->filter;
    if (!check) {
        HIPCHK(ctx, launch_filter_note(a, f->max_blocks, f->claimed_upper > 4096, ctx->stream));
    } else if (h_verdict) {
        // CheckInbound reports nothing through the status word
        a.verdict = ctx->pin.dev(h_verdict);
        HIPCHK(ctx, launch_filter_check(a, f->max_blocks, ctx->stream));
        if (int wrc = wait_stream(ctx)) return wrc;
        memcpy(verdict, h_verdict, a.n);
        return BNK_OK;
    } else {
        HIPCHK(ctx, ctx->verdict.reserve(a.n));
        a.verdict = ctx->verdict.as<uint8_t>();
        HIPCHK(ctx, launch_filter_check(a, f->max_blocks, ctx->stream));
        HIPCHK(ctx, hipMemcpyAsync(verdict, a.verdict, a.n, hipMemcpyDeviceToHost, ctx->stream));
    }
    uint32_t status = 0;
    int rc = take_status(ctx, &status, !check);
    if (rc) return rc;
    return status_to_rc(ctx, status);
}

void base_args(bnk_ctx *ctx, uint32_t n, int64_t now_ns, FilterArgs *a)
{
    *a = FilterArgs{};
    a->n = n;
    a->now = now_ns;
    a->status = ctx->d_status;
    a->rules = ctx->filter->ridx;
    a->flows = ctx->filter->flows;
}

int check_device_layout(bnk_ctx *ctx, const bnk_batch *b)
{
    if (b->n && b->bytes == 0) return fail(ctx, BNK_E_INVAL, "pkts: arena size 0");
    if (!b->offsets && !b->lens && b->n &&
        (uint64_t)(b->n - 1) * b->stride + b->len > b->bytes)
        return fail(ctx, BNK_E_INVAL, "pkts: uniform layout exceeds the arena");
    return BNK_OK;
}

// *counted (check only): the launch has counted its own verdicts (bnk_counters_get)
int filter_batch(bnk_ctx *ctx, bool check, const bnk_batch *pkts, int64_t now_ns, uint8_t *verdict,
                 bool *counted = nullptr)
{
    int rc = check_batch_common(ctx, pkts, "pkts");
    if (rc) return rc;
    const uint32_t n = pkts->n;
    if (n == 0) return BNK_OK;
    if (check && !verdict) return fail(ctx, BNK_E_INVAL, "null verdict array");
    FilterState *f = ctx->filter;
    if (!f->enforce) {
        // filter.go:124-126 / :192-194
        if (!check) return BNK_OK;
        if (pkts->mem == BNK_MEM_HOST) memset(verdict, 1, n);
        else HIPCHK(ctx, launch_fill_u8(verdict, n, 1, ctx->stream));
        return BNK_OK;
    }
    if (!check) {
        rc = flows_reserve(ctx, n);
        if (rc) return rc;
    }
    FilterArgs a;
    base_args(ctx, n, now_ns, &a);
    if (pkts->mem == BNK_MEM_DEVICE) {
        rc = check_device_layout(ctx, pkts);
        if (rc) return rc;
        a.pkts = (const uint8_t *)pkts->base;
        a.off = pkts->offsets;
        a.lens = pkts->lens;
        a.stride = pkts->stride;
        a.len = pkts->len;
        a.verdict = verdict;
        if (pkts->offsets || pkts->lens) a.limit = pkts->bytes; // the lanes check what the host cannot read
        if (check && counted && ctx->tally_on.load(std::memory_order_relaxed)) {
            a.tally = reinterpret_cast<unsigned long long *>(ctx->d_tally);
            *counted = true;
        }
        HIPCHK(ctx, check ? launch_filter_check(a, f->max_blocks, ctx->stream)
                          : launch_filter_note(a, f->max_blocks, f->claimed_upper > 4096, ctx->stream));
        return BNK_OK;
    }
    Span span;
    rc = scan_host_layout(ctx, pkts, pkts, 0, &span, "pkts");
    if (rc) return rc;
    const uint8_t *base = (const uint8_t *)pkts->base;
    uint8_t *h_verdict = nullptr;
    rc = stage_headers(
        ctx, n, [&](uint32_t i) { return base + pkt_off(pkts, i); },
        [&](uint32_t i) { return pkts->lens ? pkts->lens[i] : pkts->len; }, &a, &h_verdict);
    if (rc) return rc;
    return run_staged(ctx, check, a, h_verdict, verdict);
}

int filter_ptrs(bnk_ctx *ctx, bool check, const uint8_t *const *pkts, const uint32_t *lens,
                uint32_t n, int64_t now_ns, uint8_t *verdict)
{
    if (n == 0) return BNK_OK;
    if (!pkts || !lens) return fail(ctx, BNK_E_INVAL, "null packet list");
    if (check && !verdict) return fail(ctx, BNK_E_INVAL, "null verdict array");
    for (uint32_t i = 0; i < n; i++)
        if (lens[i] && !pkts[i]) return fail(ctx, BNK_E_INVAL, "null packet pointer");
    FilterState *f = ctx->filter;
    if (!f->enforce) {
        if (check) memset(verdict, 1, n);
        return BNK_OK;
    }
    int rc;
    if (!check) {
        rc = flows_reserve(ctx, n);
        if (rc) return rc;
    }
    FilterArgs a;
    base_args(ctx, n, now_ns, &a);
    uint8_t *h_verdict = nullptr;
    rc = stage_headers(
        ctx, n, [&](uint32_t i) { return pkts[i]; }, [&](uint32_t i) { return lens[i]; }, &a, &h_verdict);
    if (rc) return rc;
    return run_staged(ctx, check, a, h_verdict, verdict);
}

} // namespace

extern "C" {

int bnk_filter_set_rules(bnk_ctx *ctx, const bnk_rule *rules, uint32_t n)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (n && !rules) return fail(ctx, BNK_E_INVAL, "null rule array");
    HostRuleIndex h;
    std::string err;
    if (!build_rule_index(rules, n, h, err)) return fail(ctx, BNK_E_INVAL, err);
    // work already queued may still read the old tables
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, upload_rule_index(ctx->filter, h, ctx->stream));
    ctx->filter->enforce = true;
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_rules_from_netmap_json(const char *json, size_t len, bnk_rule *out, uint32_t cap,
                               uint32_t *n_tuples, int *filter_enabled, char *err, size_t err_cap)
{
    BNK_API_TRY
    if (err && err_cap) err[0] = '\0';
    if (!json || !n_tuples || !filter_enabled || (cap && !out)) return BNK_E_INVAL;
    NetmapFilter nf;
    std::string msg;
    if (!NetmapJson(json, len).parse(nf, msg)) {
        if (err && err_cap) {
            strncpy(err, msg.c_str(), err_cap - 1);
            err[err_cap - 1] = '\0';
        }
        return BNK_E_INVAL;
    }
    *n_tuples = (uint32_t)nf.tuples.size();
    *filter_enabled = nf.filter_enabled ? 1 : 0;
    const size_t k = std::min<size_t>(cap, nf.tuples.size());
    if (k) memcpy(out, nf.tuples.data(), k * sizeof(bnk_rule));
    return BNK_OK;
    }
    catch (const std::bad_alloc &) {
        if (err && err_cap) snprintf(err, err_cap, "out of host memory");
        return BNK_E_NOMEM;
    }
    catch (...) {
        if (err && err_cap) snprintf(err, err_cap, "unexpected C++ exception inside the library");
        return BNK_E_HIP;
    }
}

int bnk_filter_apply_netmap_json(bnk_ctx *ctx, const char *json, size_t len)
{
    BNK_API_TRY
    if (!ctx) return fail(nullptr, BNK_E_INVAL, "null context");
    if (!json) return fail(ctx, BNK_E_INVAL, "null document");
    NetmapFilter nf;
    std::string msg;
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        if (!NetmapJson(json, len).parse(nf, msg)) return fail(ctx, BNK_E_INVAL, msg);
    }
    // engine.go:279-283
    if (nf.filter_enabled) return bnk_filter_set_rules(ctx, nf.tuples.data(), (uint32_t)nf.tuples.size());
    return bnk_filter_set_allow_all(ctx);
    BNK_API_CATCH(ctx)
}

int bnk_filter_set_allow_all(bnk_ctx *ctx)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HostRuleIndex h;
    std::string err;
    build_rule_index(nullptr, 0, h, err);
    HIPCHK(ctx, upload_rule_index(ctx->filter, h, ctx->stream));
    ctx->filter->enforce = false;
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_filter_note_outbound_batch(bnk_ctx *ctx, const bnk_batch *pkts, int64_t now_ns)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    return filter_batch(ctx, false, pkts, now_ns, nullptr);
    BNK_API_CATCH(ctx)
}

int bnk_filter_check_inbound_batch(bnk_ctx *ctx, const bnk_batch *pkts, int64_t now_ns,
                                   uint8_t *verdict)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    bool counted = false;
    const int rc = filter_batch(ctx, true, pkts, now_ns, verdict, &counted);
    if (rc == BNK_OK && pkts && !counted) return tally_results(ctx, TALLY_CHECK, verdict, pkts->n, pkts->mem);
    return rc;
    BNK_API_CATCH(ctx)
}

int bnk_filter_note_outbound_ptrs(bnk_ctx *ctx, const uint8_t *const *pkts, const uint32_t *lens,
                                  uint32_t n, int64_t now_ns)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    return filter_ptrs(ctx, false, pkts, lens, n, now_ns, nullptr);
    BNK_API_CATCH(ctx)
}

int bnk_filter_check_inbound_ptrs(bnk_ctx *ctx, const uint8_t *const *pkts, const uint32_t *lens,
                                  uint32_t n, int64_t now_ns, uint8_t *verdict)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    const int rc = filter_ptrs(ctx, true, pkts, lens, n, now_ns, verdict);
    if (rc == BNK_OK) return tally_results(ctx, TALLY_CHECK, verdict, n, BNK_MEM_HOST);
    return rc;
    BNK_API_CATCH(ctx)
}

int bnk_filter_flow_count(bnk_ctx *ctx, uint32_t *count)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!count) return fail(ctx, BNK_E_INVAL, "null count");
    uint32_t c[FLOW_COUNTERS];
    HIPCHK(ctx, hipMemcpyAsync(c, ctx->filter->flows.counters, sizeof c, hipMemcpyDeviceToHost,
                               ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    *count = c[FLOW_LIVE];
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

int bnk_filter_flow_dump(bnk_ctx *ctx, uint64_t *key, uint8_t *proto, int64_t *expiry_ns,
                         uint32_t cap, uint32_t *count)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!count || (cap && (!key || !proto || !expiry_ns))) return fail(ctx, BNK_E_INVAL, "null output");
    const FlowTableDev &ft = ctx->filter->flows;
    const size_t slots = (size_t)ft.cap * FLOW_REGIONS;
    std::vector<FlowSlotMem> hs(slots);
    HIPCHK(ctx, hipMemcpyAsync(hs.data(), ft.slots, slots * sizeof(FlowSlotMem), hipMemcpyDeviceToHost,
                               ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    static const uint8_t class_proto[3] = {1, 6, 17};
    uint32_t k = 0;
    for (size_t idx = 0; idx < slots && k < cap; idx++) {
        if (hs[idx].key == 0 || hs[idx].exp == FLOW_TOMB) continue;
        const uint32_t region = (uint32_t)(idx / ft.cap);
        const uint64_t w = hs[idx].key;
        const uint64_t remote = ((uint64_t)(region & 1u) << 31) | ((w >> 32) & 0x7FFFFFFFu);
        key[k] = remote << 32 | (w & 0xFFFFFFFFu);
        proto[k] = class_proto[region >> 1];
        expiry_ns[k] = hs[idx].exp;
        k++;
    }
    *count = k;
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

} // extern "C"
