// C ABI of libbnkhip.so (see include/bnkhip.h): argument checking, staging of
// host batches through the context's device buffers, kernel launches.
#include "api_common.hpp"
#include "filter_host.hpp"

using namespace bnk;

namespace {

// Chunked form of a host batch: while chunk k is computed, chunk k+1 is on its
// way up and chunk k-1 on its way down (the link is full duplex).  Needs
// packets laid out in ascending, non-overlapping order in both arenas, so that
// a run of consecutive packets is one contiguous span.  Returns 1 when the
// batch does not qualify and the caller should take the single-shot route.
constexpr uint32_t PIPE_MAX_CHUNKS = 16;
constexpr uint64_t PIPE_MIN_CHUNK_BYTES = 4ull << 20;

bool ascending_layout(const bnk_batch *lay, const bnk_batch *src, int delta)
{
    const uint32_t n = src->n;
    if (!lay->offsets) {
        if (!src->lens) return (int64_t)src->len + delta <= (int64_t)lay->stride;
        for (uint32_t i = 0; i < n; i++)
            if ((int64_t)src->lens[i] + delta > (int64_t)lay->stride) return false;
        return true;
    }
    uint64_t end = 0;
    for (uint32_t i = 0; i < n; i++) {
        const uint64_t off = lay->offsets[i];
        int64_t len = (int64_t)(src->lens ? src->lens[i] : src->len) + delta;
        if (len < 0) len = 0;
        if (off < end) return false;
        end = off + (uint64_t)len;
    }
    return true;
}

int ensure_pipe(bnk_ctx *ctx, uint32_t chunks)
{
    if (!ctx->s_up) HIPCHK(ctx, hipStreamCreateWithFlags(&ctx->s_up, hipStreamNonBlocking));
    if (!ctx->s_down) HIPCHK(ctx, hipStreamCreateWithFlags(&ctx->s_down, hipStreamNonBlocking));
    while (ctx->ev_up.size() < chunks + 1u) {
        hipEvent_t e;
        HIPCHK(ctx, hipEventCreateWithFlags(&e, hipEventDisableTiming));
        ctx->ev_up.push_back(e);
    }
    while (ctx->ev_done.size() < chunks) {
        hipEvent_t e;
        HIPCHK(ctx, hipEventCreateWithFlags(&e, hipEventDisableTiming));
        ctx->ev_done.push_back(e);
    }
    return BNK_OK;
}

int aead_batch_host_chunked(bnk_ctx *ctx, bool open, const bnk_batch *in, const bnk_batch *out,
                            uint8_t *verdict, AeadArgs a)
{
    const uint32_t n = in->n;
    const int out_delta = open ? -16 : 16;
    Span sin, sout;
    int rc = scan_host_layout(ctx, in, in, 0, &sin, "in");
    if (rc) return rc;
    rc = scan_host_layout(ctx, out, in, out_delta, &sout, "out");
    if (rc) return rc;
    const uint32_t by_bytes = (uint32_t)std::min<uint64_t>(sin.size() / PIPE_MIN_CHUNK_BYTES, PIPE_MAX_CHUNKS);
    if (by_bytes < 2 || n < 2u * 64u) return 1;
    if (!ascending_layout(in, in, 0) || !ascending_layout(out, in, out_delta)) return 1;
    if (in->peer)
        for (uint32_t i = 0; i < n; i++)
            if (in->peer[i] >= a.n_peers)
                return fail(ctx, BNK_E_RANGE, "peer index " + std::to_string(in->peer[i]) + " beyond the key table");
    const uint32_t chunks = by_bytes;
    const uint32_t per = ((n + chunks - 1u) / chunks + 63u) & ~63u; // whole waves per chunk
    rc = ensure_pipe(ctx, chunks);
    if (rc) return rc;
    const bool in_place = same_layout(in, out);
    if (in_place) {
        sin.add(sout.lo, sout.hi);
        sout = sin;
    }
    // a uniform output layout comes back row by row, so the gaps between its
    // packets never need to be on the device; any other layout first takes the
    // host's bytes up so that they come back unchanged
    const bool rows_down = !in_place && !out->offsets && !in->lens;
    // offsets staging, then verdict staging: a download into pageable memory
    // would make the runtime wait for it and stall the pipeline
    HIPCHK(ctx, ctx->pin.reserve((size_t)n * 17 + 64));
    uint8_t *h_verdict = ctx->pin.as<uint8_t>() + (size_t)n * 16;
    HIPCHK(ctx, ctx->in_arena.reserve(sin.size() + 16));
    uint8_t *d_in = ctx->in_arena.as<uint8_t>(), *d_out = d_in;
    if (!in_place) {
        HIPCHK(ctx, ctx->out_arena.reserve(sout.size() + 16));
        d_out = ctx->out_arena.as<uint8_t>();
    }
    // per-packet arrays go up whole, ahead of everything, on the compute stream
    rc = upload_offsets(ctx, in, n, sin.lo, &ctx->off_in, 0, &a.in_off);
    if (rc) return rc;
    if (in_place) a.out_off = a.in_off;
    else {
        rc = upload_offsets(ctx, out, n, sout.lo, &ctx->off_out, (size_t)n * 8, &a.out_off);
        if (rc) return rc;
    }
    auto up = [&](DevBuf *dst, const void *src, size_t bytes) -> hipError_t {
        hipError_t e = dst->reserve(bytes);
        if (e != hipSuccess) return e;
        return hipMemcpyAsync(dst->p, src, bytes, hipMemcpyHostToDevice, ctx->stream);
    };
    if (in->lens) {
        HIPCHK(ctx, up(&ctx->lens, in->lens, (size_t)n * 4));
        a.lens = ctx->lens.as<uint32_t>();
        HIPCHK(ctx, ctx->order.reserve((size_t)n * 4));
        HIPCHK(ctx, ctx->hist.reserve(LEN_BINS * 4));
        HIPCHK(ctx, ctx->cursor.reserve(LEN_BINS * 4));
    }
    if (in->peer) {
        HIPCHK(ctx, up(&ctx->peer, in->peer, (size_t)n * 4));
        a.peer = ctx->peer.as<uint32_t>();
    }
    if (in->counters) {
        HIPCHK(ctx, up(&ctx->counters, in->counters, (size_t)n * 8));
        a.counters = ctx->counters.as<uint64_t>();
    }
    if (open) {
        HIPCHK(ctx, ctx->verdict.reserve(n));
        a.verdict = ctx->verdict.as<uint8_t>();
    }
    a.in = d_in;
    a.out = d_out;
    HIPCHK(ctx, hipEventRecord(ctx->ev_up[chunks], ctx->stream));
    HIPCHK(ctx, hipStreamWaitEvent(ctx->s_up, ctx->ev_up[chunks], 0));

    auto pkt_len = [&](uint32_t i) { return (uint64_t)(in->lens ? in->lens[i] : in->len); };
    const uint8_t *h_in = (const uint8_t *)in->base;
    uint8_t *h_out = (uint8_t *)out->base;
    for (uint32_t k = 0; k < chunks; k++) {
        const uint32_t lo = k * per, hi = std::min(n, lo + per);
        if (lo >= hi) break;
        // spans of this run of packets, relative to the staged arenas
        const uint64_t i0 = pkt_off(in, lo), i1 = pkt_off(in, hi - 1) + pkt_len(hi - 1);
        const int64_t last_out = std::max<int64_t>((int64_t)pkt_len(hi - 1) + out_delta, 0);
        uint64_t o0 = pkt_off(out, lo), o1 = pkt_off(out, hi - 1) + (uint64_t)last_out;
        uint64_t u0 = i0, u1 = i1;
        if (in_place) {
            u0 = std::min(i0, o0);
            u1 = std::max(i1, o1);
            o0 = u0;
            o1 = u1;
        }
        if (u1 > u0)
            HIPCHK(ctx, hipMemcpyAsync(d_in + (u0 - sin.lo), h_in + u0, u1 - u0, hipMemcpyHostToDevice, ctx->s_up));
        if (!in_place && !rows_down && o1 > o0)
            HIPCHK(ctx, hipMemcpyAsync(d_out + (o0 - sout.lo), h_out + o0, o1 - o0, hipMemcpyHostToDevice, ctx->s_up));
        HIPCHK(ctx, hipEventRecord(ctx->ev_up[k], ctx->s_up));
        HIPCHK(ctx, hipStreamWaitEvent(ctx->stream, ctx->ev_up[k], 0));
        AeadArgs c = a;
        c.first = lo;
        c.n = hi - lo;
        if (a.lens && c.n > 64) {
            HIPCHK(ctx, launch_length_sort(a.lens + lo, c.n, open ? 16 : 0, ctx->order.as<uint32_t>() + lo,
                                           ctx->hist.as<uint32_t>(), ctx->cursor.as<uint32_t>(), ctx->stream));
            c.order = ctx->order.as<uint32_t>() + lo;
        }
        HIPCHK(ctx, open ? launch_aead_open(c, ctx->stream) : launch_aead_seal(c, ctx->stream));
        HIPCHK(ctx, hipEventRecord(ctx->ev_done[k], ctx->stream));
        HIPCHK(ctx, hipStreamWaitEvent(ctx->s_down, ctx->ev_done[k], 0));
        if (rows_down) {
            const uint64_t width = (uint64_t)std::max<int64_t>((int64_t)in->len + out_delta, 0);
            if (width)
                HIPCHK(ctx, hipMemcpy2DAsync(h_out + o0, out->stride, d_out + (o0 - sout.lo), out->stride, width,
                                             hi - lo, hipMemcpyDeviceToHost, ctx->s_down));
        } else if (o1 > o0) {
            HIPCHK(ctx, hipMemcpyAsync(h_out + o0, d_out + (o0 - sout.lo), o1 - o0, hipMemcpyDeviceToHost, ctx->s_down));
        }
        if (open)
            HIPCHK(ctx, hipMemcpyAsync(h_verdict + lo, a.verdict + lo, hi - lo, hipMemcpyDeviceToHost, ctx->s_down));
    }
    HIPCHK(ctx, hipStreamSynchronize(ctx->s_down));
    if (open) memcpy(verdict, h_verdict, n);
    uint32_t status = 0;
    rc = take_status(ctx, &status);
    if (rc) return rc;
    return status_to_rc(ctx, status);
}

int aead_batch(bnk_ctx *ctx, bool open, const bnk_batch *in, const bnk_batch *out,
               uint8_t *verdict)
{
    int rc = check_batch_common(ctx, in, "in");
    if (rc) return rc;
    rc = check_batch_common(ctx, out, "out");
    if (rc) return rc;
    if (in->mem != out->mem) return fail(ctx, BNK_E_INVAL, "in and out must use the same mem kind");
    const uint32_t n = in->n;
    if (n == 0) return BNK_OK;
    if (open && !verdict) return fail(ctx, BNK_E_INVAL, "null verdict array");
    const int which = open ? BNK_KEYS_RECV : BNK_KEYS_SEND;
    if (!ctx->d_keys[which] || ctx->n_keys[which] == 0)
        return fail(ctx, BNK_E_STATE, open ? "no receive keys loaded" : "no send keys loaded");
    if (!in->peer && ctx->n_keys[which] < 1) return fail(ctx, BNK_E_RANGE, "empty key table");

    AeadArgs a{};
    a.keys = ctx->d_keys[which];
    a.n_peers = ctx->n_keys[which];
    a.status = ctx->d_status;
    a.counter0 = in->counter0;
    a.n = n;
    a.in_stride = in->stride;
    a.out_stride = out->stride;
    a.len = in->len;

    if (in->mem == BNK_MEM_DEVICE) {
        // Device batches cannot be walked on the host; check what is uniform.
        if (!in->offsets && !in->lens &&
            ((uint64_t)(n - 1) * in->stride + in->len > in->bytes))
            return fail(ctx, BNK_E_INVAL, "in: uniform layout exceeds the arena");
        if (!out->offsets && !in->lens) {
            const int64_t ol = (int64_t)in->len + (open ? -16 : 16);
            if ((uint64_t)(n - 1) * out->stride + (uint64_t)std::max<int64_t>(ol, 0) > out->bytes)
                return fail(ctx, BNK_E_INVAL, "out: uniform layout exceeds the arena");
        }
        a.in = (const uint8_t *)in->base;
        a.out = (uint8_t *)out->base;
        a.in_off = in->offsets;
        a.out_off = out->offsets;
        a.lens = in->lens;
        a.peer = in->peer;
        a.counters = in->counters;
        a.verdict = verdict;
        rc = maybe_sort(ctx, a.lens, n, open ? 16 : 0, &a.order);
        if (rc) return rc;
        HIPCHK(ctx, open ? launch_aead_open(a, ctx->stream) : launch_aead_seal(a, ctx->stream));
        return BNK_OK;
    }

    rc = aead_batch_host_chunked(ctx, open, in, out, verdict, a);
    if (rc != 1) return rc;
    Staged st;
    rc = stage_host(ctx, in, out, open ? -16 : 16, ctx->n_keys[which], &st);
    if (rc) return rc;
    a.in = st.d_in;
    a.out = st.d_out;
    a.in_off = st.d_in_off;
    a.out_off = st.d_out_off;
    a.lens = st.d_lens;
    a.peer = st.d_peer;
    a.counters = st.d_counters;
    if (open) {
        HIPCHK(ctx, ctx->verdict.reserve(n));
        a.verdict = ctx->verdict.as<uint8_t>();
    }
    rc = maybe_sort(ctx, a.lens, n, open ? 16 : 0, &a.order);
    if (rc) return rc;
    HIPCHK(ctx, open ? launch_aead_open(a, ctx->stream) : launch_aead_seal(a, ctx->stream));
    HIPCHK(ctx, hipMemcpyAsync((uint8_t *)out->base + st.sout.lo, st.d_out, st.sout.size(),
                               hipMemcpyDeviceToHost, ctx->stream));
    if (open)
        HIPCHK(ctx, hipMemcpyAsync(verdict, a.verdict, n, hipMemcpyDeviceToHost, ctx->stream));
    uint32_t status = 0;
    rc = take_status(ctx, &status);
    if (rc) return rc;
    return status_to_rc(ctx, status);
}

} // namespace

namespace bnk {

// Reads and clears the device status word; the stream must be idle.
int take_status(bnk_ctx *ctx, uint32_t *status)
{
    HIPCHK(ctx, hipMemcpyAsync(status, ctx->d_status, 4, hipMemcpyDeviceToHost, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    if (*status) HIPCHK(ctx, launch_fill_u32(ctx->d_status, 1, 0, ctx->stream));
    return BNK_OK;
}

int status_to_rc(bnk_ctx *ctx, uint32_t status)
{
    if (status & STATUS_PEER_RANGE) return fail(ctx, BNK_E_RANGE, "peer index beyond the key table");
    if (status & STATUS_FLOWS_FULL) return fail(ctx, BNK_E_NOMEM, "flow table overflow");
    return BNK_OK;
}

} // namespace bnk

extern "C" {

int bnk_init(int device_ordinal, bnk_ctx **out)
{
    if (!out) return fail(nullptr, BNK_E_INVAL, "null out pointer");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(nullptr, BNK_E_NODEV, std::string("no HIP device: ") +
                                              (e != hipSuccess ? hipGetErrorString(e) : "count is 0"));
    if (device_ordinal < 0 || device_ordinal >= count)
        return fail(nullptr, BNK_E_NODEV, "device ordinal out of range");
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device_ordinal);
    if (e != hipSuccess) return fail_hip(nullptr, "hipGetDeviceProperties", e);
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(nullptr, BNK_E_NODEV,
                    std::string("device is ") + prop.gcnArchName + ", this library is built for gfx950");
    bnk_ctx *ctx = new (std::nothrow) bnk_ctx;
    if (!ctx) return fail(nullptr, BNK_E_NOMEM, "out of host memory");
    ctx->device = device_ordinal;
    auto bail = [&](const char *what, hipError_t err) {
        int rc = fail_hip(nullptr, what, err);
        ctx->alive = true;
        bnk_shutdown(ctx);
        return rc;
    };
    if ((e = hipSetDevice(device_ordinal)) != hipSuccess) return bail("hipSetDevice", e);
    if ((e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking)) != hipSuccess)
        return bail("hipStreamCreate", e);
    if ((e = hipEventCreate(&ctx->ev0)) != hipSuccess) return bail("hipEventCreate", e);
    if ((e = hipEventCreate(&ctx->ev1)) != hipSuccess) return bail("hipEventCreate", e);
    if ((e = hipMalloc((void **)&ctx->d_status, 256)) != hipSuccess) return bail("hipMalloc", e);
    if ((e = launch_fill_u32(ctx->d_status, 64, 0, ctx->stream)) != hipSuccess)
        return bail("status clear", e);
    ctx->filter = filter_create(ctx->stream, prop.multiProcessorCount);
    if (!ctx->filter) return bail("filter state", hipErrorOutOfMemory);
    if ((e = hipStreamSynchronize(ctx->stream)) != hipSuccess) return bail("hipStreamSynchronize", e);
    ctx->alive = true;
    *out = ctx;
    return BNK_OK;
}

void bnk_shutdown(bnk_ctx *ctx)
{
    if (!ctx) return;
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        if (!ctx->alive) return;
        ctx->alive = false;
        (void)hipSetDevice(ctx->device);
        if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
        for (DevBuf *b : {&ctx->in_arena, &ctx->out_arena, &ctx->off_in, &ctx->off_out, &ctx->lens,
                          &ctx->peer, &ctx->counters, &ctx->verdict, &ctx->order, &ctx->hist,
                          &ctx->cursor, &ctx->misc, &ctx->r_plain, &ctx->r_auth, &ctx->r_pass,
                          &ctx->r_keys, &ctx->r_idx, &ctx->r_skeys, &ctx->r_sidx, &ctx->r_tmp,
                          &ctx->r_peer_out, &ctx->r_ctr_base, &ctx->r_ctr_out, &ctx->r_verdict,
                          &ctx->wg_index, &ctx->wg_remote, &ctx->wg_allowed, &ctx->wg_send_ctr,
                          &ctx->wg_peer, &ctx->wg_counter, &ctx->wg_ctlen, &ctx->wg_result,
                          &ctx->wg_outlen, &ctx->wg_padded, &ctx->wg_wirelen, &ctx->wg_skip})
            b->release();
        ctx->pin.release();
        for (int w = 0; w < 2; w++)
            if (ctx->d_keys[w]) (void)hipFree(ctx->d_keys[w]);
        if (ctx->d_status) (void)hipFree(ctx->d_status);
        if (ctx->filter) filter_destroy(ctx->filter);
        for (hipEvent_t e : ctx->ev_up) (void)hipEventDestroy(e);
        for (hipEvent_t e : ctx->ev_done) (void)hipEventDestroy(e);
        if (ctx->s_up) (void)hipStreamDestroy(ctx->s_up);
        if (ctx->s_down) (void)hipStreamDestroy(ctx->s_down);
        if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
        if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
        if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    }
    delete ctx;
}

const char *bnk_last_error(bnk_ctx *ctx) { return ctx ? ctx->err.c_str() : g_init_err.c_str(); }

int bnk_ring_alloc(bnk_ctx *ctx, size_t bytes, void **host_pinned)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!host_pinned || bytes == 0) return fail(ctx, BNK_E_INVAL, "bad ring request");
    HIPCHK(ctx, hipHostMalloc(host_pinned, bytes, hipHostMallocDefault));
    return BNK_OK;
}

int bnk_ring_free(bnk_ctx *ctx, void *host_pinned)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!host_pinned) return BNK_OK;
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipHostFree(host_pinned));
    return BNK_OK;
}

int bnk_dev_alloc(bnk_ctx *ctx, size_t bytes, void **dev)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!dev || bytes == 0) return fail(ctx, BNK_E_INVAL, "bad device allocation request");
    HIPCHK(ctx, hipMalloc(dev, bytes));
    return BNK_OK;
}

int bnk_dev_free(bnk_ctx *ctx, void *dev)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!dev) return BNK_OK;
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    HIPCHK(ctx, hipFree(dev));
    return BNK_OK;
}

int bnk_copy_to_device(bnk_ctx *ctx, void *dev, const void *host, size_t bytes)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (bytes == 0) return BNK_OK;
    if (!dev || !host) return fail(ctx, BNK_E_INVAL, "null pointer");
    HIPCHK(ctx, hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return BNK_OK;
}

int bnk_copy_to_host(bnk_ctx *ctx, void *host, const void *dev, size_t bytes)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (bytes == 0) return BNK_OK;
    if (!dev || !host) return fail(ctx, BNK_E_INVAL, "null pointer");
    HIPCHK(ctx, hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    return BNK_OK;
}

int bnk_sync(bnk_ctx *ctx)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    uint32_t status = 0;
    int rc = take_status(ctx, &status);
    if (rc) return rc;
    return status_to_rc(ctx, status);
}

void *bnk_stream(bnk_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int bnk_keys_set(bnk_ctx *ctx, int which, const uint8_t *keys32, uint32_t n_peers)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (which != BNK_KEYS_SEND && which != BNK_KEYS_RECV)
        return fail(ctx, BNK_E_INVAL, "bad key table selector");
    if (!keys32 || n_peers == 0) return fail(ctx, BNK_E_INVAL, "empty key table");
    // in-flight work may still read the old table
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    uint32_t *nk = nullptr;
    HIPCHK(ctx, hipMalloc((void **)&nk, (size_t)n_peers * 32));
    hipError_t e = hipMemcpyAsync(nk, keys32, (size_t)n_peers * 32, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(nk);
        return fail_hip(ctx, "key upload", e);
    }
    if (ctx->d_keys[which]) (void)hipFree(ctx->d_keys[which]);
    ctx->d_keys[which] = nk;
    ctx->n_keys[which] = n_peers;
    return BNK_OK;
}

int bnk_aead_seal_batch(bnk_ctx *ctx, const bnk_batch *in, const bnk_batch *out)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    return aead_batch(ctx, false, in, out, nullptr);
}

int bnk_aead_open_batch(bnk_ctx *ctx, const bnk_batch *in, const bnk_batch *out, uint8_t *verdict)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    return aead_batch(ctx, true, in, out, verdict);
}

int bnk_probe_valu(bnk_ctx *ctx, int op, uint32_t iters, double *ops_per_sec)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!ops_per_sec || iters == 0 || op < 0 || op >= PROBE_OPS) return fail(ctx, BNK_E_INVAL, "bad probe request");
    hipDeviceProp_t prop;
    HIPCHK(ctx, hipGetDeviceProperties(&prop, ctx->device));
    // 8 workgroups of 4 waves per CU: every SIMD holds 8 waves
    const uint32_t blocks = (uint32_t)prop.multiProcessorCount * 8u;
    HIPCHK(ctx, ctx->misc.reserve((size_t)blocks * PROBE_THREADS * 4));
    HIPCHK(ctx, launch_probe(op, 4, blocks, ctx->misc.as<uint32_t>(), ctx->stream)); // warm-up
    HIPCHK(ctx, hipEventRecord(ctx->ev0, ctx->stream));
    HIPCHK(ctx, launch_probe(op, iters, blocks, ctx->misc.as<uint32_t>(), ctx->stream));
    HIPCHK(ctx, hipEventRecord(ctx->ev1, ctx->stream));
    HIPCHK(ctx, hipEventSynchronize(ctx->ev1));
    float ms = 0;
    HIPCHK(ctx, hipEventElapsedTime(&ms, ctx->ev0, ctx->ev1));
    const double ops = (double)blocks * PROBE_THREADS * (double)iters * PROBE_CHAINS * PROBE_UNROLL;
    *ops_per_sec = ops / ((double)ms * 1e-3);
    return BNK_OK;
}

int bnk_probe_copy(bnk_ctx *ctx, size_t bytes, uint32_t iters, double *bytes_per_sec)
{
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!bytes_per_sec || iters == 0 || bytes < 4096 || (bytes & 15))
        return fail(ctx, BNK_E_INVAL, "bad copy probe request");
    hipDeviceProp_t prop;
    HIPCHK(ctx, hipGetDeviceProperties(&prop, ctx->device));
    const uint32_t blocks = (uint32_t)prop.multiProcessorCount * 16u;
    void *src = nullptr, *dst = nullptr;
    HIPCHK(ctx, hipMalloc(&src, bytes));
    hipError_t e = hipMalloc(&dst, bytes);
    if (e != hipSuccess) {
        (void)hipFree(src);
        return fail_hip(ctx, "hipMalloc", e);
    }
    float ms = 0;
    e = launch_fill_u32((uint32_t *)src, (uint32_t)std::min<size_t>(bytes / 4, 1u << 30), 0x5a5a5a5au,
                        ctx->stream);
    if (e == hipSuccess) e = launch_copy(src, dst, bytes, blocks, ctx->stream); // warm-up
    if (e == hipSuccess) e = hipEventRecord(ctx->ev0, ctx->stream);
    for (uint32_t i = 0; i < iters && e == hipSuccess; i++)
        e = launch_copy(src, dst, bytes, blocks, ctx->stream);
    if (e == hipSuccess) e = hipEventRecord(ctx->ev1, ctx->stream);
    if (e == hipSuccess) e = hipEventSynchronize(ctx->ev1);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, ctx->ev0, ctx->ev1);
    (void)hipFree(src);
    (void)hipFree(dst);
    if (e != hipSuccess) return fail_hip(ctx, "copy probe", e);
    // bytes read plus bytes written
    *bytes_per_sec = 2.0 * (double)bytes * iters / ((double)ms * 1e-3);
    return BNK_OK;
}

} // extern "C"
