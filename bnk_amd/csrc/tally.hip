// Hot-path counters: how many packets each entry point sealed, opened, turned
// away, and why.  The reference keeps no such counts (its filter has no drop
// counters, internal/filter/filter.go:100-145; wireguard-go counts bytes per
// peer only), so these are an addition, read through bnk_counters_get.
//
// Nothing in the packet kernels changes for them: every entry point already
// leaves one result byte per packet (verdict / result), and the counts are a
// histogram of those bytes, taken where they lie -- on the host for a host
// batch (the bytes have just come back), by one small launch behind the batch's
// own work for a device-resident one.
#include "api_common.hpp"
#include "kernels.hpp"

namespace bnk {

namespace {

// which counter a result byte feeds, per kind of call; 0xFF: none
struct TallyMap {
    uint8_t slot[16];
    uint8_t also[16]; // a second counter the same value feeds
};

constexpr uint8_t NONE = 0xFF;

TallyMap map_of(TallyKind kind)
{
    TallyMap m;
    for (uint8_t &s : m.slot) s = NONE;
    for (uint8_t &s : m.also) s = NONE;
    switch (kind) {
    case TALLY_OPEN:
        m.slot[1] = TALLY_OPENED;
        m.slot[0] = TALLY_REJECTED;
        break;
    case TALLY_CHECK:
        m.slot[1] = TALLY_ALLOWED;
        m.slot[0] = TALLY_DENIED;
        break;
    case TALLY_DECAP:
    case TALLY_DECAP_CHECK:
        // (everything but a bad header, an unknown index and a failed tag was authentic)
        m.slot[BNK_WG_OK] = TALLY_DELIVERED;
        m.slot[BNK_WG_KEEPALIVE] = TALLY_KEEPALIVE;
        m.slot[BNK_WG_BAD_HEADER] = TALLY_BAD_HEADER;
        m.slot[BNK_WG_UNKNOWN_INDEX] = TALLY_UNKNOWN_INDEX;
        m.slot[BNK_WG_AUTH_FAIL] = TALLY_REJECTED;
        m.slot[BNK_WG_BAD_IP] = TALLY_BAD_IP;
        m.slot[BNK_WG_NOT_ALLOWED] = TALLY_NOT_ALLOWED;
        m.slot[BNK_WG_FILTERED] = TALLY_DENIED;
        m.slot[BNK_WG_REPLAY] = TALLY_REPLAYED;
        // CheckInbound behind a decapsulating call saw exactly what was delivered
        if (kind == TALLY_DECAP_CHECK) m.also[BNK_WG_OK] = TALLY_ALLOWED;
        break;
    case TALLY_RELAY:
        m.slot[BNK_RELAY_OK] = TALLY_RELAYED;
        m.slot[BNK_RELAY_FORGED] = TALLY_REJECTED;
        m.slot[BNK_RELAY_DENIED] = TALLY_DENIED;
        break;
    default:
        break;
    }
    return m;
}

// One count per result value per block in LDS, then one atomic per value that
// occurred: a few hundred atomics for a batch of a million.
constexpr uint32_t TALLY_PER_THREAD = 16;
__global__ __launch_bounds__(256) void tally_kernel(const uint8_t *res, uint32_t n, TallyMap map,
                                                    unsigned long long *counters)
{
    __shared__ uint32_t hist[16];
    if (threadIdx.x < 16u) hist[threadIdx.x] = 0u;
    __syncthreads();
    const uint32_t first = blockIdx.x * (256u * TALLY_PER_THREAD);
#pragma unroll 4
    for (uint32_t k = 0; k < TALLY_PER_THREAD; k++) {
        const uint32_t i = first + k * 256u + threadIdx.x;
        if (i < n) {
            const uint8_t v = res[i];
            if (v < 16u) atomicAdd(&hist[v], 1u);
        }
    }
    __syncthreads();
    if (threadIdx.x < 16u && hist[threadIdx.x] != 0u) {
        if (map.slot[threadIdx.x] != NONE)
            atomicAdd(&counters[map.slot[threadIdx.x]], (unsigned long long)hist[threadIdx.x]);
        if (map.also[threadIdx.x] != NONE)
            atomicAdd(&counters[map.also[threadIdx.x]], (unsigned long long)hist[threadIdx.x]);
    }
}

// words that are not zero (wire lengths of an encapsulating call: 0 = not sent)
__global__ __launch_bounds__(256) void tally_nonzero_kernel(const uint32_t *words, uint32_t n, uint32_t slot,
                                                            unsigned long long *counters)
{
    __shared__ uint32_t count;
    if (threadIdx.x == 0u) count = 0u;
    __syncthreads();
    const uint32_t first = blockIdx.x * (256u * TALLY_PER_THREAD);
    uint32_t mine = 0;
#pragma unroll 4
    for (uint32_t k = 0; k < TALLY_PER_THREAD; k++) {
        const uint32_t i = first + k * 256u + threadIdx.x;
        if (i < n && words[i] != 0u) mine++;
    }
    if (mine) atomicAdd(&count, mine);
    __syncthreads();
    if (threadIdx.x == 0u && count != 0u) atomicAdd(&counters[slot], (unsigned long long)count);
}

} // namespace

void tally_add(bnk_ctx *ctx, TallySlot slot, uint64_t k)
{
    ctx->tally_host[slot].fetch_add(k, std::memory_order_relaxed);
}

int tally_results(bnk_ctx *ctx, TallyKind kind, const uint8_t *res, uint32_t n, int mem)
{
    if (!res || n == 0) return BNK_OK;
    const TallyMap map = map_of(kind);
    if (mem == BNK_MEM_HOST) {
        uint64_t hist[16] = {0};
        for (uint32_t i = 0; i < n; i++)
            if (res[i] < 16u) hist[res[i]]++;
        for (int v = 0; v < 16; v++) {
            if (hist[v] && map.slot[v] != NONE) tally_add(ctx, (TallySlot)map.slot[v], hist[v]);
            if (hist[v] && map.also[v] != NONE) tally_add(ctx, (TallySlot)map.also[v], hist[v]);
        }
        return BNK_OK;
    }
    const uint32_t blocks = (n + 256u * TALLY_PER_THREAD - 1u) / (256u * TALLY_PER_THREAD);
    hipLaunchKernelGGL(tally_kernel, dim3(blocks), dim3(256), 0, ctx->stream, res, n, map,
                       reinterpret_cast<unsigned long long *>(ctx->d_tally));
    HIPCHK(ctx, hipGetLastError());
    return BNK_OK;
}

int tally_nonzero(bnk_ctx *ctx, TallySlot slot, const uint32_t *words, uint32_t n, int mem)
{
    if (!words || n == 0) return BNK_OK;
    if (mem == BNK_MEM_HOST) {
        uint64_t k = 0;
        for (uint32_t i = 0; i < n; i++) k += words[i] != 0u;
        if (k) tally_add(ctx, slot, k);
        return BNK_OK;
    }
    const uint32_t blocks = (n + 256u * TALLY_PER_THREAD - 1u) / (256u * TALLY_PER_THREAD);
    hipLaunchKernelGGL(tally_nonzero_kernel, dim3(blocks), dim3(256), 0, ctx->stream, words, n, (uint32_t)slot,
                       reinterpret_cast<unsigned long long *>(ctx->d_tally));
    HIPCHK(ctx, hipGetLastError());
    return BNK_OK;
}

} // namespace bnk

using namespace bnk;

extern "C" int bnk_counters_get(bnk_ctx *ctx, bnk_counters *out)
{
    BNK_API_TRY
    if (!out) return ctx ? fail(ctx, BNK_E_INVAL, "null argument") : BNK_E_INVAL;
    Guard g(ctx);
    if (g.rc) return g.rc;
    uint64_t dev[TALLY_SLOTS];
    HIPCHK(ctx, hipMemcpyAsync(dev, ctx->d_tally, sizeof(dev), hipMemcpyDeviceToHost, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    uint64_t v[TALLY_SLOTS];
    for (int s = 0; s < TALLY_SLOTS; s++) v[s] = dev[s] + ctx->tally_host[s].load(std::memory_order_relaxed);
    out->sealed = v[TALLY_SEALED];
    out->opened = v[TALLY_OPENED];
    out->rejected = v[TALLY_REJECTED];
    out->allowed = v[TALLY_ALLOWED];
    out->denied = v[TALLY_DENIED];
    out->delivered = v[TALLY_DELIVERED];
    out->keepalive = v[TALLY_KEEPALIVE];
    out->replayed = v[TALLY_REPLAYED];
    out->bad_header = v[TALLY_BAD_HEADER];
    out->unknown_index = v[TALLY_UNKNOWN_INDEX];
    out->bad_ip = v[TALLY_BAD_IP];
    out->not_allowed = v[TALLY_NOT_ALLOWED];
    out->relayed = v[TALLY_RELAYED];
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

extern "C" int bnk_counters_reset(bnk_ctx *ctx)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    HIPCHK(ctx, hipMemsetAsync(ctx->d_tally, 0, TALLY_SLOTS * 8, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    for (int s = 0; s < TALLY_SLOTS; s++) ctx->tally_host[s].store(0, std::memory_order_relaxed);
    return BNK_OK;
    BNK_API_CATCH(ctx)
}
