// Hot-path counters: how many packets each entry point sealed, opened, turned
// away, and why.  The reference keeps no such counts (its filter has no drop
// counters, internal/filter/filter.go:100-145; wireguard-go counts bytes per
// peer only), so these are an addition, read through bnk_counters_get.
//
// Every entry point already leaves one result byte per packet (verdict /
// result), and the counts are a histogram of those bytes, taken where they lie:
// on the host for a host batch (the bytes have just come back); for a
// device-resident one by the launch that writes them where it is the last to
// touch them (a plain open, a CheckInbound on its own: a vote per wave and two
// atomics, see tally_bump), else by one small launch behind the batch's own work
// (the framing calls, whose results the window pass and the filter still change,
// and the relay).
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

// A thread takes 16 consecutive result bytes (one load where they are aligned).
// Within a wave the lanes vote per distinct value and lane v keeps value v's
// count in a register, so nothing is contended; lanes 0-15 of every wave then
// add into the block's 16 LDS words, and the block issues one global atomic per
// value that occurred: a few hundred atomics for a batch of a million.
constexpr uint32_t TALLY_PER_THREAD = 16;

__device__ __forceinline__ void tally_vote(uint32_t v, bool valid, uint32_t lane, uint32_t &mine)
{
    unsigned long long todo = __ballot(valid && v < 16u);
    while (todo != 0ull) {
        const int leader = __ffsll((long long)todo) - 1;
        const uint32_t lv = (uint32_t)__builtin_amdgcn_readlane((int)v, leader);
        const unsigned long long same = __ballot(valid && v == lv);
        if (lane == lv) mine += (uint32_t)__popcll(same);
        todo &= ~same;
    }
}

__global__ __launch_bounds__(256) void tally_kernel(const uint8_t *res, uint32_t n, TallyMap map,
                                                    unsigned long long *counters)
{
    __shared__ uint32_t hist[16];
    if (threadIdx.x < 16u) hist[threadIdx.x] = 0u;
    __syncthreads();
    const uint32_t lane = threadIdx.x & 63u;
    const uint64_t first = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * TALLY_PER_THREAD;
    uint32_t w[4] = {0, 0, 0, 0};
    const bool whole = first + TALLY_PER_THREAD <= n && (((uintptr_t)(res + first)) & 15u) == 0;
    if (whole) {
        const uint4 q = *reinterpret_cast<const uint4 *>(res + first);
        w[0] = q.x; w[1] = q.y; w[2] = q.z; w[3] = q.w;
    } else {
        for (uint32_t k = 0; k < TALLY_PER_THREAD; k++)
            if (first + k < n) w[k >> 2] |= (uint32_t)res[first + k] << (8u * (k & 3u));
    }
    uint32_t mine = 0; // lane v: how often value v occurred in this wave
#pragma unroll
    for (uint32_t k = 0; k < TALLY_PER_THREAD; k++)
        tally_vote((w[k >> 2] >> (8u * (k & 3u))) & 0xFFu, first + k < n, lane, mine);
    if (lane < 16u && mine != 0u) atomicAdd(&hist[lane], mine);
    __syncthreads();
    if (threadIdx.x < 16u && hist[threadIdx.x] != 0u) {
        if (map.slot[threadIdx.x] != NONE)
            tally_bump(counters, map.slot[threadIdx.x], hist[threadIdx.x]);
        if (map.also[threadIdx.x] != NONE) tally_bump(counters, map.also[threadIdx.x], hist[threadIdx.x]);
    }
}

// words that are not zero (wire lengths of an encapsulating call: 0 = not sent)
__global__ __launch_bounds__(256) void tally_nonzero_kernel(const uint32_t *words, uint32_t n, uint32_t slot,
                                                            unsigned long long *counters)
{
    __shared__ uint32_t count;
    if (threadIdx.x == 0u) count = 0u;
    __syncthreads();
    // (consecutive lanes read consecutive words)
    const uint64_t first = (uint64_t)blockIdx.x * (256u * TALLY_PER_THREAD) + threadIdx.x;
    uint32_t w[TALLY_PER_THREAD];
#pragma unroll
    for (uint32_t k = 0; k < TALLY_PER_THREAD; k++) {
        const uint64_t i = first + (uint64_t)k * 256u;
        w[k] = i < n ? words[i] : 0u;
    }
    uint32_t mine = 0;
#pragma unroll
    for (uint32_t k = 0; k < TALLY_PER_THREAD; k++) mine += w[k] != 0u ? 1u : 0u;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mine += (uint32_t)__shfl_xor((int)mine, off, 64);
    if ((threadIdx.x & 63u) == 0u && mine != 0u) atomicAdd(&count, mine);
    __syncthreads();
    if (threadIdx.x == 0u) tally_bump(counters, slot, count);
}

} // namespace

void tally_add(bnk_ctx *ctx, TallySlot slot, uint64_t k)
{
    if (!ctx->tally_on.load(std::memory_order_relaxed)) return;
    ctx->tally_host[slot].fetch_add(k, std::memory_order_relaxed);
}

int tally_results(bnk_ctx *ctx, TallyKind kind, const uint8_t *res, uint32_t n, int mem)
{
    if (!res || n == 0 || !ctx->tally_on.load(std::memory_order_relaxed)) return BNK_OK;
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
    if (!words || n == 0 || !ctx->tally_on.load(std::memory_order_relaxed)) return BNK_OK;
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
    static thread_local uint64_t dev[TALLY_SLOTS * TALLY_LANES];
    HIPCHK(ctx, hipMemcpyAsync(dev, ctx->d_tally, sizeof(dev), hipMemcpyDeviceToHost, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    uint64_t v[TALLY_SLOTS];
    for (int s = 0; s < TALLY_SLOTS; s++) {
        v[s] = ctx->tally_host[s].load(std::memory_order_relaxed);
        for (uint32_t l = 0; l < TALLY_LANES; l++) v[s] += dev[s * TALLY_LANES + l];
    }
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
    HIPCHK(ctx, hipMemsetAsync(ctx->d_tally, 0, TALLY_SLOTS * TALLY_LANES * 8, ctx->stream));
    HIPCHK(ctx, hipStreamSynchronize(ctx->stream));
    for (int s = 0; s < TALLY_SLOTS; s++) ctx->tally_host[s].store(0, std::memory_order_relaxed);
    return BNK_OK;
    BNK_API_CATCH(ctx)
}

extern "C" int bnk_counters_enable(bnk_ctx *ctx, int on)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    ctx->tally_on.store(on != 0, std::memory_order_relaxed);
    return BNK_OK;
    BNK_API_CATCH(ctx)
}
