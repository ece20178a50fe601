// bnk_aead_seal_batch_noalloc: bnk_aead_seal_batch for callers that cannot
// allocate device memory (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc).  The one scratch buffer the seal path needs
// beyond its inputs and outputs -- the length grouping's packet order,
// histogram and cursors -- lives in a file-scope device array instead of the
// context's grow-only buffers.
#include <mutex>

#include "api_common.hpp"

using namespace bnk;

constexpr size_t SCRATCH_WORDS = (size_t)BNK_NOALLOC_MAX_PACKETS + LEN_BINS + LEN_CURSOR_WORDS;

// 4 MiB + 8 KiB on every GPU the library runs on, for the life of the process.
// In host code this name is only a stand-in for the symbol: the address a
// kernel can use comes from hipGetSymbolAddress, once per device.  (Kept out
// of an unnamed namespace and free of attributes: the compiler gives a static
// device variable that host code names a visible symbol of its own, which is
// what the runtime looks up.)
static __device__ __align__(256) uint32_t scratch[SCRATCH_WORDS];

namespace {

constexpr int MAX_DEVICES = 64;
std::mutex g_mu;
uint32_t *g_scratch_ptr[MAX_DEVICES]; // per device: each GPU holds its own copy of the array
// Who used a device's array last, and the event that context recorded behind its
// launches: another context makes its stream wait for that event before it
// touches the array, so that calls of different contexts on one GPU take turns
// instead of interleaving their groupings on the same words.
bnk_ctx *g_last_user[MAX_DEVICES];

} // namespace

namespace bnk {

int noalloc_setup(bnk_ctx *ctx, int device)
{
    if (device < 0 || device >= MAX_DEVICES) return fail(ctx, BNK_E_NODEV, "device ordinal out of range");
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_scratch_ptr[device]) return BNK_OK;
    void *p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return fail_hip(ctx, "hipGetSymbolAddress(scratch)", e);
    if (!p) return fail(ctx, BNK_E_HIP, "hipGetSymbolAddress(scratch) returned a null address");
    g_scratch_ptr[device] = static_cast<uint32_t *>(p);
    return BNK_OK;
}

// A context that goes away takes its event with it (its stream has been waited for).
void noalloc_forget(bnk_ctx *ctx)
{
    if (ctx->device < 0 || ctx->device >= MAX_DEVICES) return;
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_last_user[ctx->device] == ctx) g_last_user[ctx->device] = nullptr;
}

} // namespace bnk

extern "C" int bnk_aead_seal_batch_noalloc(bnk_ctx *ctx, const bnk_batch *in, const bnk_batch *out)
{
    BNK_API_TRY
    Guard g(ctx);
    if (g.rc) return g.rc;
    if (!in || !out) return fail(ctx, BNK_E_INVAL, "null batch");
    if (in->mem != BNK_MEM_DEVICE || out->mem != BNK_MEM_DEVICE)
        return fail(ctx, BNK_E_INVAL, "bnk_aead_seal_batch_noalloc takes device-resident batches only");
    if (in->n > BNK_NOALLOC_MAX_PACKETS)
        return fail(ctx, BNK_E_INVAL, "bnk_aead_seal_batch_noalloc: more than BNK_NOALLOC_MAX_PACKETS packets");
    // held while the call enqueues its work (it does not wait for it), so that two
    // contexts' waits and records on a device pair up in one order
    std::lock_guard<std::mutex> lk(g_mu);
    uint32_t *ptr = g_scratch_ptr[ctx->device];
    if (!ptr) return fail(ctx, BNK_E_STATE, "device scratch was not set up");
    bnk_ctx *last = g_last_user[ctx->device];
    if (last && last != ctx) HIPCHK(ctx, hipStreamWaitEvent(ctx->stream, last->ev_noalloc, 0));
    // The array keeps the last call's contents: the histogram starts as zeros
    // (static storage) and every length grouping clears it again before it ends
    // (a kernel, no memset), order[] and cursor[] are written before they are read.
    const int rc = aead_batch(ctx, false, in, out, nullptr, ptr);
    // (also after a failure: part of the work may have been enqueued)
    if (hipEventRecord(ctx->ev_noalloc, ctx->stream) == hipSuccess) g_last_user[ctx->device] = ctx;
    if (rc == BNK_OK) tally_add(ctx, TALLY_SEALED, in->n); // (a host-side count: nothing is launched or allocated)
    return rc;
    BNK_API_CATCH(ctx)
}
