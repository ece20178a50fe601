// Context object and host-side helpers shared by the C ABI entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/bnkhip.h"
#include "coalesce.hpp"
#include "kernels.hpp"

namespace bnk {

// Grow-only device buffer owned by a context.
struct DevBuf {
    void *p = nullptr;
    size_t cap = 0;
    hipError_t reserve(size_t bytes)
    {
        if (bytes <= cap) return hipSuccess;
        size_t want = cap ? cap : 4096;
        while (want < bytes) want *= 2;
        void *np = nullptr;
        hipError_t e = hipMalloc(&np, want);
        if (e != hipSuccess) return e;
        if (p) (void)hipFree(p);
        p = np;
        cap = want;
        return hipSuccess;
    }
    void release()
    {
        if (p) (void)hipFree(p);
        p = nullptr;
        cap = 0;
    }
    template <class T> T *as() const { return static_cast<T *>(p); }
};

// Grow-only pinned host buffer (staging for gathers from [][]byte).
struct PinBuf {
    void *p = nullptr;
    size_t cap = 0;
    hipError_t reserve(size_t bytes)
    {
        if (bytes <= cap) return hipSuccess;
        size_t want = cap ? cap : 4096;
        while (want < bytes) want *= 2;
        void *np = nullptr;
        hipError_t e = hipHostMalloc(&np, want, hipHostMallocDefault);
        if (e != hipSuccess) return e;
        void *nd = nullptr;
        e = hipHostGetDevicePointer(&nd, np, 0);
        if (e != hipSuccess) {
            (void)hipHostFree(np);
            return e;
        }
        if (p) (void)hipHostFree(p);
        p = np;
        d = static_cast<uint8_t *>(nd);
        cap = want;
        return hipSuccess;
    }
    void release()
    {
        if (p) (void)hipHostFree(p);
        p = nullptr;
        d = nullptr;
        cap = 0;
    }
    // The address a kernel uses for a host address inside the buffer.
    template <class T> T *dev(T *host) const
    {
        return reinterpret_cast<T *>(d + ((uint8_t *)host - static_cast<uint8_t *>(p)));
    }
    uint8_t *d = nullptr;
    template <class T> T *as() const { return static_cast<T *>(p); }
};

struct FilterState; // filter_host.hpp

// A result array a kernel leaves in pinned staging, to be copied to the
// caller's array once the stream has reached the end of the call.
struct Deferred {
    void *dst;
    const void *src;
    size_t bytes;
};

// Staging of one merged window (coalesce.hpp): windows are enqueued one behind
// the other and each is waited for outside the context lock, so each needs
// staging of its own until its work is done.
struct HostStage {
    PinBuf pin;
    std::atomic<bool> busy{false}; // taken by a window's leader until it has copied its results out
};
constexpr uint32_t HOST_STAGES = 4;

} // namespace bnk

struct bnk_ctx {
    std::mutex mu;
    std::mutex err_mu; // guards err alone
    int device = -1;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    // hot-path counters: what launches counted ([slot][TALLY_LANES]) and what the host counted ([slot])
    uint64_t *d_tally = nullptr;
    std::atomic<uint64_t> tally_host[bnk::TALLY_SLOTS];
    std::atomic<bool> tally_on{true};
    hipEvent_t ev_noalloc = nullptr; // recorded behind every bnk_aead_seal_batch_noalloc of this context
    // chunked host batches: upload and download streams, one event pair per chunk
    hipStream_t s_up = nullptr, s_down = nullptr;
    std::vector<hipEvent_t> ev_up, ev_done;
    std::string err;
    bool alive = false;

    uint32_t *d_keys[2] = {nullptr, nullptr};
    uint32_t n_keys[2] = {0, 0};
    uint32_t *d_status = nullptr; // the device's address of h_status, see STATUS_*

    // staging for BNK_MEM_HOST batches and scratch for the length sort
    bnk::DevBuf in_arena, out_arena, off_in, off_out, lens, peer, counters, verdict;
    bnk::DevBuf order, hist, cursor, misc;
    bnk::PinBuf pin;
    // Which pinned staging the small-batch routes of the call being enqueued
    // use, and whether that call returns as soon as its work is enqueued (defer
    // non-null: the result copies are appended there and the caller waits for
    // the stream itself, see finish_direct and coalesce.hip) or waits itself.
    bnk::PinBuf *pin_cur = &pin;
    std::vector<bnk::Deferred> *defer = nullptr;
    bool defer_status = false; // the deferred call wants the status words read when it is done
    bnk::HostStage stages[bnk::HOST_STAGES];
    // Pinned rings handed out by bnk_ring_alloc: kernels may read and write
    // them in place (small host batches skip the copies).
    struct Ring { uintptr_t host; uint8_t *dev; size_t bytes; };
    std::vector<Ring> rings;
    std::mutex rings_mu; // held (with mu) while `rings` changes, and alone by readers that do not hold mu
    bnk::Coalescer co;   // merging of small host calls, see coalesce.hpp
    uint32_t *h_status = nullptr; // pinned status words the kernels write
    uint32_t wait_seq = 0;        // number of the last wait_stream(), see STATUS_DONE_WORD
    bool wait_sync_only = false;  // BNK_WAIT_SYNC=1: wait with hipStreamSynchronize, never by watching the word
    uint32_t spread_max = bnk::SPREAD_MAX_PACKETS; // see AeadArgs::spread_max
    // fused relay: plaintext scratch, per-packet flags, sort buffers, staged arrays
    bnk::DevBuf r_plain, r_auth, r_pass, r_keys, r_idx, r_skeys, r_sidx, r_tmp;
    bnk::DevBuf r_heads; // 32 bytes per packet: AeadArgs::heads of the relay's open
    bnk::DevBuf r_peer_out, r_ctr_base, r_ctr_out, r_verdict;

    // WireGuard framing: peer tables and per-packet scratch
    bnk::DevBuf wg_index, wg_remote, wg_allowed, wg_send_ctr;
    uint32_t n_wg_peers = 0;
    std::vector<bnk_wg_peer> wg_rows; // host copy of the peer table, row by row
    // anti-replay windows, one per row, and the scratch of a replay pass
    uint64_t *wg_replay = nullptr;
    uint32_t wg_replay_rows = 0;
    bnk::DevBuf wg_hash;      // receiver index -> row, hash table form
    uint32_t wg_hash_bits = 0;
    uint32_t wg_replay_parity = 0; // WgReplayScratch::parity of the next pass over a large batch
    bool wg_replay_on = true;
    bool wg_unfused = false; // framing of lane-per-packet launches in kernels of its own
    bnk::DevBuf wg_sctr, wg_sval, wg_pmax, wg_lastb, wg_rtable, wg_rflags;
    bnk::DevBuf wg_peer, wg_counter, wg_ctlen, wg_result, wg_outlen, wg_padded, wg_wirelen, wg_skip;

    bnk::FilterState *filter = nullptr;
};
