// WireGuard transport framing around the AEAD kernels: header parse and
// build, receiver-index lookup, zero padding, IPv4 length trim, allowed-IP
// check.  Follows the WireGuard protocol paper (section 5.4.6) and
// wireguard-go's documented behaviour; wireguard-go itself is not part of the
// reference tree (the reference only instantiates it,
// internal/dataplane/engine.go:51, and gives every peer one /32 allowed IP,
// engine.go:292-299).
#include "../../include/bnkhip.h"
#include "kernels.hpp"
#include "wg_dev.hpp"

namespace bnk {

#define BNK_DEV __device__ __forceinline__

BNK_DEV uint32_t wg_ld32(const uint8_t *p)
{
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}

BNK_DEV void wg_st32(uint8_t *p, uint32_t v) { __builtin_memcpy(p, &v, 4); }

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 __attribute__((aligned(1))) u32x4_unaligned;

constexpr uint32_t WG_LDS_PEERS_MAX = 8192; // 64 KiB of (index, peer) pairs

// Header checks and receiver-index lookup of received datagrams.  The sorted
// index table is searched in LDS when it fits (ten dependent reads per packet
// would otherwise each go out to L2); the header comes in with one load.
__global__ __launch_bounds__(256) void wg_parse_kernel(WgBatch b, WgPeersDev pe, uint32_t *peer,
                                                       uint64_t *counter, uint32_t *ct_len,
                                                       uint8_t *result, uint32_t *status)
{
    extern __shared__ uint2 ltab[];
    const bool in_lds = pe.n <= WG_LDS_PEERS_MAX;
    if (in_lds) {
        for (uint32_t q = threadIdx.x; q < pe.n; q += 256u) ltab[q] = pe.index_sorted[q];
        __syncthreads();
    }
    const uint2 *tab = in_lds ? ltab : pe.index_sorted;
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= b.n) return;
    const uint32_t i = b.first + t;
    const uint64_t at = b.off ? b.off[i] : (uint64_t)i * b.stride;
    const uint8_t *w = b.base + at;
    const uint32_t len = b.lens ? b.lens[i] : b.len;
    peer[i] = 0xFFFFFFFFu;
    counter[i] = 0;
    ct_len[i] = 0;
    if (beyond_arena(at, len, b.limit)) {
        status_raise(status, STATUS_BOUNDS);
        result[i] = BNK_WG_BAD_HEADER;
        return;
    }
    if (len < 32u) {
        result[i] = BNK_WG_BAD_HEADER;
        return;
    }
    const u32x4 h = *reinterpret_cast<const u32x4_unaligned *>(w);
    if (h.x != 4u) {
        result[i] = BNK_WG_BAD_HEADER;
        return;
    }
    const uint32_t idx = h.y;
    uint32_t lo = 0, hi = pe.n;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) >> 1;
        if (tab[mid].x < idx) lo = mid + 1;
        else hi = mid;
    }
    if (lo >= pe.n || tab[lo].x != idx) {
        result[i] = BNK_WG_UNKNOWN_INDEX;
        return;
    }
    peer[i] = tab[lo].y;
    counter[i] = (uint64_t)h.z | (uint64_t)h.w << 32;
    ct_len[i] = len - 16u;
    result[i] = BNK_WG_OK; // so far
}

// After the open: keepalive, IP version, length trim, allowed source.
__global__ __launch_bounds__(256) void wg_finish_kernel(WgBatch out, uint32_t out_skip, WgPeersDev pe,
                                                        const uint32_t *peer, const uint32_t *ct_len,
                                                        const uint8_t *auth, uint8_t *result,
                                                        uint32_t *out_len)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= out.n) return;
    const uint32_t i = out.first + t;
    out_len[i] = 0;
    if (result[i] != BNK_WG_OK) return;
    if (!auth[i]) {
        result[i] = BNK_WG_AUTH_FAIL;
        return;
    }
    const uint32_t plen = ct_len[i] - 16u;
    if (plen == 0u) {
        result[i] = BNK_WG_KEEPALIVE;
        return;
    }
    const uint8_t *p = out.base + (out.off ? out.off[i] : (uint64_t)i * out.stride) + out_skip;
    if (plen < 16u) {
        // too short for either header; only the version nibble could matter and
        // every version is refused at this length
        result[i] = BNK_WG_BAD_IP;
        return;
    }
    // the first 16 bytes hold every field looked at below, in one load
    const u32x4 hw = *reinterpret_cast<const u32x4_unaligned *>(p);
    const uint32_t version = (hw.x >> 4) & 0xFu;
    if (version == 4u) {
        if (plen < 20u) { result[i] = BNK_WG_BAD_IP; return; }
        const uint32_t total = __builtin_bswap32(hw.x) & 0xFFFFu;
        if (total > plen || total < 20u) { result[i] = BNK_WG_BAD_IP; return; }
        const uint32_t src = __builtin_bswap32(hw.w);
        const uint2 al = pe.allowed[peer[i]];
        if ((src & al.y) != (al.x & al.y)) { result[i] = BNK_WG_NOT_ALLOWED; return; }
        out_len[i] = total;
        return;
    }
    if (version == 6u) {
        if (plen < 40u) { result[i] = BNK_WG_BAD_IP; return; }
        const uint32_t total = (__builtin_bswap32(hw.y) >> 16) + 40u;
        result[i] = total > plen ? BNK_WG_BAD_IP : BNK_WG_NOT_ALLOWED; // peers own IPv4 addresses only
        return;
    }
    result[i] = BNK_WG_BAD_IP;
}

// Sort keys for the per-peer counter assignment of an outgoing batch.
__global__ __launch_bounds__(256) void wg_keys_kernel(const uint32_t *peer, uint32_t n_peers, uint32_t n,
                                                      uint32_t *keys, uint32_t *idx, uint32_t *status)
{
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n) return;
    uint32_t k = peer ? peer[i] : 0u;
    if (k >= n_peers) {
        status_raise(status, STATUS_PEER_RANGE);
        k = 0xFFFFFFFFu;
    }
    keys[i] = k;
    idx[i] = i;
}

// Writes the transport header into the slot's headroom, zero-pads the
// plaintext, and reports the padded and wire lengths.  The header goes to
// hdr_base (same offsets as b.base): the arena the sealed packet is written
// to, when that is not the one the plaintext is read from.
__global__ __launch_bounds__(256) void wg_encap_prep_kernel(WgBatch b, uint8_t *hdr_base, WgPeersDev pe, const uint32_t *peer,
                                                            const uint64_t *counter, uint32_t mtu,
                                                            uint32_t *padded_len, uint32_t *wire_len,
                                                            uint8_t *skip, uint32_t *status)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= b.n) return;
    const uint32_t i = b.first + t;
    const uint32_t pr = peer ? peer[i] : 0u;
    const uint32_t len = b.lens ? b.lens[i] : b.len;
    // a peer beyond the table, or a keypair that has used up its nonces
    // (wireguard-go device/send.go: nothing is sent at RejectAfterMessages)
    const uint64_t c = pr < pe.n ? counter[i] : 0;
    const uint64_t at = b.off ? b.off[i] : (uint64_t)i * b.stride;
    const uint32_t pad = wg_padding(len, mtu);
    const bool outside = beyond_arena(at, 16ull + len + pad + 16ull, b.limit) ||
                         (len > MAX_PACKET_BYTES && b.limit != 0); // len + pad must not wrap
    if (outside) status_raise(status, STATUS_BOUNDS);
    if (pr >= pe.n || c >= WG_REJECT_AFTER_MESSAGES || outside) {
        skip[i] = 1;
        padded_len[i] = 0;
        wire_len[i] = 0;
        return;
    }
    uint8_t *w = const_cast<uint8_t *>(b.base) + at;
    const u32x4 hdr = {4u, pe.remote_index[pr], (uint32_t)c, (uint32_t)(c >> 32)};
    *reinterpret_cast<u32x4_unaligned *>(hdr_base + at) = hdr;
    for (uint32_t k = 0; k < pad; k++) w[16u + len + k] = 0;
    skip[i] = 0;
    padded_len[i] = len + pad;
    wire_len[i] = 16u + len + pad + 16u;
}

static dim3 grid_of(uint32_t n) { return dim3((n + 255u) / 256u); }

hipError_t launch_wg_parse(const WgBatch &b, const WgPeersDev &pe, uint32_t *peer, uint64_t *counter,
                           uint32_t *ct_len, uint8_t *result, uint32_t *status, hipStream_t s)
{
    if (b.n == 0) return hipSuccess;
    const uint32_t lds = pe.n <= WG_LDS_PEERS_MAX ? pe.n * 8u : 0u;
    if (lds > 48u * 1024u) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(wg_parse_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)(WG_LDS_PEERS_MAX * 8u));
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(wg_parse_kernel, grid_of(b.n), dim3(256), lds, s, b, pe, peer, counter, ct_len, result, status);
    return hipGetLastError();
}

hipError_t launch_wg_finish(const WgBatch &out, uint32_t out_skip, const WgPeersDev &pe,
                            const uint32_t *peer, const uint32_t *ct_len, const uint8_t *auth,
                            uint8_t *result, uint32_t *out_len, hipStream_t s)
{
    if (out.n == 0) return hipSuccess;
    hipLaunchKernelGGL(wg_finish_kernel, grid_of(out.n), dim3(256), 0, s, out, out_skip, pe, peer, ct_len,
                       auth, result, out_len);
    return hipGetLastError();
}

hipError_t launch_wg_keys(const uint32_t *peer, uint32_t n_peers, uint32_t n, uint32_t *keys,
                          uint32_t *idx, uint32_t *status, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(wg_keys_kernel, grid_of(n), dim3(256), 0, s, peer, n_peers, n, keys, idx, status);
    return hipGetLastError();
}

hipError_t launch_wg_encap_prep(const WgBatch &b, uint8_t *hdr_base, const WgPeersDev &pe, const uint32_t *peer,
                                const uint64_t *counter, uint32_t mtu, uint32_t *padded_len,
                                uint32_t *wire_len, uint8_t *skip, uint32_t *status, hipStream_t s)
{
    if (b.n == 0) return hipSuccess;
    hipLaunchKernelGGL(wg_encap_prep_kernel, grid_of(b.n), dim3(256), 0, s, b, hdr_base, pe, peer, counter, mtu,
                       padded_len, wire_len, skip, status);
    return hipGetLastError();
}

} // namespace bnk
