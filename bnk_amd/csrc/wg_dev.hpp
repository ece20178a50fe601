// Device-side views for the WireGuard transport framing kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bnk {

struct WgPeersDev {
    const uint2 *index_sorted;   // (local receiver index, peer), ascending by index
    const uint32_t *remote_index; // [n] index the peer expects in the header
    const uint2 *allowed;         // [n] (net, mask) of the peer's allowed IPv4 prefix
    uint64_t *send_ctr;           // [n] next nonce counter per peer
    uint32_t n;
};

struct WgBatch {
    const uint8_t *base;
    const uint64_t *off;  // or nullptr: i * stride
    const uint32_t *lens; // or nullptr: len
    uint32_t n, stride, len;
    uint32_t first; // the launch covers packets first .. first+n-1 of the arrays
    uint64_t limit; // arena size when the host could not check the layout (device-resident
                    // per-packet arrays), else 0: see AeadArgs::in_limit
};

hipError_t launch_wg_parse(const WgBatch &b, const WgPeersDev &pe, uint32_t *peer, uint64_t *counter,
                           uint32_t *ct_len, uint8_t *result, uint32_t *status, hipStream_t s);
hipError_t launch_wg_finish(const WgBatch &out, uint32_t out_skip, const WgPeersDev &pe,
                            const uint32_t *peer, const uint32_t *ct_len, const uint8_t *auth,
                            uint8_t *result, uint32_t *out_len, hipStream_t s);
hipError_t launch_wg_keys(const uint32_t *peer, uint32_t n_peers, uint32_t n, uint32_t *keys,
                          uint32_t *idx, uint32_t *status, hipStream_t s);
hipError_t launch_wg_encap_prep(const WgBatch &b, uint8_t *hdr_base, const WgPeersDev &pe, const uint32_t *peer,
                                const uint64_t *counter, uint32_t mtu, uint32_t *padded_len,
                                uint32_t *wire_len, uint8_t *skip, uint32_t *status, hipStream_t s);

// result[i] = BNK_WG_FILTERED where it was BNK_WG_OK and pass[i] == 0.
hipError_t launch_wg_mark_filtered(uint8_t *result, const uint8_t *pass, uint32_t n, hipStream_t s);

} // namespace bnk
