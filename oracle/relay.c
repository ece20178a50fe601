/*
 * relay.c -- CPU definition of the fused relay step open -> filter ->
 * re-seal.  Test infrastructure only: see bnk_oracle.h.
 *
 * The reference has no such function: its server forwards ciphertext
 * unopened (internal/coord/server/server.go:439-453).  The step is the
 * composition of wireguard-go's transport open, internal/filter's
 * CheckInbound (filter.go:121-147) and a transport seal under the outbound
 * peer's key, with the outbound counter assigned only to packets that
 * survive, in batch order.
 */
#include "bnk_oracle.h"

#include <stdlib.h>
#include <string.h>

void bnko_relay_fused_batch(bnko_filter *f, const uint8_t *keys_in,
                            const uint32_t *peer_in, const uint64_t *ctr_in,
                            const uint8_t *keys_out, const uint32_t *peer_out,
                            const uint64_t *ctr_base_out, uint32_t n_peers_out,
                            const uint8_t *in, const uint64_t *in_off,
                            const uint32_t *in_len, uint8_t *out,
                            const uint64_t *out_off, int64_t now_ns,
                            uint8_t *verdict, uint64_t *ctr_out, uint32_t n)
{
    uint64_t *next = (uint64_t *)malloc(sizeof(uint64_t) *
                                        (n_peers_out ? n_peers_out : 1));
    memcpy(next, ctr_base_out, sizeof(uint64_t) * n_peers_out);
    uint8_t *pt = NULL;
    size_t pt_cap = 0;
    for (uint32_t i = 0; i < n; i++) {
        ctr_out[i] = 0;
        uint32_t len = in_len[i];
        if (len < 16) {
            verdict[i] = BNKO_RELAY_FORGED;
            continue;
        }
        if (pt_cap < len) {
            pt_cap = (size_t)len * 2;
            pt = (uint8_t *)realloc(pt, pt_cap);
        }
        uint8_t nonce[12];
        bnko_wg_nonce(ctr_in[i], nonce);
        if (!bnko_aead_open(keys_in + 32 * (size_t)peer_in[i], nonce,
                            in + in_off[i], len, NULL, 0, pt)) {
            verdict[i] = BNKO_RELAY_FORGED;
            continue;
        }
        if (!bnko_filter_check_inbound(f, pt, len - 16, now_ns)) {
            verdict[i] = BNKO_RELAY_DENIED;
            continue;
        }
        uint32_t po = peer_out[i];
        uint64_t c = next[po]++;
        bnko_wg_nonce(c, nonce);
        bnko_aead_seal(keys_out + 32 * (size_t)po, nonce, pt, len - 16, NULL, 0,
                       out + out_off[i]);
        verdict[i] = BNKO_RELAY_OK;
        ctr_out[i] = c;
    }
    free(pt);
    free(next);
}
