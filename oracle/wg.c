/*
 * wg.c -- CPU restatement of WireGuard transport framing around the AEAD:
 * header, padding, receiver-index lookup, IPv4 trim, allowed-IP check, replay
 * window.  Test infrastructure only, and PARITY UNPINNED: wireguard-go is not
 * vendored in the reference tree (go.mod:10), so this follows the protocol
 * paper and wireguard-go's documented behaviour; see bnk_oracle.h.
 */
#include "bnk_oracle.h"

#include <string.h>

static void st32le(uint8_t *p, uint32_t v)
{
    p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); p[2] = (uint8_t)(v >> 16); p[3] = (uint8_t)(v >> 24);
}
static uint32_t ld32le(const uint8_t *p)
{
    return (uint32_t)p[0] | (uint32_t)p[1] << 8 | (uint32_t)p[2] << 16 | (uint32_t)p[3] << 24;
}

/* Pad to a multiple of 16, but never beyond the MTU; a packet longer than the
 * MTU is padded as its remainder modulo the MTU would be. */
uint32_t bnko_wg_padding(uint32_t packet_len, uint32_t mtu)
{
    uint32_t last = packet_len;
    if (mtu == 0) return ((last + 15u) & ~15u) - last;
    if (last > mtu) last %= mtu;
    uint32_t padded = (last + 15u) & ~15u;
    if (padded > mtu) padded = mtu;
    return padded - last;
}

uint32_t bnko_wg_encap(uint8_t *slot, uint32_t len, uint32_t mtu, const uint8_t key[32],
                       uint32_t remote_index, uint64_t counter)
{
    const uint32_t pad = bnko_wg_padding(len, mtu);
    st32le(slot, 4);                 /* type 4, three reserved zero bytes */
    st32le(slot + 4, remote_index);
    st32le(slot + 8, (uint32_t)counter);
    st32le(slot + 12, (uint32_t)(counter >> 32));
    memset(slot + 16 + len, 0, pad);
    uint8_t nonce[12];
    bnko_wg_nonce(counter, nonce);
    bnko_aead_seal(key, nonce, slot + 16, len + pad, NULL, 0, slot + 16);
    return 16 + len + pad + 16;
}

int bnko_wg_decap(const uint8_t *wire, uint32_t wire_len, const bnko_wg_peer *peers,
                  const uint8_t *keys_recv, uint32_t n_peers, uint8_t *out, uint32_t *out_len,
                  uint32_t *peer, uint64_t *counter)
{
    *out_len = 0;
    *peer = 0xFFFFFFFFu;
    *counter = 0;
    if (wire_len < 32 || ld32le(wire) != 4) return BNKO_WG_BAD_HEADER;
    const uint32_t idx = ld32le(wire + 4);
    uint32_t p = 0xFFFFFFFFu;
    for (uint32_t i = 0; i < n_peers; i++)
        if (peers[i].local_index == idx) {
            p = i;
            break;
        }
    if (p == 0xFFFFFFFFu) return BNKO_WG_UNKNOWN_INDEX;
    *peer = p;
    *counter = (uint64_t)ld32le(wire + 8) | (uint64_t)ld32le(wire + 12) << 32;
    uint8_t nonce[12];
    bnko_wg_nonce(*counter, nonce);
    const uint32_t plen = wire_len - 32;
    if (!bnko_aead_open(keys_recv + 32 * (size_t)p, nonce, wire + 16, wire_len - 16, NULL, 0, out))
        return BNKO_WG_AUTH_FAIL;
    if (plen == 0) return BNKO_WG_KEEPALIVE;
    const uint32_t version = out[0] >> 4;
    if (version == 4) {
        if (plen < 20) return BNKO_WG_BAD_IP;
        const uint32_t total = (uint32_t)out[2] << 8 | out[3];
        if (total > plen || total < 20) return BNKO_WG_BAD_IP;
        const uint32_t src = (uint32_t)out[12] << 24 | (uint32_t)out[13] << 16 |
                             (uint32_t)out[14] << 8 | out[15];
        if ((src & peers[p].allowed_mask) != (peers[p].allowed_net & peers[p].allowed_mask))
            return BNKO_WG_NOT_ALLOWED;
        *out_len = total;
        return BNKO_WG_OK;
    }
    if (version == 6) {
        if (plen < 40) return BNKO_WG_BAD_IP;
        const uint32_t total = ((uint32_t)out[4] << 8 | out[5]) + 40u;
        if (total > plen) return BNKO_WG_BAD_IP;
        return BNKO_WG_NOT_ALLOWED; /* bnk hands every peer one IPv4 /32 only */
    }
    return BNKO_WG_BAD_IP;
}

/* RFC 6479, ring of 128 64-bit blocks, window (128 - 1) * 64 = 8128 */
#define RING_BLOCKS 128u
#define BLOCK_BITS 64u
#define WINDOW ((RING_BLOCKS - 1u) * BLOCK_BITS)

void bnko_replay_reset(bnko_replay *f) { memset(f, 0, sizeof *f); }

int bnko_replay_validate(bnko_replay *f, uint64_t counter, uint64_t limit)
{
    if (counter >= limit) return 0;
    uint64_t index_block = counter >> 6;
    if (counter > f->last) {
        const uint64_t current = f->last >> 6;
        uint64_t diff = index_block - current;
        if (diff > RING_BLOCKS) diff = RING_BLOCKS;
        for (uint64_t i = current + 1; i <= current + diff; i++) f->ring[i & (RING_BLOCKS - 1u)] = 0;
        f->last = counter;
    } else if (f->last - counter > WINDOW) {
        return 0;
    }
    index_block &= RING_BLOCKS - 1u;
    const uint64_t bit = 1ull << (counter & (BLOCK_BITS - 1u));
    const uint64_t old = f->ring[index_block];
    f->ring[index_block] = old | bit;
    return (old & bit) == 0;
}
