/*
 * aead.c -- CPU restatement of RFC 8439 (ChaCha20, Poly1305,
 * AEAD_CHACHA20_POLY1305) and of the WireGuard transport nonce.
 *
 * Test infrastructure only: see bnk_oracle.h.  The arithmetic follows the
 * RFC text section by section; golang.org/x/crypto v0.55.0
 * chacha20poly1305 (reference go.mod:8), which wireguard-go calls for every
 * transport packet behind device.NewDevice
 * (reference internal/dataplane/engine.go:51), implements the same RFC.
 */
#include "bnk_oracle.h"

#include <pthread.h>
#include <stdlib.h>
#include <string.h>

typedef unsigned __int128 u128;

static uint32_t ld32(const uint8_t *p)
{
    return (uint32_t)p[0] | (uint32_t)p[1] << 8 | (uint32_t)p[2] << 16 |
           (uint32_t)p[3] << 24;
}
static uint64_t ld64(const uint8_t *p)
{
    return (uint64_t)ld32(p) | (uint64_t)ld32(p + 4) << 32;
}
static void st32(uint8_t *p, uint32_t v)
{
    p[0] = (uint8_t)v;
    p[1] = (uint8_t)(v >> 8);
    p[2] = (uint8_t)(v >> 16);
    p[3] = (uint8_t)(v >> 24);
}
static void st64(uint8_t *p, uint64_t v)
{
    st32(p, (uint32_t)v);
    st32(p + 4, (uint32_t)(v >> 32));
}
static uint32_t rotl(uint32_t v, int c) { return v << c | v >> (32 - c); }

/* RFC 8439 section 2.1 */
#define QR(a, b, c, d)      \
    do {                    \
        a += b;             \
        d ^= a;             \
        d = rotl(d, 16);    \
        c += d;             \
        b ^= c;             \
        b = rotl(b, 12);    \
        a += b;             \
        d ^= a;             \
        d = rotl(d, 8);     \
        c += d;             \
        b ^= c;             \
        b = rotl(b, 7);     \
    } while (0)

/* RFC 8439 section 2.3 */
void bnko_chacha20_block(const uint8_t key[32], uint32_t counter,
                         const uint8_t nonce[12], uint8_t out[64])
{
    uint32_t s[16], x[16];
    s[0] = 0x61707865;
    s[1] = 0x3320646e;
    s[2] = 0x79622d32;
    s[3] = 0x6b206574;
    for (int i = 0; i < 8; i++) s[4 + i] = ld32(key + 4 * i);
    s[12] = counter;
    for (int i = 0; i < 3; i++) s[13 + i] = ld32(nonce + 4 * i);
    memcpy(x, s, sizeof x);
    for (int i = 0; i < 10; i++) {
        QR(x[0], x[4], x[8], x[12]);
        QR(x[1], x[5], x[9], x[13]);
        QR(x[2], x[6], x[10], x[14]);
        QR(x[3], x[7], x[11], x[15]);
        QR(x[0], x[5], x[10], x[15]);
        QR(x[1], x[6], x[11], x[12]);
        QR(x[2], x[7], x[8], x[13]);
        QR(x[3], x[4], x[9], x[14]);
    }
    for (int i = 0; i < 16; i++) st32(out + 4 * i, x[i] + s[i]);
}

/* RFC 8439 section 2.4 */
void bnko_chacha20_xor(const uint8_t key[32], uint32_t counter,
                       const uint8_t nonce[12], const uint8_t *in,
                       uint8_t *out, size_t len)
{
    uint8_t ks[64];
    size_t pos = 0;
    while (pos < len) {
        size_t n = len - pos < 64 ? len - pos : 64;
        bnko_chacha20_block(key, counter++, nonce, ks);
        for (size_t i = 0; i < n; i++) out[pos + i] = in[pos + i] ^ ks[i];
        pos += n;
    }
}

/*
 * RFC 8439 section 2.5.  The accumulator is three 64-bit words
 * h = h0 + h1*2^64 + h2*2^128 with h2 kept tiny; r = r0 + r1*2^64 after the
 * clamp.  Because the clamp clears the low two bits of r1,
 * 2^128 * r1 = 2^130 * (r1/4) == 5 * (r1/4) (mod 2^130-5), so products that
 * land at 2^128 fold back with the multiplier s1 = r1 + r1/4.
 */
typedef struct {
    uint64_t r0, r1, s1;
    uint64_t h0, h1, h2;
    uint64_t pad0, pad1;
} poly_st;

static void poly_init(poly_st *st, const uint8_t key[32])
{
    st->r0 = ld64(key) & 0x0ffffffc0fffffffULL;
    st->r1 = ld64(key + 8) & 0x0ffffffc0ffffffcULL;
    st->s1 = st->r1 + (st->r1 >> 2);
    st->h0 = st->h1 = st->h2 = 0;
    st->pad0 = ld64(key + 16);
    st->pad1 = ld64(key + 24);
}

/* One 16-byte block with the given value for bit 128 (1 for every block
 * the RFC appends 0x01 to). */
static void poly_block(poly_st *st, uint64_t m0, uint64_t m1, uint64_t hibit)
{
    u128 t = (u128)st->h0 + m0;
    uint64_t h0 = (uint64_t)t;
    t = (u128)st->h1 + m1 + (uint64_t)(t >> 64);
    uint64_t h1 = (uint64_t)t;
    uint64_t h2 = st->h2 + hibit + (uint64_t)(t >> 64);

    u128 d0 = (u128)h0 * st->r0 + (u128)h1 * st->s1;
    u128 d1 = (u128)h0 * st->r1 + (u128)h1 * st->r0 + (u128)(h2 * st->s1);
    uint64_t d2 = h2 * st->r0;

    d1 += (uint64_t)(d0 >> 64);
    h0 = (uint64_t)d0;
    h1 = (uint64_t)d1;
    h2 = d2 + (uint64_t)(d1 >> 64);

    /* fold everything at and above 2^130 back in, times 5 */
    uint64_t c = (h2 >> 2) * 5;
    h2 &= 3;
    t = (u128)h0 + c;
    h0 = (uint64_t)t;
    t = (u128)h1 + (uint64_t)(t >> 64);
    h1 = (uint64_t)t;
    h2 += (uint64_t)(t >> 64);
    st->h0 = h0;
    st->h1 = h1;
    st->h2 = h2;
}

static void poly_update(poly_st *st, const uint8_t *m, size_t len)
{
    while (len >= 16) {
        poly_block(st, ld64(m), ld64(m + 8), 1);
        m += 16;
        len -= 16;
    }
    if (len) {
        /* RFC 2.5.1: append 0x01 then zero-pad to 17 bytes */
        uint8_t buf[16] = {0};
        memcpy(buf, m, len);
        buf[len] = 1;
        poly_block(st, ld64(buf), ld64(buf + 8), 0);
    }
}

static void poly_finish(poly_st *st, uint8_t tag[16])
{
    /* full reduction mod 2^130-5: h >= p  <=>  h + 5 >= 2^130 */
    uint64_t h0 = st->h0, h1 = st->h1, h2 = st->h2;
    u128 t = (u128)h0 + 5;
    uint64_t g0 = (uint64_t)t;
    t = (u128)h1 + (uint64_t)(t >> 64);
    uint64_t g1 = (uint64_t)t;
    uint64_t g2 = h2 + (uint64_t)(t >> 64);
    if (g2 >> 2) {
        h0 = g0;
        h1 = g1;
    }
    /* tag = (h + s) mod 2^128 */
    t = (u128)h0 + st->pad0;
    h0 = (uint64_t)t;
    h1 = h1 + st->pad1 + (uint64_t)(t >> 64);
    st64(tag, h0);
    st64(tag + 8, h1);
}

void bnko_poly1305(const uint8_t key[32], const uint8_t *msg, size_t len,
                   uint8_t tag[16])
{
    poly_st st;
    poly_init(&st, key);
    poly_update(&st, msg, len);
    poly_finish(&st, tag);
}

/* RFC 8439 section 2.6 */
void bnko_poly1305_keygen(const uint8_t key[32], const uint8_t nonce[12],
                          uint8_t otk[32])
{
    uint8_t blk[64];
    bnko_chacha20_block(key, 0, nonce, blk);
    memcpy(otk, blk, 32);
}

/* RFC 8439 section 2.8: mac_data = aad | pad16 | ct | pad16 | len(aad) |
 * len(ct), both lengths 64-bit little-endian. */
static void aead_tag(const uint8_t otk[32], const uint8_t *aad, size_t aad_len,
                     const uint8_t *ct, size_t len, uint8_t tag[16])
{
    poly_st st;
    uint8_t lens[16];
    poly_init(&st, otk);
    /* zero padding makes every data block a full 16-byte block, so each
     * gets the 2^128 bit; feed whole blocks, then the padded remainder */
    size_t full = aad_len & ~(size_t)15;
    poly_update(&st, aad, full);
    if (aad_len & 15) {
        uint8_t b[16] = {0};
        memcpy(b, aad + full, aad_len & 15);
        poly_update(&st, b, 16);
    }
    full = len & ~(size_t)15;
    poly_update(&st, ct, full);
    if (len & 15) {
        uint8_t b[16] = {0};
        memcpy(b, ct + full, len & 15);
        poly_update(&st, b, 16);
    }
    st64(lens, (uint64_t)aad_len);
    st64(lens + 8, (uint64_t)len);
    poly_update(&st, lens, 16);
    poly_finish(&st, tag);
}

void bnko_aead_seal(const uint8_t key[32], const uint8_t nonce[12],
                    const uint8_t *pt, size_t len, const uint8_t *aad,
                    size_t aad_len, uint8_t *out)
{
    uint8_t otk[32];
    bnko_poly1305_keygen(key, nonce, otk);
    bnko_chacha20_xor(key, 1, nonce, pt, out, len);
    aead_tag(otk, aad, aad_len, out, len, out + len);
}

int bnko_aead_open(const uint8_t key[32], const uint8_t nonce[12],
                   const uint8_t *ct, size_t ct_len, const uint8_t *aad,
                   size_t aad_len, uint8_t *out)
{
    if (ct_len < 16) return 0;
    size_t len = ct_len - 16;
    uint8_t otk[32], tag[16];
    bnko_poly1305_keygen(key, nonce, otk);
    aead_tag(otk, aad, aad_len, ct, len, tag);
    /* compare all 16 bytes, no early exit */
    uint8_t diff = 0;
    for (int i = 0; i < 16; i++) diff |= tag[i] ^ ct[len + i];
    if (diff) {
        memset(out, 0, len);
        return 0;
    }
    bnko_chacha20_xor(key, 1, nonce, ct, out, len);
    return 1;
}

void bnko_wg_nonce(uint64_t counter, uint8_t nonce[12])
{
    memset(nonce, 0, 4);
    st64(nonce + 4, counter);
}

/* ---------------- batches ---------------- */

typedef struct {
    int open;
    const uint8_t *keys;
    const uint32_t *peer;
    const uint64_t *counters;
    const uint8_t *in;
    const uint64_t *in_off;
    const uint32_t *in_len;
    uint8_t *out;
    const uint64_t *out_off;
    uint8_t *verdict;
    uint32_t lo, hi;
} batch_job;

static void *batch_run(void *arg)
{
    batch_job *j = (batch_job *)arg;
    for (uint32_t i = j->lo; i < j->hi; i++) {
        const uint8_t *key = j->keys + 32 * (size_t)(j->peer ? j->peer[i] : 0);
        uint8_t nonce[12];
        bnko_wg_nonce(j->counters[i], nonce);
        const uint8_t *src = j->in + j->in_off[i];
        uint8_t *dst = j->out + j->out_off[i];
        if (j->open)
            j->verdict[i] = (uint8_t)bnko_aead_open(key, nonce, src,
                                                    j->in_len[i], NULL, 0, dst);
        else
            bnko_aead_seal(key, nonce, src, j->in_len[i], NULL, 0, dst);
    }
    return NULL;
}

static void batch_dispatch(batch_job *proto, uint32_t n, int nthreads)
{
    if (nthreads < 1) nthreads = 1;
    if ((uint32_t)nthreads > n) nthreads = n ? (int)n : 1;
    if (nthreads == 1) {
        proto->lo = 0;
        proto->hi = n;
        batch_run(proto);
        return;
    }
    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)nthreads);
    batch_job *jobs = (batch_job *)malloc(sizeof(batch_job) * (size_t)nthreads);
    for (int t = 0; t < nthreads; t++) {
        jobs[t] = *proto;
        jobs[t].lo = (uint32_t)((uint64_t)n * (uint64_t)t / (uint64_t)nthreads);
        jobs[t].hi =
            (uint32_t)((uint64_t)n * (uint64_t)(t + 1) / (uint64_t)nthreads);
        pthread_create(&th[t], NULL, batch_run, &jobs[t]);
    }
    for (int t = 0; t < nthreads; t++) pthread_join(th[t], NULL);
    free(jobs);
    free(th);
}

void bnko_seal_batch(const uint8_t *keys, const uint32_t *peer,
                     const uint64_t *counters, const uint8_t *in,
                     const uint64_t *in_off, const uint32_t *in_len,
                     uint8_t *out, const uint64_t *out_off, uint32_t n,
                     int nthreads)
{
    batch_job j = {0,  keys, peer,    counters, in, in_off,
                   in_len, out,  out_off, NULL,     0,  0};
    batch_dispatch(&j, n, nthreads);
}

void bnko_open_batch(const uint8_t *keys, const uint32_t *peer,
                     const uint64_t *counters, const uint8_t *in,
                     const uint64_t *in_off, const uint32_t *in_len,
                     uint8_t *out, const uint64_t *out_off, uint8_t *verdict,
                     uint32_t n, int nthreads)
{
    batch_job j = {1,  keys, peer,    counters, in, in_off,
                   in_len, out,  out_off, verdict,  0,  0};
    batch_dispatch(&j, n, nthreads);
}
