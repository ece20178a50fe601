// Per-lane ChaCha20-Poly1305 building blocks for gfx950.
//
// One lane owns one packet end to end: the 16-word ChaCha20 state and the
// Poly1305 accumulator stay in VGPRs for the packet's whole life, there is no
// cross-lane traffic and no LDS.  32-bit add/xor/rotate (v_alignbit_b32) for
// ChaCha20; Poly1305 with v_mad_u64_u32 partial products (radix 2^32 in the
// kernels; the radix 2^26 layout is kept as an independent cross-check).
#pragma once

#include <stdint.h>

// The arithmetic in this header is plain 32/64-bit integer C++, so the same
// source also compiles for the host: tests/cpp/lane_test.cpp runs it on the
// CPU against the RFC 8439 vectors (including Poly1305 carry edge cases that
// random packets never reach).  The library itself only ever uses it on the GPU.
#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define BNK_DEV __device__ __forceinline__
#else
#define BNK_DEV inline
#endif

namespace bnk {

BNK_DEV uint32_t rotl32(uint32_t v, int c) { return v << c | v >> (32 - c); }
// low 32 bits of (hi:lo) >> s, 0 < s < 32 (one v_alignbit_b32 on the GPU)
BNK_DEV uint32_t funnel(uint32_t hi, uint32_t lo, int s) { return lo >> s | hi << (32 - s); }
// a + b + cin (cin 0 or 1) as 32 bits and a carry
BNK_DEV uint32_t addc32(uint32_t a, uint32_t b, uint32_t cin, uint32_t &cout)
{
#if defined(__HIP_DEVICE_COMPILE__)
    unsigned int co;
    const uint32_t r = __builtin_addc(a, b, cin, &co);
    cout = co;
    return r;
#else
    const uint64_t t = (uint64_t)a + b + cin;
    cout = (uint32_t)(t >> 32);
    return (uint32_t)t;
#endif
}

#if defined(__HIP_DEVICE_COMPILE__)
// Four quarter rounds side by side.  A SIMD issues adds and xors of two waves
// together but rotates (v_alignbit_b32) of one wave at a time, and serves its
// older wave first: the younger wave's rotates then wait about four of the
// older wave's issue slots each.  The four rotates of a step therefore run at
// raised wave priority, so that whichever wave is rotating owns the SIMD and the
// other fills in with its adds and xors (measured on the bare quarter-round
// stream at two waves per SIMD: 41.9 -> 50.1 T lane-instructions/s).
#define BNK_ROT4(n, a, b, c, d)                                                        \
    asm volatile("s_setprio 1\n\t"                                                     \
                 "v_alignbit_b32 %0, %0, %0, " #n "\n\tv_alignbit_b32 %1, %1, %1, " #n "\n\t" \
                 "v_alignbit_b32 %2, %2, %2, " #n "\n\tv_alignbit_b32 %3, %3, %3, " #n "\n\t" \
                 "s_setprio 0"                                                         \
                 : "+v"(a), "+v"(b), "+v"(c), "+v"(d))
#define BNK_QR4(a0, b0, c0, d0, a1, b1, c1, d1, a2, b2, c2, d2, a3, b3, c3, d3)       \
    a0 += b0; a1 += b1; a2 += b2; a3 += b3; d0 ^= a0; d1 ^= a1; d2 ^= a2; d3 ^= a3;    \
    BNK_ROT4(16, d0, d1, d2, d3);                                                      \
    c0 += d0; c1 += d1; c2 += d2; c3 += d3; b0 ^= c0; b1 ^= c1; b2 ^= c2; b3 ^= c3;    \
    BNK_ROT4(20, b0, b1, b2, b3);                                                      \
    a0 += b0; a1 += b1; a2 += b2; a3 += b3; d0 ^= a0; d1 ^= a1; d2 ^= a2; d3 ^= a3;    \
    BNK_ROT4(24, d0, d1, d2, d3);                                                      \
    c0 += d0; c1 += d1; c2 += d2; c3 += d3; b0 ^= c0; b1 ^= c1; b2 ^= c2; b3 ^= c3;    \
    BNK_ROT4(25, b0, b1, b2, b3)
// The same for two blocks side by side: eight rotates per pair of priority changes.
#define BNK_ROT8(n, a, b, c, d, e, f, g, h)                                            \
    asm volatile("s_setprio 1\n\t"                                                     \
                 "v_alignbit_b32 %0, %0, %0, " #n "\n\tv_alignbit_b32 %1, %1, %1, " #n "\n\t" \
                 "v_alignbit_b32 %2, %2, %2, " #n "\n\tv_alignbit_b32 %3, %3, %3, " #n "\n\t" \
                 "v_alignbit_b32 %4, %4, %4, " #n "\n\tv_alignbit_b32 %5, %5, %5, " #n "\n\t" \
                 "v_alignbit_b32 %6, %6, %6, " #n "\n\tv_alignbit_b32 %7, %7, %7, " #n "\n\t" \
                 "s_setprio 0"                                                         \
                 : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(e), "+v"(f), "+v"(g), "+v"(h))
#define BNK_HALF8(x, y, a0, b0, d0, a1, b1, d1, a2, b2, d2, a3, b3, d3, n)             \
    x[a0] += x[b0]; x[a1] += x[b1]; x[a2] += x[b2]; x[a3] += x[b3];                    \
    x[d0] ^= x[a0]; x[d1] ^= x[a1]; x[d2] ^= x[a2]; x[d3] ^= x[a3];                    \
    y[a0] += y[b0]; y[a1] += y[b1]; y[a2] += y[b2]; y[a3] += y[b3];                    \
    y[d0] ^= y[a0]; y[d1] ^= y[a1]; y[d2] ^= y[a2]; y[d3] ^= y[a3];                    \
    BNK_ROT8(n, x[d0], x[d1], x[d2], x[d3], y[d0], y[d1], y[d2], y[d3])
#define BNK_QR8(x, y, a0, b0, c0, d0, a1, b1, c1, d1, a2, b2, c2, d2, a3, b3, c3, d3)  \
    BNK_HALF8(x, y, a0, b0, d0, a1, b1, d1, a2, b2, d2, a3, b3, d3, 16);               \
    BNK_HALF8(x, y, c0, d0, b0, c1, d1, b1, c2, d2, b2, c3, d3, b3, 20);               \
    BNK_HALF8(x, y, a0, b0, d0, a1, b1, d1, a2, b2, d2, a3, b3, d3, 24);               \
    BNK_HALF8(x, y, c0, d0, b0, c1, d1, b1, c2, d2, b2, c3, d3, b3, 25)
#else
#define BNK_QR(a, b, c, d)                          \
    a += b; d ^= a; d = rotl32(d, 16);              \
    c += d; b ^= c; b = rotl32(b, 12);              \
    a += b; d ^= a; d = rotl32(d, 8);               \
    c += d; b ^= c; b = rotl32(b, 7)
#define BNK_QR4(a0, b0, c0, d0, a1, b1, c1, d1, a2, b2, c2, d2, a3, b3, c3, d3)       \
    BNK_QR(a0, b0, c0, d0); BNK_QR(a1, b1, c1, d1); BNK_QR(a2, b2, c2, d2); BNK_QR(a3, b3, c3, d3)
#define BNK_QR8(x, y, a0, b0, c0, d0, a1, b1, c1, d1, a2, b2, c2, d2, a3, b3, c3, d3)  \
    BNK_QR4(x[a0], x[b0], x[c0], x[d0], x[a1], x[b1], x[c1], x[d1], x[a2], x[b2], x[c2], x[d2], x[a3], x[b3], x[c3], x[d3]); \
    BNK_QR4(y[a0], y[b0], y[c0], y[d0], y[a1], y[b1], y[c1], y[d1], y[a2], y[b2], y[c2], y[d2], y[a3], y[b3], y[c3], y[d3])
#endif

// RFC 8439 section 2.3 with the WireGuard nonce: words 13..15 of the state
// are 0, counter low, counter high.
BNK_DEV void chacha_block(const uint32_t (&k)[8], uint32_t blk, uint32_t n1,
                          uint32_t n2, uint32_t (&x)[16])
{
    x[0] = 0x61707865u; x[1] = 0x3320646eu; x[2] = 0x79622d32u; x[3] = 0x6b206574u;
#pragma unroll
    for (int i = 0; i < 8; i++) x[4 + i] = k[i];
    x[12] = blk; x[13] = 0; x[14] = n1; x[15] = n2;
#pragma unroll 1
    for (int r = 0; r < 10; r++) {
        BNK_QR4(x[0], x[4], x[8], x[12], x[1], x[5], x[9], x[13], x[2], x[6], x[10], x[14], x[3], x[7], x[11], x[15]);
        BNK_QR4(x[0], x[5], x[10], x[15], x[1], x[6], x[11], x[12], x[2], x[7], x[8], x[13], x[3], x[4], x[9], x[14]);
    }
    x[0] += 0x61707865u; x[1] += 0x3320646eu; x[2] += 0x79622d32u; x[3] += 0x6b206574u;
#pragma unroll
    for (int i = 0; i < 8; i++) x[4 + i] += k[i];
    x[12] += blk; x[14] += n1; x[15] += n2;
}

// Blocks blk and blk + 1 at once, their rounds interleaved.
BNK_DEV void chacha_block2(const uint32_t (&k)[8], uint32_t blk, uint32_t n1, uint32_t n2,
                           uint32_t (&x)[16], uint32_t (&y)[16])
{
    x[0] = y[0] = 0x61707865u; x[1] = y[1] = 0x3320646eu; x[2] = y[2] = 0x79622d32u; x[3] = y[3] = 0x6b206574u;
#pragma unroll
    for (int i = 0; i < 8; i++) x[4 + i] = y[4 + i] = k[i];
    x[12] = blk; y[12] = blk + 1u; x[13] = y[13] = 0; x[14] = y[14] = n1; x[15] = y[15] = n2;
#pragma unroll 1
    for (int r = 0; r < 10; r++) {
        BNK_QR8(x, y, 0, 4, 8, 12, 1, 5, 9, 13, 2, 6, 10, 14, 3, 7, 11, 15);
        BNK_QR8(x, y, 0, 5, 10, 15, 1, 6, 11, 12, 2, 7, 8, 13, 3, 4, 9, 14);
    }
    x[0] += 0x61707865u; x[1] += 0x3320646eu; x[2] += 0x79622d32u; x[3] += 0x6b206574u;
    y[0] += 0x61707865u; y[1] += 0x3320646eu; y[2] += 0x79622d32u; y[3] += 0x6b206574u;
#pragma unroll
    for (int i = 0; i < 8; i++) { x[4 + i] += k[i]; y[4 + i] += k[i]; }
    x[12] += blk; y[12] += blk + 1u; x[14] += n1; y[14] += n1; x[15] += n2; y[15] += n2;
}

// What the blocks of one packet share: the block counter sits in the first column of
// the state, so the first column round leaves the other three columns the same for
// every block, and the first addition of the first column as well.
struct ChachaShared {
    uint32_t a0;     // constant 0 + key word 0
    uint32_t col[12]; // words 1, 5, 9, 13, 2, 6, 10, 14, 3, 7, 11, 15 after the first column round
};

BNK_DEV void chacha_shared(const uint32_t (&k)[8], uint32_t n1, uint32_t n2, ChachaShared &sh)
{
    const uint32_t c[4] = {0x61707865u, 0x3320646eu, 0x79622d32u, 0x6b206574u};
    const uint32_t n[4] = {0, 0, n1, n2};
    sh.a0 = c[0] + k[0];
#pragma unroll
    for (int j = 1; j < 4; j++) {
        uint32_t a = c[j], b = k[j], cc = k[4 + j], d = n[j];
        a += b; d ^= a; d = rotl32(d, 16);
        cc += d; b ^= cc; b = rotl32(b, 12);
        a += b; d ^= a; d = rotl32(d, 8);
        cc += d; b ^= cc; b = rotl32(b, 7);
        sh.col[4 * (j - 1)] = a; sh.col[4 * (j - 1) + 1] = b; sh.col[4 * (j - 1) + 2] = cc; sh.col[4 * (j - 1) + 3] = d;
    }
}

// chacha_block2 from what the packet's blocks share: the first column round is only
// the counter's column, once per block.
BNK_DEV void chacha_block2_shared(const uint32_t (&k)[8], const ChachaShared &sh, uint32_t blk, uint32_t n1,
                                  uint32_t n2, uint32_t (&x)[16], uint32_t (&y)[16])
{
    x[0] = y[0] = sh.a0;
    x[12] = rotl32(blk ^ x[0], 16); y[12] = rotl32((blk + 1u) ^ y[0], 16);
    x[8] = k[4] + x[12]; y[8] = k[4] + y[12];
    x[4] = rotl32(k[0] ^ x[8], 12); y[4] = rotl32(k[0] ^ y[8], 12);
    x[0] += x[4]; y[0] += y[4];
    x[12] = rotl32(x[12] ^ x[0], 8); y[12] = rotl32(y[12] ^ y[0], 8);
    x[8] += x[12]; y[8] += y[12];
    x[4] = rotl32(x[4] ^ x[8], 7); y[4] = rotl32(y[4] ^ y[8], 7);
#pragma unroll
    for (int j = 1; j < 4; j++) {
        x[j] = y[j] = sh.col[4 * (j - 1)];
        x[4 + j] = y[4 + j] = sh.col[4 * (j - 1) + 1];
        x[8 + j] = y[8 + j] = sh.col[4 * (j - 1) + 2];
        x[12 + j] = y[12 + j] = sh.col[4 * (j - 1) + 3];
    }
    BNK_QR8(x, y, 0, 5, 10, 15, 1, 6, 11, 12, 2, 7, 8, 13, 3, 4, 9, 14);
#pragma unroll 1
    for (int r = 1; r < 10; r++) {
        BNK_QR8(x, y, 0, 4, 8, 12, 1, 5, 9, 13, 2, 6, 10, 14, 3, 7, 11, 15);
        BNK_QR8(x, y, 0, 5, 10, 15, 1, 6, 11, 12, 2, 7, 8, 13, 3, 4, 9, 14);
    }
    x[0] += 0x61707865u; x[1] += 0x3320646eu; x[2] += 0x79622d32u; x[3] += 0x6b206574u;
    y[0] += 0x61707865u; y[1] += 0x3320646eu; y[2] += 0x79622d32u; y[3] += 0x6b206574u;
#pragma unroll
    for (int i = 0; i < 8; i++) { x[4 + i] += k[i]; y[4 + i] += k[i]; }
    x[12] += blk; y[12] += blk + 1u; x[14] += n1; y[14] += n1; x[15] += n2; y[15] += n2;
}

// Poly1305 (RFC 8439 section 2.5), radix 2^26.
struct Poly26 {
    uint32_t r0, r1, r2, r3, r4;
    uint32_t s1, s2, s3, s4; // 5 * r
    uint32_t h0, h1, h2, h3, h4;
    uint32_t pad0, pad1, pad2, pad3;

    // otk = first 8 words of ChaCha20 block 0
    BNK_DEV void init(const uint32_t (&x)[16])
    {
        const uint32_t t0 = x[0] & 0x0fffffffu, t1 = x[1] & 0x0ffffffcu;
        const uint32_t t2 = x[2] & 0x0ffffffcu, t3 = x[3] & 0x0ffffffcu;
        r0 = t0 & 0x3ffffffu;
        r1 = ((t0 >> 26) | (t1 << 6)) & 0x3ffffffu;
        r2 = ((t1 >> 20) | (t2 << 12)) & 0x3ffffffu;
        r3 = ((t2 >> 14) | (t3 << 18)) & 0x3ffffffu;
        r4 = t3 >> 8;
        s1 = r1 * 5; s2 = r2 * 5; s3 = r3 * 5; s4 = r4 * 5;
        h0 = h1 = h2 = h3 = h4 = 0;
        pad0 = x[4]; pad1 = x[5]; pad2 = x[6]; pad3 = x[7];
    }

    // One full 16-byte block (little-endian words w0..w3) with bit 128 set.
    BNK_DEV void block(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3)
    {
        const uint32_t a0 = h0 + (w0 & 0x3ffffffu);
        const uint32_t a1 = h1 + (funnel(w1, w0, 26) & 0x3ffffffu);
        const uint32_t a2 = h2 + (funnel(w2, w1, 20) & 0x3ffffffu);
        const uint32_t a3 = h3 + (funnel(w3, w2, 14) & 0x3ffffffu);
        const uint32_t a4 = h4 + ((w3 >> 8) | (1u << 24));

        uint64_t d0 = (uint64_t)a0 * r0 + (uint64_t)a1 * s4 + (uint64_t)a2 * s3 +
                      (uint64_t)a3 * s2 + (uint64_t)a4 * s1;
        uint64_t d1 = (uint64_t)a0 * r1 + (uint64_t)a1 * r0 + (uint64_t)a2 * s4 +
                      (uint64_t)a3 * s3 + (uint64_t)a4 * s2;
        uint64_t d2 = (uint64_t)a0 * r2 + (uint64_t)a1 * r1 + (uint64_t)a2 * r0 +
                      (uint64_t)a3 * s4 + (uint64_t)a4 * s3;
        uint64_t d3 = (uint64_t)a0 * r3 + (uint64_t)a1 * r2 + (uint64_t)a2 * r1 +
                      (uint64_t)a3 * r0 + (uint64_t)a4 * s4;
        uint64_t d4 = (uint64_t)a0 * r4 + (uint64_t)a1 * r3 + (uint64_t)a2 * r2 +
                      (uint64_t)a3 * r1 + (uint64_t)a4 * r0;

        uint32_t c;
        c = (uint32_t)(d0 >> 26); h0 = (uint32_t)d0 & 0x3ffffffu; d1 += c;
        c = (uint32_t)(d1 >> 26); h1 = (uint32_t)d1 & 0x3ffffffu; d2 += c;
        c = (uint32_t)(d2 >> 26); h2 = (uint32_t)d2 & 0x3ffffffu; d3 += c;
        c = (uint32_t)(d3 >> 26); h3 = (uint32_t)d3 & 0x3ffffffu; d4 += c;
        c = (uint32_t)(d4 >> 26); h4 = (uint32_t)d4 & 0x3ffffffu;
        h0 += c * 5;
        c = h0 >> 26; h0 &= 0x3ffffffu;
        h1 += c;
    }

    // tag = ((h mod 2^130-5) + s) mod 2^128 as four little-endian words
    BNK_DEV void finish(uint32_t (&tag)[4])
    {
        uint32_t c;
        c = h1 >> 26; h1 &= 0x3ffffffu; h2 += c;
        c = h2 >> 26; h2 &= 0x3ffffffu; h3 += c;
        c = h3 >> 26; h3 &= 0x3ffffffu; h4 += c;
        c = h4 >> 26; h4 &= 0x3ffffffu; h0 += c * 5;
        c = h0 >> 26; h0 &= 0x3ffffffu; h1 += c;

        // g = h + 5 - 2^130; keep g when it did not go negative (h >= p)
        uint32_t g0 = h0 + 5; c = g0 >> 26; g0 &= 0x3ffffffu;
        uint32_t g1 = h1 + c; c = g1 >> 26; g1 &= 0x3ffffffu;
        uint32_t g2 = h2 + c; c = g2 >> 26; g2 &= 0x3ffffffu;
        uint32_t g3 = h3 + c; c = g3 >> 26; g3 &= 0x3ffffffu;
        uint32_t g4 = h4 + c - (1u << 26);
        const uint32_t take_g = (g4 >> 31) - 1; // all ones when g4 >= 0
        h0 = (h0 & ~take_g) | (g0 & take_g);
        h1 = (h1 & ~take_g) | (g1 & take_g);
        h2 = (h2 & ~take_g) | (g2 & take_g);
        h3 = (h3 & ~take_g) | (g3 & take_g);
        h4 = (h4 & ~take_g) | (g4 & take_g);

        const uint32_t w0 = h0 | (h1 << 26);
        const uint32_t w1 = (h1 >> 6) | (h2 << 20);
        const uint32_t w2 = (h2 >> 12) | (h3 << 14);
        const uint32_t w3 = (h3 >> 18) | (h4 << 8);
        uint64_t f;
        f = (uint64_t)w0 + pad0;             tag[0] = (uint32_t)f;
        f = (uint64_t)w1 + pad1 + (f >> 32); tag[1] = (uint32_t)f;
        f = (uint64_t)w2 + pad2 + (f >> 32); tag[2] = (uint32_t)f;
        f = (uint64_t)w3 + pad3 + (f >> 32); tag[3] = (uint32_t)f;
    }
};

// Poly1305 in radix 2^32: the accumulator is four 32-bit words plus a small
// fifth, r is its four clamped words.  The clamp clears the low two bits of
// r1..r3, so a product that lands at 2^128 or above folds back exactly with
// s_j = r_j + r_j/4 = 5*r_j/4 (2^130 = 5 mod p).  Message words are used as
// they are: no limb extraction, 20 multiplies per block.
struct Poly32 {
    uint32_t r0, r1, r2, r3;
    uint32_t s1, s2, s3;
    uint32_t h0, h1, h2, h3, h4;
    uint32_t pad0, pad1, pad2, pad3;

    // otk = first 8 words of ChaCha20 block 0
    BNK_DEV void init(const uint32_t (&x)[16])
    {
        r0 = x[0] & 0x0fffffffu; r1 = x[1] & 0x0ffffffcu;
        r2 = x[2] & 0x0ffffffcu; r3 = x[3] & 0x0ffffffcu;
        s1 = r1 + (r1 >> 2); s2 = r2 + (r2 >> 2); s3 = r3 + (r3 >> 2);
        h0 = h1 = h2 = h3 = h4 = 0;
        pad0 = x[4]; pad1 = x[5]; pad2 = x[6]; pad3 = x[7];
    }

    // One full 16-byte block (little-endian words w0..w3) with bit 128 set.
    // Additions go 32 bits at a time with an explicit carry (add-with-carry
    // instructions on the GPU; written as 64-bit sums the compiler builds each
    // zero-extended operand with a move first: 68 instructions a block against 47).
    // The block runs at raised wave priority for the same reason as the rotates of
    // ChaCha20: nearly all of it is multiplies and carries, which a SIMD takes
    // from one wave at a time.
    BNK_DEV void block(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        __builtin_amdgcn_s_setprio(1);
#endif
        uint32_t c;
        const uint32_t a0 = addc32(h0, w0, 0, c);
        const uint32_t a1 = addc32(h1, w1, c, c);
        const uint32_t a2 = addc32(h2, w2, c, c);
        const uint32_t a3 = addc32(h3, w3, c, c);
        const uint32_t a4 = h4 + 1u + c; // at most 9

        // a_i < 2^32, r_j < 2^28, s_j < 1.25 * 2^28: four terms stay below 2^63,
        // and a4 * s_j below 2^32
        const uint64_t d0 = (uint64_t)a0 * r0 + (uint64_t)a1 * s3 + (uint64_t)a2 * s2 + (uint64_t)a3 * s1;
        const uint64_t d1 = (uint64_t)a0 * r1 + (uint64_t)a1 * r0 + (uint64_t)a2 * s3 + (uint64_t)a3 * s2 +
                            (uint64_t)a4 * s1;
        const uint64_t d2 = (uint64_t)a0 * r2 + (uint64_t)a1 * r1 + (uint64_t)a2 * r0 + (uint64_t)a3 * s3 +
                            (uint64_t)a4 * s2;
        const uint64_t d3 = (uint64_t)a0 * r3 + (uint64_t)a1 * r2 + (uint64_t)a2 * r1 + (uint64_t)a3 * r0 +
                            (uint64_t)a4 * s3;
        uint32_t e4 = a4 * r0; // stays at 2^128; below 2^32 because a4 <= 9

        // each column's upper half goes into the next column
        const uint32_t l1 = addc32((uint32_t)d1, (uint32_t)(d0 >> 32), 0, c);
        const uint32_t u1 = (uint32_t)(d1 >> 32) + c;
        const uint32_t l2 = addc32((uint32_t)d2, u1, 0, c);
        const uint32_t u2 = (uint32_t)(d2 >> 32) + c;
        const uint32_t l3 = addc32((uint32_t)d3, u2, 0, c);
        const uint32_t u3 = (uint32_t)(d3 >> 32) + c;
        e4 += u3;
        // everything at and above 2^130 comes back times 5
        const uint32_t f = (e4 >> 2) * 5u;
        h0 = addc32((uint32_t)d0, f, 0, c);
        h1 = addc32(l1, 0, c, c);
        h2 = addc32(l2, 0, c, c);
        h3 = addc32(l3, 0, c, c);
        h4 = (e4 & 3u) + c;
#if defined(__HIP_DEVICE_COMPILE__)
        __builtin_amdgcn_s_setprio(0);
#endif
    }

    // tag = ((h mod 2^130-5) + s) mod 2^128 as four little-endian words
    BNK_DEV void finish(uint32_t (&tag)[4])
    {
        // h < 2^130 + small: h >= p  <=>  h + 5 >= 2^130
        uint64_t t;
        t = (uint64_t)h0 + 5u;         const uint32_t g0 = (uint32_t)t;
        t = (uint64_t)h1 + (t >> 32);  const uint32_t g1 = (uint32_t)t;
        t = (uint64_t)h2 + (t >> 32);  const uint32_t g2 = (uint32_t)t;
        t = (uint64_t)h3 + (t >> 32);  const uint32_t g3 = (uint32_t)t;
        const uint32_t g4 = h4 + (uint32_t)(t >> 32);
        const uint32_t take_g = 0u - (uint32_t)((g4 >> 2) != 0); // all ones when h + 5 >= 2^130
        const uint32_t f0 = (h0 & ~take_g) | (g0 & take_g);
        const uint32_t f1 = (h1 & ~take_g) | (g1 & take_g);
        const uint32_t f2 = (h2 & ~take_g) | (g2 & take_g);
        const uint32_t f3 = (h3 & ~take_g) | (g3 & take_g);
        t = (uint64_t)f0 + pad0;             tag[0] = (uint32_t)t;
        t = (uint64_t)f1 + pad1 + (t >> 32); tag[1] = (uint32_t)t;
        t = (uint64_t)f2 + pad2 + (t >> 32); tag[2] = (uint32_t)t;
        t = (uint64_t)f3 + pad3 + (t >> 32); tag[3] = (uint32_t)t;
    }
};

// ---------------------------------------------------------------------------
// One packet spread over the lanes of a wave (small batches, where a packet
// per lane would leave the chip empty and a call would last as long as one
// lane takes for a whole packet).  Lane 0 runs ChaCha20 block 0 (the one-time
// key) and owns the AEAD length block, lane l >= 1 owns keystream block l and
// its four 16-byte cells.  With C MAC cells m_0 .. m_{C-1} the tag is
// sum m_j r^(C-j) + s: each lane evaluates its own cells by Horner's rule,
// lifts the result by r^(cells after its last one), and the lanes' terms are
// added.  General multipliers (powers of r are not clamped) need the radix
// 2^26 form.
// ---------------------------------------------------------------------------

// Element of GF(2^130 - 5), five limbs of 26 bits; arithmetic keeps limbs
// below 2^27 and accepts limbs below 2^28 in the left operand of fe_mul.
struct Fe26 {
    uint32_t v0, v1, v2, v3, v4;
};

BNK_DEV Fe26 fe_small(uint32_t x) { return Fe26{x, 0, 0, 0, 0}; }

// A 16-byte cell (little-endian words) with bit 128 set.
BNK_DEV Fe26 fe_cell(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3)
{
    return Fe26{w0 & 0x3ffffffu, funnel(w1, w0, 26) & 0x3ffffffu, funnel(w2, w1, 20) & 0x3ffffffu,
                funnel(w3, w2, 14) & 0x3ffffffu, (w3 >> 8) | (1u << 24)};
}

// r from the first four words of ChaCha20 block 0, clamped.
BNK_DEV Fe26 fe_clamped_r(uint32_t x0, uint32_t x1, uint32_t x2, uint32_t x3)
{
    Fe26 r = fe_cell(x0 & 0x0fffffffu, x1 & 0x0ffffffcu, x2 & 0x0ffffffcu, x3 & 0x0ffffffcu);
    r.v4 &= 0xffffffu; // no bit 128
    return r;
}

BNK_DEV Fe26 fe_add(const Fe26 &a, const Fe26 &b)
{
    return Fe26{a.v0 + b.v0, a.v1 + b.v1, a.v2 + b.v2, a.v3 + b.v3, a.v4 + b.v4};
}

BNK_DEV Fe26 fe_select(bool take_a, const Fe26 &a, const Fe26 &b)
{
    return Fe26{take_a ? a.v0 : b.v0, take_a ? a.v1 : b.v1, take_a ? a.v2 : b.v2,
                take_a ? a.v3 : b.v3, take_a ? a.v4 : b.v4};
}

// a * b mod 2^130 - 5.  a's limbs below 2^28, b's below 2^27: a product is
// below 2^28 * 5 * 2^27 < 2^58 and five of them stay below 2^61.
BNK_DEV Fe26 fe_mul(const Fe26 &a, const Fe26 &b)
{
    const uint32_t s1 = b.v1 * 5, s2 = b.v2 * 5, s3 = b.v3 * 5, s4 = b.v4 * 5;
    uint64_t d0 = (uint64_t)a.v0 * b.v0 + (uint64_t)a.v1 * s4 + (uint64_t)a.v2 * s3 +
                  (uint64_t)a.v3 * s2 + (uint64_t)a.v4 * s1;
    uint64_t d1 = (uint64_t)a.v0 * b.v1 + (uint64_t)a.v1 * b.v0 + (uint64_t)a.v2 * s4 +
                  (uint64_t)a.v3 * s3 + (uint64_t)a.v4 * s2;
    uint64_t d2 = (uint64_t)a.v0 * b.v2 + (uint64_t)a.v1 * b.v1 + (uint64_t)a.v2 * b.v0 +
                  (uint64_t)a.v3 * s4 + (uint64_t)a.v4 * s3;
    uint64_t d3 = (uint64_t)a.v0 * b.v3 + (uint64_t)a.v1 * b.v2 + (uint64_t)a.v2 * b.v1 +
                  (uint64_t)a.v3 * b.v0 + (uint64_t)a.v4 * s4;
    uint64_t d4 = (uint64_t)a.v0 * b.v4 + (uint64_t)a.v1 * b.v3 + (uint64_t)a.v2 * b.v2 +
                  (uint64_t)a.v3 * b.v1 + (uint64_t)a.v4 * b.v0;
    Fe26 o;
    uint64_t c;
    c = d0 >> 26; o.v0 = (uint32_t)d0 & 0x3ffffffu; d1 += c;
    c = d1 >> 26; o.v1 = (uint32_t)d1 & 0x3ffffffu; d2 += c;
    c = d2 >> 26; o.v2 = (uint32_t)d2 & 0x3ffffffu; d3 += c;
    c = d3 >> 26; o.v3 = (uint32_t)d3 & 0x3ffffffu; d4 += c;
    c = d4 >> 26; o.v4 = (uint32_t)d4 & 0x3ffffffu;
    // c < 2^36: times five it still fits 64 bits, and two more carries settle it
    c = (uint64_t)o.v0 + c * 5;
    o.v0 = (uint32_t)c & 0x3ffffffu;
    c = (uint64_t)o.v1 + (c >> 26);
    o.v1 = (uint32_t)c & 0x3ffffffu;
    o.v2 += (uint32_t)(c >> 26);
    return o;
}

// One lane's share of the tag polynomial: its k (0..4) cells m[4t .. 4t+3]
// evaluated as sum_t m_t r^(k-t), times r^e.  e_max bounds e over the wave
// (it only limits the length of the square-and-multiply loop, so every lane
// of a wave runs the same trip count).
BNK_DEV Fe26 spread_term(const Fe26 &r, const uint32_t (&m)[16], uint32_t k, uint32_t e, uint32_t e_max)
{
    Fe26 acc = fe_small(0);
#pragma unroll
    for (uint32_t t = 0; t < 4; t++) {
        const Fe26 nx = fe_mul(fe_add(acc, fe_cell(m[4 * t], m[4 * t + 1], m[4 * t + 2], m[4 * t + 3])), r);
        acc = fe_select(t < k, nx, acc);
    }
    Fe26 lift = fe_small(1), pw = r;
#pragma unroll 1
    for (uint32_t b = 0; (1u << b) <= e_max; b++) {
        const Fe26 nl = fe_mul(lift, pw);
        lift = fe_select(((e >> b) & 1u) != 0, nl, lift);
        pw = fe_mul(pw, pw);
    }
    return fe_mul(acc, lift);
}

// Tag from the limb-wise sum of the lanes' terms (each sum below 2^34) and the
// second half of the one-time key.
BNK_DEV void spread_finish(const uint64_t (&sum)[5], const uint32_t (&pad)[4], uint32_t (&tag)[4])
{
    uint64_t t0 = sum[0], t1 = sum[1], t2 = sum[2], t3 = sum[3], t4 = sum[4];
#pragma unroll
    for (int pass = 0; pass < 2; pass++) {
        t1 += t0 >> 26; t0 &= 0x3ffffffu;
        t2 += t1 >> 26; t1 &= 0x3ffffffu;
        t3 += t2 >> 26; t2 &= 0x3ffffffu;
        t4 += t3 >> 26; t3 &= 0x3ffffffu;
        t0 += (t4 >> 26) * 5; t4 &= 0x3ffffffu;
    }
    Poly26 p;
    p.h0 = (uint32_t)t0; p.h1 = (uint32_t)t1; p.h2 = (uint32_t)t2; p.h3 = (uint32_t)t3; p.h4 = (uint32_t)t4;
    p.pad0 = pad[0]; p.pad1 = pad[1]; p.pad2 = pad[2]; p.pad3 = pad[3];
    p.finish(tag);
}

// Which cells lane l owns in a packet of `len` ciphertext bytes, and how far
// its term is lifted.  Lane 0: the length block, last in the MAC input, so it
// is lifted by nothing.  Lane l >= 1: data cells 4(l-1) .. of ceil(len/16).
struct SpreadShare {
    uint32_t k, e;
};
BNK_DEV SpreadShare spread_share(uint32_t lane, uint32_t len)
{
    const uint32_t cd = (len + 15u) >> 4;
    if (lane == 0) return SpreadShare{1u, 0u};
    const uint32_t first = 4u * (lane - 1u);
    if (first >= cd) return SpreadShare{0u, 0u};
    const uint32_t k = cd - first < 4u ? cd - first : 4u;
    return SpreadShare{k, cd - first - k + 1u}; // the cells after mine, and the length block
}
// Largest lift in the wave: lane 1's.
BNK_DEV uint32_t spread_e_max(uint32_t len)
{
    const uint32_t cd = (len + 15u) >> 4;
    return cd > 4u ? cd - 3u : 1u;
}
constexpr uint32_t SPREAD_MAX_LEN = 63u * 64u; // data blocks on lanes 1..63

} // namespace bnk
