// CPU check of the per-lane arithmetic the HIP kernels use
// (bnk_amd/csrc/aead_lane.hpp compiles for the host too): ChaCha20 blocks and
// both Poly1305 limb layouts against RFC 8439 vectors -- including the
// appendix A.3 carry and wrap-around cases, which need chosen r and s and so
// can never be reached through packets -- and against the C oracle on random
// input.  Prints PASS/FAIL lines; exit status is the number of failures.
#include <stdio.h>
#include <string.h>

#include <vector>

#include "../../bnk_amd/csrc/aead_lane.hpp"
#include "../../oracle/bnk_oracle.h"

using namespace bnk;

static int failures = 0;
static void expect(bool ok, const char *what)
{
    if (!ok) {
        printf("FAIL %s\n", what);
        failures++;
    }
}

static uint32_t ld32(const uint8_t *p) { return p[0] | p[1] << 8 | p[2] << 16 | (uint32_t)p[3] << 24; }

// Poly1305 of msg under a raw 32-byte key, with the limb layout P, the way the
// AEAD uses it: whole 16-byte blocks with bit 128 set.
template <class P> static void poly_full_blocks(const uint8_t key[32], const uint8_t *msg, size_t len, uint8_t tag[16])
{
    uint32_t x[16] = {0};
    for (int i = 0; i < 8; i++) x[i] = ld32(key + 4 * i);
    P mac;
    mac.init(x);
    for (size_t o = 0; o + 16 <= len; o += 16)
        mac.block(ld32(msg + o), ld32(msg + o + 4), ld32(msg + o + 8), ld32(msg + o + 12));
    uint32_t t[4];
    mac.finish(t);
    for (int i = 0; i < 4; i++) {
        tag[4 * i] = (uint8_t)t[i]; tag[4 * i + 1] = (uint8_t)(t[i] >> 8);
        tag[4 * i + 2] = (uint8_t)(t[i] >> 16); tag[4 * i + 3] = (uint8_t)(t[i] >> 24);
    }
}

static std::vector<uint8_t> hex(const char *s)
{
    std::vector<uint8_t> v;
    for (; s[0] && s[1]; s += 2) {
        unsigned b;
        sscanf(s, "%2x", &b);
        v.push_back((uint8_t)b);
    }
    return v;
}

struct Vec { const char *key, *msg, *tag; };

template <class P> static void run_poly(const char *name)
{
    // RFC 8439 A.3 vectors whose messages are whole blocks (#1, #5 - #11)
    static const Vec a3[] = {
        {"0000000000000000000000000000000000000000000000000000000000000000",
         "00000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000000",
         "00000000000000000000000000000000"},
        {"0200000000000000000000000000000000000000000000000000000000000000", "ffffffffffffffffffffffffffffffff",
         "03000000000000000000000000000000"},
        {"02000000000000000000000000000000ffffffffffffffffffffffffffffffff", "02000000000000000000000000000000",
         "03000000000000000000000000000000"},
        {"0100000000000000000000000000000000000000000000000000000000000000",
         "fffffffffffffffffffffffffffffffff0ffffffffffffffffffffffffffffff11000000000000000000000000000000",
         "05000000000000000000000000000000"},
        {"0100000000000000000000000000000000000000000000000000000000000000",
         "fffffffffffffffffffffffffffffffffbfefefefefefefefefefefefefefefe01010101010101010101010101010101",
         "00000000000000000000000000000000"},
        {"0200000000000000000000000000000000000000000000000000000000000000", "fdffffffffffffffffffffffffffffff",
         "faffffffffffffffffffffffffffffff"},
        {"0100000000000000040000000000000000000000000000000000000000000000",
         "e33594d7505e43b900000000000000003394d7505e4379cd01000000000000000000000000000000000000000000000001000000000000000000000000000000",
         "14000000000000005500000000000000"},
        {"0100000000000000040000000000000000000000000000000000000000000000",
         "e33594d7505e43b900000000000000003394d7505e4379cd010000000000000000000000000000000000000000000000",
         "13000000000000000000000000000000"},
    };
    char what[128];
    for (size_t i = 0; i < sizeof a3 / sizeof a3[0]; i++) {
        auto key = hex(a3[i].key), msg = hex(a3[i].msg), want = hex(a3[i].tag);
        uint8_t tag[16], otag[16];
        poly_full_blocks<P>(key.data(), msg.data(), msg.size(), tag);
        bnko_poly1305(key.data(), msg.data(), msg.size(), otag);
        snprintf(what, sizeof what, "%s A.3 vector %zu", name, i);
        expect(memcmp(tag, want.data(), 16) == 0 && memcmp(otag, want.data(), 16) == 0, what);
    }
    // random keys and messages, plus saturated ones, against the oracle
    uint64_t st = 0x9E3779B97F4A7C15ull;
    auto rnd = [&]() { st ^= st << 13; st ^= st >> 7; st ^= st << 17; return st; };
    for (int trial = 0; trial < 3000; trial++) {
        uint8_t key[32];
        std::vector<uint8_t> msg(16 * (1 + rnd() % 100));
        for (auto &b : key) b = (uint8_t)rnd();
        for (auto &b : msg) b = (uint8_t)rnd();
        if (trial % 5 == 0) memset(key, 0xFF, 16);
        if (trial % 7 == 0) memset(msg.data(), 0xFF, msg.size());
        if (trial % 11 == 0) memset(key + 16, 0xFF, 16);
        uint8_t tag[16], otag[16];
        poly_full_blocks<P>(key, msg.data(), msg.size(), tag);
        bnko_poly1305(key, msg.data(), msg.size(), otag);
        if (memcmp(tag, otag, 16) != 0) {
            snprintf(what, sizeof what, "%s random trial %d", name, trial);
            expect(false, what);
            break;
        }
    }
}

// The tag of `len` ciphertext bytes the way a wave computes it when one packet
// is spread over its lanes: 64 lane terms, each evaluated independently.
static void spread_tag(const uint32_t (&otk)[16], const uint8_t *ct, uint32_t len, uint32_t (&tag)[4])
{
    const Fe26 r = fe_clamped_r(otk[0], otk[1], otk[2], otk[3]);
    const uint32_t e_max = spread_e_max(len);
    uint64_t sum[5] = {0, 0, 0, 0, 0};
    for (uint32_t lane = 0; lane < 64; lane++) {
        uint32_t m[16] = {0};
        if (lane == 0) {
            m[2] = len;
        } else {
            uint8_t buf[64] = {0};
            const uint32_t at = 64 * (lane - 1);
            if (at < len) memcpy(buf, ct + at, len - at < 64 ? len - at : 64);
            for (int i = 0; i < 16; i++) m[i] = ld32(buf + 4 * i);
        }
        const SpreadShare sh = spread_share(lane, len);
        const Fe26 t = spread_term(r, m, sh.k, sh.e, e_max);
        sum[0] += t.v0; sum[1] += t.v1; sum[2] += t.v2; sum[3] += t.v3; sum[4] += t.v4;
    }
    const uint32_t pad[4] = {otk[4], otk[5], otk[6], otk[7]};
    spread_finish(sum, pad, tag);
}

// The same tag serially: zero-padded cells, then the length block.
static void serial_tag(const uint32_t (&otk)[16], const uint8_t *ct, uint32_t len, uint32_t (&tag)[4])
{
    Poly32 mac;
    mac.init(otk);
    for (uint32_t o = 0; o < len; o += 16) {
        uint8_t cell[16] = {0};
        memcpy(cell, ct + o, len - o < 16 ? len - o : 16);
        mac.block(ld32(cell), ld32(cell + 4), ld32(cell + 8), ld32(cell + 12));
    }
    mac.block(0, 0, len, 0);
    mac.finish(tag);
}

static void run_spread()
{
    uint64_t st = 777;
    auto rnd = [&]() { st ^= st << 13; st ^= st >> 7; st ^= st << 17; return st; };
    std::vector<uint8_t> ct(SPREAD_MAX_LEN);
    int bad = 0, cases = 0;
    auto check = [&](const uint32_t (&otk)[16], uint32_t len) {
        uint32_t a[4], b[4];
        spread_tag(otk, ct.data(), len, a);
        serial_tag(otk, ct.data(), len, b);
        cases++;
        if (memcmp(a, b, 16) != 0) bad++;
    };
    // every length class around cell, block and lane boundaries, random keys
    for (uint32_t len = 0; len <= SPREAD_MAX_LEN; len += (len < 300 || len > SPREAD_MAX_LEN - 80) ? 1 : 37) {
        uint32_t otk[16];
        for (auto &w : otk) w = (uint32_t)rnd();
        for (auto &b : ct) b = (uint8_t)rnd();
        check(otk, len);
    }
    // extreme limbs: r with every clamped bit set, all-ones and all-zero data
    // (drives the carries of the limb products and of the lane sum to their
    // largest), and the RFC 8439 A.3 keys r = 1, 2 with s = 0 or all ones
    for (int data = 0; data < 3; data++)
        for (int key = 0; key < 4; key++) {
            uint32_t otk[16] = {0};
            if (key == 0) { otk[0] = 0x0fffffffu; otk[1] = otk[2] = otk[3] = 0x0ffffffcu; }
            if (key == 1) otk[0] = 1;
            if (key == 2) { otk[0] = 2; otk[4] = otk[5] = otk[6] = otk[7] = 0xffffffffu; }
            if (key == 3) { otk[0] = 0x0fffffffu; otk[1] = otk[2] = otk[3] = 0x0ffffffcu;
                            otk[4] = otk[5] = otk[6] = otk[7] = 0xffffffffu; }
            for (auto &b : ct) b = data == 0 ? 0xff : data == 1 ? 0x00 : (uint8_t)rnd();
            for (uint32_t len : {0u, 1u, 15u, 16u, 17u, 63u, 64u, 65u, 256u, 1420u, 1436u, 4000u, 4031u, 4032u})
                check(otk, len);
        }
    printf("spread tags: %d cases, %d differ from the serial form\n", cases, bad);
    expect(bad == 0, "one packet spread over the lanes of a wave");
}

int main()
{
    // ChaCha20 block, RFC 8439 2.3.2 through the WireGuard-shaped state
    // (nonce word 13 is zero there, so use the oracle for arbitrary nonces)
    uint64_t st = 12345;
    auto rnd = [&]() { st ^= st << 13; st ^= st >> 7; st ^= st << 17; return st; };
    for (int trial = 0; trial < 200; trial++) {
        uint8_t key[32], nonce[12] = {0}, want[64];
        for (auto &b : key) b = (uint8_t)rnd();
        const uint64_t ctr = trial < 4 ? (uint64_t[]){0, 1, 0xFFFFFFFFull, ~0ull}[trial] : rnd();
        const uint32_t blk = trial % 3 == 0 ? 0xFFFFFFFFu : (uint32_t)(rnd() % 70000);
        memcpy(nonce + 4, &ctr, 8);
        bnko_chacha20_block(key, blk, nonce, want);
        uint32_t k[8], x[16], y[16];
        for (int i = 0; i < 8; i++) k[i] = ld32(key + 4 * i);
        chacha_block(k, blk, (uint32_t)ctr, (uint32_t)(ctr >> 32), x);
        bool ok = true;
        for (int i = 0; i < 16; i++) ok = ok && x[i] == ld32(want + 4 * i);
        expect(ok, "chacha_block against the oracle");
        // two blocks side by side, plainly and from what a packet's blocks share
        uint8_t want2[64];
        bnko_chacha20_block(key, blk + 1u, nonce, want2);
        uint32_t x2[16];
        chacha_block2(k, blk, (uint32_t)ctr, (uint32_t)(ctr >> 32), x2, y);
        ok = true;
        for (int i = 0; i < 16; i++) ok = ok && x2[i] == ld32(want + 4 * i) && y[i] == ld32(want2 + 4 * i);
        expect(ok, "chacha_block2 against the oracle");
        ChachaShared sh;
        chacha_shared(k, (uint32_t)ctr, (uint32_t)(ctr >> 32), sh);
        chacha_block2_shared(k, sh, blk, (uint32_t)ctr, (uint32_t)(ctr >> 32), x2, y);
        ok = true;
        for (int i = 0; i < 16; i++) ok = ok && x2[i] == ld32(want + 4 * i) && y[i] == ld32(want2 + 4 * i);
        expect(ok, "chacha_block2_shared against the oracle");
    }
    run_poly<Poly26>("Poly26");
    run_poly<Poly32>("Poly32");
    run_spread();
    printf(failures ? "FAILED %d\n" : "PASS lane arithmetic (%d failures)\n", failures);
    return failures;
}
