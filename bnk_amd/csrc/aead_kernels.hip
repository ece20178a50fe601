// Batched WireGuard transport seal/open for gfx950: one lane per packet for
// the arithmetic, wave-cooperative coalesced memory traffic through LDS.
//
// Stands behind wireguard-go's AEAD.Seal / AEAD.Open calls on transport
// packets (reached in the reference through device.NewDevice,
// internal/dataplane/engine.go:51): RFC 8439 with nonce 00000000 ||
// LE64(counter) and empty AAD.  Block 0 of the keystream gives the Poly1305
// one-time key; data uses blocks 1..; the MAC covers the zero-padded
// ciphertext and one length block.
#include "aead_lane.hpp"
#include <stdlib.h>

#include <algorithm>

#include "../../include/bnkhip.h"
#include "kernels.hpp"

namespace bnk {

// Packet pointers travel between lanes as integers, which would leave the
// compiler with flat accesses (and flat accesses also tick the LDS counter,
// stalling LDS waits behind loads still in flight): name the global address
// space explicitly.
#define BNK_GLOBAL __attribute__((address_space(1)))
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 __attribute__((aligned(1))) u32x4_unaligned;

// 16 bytes of global memory at any byte alignment (the hardware handles
// misaligned dwordx4 accesses; aligned ones cost nothing extra).
BNK_DEV uint4 ld16(const uint8_t *p)
{
    const u32x4 v = *reinterpret_cast<const BNK_GLOBAL u32x4_unaligned *>((uintptr_t)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

BNK_DEV void st16(uint8_t *p, uint4 v)
{
    const u32x4 t = {v.x, v.y, v.z, v.w};
    *reinterpret_cast<BNK_GLOBAL u32x4_unaligned *>((uintptr_t)p) = t;
}

// The same for addresses known to be 16-byte aligned.
BNK_DEV uint4 ld16a(const uint8_t *p)
{
    const u32x4 v = *reinterpret_cast<const BNK_GLOBAL u32x4 *>((uintptr_t)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

BNK_DEV void st16a(uint8_t *p, uint4 v)
{
    const u32x4 t = {v.x, v.y, v.z, v.w};
    *reinterpret_cast<BNK_GLOBAL u32x4 *>((uintptr_t)p) = t;
}

// Whole-line output that nothing in the launch reads again goes out with the
// non-temporal hint, so that it does not push packets still to be read out of
// the caches (2 % on large batches).  Only for aligned 16-byte stores of the
// line path: on misaligned stores the hint halves the rate, and on the short
// path and the tags it changes nothing.
BNK_DEV void st16a_out(uint8_t *p, uint4 v)
{
    const u32x4 t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<BNK_GLOBAL u32x4 *>((uintptr_t)p));
}

BNK_DEV uint8_t ld8(const uint8_t *p) { return *reinterpret_cast<const BNK_GLOBAL uint8_t *>((uintptr_t)p); }
BNK_DEV void st8(uint8_t *p, uint8_t v) { *reinterpret_cast<BNK_GLOBAL uint8_t *>((uintptr_t)p) = v; }
BNK_DEV void st4a(uint8_t *p, uint32_t v) { *reinterpret_cast<BNK_GLOBAL uint32_t *>((uintptr_t)p) = v; }

typedef uint32_t __attribute__((aligned(1))) u32_unaligned;
typedef uint16_t __attribute__((aligned(1))) u16_unaligned;

// m in 1..15 bytes at p (any alignment), zero-extended to 16, without touching
// a byte beyond them: whole words first, then a halfword, then a byte.
BNK_DEV uint4 ld_partial(const uint8_t *p, uint32_t m)
{
    uint32_t w[4] = {0, 0, 0, 0};
    const uint32_t nd = m >> 2;
#pragma unroll
    for (int q = 0; q < 3; q++)
        if ((uint32_t)q < nd) w[q] = *reinterpret_cast<const BNK_GLOBAL u32_unaligned *>((uintptr_t)(p + 4 * q));
    uint32_t last = 0;
    if (m & 2u) last = *reinterpret_cast<const BNK_GLOBAL u16_unaligned *>((uintptr_t)(p + 4u * nd));
    if (m & 1u) last |= (uint32_t)ld8(p + 4u * nd + (m & 2u)) << (8u * (m & 2u));
    if (nd == 0) w[0] = last;
    else if (nd == 1) w[1] = last;
    else if (nd == 2) w[2] = last;
    else w[3] = last;
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// The same with every load issued whatever m is (from `safe`, 4 readable bytes at an even
// address, where the packet has nothing there), for a caller whose other loads should not
// queue behind a branch: m may be 0, the result is then zero.
BNK_DEV uint4 ld_partial_flat(const uint8_t *p, uint32_t m, const uint8_t *safe)
{
    const uint32_t nd = m >> 2;
    uint32_t w[4];
#pragma unroll
    for (int q = 0; q < 3; q++)
        w[q] = *reinterpret_cast<const BNK_GLOBAL u32_unaligned *>((uintptr_t)((uint32_t)q < nd ? p + 4 * q : safe));
    const uint32_t half = *reinterpret_cast<const BNK_GLOBAL u16_unaligned *>((uintptr_t)((m & 2u) ? p + 4u * nd : safe));
    const uint32_t byte = ld8((m & 1u) ? p + 4u * nd + (m & 2u) : safe);
#pragma unroll
    for (int q = 0; q < 3; q++)
        if ((uint32_t)q >= nd) w[q] = 0;
    w[3] = 0;
    uint32_t last = (m & 2u) ? half : 0u;
    if (m & 1u) last |= byte << (8u * (m & 2u));
    if (nd == 0) w[0] = last;
    else if (nd == 1) w[1] = last;
    else if (nd == 2) w[2] = last;
    else w[3] = last;
    return make_uint4(w[0], w[1], w[2], w[3]);
}

BNK_DEV void st_partial(uint8_t *p, uint4 v, uint32_t m)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    const uint32_t nd = m >> 2;
#pragma unroll
    for (int q = 0; q < 3; q++)
        if ((uint32_t)q < nd) *reinterpret_cast<BNK_GLOBAL u32_unaligned *>((uintptr_t)(p + 4 * q)) = w[q];
    const uint32_t last = nd == 0 ? w[0] : nd == 1 ? w[1] : nd == 2 ? w[2] : w[3];
    if (m & 2u) *reinterpret_cast<BNK_GLOBAL u16_unaligned *>((uintptr_t)(p + 4u * nd)) = (uint16_t)last;
    if (m & 1u) st8(p + 4u * nd + (m & 2u), (uint8_t)(last >> (8u * (m & 2u))));
}

// Keeps the low m (0..16) bytes of a 16-byte little-endian value.
BNK_DEV uint4 keep_bytes(uint4 v, uint32_t m)
{
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int valid = (int)m - 4 * q;
        const uint32_t mask = valid >= 4 ? 0xffffffffu
                              : valid <= 0 ? 0u
                                           : ((1u << (8 * valid)) - 1u);
        w[q] &= mask;
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

BNK_DEV uint64_t shfl64(uint64_t v, int src_lane)
{
    const uint32_t lo = (uint32_t)__shfl((int)(uint32_t)v, src_lane, 64);
    const uint32_t hi = (uint32_t)__shfl((int)(uint32_t)(v >> 32), src_lane, 64);
    return (uint64_t)hi << 32 | lo;
}

// Orders this wave's LDS traffic: the lanes of a wave run in lockstep and the
// LDS serves one wave's instructions in order, so no hardware wait is needed,
// only a barrier the compiler will not move memory operations across.
BNK_DEV void wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// One wave = 64 packets, one lane per packet for the arithmetic.  Memory is
// touched cooperatively through a per-wave LDS tile (body_lines, body_short,
// body_generic).
//
// Line path (every packet of the wave 16-byte aligned, source and destination
// at the same offset within a 128-byte line): the wave moves whole aligned
// 128-byte lines, eight adjacent lanes per line, so every HBM/L2 access is a
// full line touched exactly once.  A packet rarely starts on a line boundary,
// so each LDS row is a ring of two lines: step s consumes packet bytes
// [128s, 128s+128), which live in lines s and s+1 of the packet; line s+2 is
// on its way into registers meanwhile, line s is complete after the step and
// leaves before line s+2 takes its place.  Only the 16-byte cells that belong
// to the packet are ever read or written, so neighbours sharing a line are
// never disturbed.
//
// Unaligned path (any other layout): the same ring over 128-byte pieces of the
// packet itself, at whatever alignment it has; where every destination of the
// wave is 4-byte aligned the output still leaves as whole aligned cells of the
// destination's lines (see body_lines).
//
// Generic path (packets beyond the wave-per-packet kernel's reach in small
// batches): 64 bytes per packet per step, four adjacent lanes per packet, any
// byte alignment.
constexpr uint32_t LDS_ROW = 80;    // generic: 64 data bytes + 16 pad
constexpr uint32_t RING_ROW = 272;  // line path: 2 x 128-byte lines + 16 pad (where the shifted output keeps a copy of the first cell)
constexpr uint32_t WAVES_PER_BLOCK = 4;
// The lane-per-packet launches run workgroups of one wave: their waves share nothing, and a
// wave that has finished gives its place to the next at once instead of waiting for the
// other waves of a workgroup of four (IMIX and the relay 1.3 % faster, uniform 1420-byte
// batches the same).
#define LANE_KERNEL_WAVES 1
constexpr uint32_t LANE_BLOCK = 64u * LANE_KERNEL_WAVES;
// Short path: a wave whose packets all have at most SHORT_BLOCKS data blocks
// (128 plaintext bytes: at most eight cells, in at most two lines) brings each
// packet in whole, computes it in one go and writes it back, with rows that
// hold the packet's cells from its first one.  Straight-line code, every load
// of the wave in flight at once: 2^20 x 60 bytes seal in 101 us against 113 us
// through the ring.  (Running such waves three to a SIMD on smaller rows was
// tried too: the 168 registers that allows cost the long packets 15 % and the
// short ones gained nothing.)
constexpr uint32_t SHORT_BLOCKS = 2;
constexpr uint32_t SHORT_ROW = 144;          // 8 cells + 16 pad
#ifndef SHORT_WAVES_PER_SIMD
#define SHORT_WAVES_PER_SIMD 3
#endif

// v: the cell's 16 bytes, read from `cell` beforehand (before the keystream block was
// computed, so that the LDS read is not waited for)
template <bool OPEN>
BNK_DEV void crypt_cell_v(Poly32 &mac, const uint32_t (&x)[16], int j, const uint4 v, uint8_t *cell)
{
    const uint4 o = make_uint4(v.x ^ x[4 * j], v.y ^ x[4 * j + 1], v.z ^ x[4 * j + 2],
                               v.w ^ x[4 * j + 3]);
    if (OPEN) mac.block(v.x, v.y, v.z, v.w);
    else mac.block(o.x, o.y, o.z, o.w);
    *reinterpret_cast<uint4 *>(cell) = o;
}

template <bool OPEN>
BNK_DEV void crypt_cell(Poly32 &mac, const uint32_t (&x)[16], int j, uint8_t *cell)
{
    const uint4 v = *reinterpret_cast<const uint4 *>(cell);
    const uint4 o = make_uint4(v.x ^ x[4 * j], v.y ^ x[4 * j + 1], v.z ^ x[4 * j + 2],
                               v.w ^ x[4 * j + 3]);
    if (OPEN) mac.block(v.x, v.y, v.z, v.w);
    else mac.block(o.x, o.y, o.z, o.w);
    *reinterpret_cast<uint4 *>(cell) = o;
}

// A cell at the end of a packet: m_in of its bytes are input (the rest count as
// zeros: WireGuard's padding, which is not in memory) and m_out come out,
// m_in <= m_out <= 16.  Without padding both are the packet's last 1..15 bytes.
// This one goes straight from and to global memory; `cell` is where the
// packet's cell of that number lives in the lane's LDS row, and the output is
// left there as well (zero-extended), for capture_head().
template <bool OPEN>
BNK_DEV void crypt_tail(Poly32 &mac, const uint32_t (&x)[16], int j, const uint8_t *s, uint8_t *d,
                        uint32_t m_in, uint32_t m_out, uint8_t *cell)
{
    const uint4 v = ld_partial(s, m_in);
    const uint4 o = keep_bytes(make_uint4(v.x ^ x[4 * j], v.y ^ x[4 * j + 1], v.z ^ x[4 * j + 2],
                                          v.w ^ x[4 * j + 3]), m_out);
    // the MAC sees the ciphertext zero-padded to 16 bytes
    if (OPEN) mac.block(v.x, v.y, v.z, v.w);
    else mac.block(o.x, o.y, o.z, o.w);
    st_partial(d, o, m_out);
    if (OPEN) *reinterpret_cast<uint4 *>(cell) = o;
}

// The same when the cell has come into LDS with the rest of its line (bytes
// beyond the input are whatever memory held: masked off).  A whole cell of
// output stays in LDS and leaves with its line; fewer bytes are written here,
// to a 16-byte aligned destination.
template <bool OPEN>
BNK_DEV void crypt_tail_lds(Poly32 &mac, const uint32_t (&x)[16], int j, uint8_t *cell, uint8_t *d,
                            uint32_t m_in, uint32_t m_out)
{
    const uint4 raw = *reinterpret_cast<const uint4 *>(cell);
    const uint4 v = keep_bytes(raw, m_in);
    const uint4 o = keep_bytes(make_uint4(v.x ^ x[4 * j], v.y ^ x[4 * j + 1], v.z ^ x[4 * j + 2],
                                          v.w ^ x[4 * j + 3]), m_out);
    if (OPEN) mac.block(v.x, v.y, v.z, v.w);
    else mac.block(o.x, o.y, o.z, o.w);
    if (m_out < 16u) st_partial(d, o, m_out);
    if (OPEN || m_out == 16u) *reinterpret_cast<uint4 *>(cell) = o;
}

// Open only: what a lane keeps of its plaintext's first bytes for the packet's
// record in AeadArgs::heads, read from its LDS row once the first data block has
// been through (cells c0 and c1 of the packet; bytes beyond a packet shorter
// than that are whatever the row held).
struct Head {
    uint4 c0, c1;
    bool on; // the launch writes records (the same for every lane)
};

BNK_DEV void capture_head(Head &h, const uint8_t *c0, const uint8_t *c1)
{
    if (h.on) {
        h.c0 = *reinterpret_cast<const uint4 *>(c0);
        h.c1 = *reinterpret_cast<const uint4 *>(c1);
    }
}

template <bool OPEN>
BNK_DEV void body_generic(uint8_t *tile, uint32_t lane, const uint8_t *src, uint8_t *dst,
                          uint32_t len, const uint8_t *safe, const uint32_t (&k)[8], uint32_t n1,
                          uint32_t n2, Poly32 &mac, uint32_t (&x)[16], Head &head)
{
    const uint32_t nfull = len >> 6, rem = len & 63u;
    const uint32_t steps = nfull + (rem ? 1u : 0u);
    // the four (packet, 16-byte column) cells this lane moves per step
    const uint32_t col = lane & 3u;
    const uint8_t *csrc[4];
    uint8_t *cdst[4];
    uint32_t clen[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int owner = 16 * j + (int)(lane >> 2);
        csrc[j] = reinterpret_cast<const uint8_t *>(shfl64((uint64_t)(uintptr_t)src, owner)) + 16u * col;
        cdst[j] = reinterpret_cast<uint8_t *>(shfl64((uint64_t)(uintptr_t)dst, owner)) + 16u * col;
        clen[j] = (uint32_t)__shfl((int)len, owner, 64);
    }
    // The cells of step b+1 are fetched into registers while step b is
    // computed.  Every lane loads every time, from a harmless address (`safe`,
    // 16 readable bytes) when the cell is not a packet's: a load under a branch
    // would make the wave wait for it before the branch closes.
    uint4 pre[4];
#pragma unroll
    for (int j = 0; j < 4; j++) pre[j] = ld16(16u * col + 16u <= clen[j] ? csrc[j] : safe);
    chacha_block(k, 0, n1, n2, x);
    mac.init(x);
    for (uint32_t b = 0; __ballot(b < steps) != 0ull; b++) {
        const uint32_t pos = 64u * b + 16u * col;
        // registers -> LDS, all 64 lanes, only 16-byte cells that lie fully inside a packet
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (pos + 16u <= clen[j])
                *reinterpret_cast<uint4 *>(tile + (16u * j + (lane >> 2)) * LDS_ROW + 16u * col) = pre[j];
        }
        wave_sync();
#pragma unroll
        for (int j = 0; j < 4; j++)
            pre[j] = ld16(pos + 64u + 16u <= clen[j] ? csrc[j] + 64u * (b + 1u) : safe);
        if (b < steps) {
            chacha_block(k, b + 1, n1, n2, x);
            uint8_t *row = tile + lane * LDS_ROW;
            if (b < nfull) {
#pragma unroll
                for (int j = 0; j < 4; j++) crypt_cell<OPEN>(mac, x, j, row + 16 * j);
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if (rem >= 16u * (j + 1)) crypt_cell<OPEN>(mac, x, j, row + 16 * j);
                    else if (rem > 16u * j)
                        crypt_tail<OPEN>(mac, x, j, src + 64u * b + 16 * j, dst + 64u * b + 16 * j,
                                         rem - 16u * j, rem - 16u * j, row + 16 * j);
                }
            }
            if (OPEN && b == 0) capture_head(head, row, row + 16);
        }
        wave_sync();
        // LDS -> global
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (pos + 16u <= clen[j]) {
                const uint4 v = *reinterpret_cast<const uint4 *>(
                    tile + (16u * j + (lane >> 2)) * LDS_ROW + 16u * col);
                st16(cdst[j] + 64u * b, v);
            }
        }
        wave_sync();
    }
}

// ALIGNED: every packet of the wave 16-byte aligned, source and destination at
// the same place within a 128-byte line: the stream of cells starts at the line
// holding the packet's first byte and every access is a whole aligned cell.
// Otherwise the stream starts at the packet itself (any alignment, source and
// destination independent): the same pipeline over 128-byte pieces of the
// packet, which then straddle two lines each.
// SHIFT (not ALIGNED, every destination of the wave 4-byte aligned): the input
// comes in as such pieces, but the output leaves as whole aligned 16-byte cells
// of the destination's own 128-byte lines.  A lane that moves such a cell reads
// its four words from where they lie in the ring, a multiple of 4 bytes into a
// ring cell (the 16 bytes behind a row's ring repeat its first cell, so that
// such a read never wraps); the first and the last cell of a packet, which it
// shares with its neighbours, leave word by word.  (Misaligned 16-byte stores run at half rate and leave
// every line in two parts.)  A destination line lags the packet's pieces by up to
// 124 bytes, so a piece enters the ring one step later than otherwise: just
// before it is needed, after the line that still holds the end of the piece
// two before it has left.
template <bool OPEN, bool ALIGNED, bool SHIFT = false>
BNK_DEV void body_lines(uint8_t *tile, uint32_t lane, const uint8_t *src, uint8_t *dst, uint32_t len,
                        uint32_t len_in, const uint8_t *safe, const uint32_t (&k)[8], uint32_t n1, uint32_t n2,
                        Poly32 &mac, uint32_t (&x)[16], Head &head)
{
    // len_in <= len: the packet's bytes in memory; the up to 15 between the two
    // are padding that counts as zeros (a sealing WireGuard launch; otherwise
    // the two are equal)
    const uint32_t ncell_in = len_in >> 4;
    // Cells are 16 bytes; a packet's cell kc sits at stream position c0 + kc,
    // where the stream starts at the 128-byte line holding the packet's first
    // byte.  Stream position K lives in line K / 8 and in ring cell K % 16.
    const uint32_t skew = ALIGNED ? (uint32_t)(uintptr_t)src & 127u : 0u;
    const uint32_t c0 = skew >> 4;
    const uint32_t ncell = len >> 4; // whole cells; the last 1-15 bytes are written by their owner,
                                     // but their cell comes in with the others
    const uint32_t steps = (len + 127u) >> 7;
    const uint32_t sub = lane & 7u;
    // the eight (packet, cell-of-line) positions this lane moves per line
    const uint8_t *csrc[8];
    uint8_t *cdst[8];
    uint32_t cfirst[8], cend[8], cend_ld[8];
    int32_t pofs[8];
    uint32_t whole[8];
#pragma unroll
    for (int q = 0; q < 8; q++) {
        const int owner = 8 * q + (int)(lane >> 3);
        csrc[q] = reinterpret_cast<const uint8_t *>(shfl64((uint64_t)(uintptr_t)(src - skew), owner)) + 16u * sub;
        cdst[q] = reinterpret_cast<uint8_t *>(shfl64((uint64_t)(uintptr_t)(dst - skew), owner)) + 16u * sub;
        cfirst[q] = (uint32_t)__shfl((int)c0, owner, 64);
        const uint32_t olen = (uint32_t)__shfl((int)len, owner, 64);
        cend[q] = cfirst[q] + (olen >> 4);
        // (a cell that is not aligned may reach into the next page: only aligned ones
        // are fetched beyond the packet's last byte)
        cend_ld[q] = cfirst[q] + ((olen + (ALIGNED ? 15u : 0u)) >> 4);
        if (SHIFT) {
            const uint64_t od = shfl64((uint64_t)(uintptr_t)dst, owner);
            const uint32_t skd = (uint32_t)od & 127u;
            cdst[q] = reinterpret_cast<uint8_t *>(od - skd) + 16u * sub; // my cell of the line holding the packet's first byte
            pofs[q] = (int32_t)(16u * sub) - (int32_t)skd;               // where that cell starts within the packet
            whole[q] = olen & ~15u;                                      // bytes of it that go through the ring
        }
    }
    uint32_t maxsteps = steps;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)maxsteps, off, 64);
        maxsteps = o > maxsteps ? o : maxsteps;
    }
    maxsteps = __builtin_amdgcn_readfirstlane(maxsteps);

    // Lines m_lo <= m < m_hi lie wholly inside every packet of the wave: those
    // move without per-cell bounds checks.
    uint32_t maxc0 = c0, minend = c0 + ncell;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const uint32_t a = (uint32_t)__shfl_xor((int)maxc0, off, 64);
        const uint32_t b = (uint32_t)__shfl_xor((int)minend, off, 64);
        maxc0 = a > maxc0 ? a : maxc0;
        minend = b < minend ? b : minend;
    }
    const uint32_t m_lo = __builtin_amdgcn_readfirstlane(maxc0) ? 1u : 0u;
    const uint32_t m_hi = __builtin_amdgcn_readfirstlane(minend) >> 3;

    // Lines are fetched one iteration ahead into registers (issue), so the
    // loads fly while the wave computes, and only then moved into the ring
    // (commit), which overwrites the half whose line was written back last.
    uint4 pre0 = make_uint4(0, 0, 0, 0), pre1 = pre0, pre2 = pre0, pre3 = pre0, pre4 = pre0,
          pre5 = pre0, pre6 = pre0, pre7 = pre0;
    uint8_t *mycell = tile + (lane >> 3) * RING_ROW;
#define BNK_INSIDE(q, m) (8u * (m) + sub >= cfirst[q] && 8u * (m) + sub < cend[q])
#define BNK_INSIDE_LD(q, m) (8u * (m) + sub >= cfirst[q] && 8u * (m) + sub < cend_ld[q])
#define BNK_SLOT(q, m) reinterpret_cast<uint4 *>(mycell + 8u * q * RING_ROW + (((8u * (m) + sub) & 15u) << 4))
    // Boundary lines: a load under a branch makes the wave wait for it before the
    // branch closes, eight times per line; loading unconditionally from a harmless
    // address instead keeps all eight in flight (cells outside the packet are
    // fetched from `safe` and never leave their register).
#define BNK_LD(p) (ALIGNED ? ld16a(p) : ld16(p))
#define BNK_ST(p, v) do { if (ALIGNED) st16a_out(p, v); else st16(p, v); } while (0)
#define BNK_ISSUE(q, m) pre##q = BNK_LD(BNK_INSIDE_LD(q, m) ? csrc[q] + 128u * (m) : safe)
#define BNK_ISSUE_ALL(q, m) pre##q = BNK_LD(csrc[q] + 128u * (m))
#define BNK_COMMIT(q, m) if (BNK_INSIDE_LD(q, m)) *BNK_SLOT(q, m) = pre##q
#define BNK_COMMIT_ALL(q, m) *BNK_SLOT(q, m) = pre##q
    // A finished line leaves in two parts: out of the ring into registers
    // (unconditionally, for the same reason), and to memory only after the next
    // line's loads have been issued.  The wave's memory operations complete in
    // the order they were issued and one counter covers loads and stores, so a
    // wait for a line's loads also waits for every store issued after them:
    // stores issued just before the wait (a finished line, then straight on to
    // the next line's arrival) cost 24-31 % of a wave's time; issued after the
    // following loads, the next wait that covers them is a whole step away.
#define BNK_TAKE(q, m) out##q = *BNK_SLOT(q, m)
#define BNK_PUT(q, m) if (BNK_INSIDE(q, m)) BNK_ST(cdst[q] + 128u * (m), out##q)
#define BNK_PUT_ALL(q, m) BNK_ST(cdst[q] + 128u * (m), out##q)
    // SHIFT: my cell of destination line m starts pofs[q] + 128 m bytes into the packet
    // (before it when negative), a multiple of 4: its four words from that place of the ring
    // on, running into the copy of the ring's first cell behind its end where they would wrap
#define BNK_TAKE_SHIFT(q, m)                                                                \
    do {                                                                                    \
        const uint32_t at_##q = (uint32_t)(pofs[q] + (int32_t)(128u * (m))) & 255u;         \
        const uint32_t *const w_##q = reinterpret_cast<const uint32_t *>(mycell + 8u * q * RING_ROW + at_##q); \
        out##q = make_uint4(w_##q[0], w_##q[1], w_##q[2], w_##q[3]);                        \
    } while (0)
#define BNK_PUT_SHIFT(q, m)                                                                 \
    do {                                                                                    \
        const uint32_t at_##q = (uint32_t)(pofs[q] + (int32_t)(128u * (m)));                \
        uint8_t *const to_##q = cdst[q] + 128u * (m);                                       \
        if (at_##q < whole[q] && at_##q + 12u < whole[q]) st16a_out(to_##q, out##q);        \
        else {                                                                              \
            if (at_##q < whole[q]) st4a(to_##q, out##q.x);                                  \
            if (at_##q + 4u < whole[q]) st4a(to_##q + 4, out##q.y);                         \
            if (at_##q + 8u < whole[q]) st4a(to_##q + 8, out##q.z);                         \
            if (at_##q + 12u < whole[q]) st4a(to_##q + 12, out##q.w);                       \
        }                                                                                   \
    } while (0)
#define BNK_PUT_SHIFT_ALL(q, m) st16a_out(cdst[q] + 128u * (m), out##q)
#define BNK_EIGHT(OP, m)                                                                    \
    do {                                                                                    \
        OP(0, m); OP(1, m); OP(2, m); OP(3, m); OP(4, m); OP(5, m); OP(6, m); OP(7, m);     \
    } while (0)
#define BNK_LINE(OP, m)                                                                     \
    do {                                                                                    \
        if ((m) >= m_lo && (m) < m_hi) BNK_EIGHT(OP##_ALL, m);                              \
        else BNK_EIGHT(OP, m);                                                              \
    } while (0)
#define BNK_ISSUE_LINE(m) BNK_LINE(BNK_ISSUE, m)
#define BNK_COMMIT_LINE(m) BNK_LINE(BNK_COMMIT, m)
    uint4 out0 = pre0, out1 = pre0, out2 = pre0, out3 = pre0, out4 = pre0, out5 = pre0, out6 = pre0, out7 = pre0;

    uint8_t *row = tile + lane * RING_ROW;
    BNK_ISSUE_LINE(0u);
    // keystream block 0 (the Poly1305 key) is computed while the first line flies
    chacha_block(k, 0, n1, n2, x);
    mac.init(x);
    ChachaShared shared;
    chacha_shared(k, n1, n2, shared);
    // (with SHIFT a piece enters the ring, and the next one starts flying, one step later)
    constexpr uint32_t AHEAD = SHIFT ? 0u : 1u;
    if (!SHIFT) {
        BNK_COMMIT_LINE(0u);
        BNK_ISSUE_LINE(1u);
    }
    // iteration s: line s-1 (complete since the step before) leaves the ring,
    // line s+1 enters it, line s+2 starts flying, line s-1 goes to memory,
    // packet bytes [128s, 128s+128) are processed; the extra last iteration
    // only writes back the final line
    for (uint32_t s = 0; s <= maxsteps + 1; s++) {
        if (s >= 1) {
            if (SHIFT) BNK_EIGHT(BNK_TAKE_SHIFT, s - 1);
            else BNK_EIGHT(BNK_TAKE, s - 1);
        }
        wave_sync();
        BNK_COMMIT_LINE(s + AHEAD);
        // Sealing: nothing of the wave's is in flight here but the stores of the line that left
        // a step ago.  Waiting for them by hand tells the compiler that the registers the next
        // loads fill are free: otherwise it protects them with a wait of its own, for
        // everything, which lands behind the first seven of those loads (the eighth is shared
        // by the two forms of the line and issued after them) and makes the wave sit out their
        // whole way to memory and back in every step: 5 % of a sealing launch.  (The opening
        // code comes out without that wait, and with this one it is 1 % slower.
        // tests/test_kernel_isa.py looks for the pattern in both.)
        if (!OPEN) __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
        if (s + AHEAD + 1u <= maxsteps) BNK_ISSUE_LINE(s + AHEAD + 1u);
        if (s >= 1) {
            if (SHIFT) {
                // whole lines of every packet of the wave: not the first, and ending within its whole cells
                if (s - 1 >= 1u && s - 1 < m_hi) BNK_EIGHT(BNK_PUT_SHIFT_ALL, s - 1);
                else BNK_EIGHT(BNK_PUT_SHIFT, s - 1);
            } else if (s - 1 >= m_lo && s - 1 < m_hi) BNK_EIGHT(BNK_PUT_ALL, s - 1);
            else BNK_EIGHT(BNK_PUT, s - 1);
        }
        wave_sync();
        if (s < steps) {
            if (8u * s + 8u <= ncell_in) {
                // all eight cells of this step are whole cells of the packet: its two
                // keystream blocks side by side
                uint32_t y[16];
                const uint32_t r0 = c0 + 8u * s;
                // The step's first cell leaves LDS while the keystream is computed, every other
                // one while the cell before it goes through the cipher and the MAC (a read
                // where the cell is used costs open 1 %; reading four ahead of the keystream,
                // which seal had registers for, is no faster than this).
                uint4 cur = *reinterpret_cast<const uint4 *>(row + ((r0 & 15u) << 4));
                chacha_block2_shared(k, shared, 2u * s + 1u, n1, n2, x, y);
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    uint4 nxt = cur;
                    if (j < 7) nxt = *reinterpret_cast<const uint4 *>(row + (((r0 + j + 1u) & 15u) << 4));
                    if (j < 4) crypt_cell_v<OPEN>(mac, x, j, cur, row + (((r0 + j) & 15u) << 4));
                    else crypt_cell_v<OPEN>(mac, y, j - 4, cur, row + (((r0 + j) & 15u) << 4));
                    cur = nxt;
                }
            } else {
#pragma unroll 1
                for (uint32_t h = 0; h < 2; h++) {
                    const uint32_t b = 2u * s + h;
                    if (64u * b < len) {
                        chacha_block(k, b + 1, n1, n2, x);
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const uint32_t kc = 4u * b + j;
                            uint8_t *cell = row + (((c0 + kc) & 15u) << 4);
                            if (kc < ncell_in) crypt_cell<OPEN>(mac, x, j, cell);
                            else if (kc < ncell || (kc == ncell && (len & 15u))) {
                                const uint32_t m_out = kc < ncell ? 16u : len & 15u;
                                const uint32_t m_in = len_in > 16u * kc ? min(len_in - 16u * kc, m_out) : 0u;
                                // (not aligned: only whole cells of the packet have come into LDS)
                                if (ALIGNED || kc < ncell)
                                    crypt_tail_lds<OPEN>(mac, x, j, cell, dst + 16u * kc, m_in, m_out);
                                else
                                    crypt_tail<OPEN>(mac, x, j, src + 16u * kc, dst + 16u * kc, m_in, m_out, cell);
                            }
                        }
                    }
                }
            }
            if (OPEN && s == 0) capture_head(head, row + (c0 << 4), row + (((c0 + 1u) & 15u) << 4));
            // SHIFT: a step that has written the ring's first cell (every second one: the ring
            // holds a packet from its first byte) repeats it behind the ring's end
            static_assert(!SHIFT || RING_ROW >= 256u + 16u, "no room behind the ring for the copy of its first cell");
            if (SHIFT && (s & 1u) == 0u)
                *reinterpret_cast<uint4 *>(row + 256) = *reinterpret_cast<const uint4 *>(row);
        }
        wave_sync();
    }
#undef BNK_INSIDE
#undef BNK_LD
#undef BNK_ST
#undef BNK_INSIDE_LD
#undef BNK_SLOT
#undef BNK_ISSUE
#undef BNK_ISSUE_ALL
#undef BNK_COMMIT
#undef BNK_COMMIT_ALL
#undef BNK_TAKE
#undef BNK_PUT
#undef BNK_PUT_ALL
#undef BNK_TAKE_SHIFT
#undef BNK_PUT_SHIFT
#undef BNK_PUT_SHIFT_ALL
#undef BNK_EIGHT
#undef BNK_LINE
#undef BNK_ISSUE_LINE
#undef BNK_COMMIT_LINE
}

// Short path (see SHORT_BLOCKS): cell j of a packet lives at row + 16 j.  Same
// cooperative movement as body_lines: eight adjacent lanes per aligned
// 128-byte line, only cells of the packet read into LDS or written back.
// LEAN (the launch that holds more such waves per SIMD): where each cell goes is
// worked out again after the cipher instead of being kept in registers across it.
template <bool OPEN, bool LEAN = false>
BNK_DEV void body_short(uint8_t *tile, uint32_t lane, const uint8_t *src, uint8_t *dst, uint32_t len,
                        uint32_t len_in, const uint8_t *safe, const uint32_t (&k)[8], uint32_t n1, uint32_t n2,
                        Poly32 &mac, uint32_t (&x)[16], Head &head)
{
    const uint32_t ncell_in = len_in >> 4; // see body_lines
    const uint32_t skew = (uint32_t)(uintptr_t)src & 127u;
    const uint32_t c0 = skew >> 4;
    const uint32_t ncell = len >> 4;           // whole cells, stored cooperatively
    const uint32_t sub = lane & 7u;
    // does any packet of the wave reach into a second line?
    const bool two = __ballot(c0 + ((len + 15u) >> 4) > 8u) != 0ull;
    uint8_t *rows = tile + (lane >> 3) * SHORT_ROW;
    uint4 pre[2][8];
    uint32_t jcell[8], nst[8], nld[8]; // my cell's index in the owner's packet for line 0; its cell counts
    const uint8_t *csrc[8];
    uint8_t *cdst[8];
#pragma unroll
    for (int q = 0; q < 8; q++) {
        const int owner = 8 * q + (int)(lane >> 3);
        csrc[q] = reinterpret_cast<const uint8_t *>(shfl64((uint64_t)(uintptr_t)(src - skew), owner)) + 16u * sub;
        cdst[q] = reinterpret_cast<uint8_t *>(shfl64((uint64_t)(uintptr_t)(dst - skew), owner)) + 16u * sub;
        const uint32_t olen = (uint32_t)__shfl((int)len, owner, 64);
        jcell[q] = sub - (uint32_t)__shfl((int)c0, owner, 64); // wraps below zero for cells before the packet
        nst[q] = olen >> 4;
        nld[q] = (olen + 15u) >> 4;
    }
    // unconditional loads, from a harmless address when the cell is not the
    // packet's (a load under a branch is waited for where the branch closes)
#pragma unroll
    for (int q = 0; q < 8; q++) pre[0][q] = ld16a(jcell[q] < nld[q] ? csrc[q] : safe);
    if (two) {
#pragma unroll
        for (int q = 0; q < 8; q++) pre[1][q] = ld16a(jcell[q] + 8u < nld[q] ? csrc[q] + 128u : safe);
    }
    // keystream blocks 0 (the Poly1305 key) and 1 side by side while the loads fly
    uint32_t y[16];
    {
        ChachaShared shared;
        chacha_shared(k, n1, n2, shared);
        chacha_block2_shared(k, shared, 0, n1, n2, x, y);
    }
    mac.init(x);
#pragma unroll
    for (int q = 0; q < 8; q++)
        if (jcell[q] < nld[q]) *reinterpret_cast<uint4 *>(rows + 8u * q * SHORT_ROW + (jcell[q] << 4)) = pre[0][q];
    if (two) {
#pragma unroll
        for (int q = 0; q < 8; q++)
            if (jcell[q] + 8u < nld[q])
                *reinterpret_cast<uint4 *>(rows + 8u * q * SHORT_ROW + ((jcell[q] + 8u) << 4)) = pre[1][q];
    }
    wave_sync();
    uint8_t *row = tile + lane * SHORT_ROW;
    // block b's four cells with keystream ks
    auto crypt_block = [&](uint32_t b, const uint32_t (&ks)[16], const uint4 (&v)[4]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t kc = 4u * b + j;
            if (kc < ncell_in) crypt_cell_v<OPEN>(mac, ks, j, v[j], row + (kc << 4));
            else if (kc < ncell || (kc == ncell && (len & 15u))) {
                const uint32_t m_out = kc < ncell ? 16u : len & 15u;
                const uint32_t m_in = len_in > 16u * kc ? min(len_in - 16u * kc, m_out) : 0u;
                crypt_tail_lds<OPEN>(mac, ks, j, row + (kc << 4), dst + 16u * kc, m_in, m_out);
            }
        }
    };
    static_assert(SHORT_BLOCKS == 2, "the short path is written out for two data blocks");
    uint4 v[4];
    if (len != 0) {
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = *reinterpret_cast<const uint4 *>(row + (j << 4));
        crypt_block(0, y, v);
    }
    if (len > 64u) {
        // the second block's cells leave LDS while its keystream is computed
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = *reinterpret_cast<const uint4 *>(row + ((4 + j) << 4));
        chacha_block(k, 2, n1, n2, x);
        crypt_block(1, x, v);
    }
    if (OPEN) capture_head(head, row, row + 16);
    wave_sync();
    if (LEAN) {
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const int owner = 8 * q + (int)(lane >> 3);
            uint8_t *to = reinterpret_cast<uint8_t *>(shfl64((uint64_t)(uintptr_t)(dst - skew), owner)) + 16u * sub;
            const uint32_t jc = sub - (uint32_t)__shfl((int)c0, owner, 64);
            const uint32_t ns = (uint32_t)__shfl((int)len, owner, 64) >> 4;
            const uint4 v0 = *reinterpret_cast<const uint4 *>(rows + 8u * q * SHORT_ROW + ((jc < 8u ? jc : 0u) << 4));
            if (jc < ns) st16a(to, v0);
            if (two) {
                const uint32_t j1 = jc + 8u;
                const uint4 v1 = *reinterpret_cast<const uint4 *>(rows + 8u * q * SHORT_ROW + ((j1 < 8u ? j1 : 0u) << 4));
                if (j1 < ns) st16a(to + 128u, v1);
            }
        }
        return;
    }
#pragma unroll
    for (int q = 0; q < 8; q++) {
        // read first, unconditionally (from cell 0 when mine is not the packet's)
        const uint4 v = *reinterpret_cast<const uint4 *>(rows + 8u * q * SHORT_ROW + ((jcell[q] < 8u ? jcell[q] : 0u) << 4));
        if (jcell[q] < nst[q]) st16a(cdst[q], v);
    }
    if (two) {
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const uint32_t j1 = jcell[q] + 8u;
            const uint4 v = *reinterpret_cast<const uint4 *>(rows + 8u * q * SHORT_ROW + ((j1 < 8u ? j1 : 0u) << 4));
            if (j1 < nst[q]) st16a(cdst[q] + 128u, v);
        }
    }
}

// Tag and verdict of each lane's packet once its bytes have gone through the
// MAC, and the zero-fill of rejected plaintexts.
// Returns whether the lane's packet was rejected.
template <bool OPEN>
BNK_DEV bool lane_finish(const AeadArgs &a, uint32_t lane, bool have, uint32_t i, uint32_t len,
                         const uint8_t *src, uint8_t *dst, Poly32 &mac, const Head &head, uint8_t *record,
                         bool decap = false, uint32_t pr = 0)
{
    bool reject = false;
    if (have) {
        // LE64(len(aad) = 0) || LE64(len(ciphertext))
        mac.block(0, 0, len, 0);
        uint32_t tag[4];
        mac.finish(tag);
        if (!OPEN) {
            st16(dst + len, make_uint4(tag[0], tag[1], tag[2], tag[3]));
        } else {
            const uint4 tg = ld16(src + len);
            // all 16 bytes are compared, no early exit
            const uint32_t diff = (tg.x ^ tag[0]) | (tg.y ^ tag[1]) | (tg.z ^ tag[2]) |
                                  (tg.w ^ tag[3]);
            reject = diff != 0;
            if (a.verdict) a.verdict[i] = reject ? 0 : 1;
        }
    }
    if (OPEN && decap) {
        // what WireGuard does with an opened datagram: keepalive, IP version, the
        // trim to the IP header's total length, the sender's allowed prefix (the
        // header's first 16 bytes were kept when they went through the cipher)
        uint32_t res = BNK_WG_OK, out_len = 0;
        const uint32_t version = (head.c0.x >> 4) & 0xFu;
        if (!have || reject) res = BNK_WG_AUTH_FAIL; // (no packet here: it reached beyond the output arena)
        else if (len == 0u) res = BNK_WG_KEEPALIVE;
        else if (len < 16u) res = BNK_WG_BAD_IP; // too short for either header
        else if (version == 4u) {
            const uint32_t total = __builtin_bswap32(head.c0.x) & 0xFFFFu;
            const uint2 al = a.wg.allowed[pr];
            if (len < 20u || total > len || total < 20u) res = BNK_WG_BAD_IP;
            else if ((__builtin_bswap32(head.c0.w) & al.y) != (al.x & al.y)) res = BNK_WG_NOT_ALLOWED;
            else out_len = total;
        } else if (version == 6u) {
            // peers own IPv4 addresses only
            const uint32_t total = (__builtin_bswap32(head.c0.y) >> 16) + 40u;
            res = (len < 40u || total > len) ? BNK_WG_BAD_IP : BNK_WG_NOT_ALLOWED;
        } else res = BNK_WG_BAD_IP;
        a.wg.result[i] = (uint8_t)res;
        a.wg.out_len[i] = out_len;
        if (a.wg.replay_keys) {
            const uint32_t sender = res != BNK_WG_AUTH_FAIL ? pr : 0xFFFFFFFFu;
            if (a.wg.replay_index_bits) {
                a.wg.replay_keys[i - a.first] = wg_replay_pack(sender, i - a.first, a.wg.replay_index_bits);
            } else {
                a.wg.replay_keys[i - a.first] = sender;
                a.wg.replay_idx[i - a.first] = i - a.first;
            }
        }
    }
    if (OPEN && record) {
        // bytes 0-23 of the plaintext, its length, 1 if it is authentic: the lanes'
        // records lie side by side
        st16a(record, head.c0);
        st16a(record + 16, make_uint4(head.c1.x, head.c1.y, len, have && !reject ? 1u : 0u));
    }
    if (OPEN) {
        unsigned long long rej = __ballot(reject);
        if (rej != 0ull) {
            // the plaintext cells were stored by other lanes of this wave: wait
            // until those stores have been acknowledged (a workgroup-scope
            // release is just that wait; a wider fence would write back the
            // whole L2), then the wave clears each rejected packet together
            // (chacha20poly1305.Open leaves zeros behind)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            while (rej != 0ull) {
                const int r = __ffsll((long long)rej) - 1;
                rej &= rej - 1ull;
                uint8_t *d = reinterpret_cast<uint8_t *>(shfl64((uint64_t)(uintptr_t)dst, r));
                const uint32_t L = (uint32_t)__shfl((int)len, r, 64);
                for (uint32_t pos = 16u * lane; pos + 16u <= L; pos += 1024u)
                    st16(d + pos, make_uint4(0, 0, 0, 0));
                if (lane < (L & 15u)) st8(d + (L & ~15u) + lane, 0);
            }
        }
    }
    return reject;
}

// A lane per packet.  SHORT_ONLY: the launch for batches in which every wave
// takes the short path (see aead_short_kernel).
template <bool OPEN, bool SHORT_ONLY>
BNK_DEV void wave_main(const AeadArgs &a, uint8_t *tile)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t t = blockIdx.x * LANE_BLOCK + threadIdx.x;
    const uint32_t t_end = a.n;

    // ---- this lane's packet ----
    // Straight-line code: every load below is issued whether or not the lane
    // has a packet (from packet 0's entries or from `safe` when it has none or
    // the array is absent), because a load under a branch makes the wave wait
    // for it where the branch closes, and these form a chain (order -> lengths,
    // offsets, peer -> key) that the first data loads should not queue behind.
    // Worth 2 % on batches with every per-packet array present (the relay), a
    // wash elsewhere.
    const uint32_t *safe32 = a.keys;
    const uint64_t *safe64 = reinterpret_cast<const uint64_t *>(a.keys);
    const bool in_batch = t < t_end;
    const uint32_t tt = in_batch ? t : 0u;
    const uint32_t ord = *(a.order ? a.order + tt : safe32);
    const uint32_t i = a.first + (a.order ? ord : tt);
    const uint32_t len_ld = *(a.lens ? a.lens + i : safe32);
    const uint32_t peer_ld = *(a.peer ? a.peer + i : safe32);
    const uint8_t skip_ld = *(a.skip ? a.skip + i : reinterpret_cast<const uint8_t *>(a.keys));
    const uint64_t in_off_ld = *(a.in_off ? a.in_off + i : safe64);
    const uint64_t out_off_ld = *(a.out_off ? a.out_off + i : safe64);
    const uint64_t ctr_ld = *(a.counters ? a.counters + i : safe64);
    uint32_t len = a.lens ? len_ld : a.len;
    if (!OPEN) len = len >= a.trim ? len - a.trim : 0u;
    // Opening with WireGuard's framing (a.wg.mode, in_skip = 16: a packet's
    // offset and length are its datagram's): the header names the sender and
    // the counter.  A datagram that fails here is reported and not opened.
    const bool decap = OPEN && a.wg.mode == WG_FUSE_DECAP;
    uint32_t wg_peer = 0;
    uint64_t wg_ctr = 0;
    uint32_t wg_res = BNK_WG_OK;
    if (decap) {
        const uint64_t at = a.in_off ? in_off_ld : (uint64_t)i * a.in_stride;
        // the datagram where it is read, and the plaintext where it would be written
        const bool beyond = beyond_arena(at, len, a.in_limit) ||
                            beyond_arena((a.out_off ? out_off_ld : (uint64_t)i * a.out_stride) + a.out_skip,
                                         len >= 32u ? len - 32u : 0u, a.out_limit);
        if (in_batch && beyond) status_raise(a.status, STATUS_BOUNDS);
        if (beyond || len < 32u) wg_res = BNK_WG_BAD_HEADER;
        const uint4 h = ld16(wg_res == BNK_WG_OK && in_batch ? a.in + at : reinterpret_cast<const uint8_t *>(a.keys));
        if (wg_res == BNK_WG_OK && h.x != 4u) wg_res = BNK_WG_BAD_HEADER;
        if (wg_res == BNK_WG_OK) {
            const uint32_t mask = (1u << a.wg.hash_bits) - 1u;
            uint32_t slot = wg_hash_slot(h.y, a.wg.hash_bits);
            wg_res = BNK_WG_UNKNOWN_INDEX;
            // the table is never full: an empty slot ends the walk
            for (uint32_t probe = 0; probe <= mask; probe++) {
                const uint2 e = a.wg.index_hash[slot];
                if (e.y == WG_HASH_EMPTY) break;
                if (e.x == h.y) {
                    wg_peer = e.y;
                    wg_res = BNK_WG_OK;
                    break;
                }
                slot = (slot + 1u) & mask;
            }
        }
        wg_ctr = (uint64_t)h.z | (uint64_t)h.w << 32;
        len = len >= 16u ? len - 16u : 0u; // what goes through the cipher, tag included
    }
    // Sealing with WireGuard's framing (a.wg.mode, with in_skip = out_skip = 16:
    // a packet's offset is where its header goes): the bytes after the
    // plaintext up to its padded length count as zeros without being in memory.
    const bool encap = !OPEN && a.wg.mode == WG_FUSE_ENCAP;
    const uint32_t len_plain = len;
    // a length word of a device-resident batch may be garbage: one so large that
    // the sums below would wrap is beyond any arena
    const bool wraps = len > MAX_PACKET_BYTES;
    if (encap && !wraps) len += wg_padding(len, a.wg.mtu);
    const uint32_t pr = decap ? wg_peer : a.peer ? peer_ld : 0u;
    const bool skipped = (a.skip != nullptr && skip_ld != 0) || wg_res != BNK_WG_OK;
    const bool bad_peer = pr >= a.n_peers;
    const bool too_short = OPEN && len < 16u;
    const uint64_t in_at = (a.in_off ? in_off_ld : (uint64_t)i * a.in_stride) + a.in_skip;
    const uint64_t out_at = (a.out_off ? out_off_ld : (uint64_t)i * a.out_stride) + a.out_skip;
    // seal reads len and writes len + 16, open reads len (tag included) and writes len - 16
    const bool outside = beyond_arena(in_at, len, a.in_limit) ||
                         beyond_arena(out_at, OPEN ? (too_short ? 0u : len - 16u) : (uint64_t)len + 16u, a.out_limit) ||
                         (wraps && (a.in_limit | a.out_limit) != 0);
    const uint64_t ctr = decap ? wg_ctr : a.counters ? ctr_ld : a.counter0 + i;
    // a keypair that has used up its nonces sends nothing more (wireguard-go device/send.go)
    const bool spent = encap && ctr >= WG_REJECT_AFTER_MESSAGES;
    const bool have = in_batch && !skipped && !bad_peer && !too_short && !outside && !spent;
    // the key table has at least one row
    const uint4 *kp = reinterpret_cast<const uint4 *>(a.keys + 8u * (bad_peer ? 0u : pr));
    const uint4 k0 = kp[0], k1 = kp[1];
    if (OPEN) len -= 16u;
    len = have ? len : 0u;
    const uint32_t len_in = encap ? min(len_plain, len) : len; // bytes of it in memory
    const uint8_t *src = have ? a.in + in_at : nullptr;
    uint8_t *dst = have ? a.out + out_at : nullptr;
    const bool lane_lines = (((uintptr_t)src | (uintptr_t)dst) & 15u) == 0 &&
                            (((uintptr_t)src ^ (uintptr_t)dst) & 127u) == 0;
    // which launch does this wave's packets: nothing has been written so far
    const bool all_lines = __ballot(!lane_lines) == 0ull;
    const bool all_short = all_lines && __ballot(len > 64u * SHORT_BLOCKS) == 0ull;
    if (SHORT_ONLY && !all_short) {
        // (the host launches this kernel only where no wave can come here)
        status_raise(a.status, STATUS_INTERNAL);
        return;
    }
    // what the checks above leave behind per packet
    if (decap && in_batch) {
        const bool ok = wg_res == BNK_WG_OK;
        a.wg.peer_out[i] = ok ? wg_peer : 0xFFFFFFFFu;
        a.wg.counter_out[i] = ok ? wg_ctr : 0ull;
        if (!ok) {
            a.wg.result[i] = (uint8_t)wg_res;
            a.wg.out_len[i] = 0;
            if (a.wg.replay_keys) {
                if (a.wg.replay_index_bits) {
                    a.wg.replay_keys[i - a.first] = wg_replay_pack(0xFFFFFFFFu, i - a.first, a.wg.replay_index_bits);
                } else {
                    a.wg.replay_keys[i - a.first] = 0xFFFFFFFFu;
                    a.wg.replay_idx[i - a.first] = i - a.first;
                }
            }
        }
    }
    if (in_batch && !skipped && (bad_peer || too_short || outside)) {
        if (bad_peer) status_raise(a.status, STATUS_PEER_RANGE);
        else if (outside) status_raise(a.status, STATUS_BOUNDS);
        if (OPEN && a.verdict) a.verdict[i] = 0;
    }
    if (encap && in_batch && !skipped) {
        // the transport header: type 4, the receiver's index, the counter
        if (have) st16(dst - 16, make_uint4(4u, a.wg.remote_index[pr], (uint32_t)ctr, (uint32_t)(ctr >> 32)));
        a.wg.wire_len[i] = have ? 16u + len + 16u : 0u;
    }
    const uint32_t k[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};

    const uint32_t n1 = (uint32_t)ctr, n2 = (uint32_t)(ctr >> 32);
    uint32_t x[16];
    Poly32 mac; // keyed from keystream block 0 inside the body, once its first loads are out

    const uint8_t *safe = reinterpret_cast<const uint8_t *>(a.keys);
    Head head;
    head.on = OPEN && (a.heads != nullptr || decap);
    head.c0 = head.c1 = make_uint4(0, 0, 0, 0);
    if (SHORT_ONLY) body_short<OPEN, true>(tile, lane, src, dst, len, len_in, safe, k, n1, n2, mac, x, head);
    else if (all_short) body_short<OPEN>(tile, lane, src, dst, len, len_in, safe, k, n1, n2, mac, x, head);
    else if (!all_lines) {
        if (__ballot(((uintptr_t)dst & 3u) != 0) == 0ull)
            body_lines<OPEN, false, true>(tile, lane, src, dst, len, len_in, safe, k, n1, n2, mac, x, head);
        else body_lines<OPEN, false>(tile, lane, src, dst, len, len_in, safe, k, n1, n2, mac, x, head);
    }
    else body_lines<OPEN, true>(tile, lane, src, dst, len, len_in, safe, k, n1, n2, mac, x, head);

    const bool reject = lane_finish<OPEN>(a, lane, have, i, len, src, dst, mac, head,
                                          in_batch && a.heads ? a.heads + 32ull * t : nullptr,
                                          decap && in_batch && wg_res == BNK_WG_OK, pr);
    if (OPEN && a.tally) {
        // a plain open counting its own verdicts: verdict 1 exactly where the lane had a packet
        // whose tag verified
        const unsigned long long ok = __ballot(have && !reject), all = __ballot(in_batch);
        if (lane == 0u) {
            tally_bump(a.tally, TALLY_OPENED, (uint32_t)__popcll(ok));
            tally_bump(a.tally, TALLY_REJECTED, (uint32_t)__popcll(all & ~ok));
        }
    }
}

template <bool OPEN>
__global__ __launch_bounds__(LANE_BLOCK) __attribute__((amdgpu_waves_per_eu(2, 2))) void aead_wave_kernel(AeadArgs a)
{
    __shared__ __attribute__((aligned(16))) uint8_t tile_all[LANE_KERNEL_WAVES][64 * RING_ROW];
    static_assert(RING_ROW >= LDS_ROW && RING_ROW >= SHORT_ROW, "the other paths reuse the tile");
    wave_main<OPEN, false>(a, tile_all[threadIdx.x >> 6]);
}

// Batches in which the host can tell that every wave takes the short path
// (every_wave_short): without the ring and the line paths' registers three such
// waves fit a SIMD where the launch above holds two, worth 8-11 % at 60 bytes
// (2^20 packets seal in 83 us against 93).  Handing the short waves of a mixed
// batch to this kernel in a second launch was measured too and loses: every wave
// of both launches walks its metadata before it knows whose it is (IMIX 9 %
// slower, the relay 3.5 %).
template <bool OPEN>
__global__ __launch_bounds__(LANE_BLOCK) __attribute__((amdgpu_waves_per_eu(SHORT_WAVES_PER_SIMD, SHORT_WAVES_PER_SIMD)))
void aead_short_kernel(AeadArgs a)
{
    __shared__ __attribute__((aligned(16))) uint8_t tile_all[LANE_KERNEL_WAVES][64 * SHORT_ROW];
    wave_main<OPEN, true>(a, tile_all[threadIdx.x >> 6]);
}

// One wave = one packet, for batches too small to fill the chip with a packet
// per lane (there a call lasts as long as one lane needs for a whole packet:
// about 85 us at 1420 bytes, however few the packets).  Lane 0 computes
// ChaCha20 block 0 and owns the length block, lane l >= 1 computes block l and
// moves bytes [64(l-1), 64l) of the packet; the tag is the sum of the lanes'
// terms (aead_lane.hpp).  All loads of a packet are issued before any store,
// and a lane stores only what it loaded, so sealing in place is safe.  A
// packet longer than 63 blocks is done by lane 0 alone, the per-lane way.
//
// With WG set the wave also does the packet's WireGuard framing (a.wg): on the
// way out it writes the transport header and treats the bytes between the
// plaintext and its padded length as zeros without their being in memory; on
// the way in it checks the header, finds the sender by its receiver index (a
// 64-way search of the sorted table, the lanes probing together), and after
// the tag check looks at the inner IP header while it is still in registers.
// Same results as wg_parse_kernel / wg_encap_prep_kernel / wg_finish_kernel
// around a plain launch.
template <bool OPEN, bool WG>
__global__ __launch_bounds__(256) void aead_spread_kernel(AeadArgs a)
{
    __shared__ __attribute__((aligned(16))) uint8_t tile_all[WAVES_PER_BLOCK][64 * LDS_ROW];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t w = blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
    if (w >= a.n) return;
    // everything up to the per-lane work below is uniform across the wave
    const uint32_t i = a.first + w;
    // The packet's entries in the per-packet arrays, every one loaded whether or not the
    // array is there (from the key table where it is not): a load under a branch is waited
    // for where the branch closes, and a host batch's arrays lie in host memory, a trip over
    // the link for each wait.
    const uint8_t *const safe = reinterpret_cast<const uint8_t *>(a.keys);
    const uint32_t *const safe32 = a.keys;
    const uint64_t *const safe64 = reinterpret_cast<const uint64_t *>(a.keys);
    const uint32_t len_ld = *(a.lens ? a.lens + i : safe32);
    const uint32_t peer_ld = *(a.peer ? a.peer + i : safe32);
    const uint64_t in_off_ld = *(a.in_off ? a.in_off + i : safe64);
    const uint64_t out_off_ld = *(a.out_off ? a.out_off + i : safe64);
    const uint64_t ctr_ld = *(a.counters ? a.counters + i : safe64);
    const uint8_t skip_ld = *(a.skip ? a.skip + i : safe);
    uint32_t len = a.lens ? len_ld : a.len;
    if (!OPEN) len = len >= a.trim ? len - a.trim : 0u;
    uint32_t pr = a.peer ? peer_ld : 0u;
    const uint8_t *src = a.in + (a.in_off ? in_off_ld : (uint64_t)i * a.in_stride) + a.in_skip;
    uint8_t *dst = a.out + (a.out_off ? out_off_ld : (uint64_t)i * a.out_stride) + a.out_skip;
    const bool skipped = a.skip != nullptr && skip_ld != 0;
    uint64_t ctr = 0;
    if (!WG) {
        // (framing launches only run on layouts the host has checked)
        const uint64_t in_at = (uint64_t)(src - a.in), out_at = (uint64_t)(dst - a.out);
        const bool short_ct = OPEN && len < 16u;
        if (beyond_arena(in_at, len, a.in_limit) ||
            beyond_arena(out_at, OPEN ? (short_ct ? 0u : len - 16u) : (uint64_t)len + 16u, a.out_limit) ||
            (len > MAX_PACKET_BYTES && (a.in_limit | a.out_limit) != 0)) {
            if (lane == 0 && !skipped) {
                status_raise(a.status, STATUS_BOUNDS);
                if (OPEN) a.verdict[i] = 0;
            }
            return;
        }
    }

    // ---- my 64 bytes: loads first, they fly while everything below is looked
    // up and the block is computed.  Where the AEAD data lies and how long it
    // is follows from the length alone, so the loads need not wait for the
    // header, the index search or the key; a packet that is then turned away
    // has loaded bytes of its own datagram for nothing.
    const uint8_t *data = src + (WG ? 16 : 0);
    uint32_t data_len; // bytes through the cipher, when the packet is taken at all
    uint32_t data_there; // of which in memory
    if (!WG) {
        data_len = OPEN ? (len >= 16u ? len - 16u : 0u) : len;
        data_there = data_len <= SPREAD_MAX_LEN ? data_len : 0u; // longer ones go the per-lane way
    } else if (!OPEN) {
        const bool fits = len + 15u <= WG_FUSE_MAX_LEN;
        data_there = fits ? len : 0u;
        data_len = fits ? len + wg_padding(len, a.wg.mtu) : 0u;
    } else {
        data_len = (len >= 32u && len - 32u <= WG_FUSE_MAX_LEN) ? len - 32u : 0u;
        data_there = data_len;
    }
    const uint32_t at = 64u * (lane - 1u);
    const uint32_t mine = (lane == 0 || at >= data_len) ? 0u : min(data_len - at, 64u);
    const uint32_t there = (lane == 0 || at >= data_there) ? 0u : min(data_there - at, 64u);
    // The wave fetches the packet in pieces of 1 KB, lane l taking bytes [16 l,
    // 16 l + 16) of each piece, so that an instruction reads 1 KB in a row; the
    // lanes pick their own 64-byte blocks out of LDS further down.  (A lane
    // fetching its own block reads 16 bytes every 64: sixty-four small requests
    // an instruction, which a packet that lies in host memory pays for with a
    // read of its own over the link for each.)
    // What the packet's bytes wait for goes out ahead of them, so that a wait for it does
    // not wait for them as well (a wave's loads complete in the order they were issued): the
    // sender's key where the sender is known by now, with the receiver's index for the
    // header on the way out; on the way in the header, which names the sender.
    uint4 key_lo = make_uint4(0, 0, 0, 0), key_hi = key_lo, wg_head = key_lo;
    uint32_t wg_remote = 0;
    if (!(WG && OPEN)) {
        const uint32_t known = pr < (WG ? a.wg.n_peers : a.n_peers) ? pr : 0u; // (the table has a row 0)
        const uint4 *kp = reinterpret_cast<const uint4 *>(a.keys + 8u * known);
        key_lo = kp[0];
        key_hi = kp[1];
        if (WG) wg_remote = a.wg.remote_index[known];
    } else {
        wg_head = ld16(len >= 32u && len - 32u <= WG_FUSE_MAX_LEN ? src : safe);
    }
    // Every load below is issued whatever the lane's share is (from the key table where it
    // has none), so that they are all in flight together: the pieces, the last 1-15 bytes of
    // the packet (one lane's, by words, a halfword and a byte: nothing beyond the packet is
    // touched), and the tag.
    uint4 pre[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t off = 1024u * j + 16u * lane;
        pre[j] = ld16(off + 16u <= data_there ? data + off : safe);
    }
    const uint32_t odd = data_there & 15u, odd_at = data_there & ~15u; // the packet's last, partial cell
    const bool odd_mine = odd != 0u && ((odd_at >> 4) & 63u) == lane;
    const uint4 odd_cell = ld_partial_flat(data + odd_at, odd_mine ? odd : 0u, safe);
    const bool tagged = OPEN && (WG ? len >= 32u && len - 32u <= WG_FUSE_MAX_LEN : len >= 16u && data_len <= SPREAD_MAX_LEN);
    uint4 want_tag = ld16(tagged ? data + data_len : safe);
    // (what the lanes without a share have fetched is set aside where the pieces are used,
    // further down: looking at it here would make the key wait for the packet)

    if (!WG) {
        if (skipped) return;
        if (pr >= a.n_peers) {
            if (lane == 0) {
                status_raise(a.status, STATUS_PEER_RANGE);
                if (OPEN) a.verdict[i] = 0;
            }
            return;
        }
        if (OPEN && len < 16u) {
            if (lane == 0) a.verdict[i] = 0;
            return;
        }
        if (OPEN) len -= 16u;
        ctr = a.counters ? ctr_ld : a.counter0 + i;
    } else if (!OPEN) {
        // ---- encapsulate: header into the headroom, padding as implied zeros ----
        if (pr >= a.wg.n_peers || len + 15u > WG_FUSE_MAX_LEN) {
            if (lane == 0) a.wg.wire_len[i] = 0;
            return;
        }
        ctr = ctr_ld;
        if (ctr >= WG_REJECT_AFTER_MESSAGES) { // the keypair has used up its nonces
            if (lane == 0) a.wg.wire_len[i] = 0;
            return;
        }
        len += wg_padding(len, a.wg.mtu);
        if (lane == 0) {
            st16(dst, make_uint4(4u, wg_remote, (uint32_t)ctr, (uint32_t)(ctr >> 32)));
            a.wg.wire_len[i] = 16u + len + 16u;
        }
        src += 16;
        dst += 16;
    } else {
        // ---- decapsulate: header checks and the receiver-index lookup ----
        uint8_t res = BNK_WG_OK;
        uint4 h = make_uint4(0, 0, 0, 0);
        if (len < 32u || len - 32u > WG_FUSE_MAX_LEN) res = BNK_WG_BAD_HEADER;
        else h = wg_head;
        if (res == BNK_WG_OK && h.x != 4u) res = BNK_WG_BAD_HEADER;
        if (res == BNK_WG_OK) {
            // narrow [lo, hi) to at most 64 entries, 64 probes at a time
            uint32_t lo = 0, hi = a.wg.n_peers;
            while (hi - lo > 64u) {
                const uint32_t step = (hi - lo + 63u) / 64u;
                const uint32_t at = min(lo + lane * step, hi - 1u);
                const bool le = a.wg.index_sorted[at].x <= h.y;
                const unsigned long long m = __ballot(le);
                // lanes probe ascending positions: those at or below the index form a prefix
                const uint32_t below = (uint32_t)__popcll(m);
                if (below == 0u) { hi = lo; break; }
                const uint32_t nlo = min(lo + (below - 1u) * step, hi - 1u);
                hi = min(nlo + step, hi);
                lo = nlo;
            }
            uint2 e = make_uint2(0, 0);
            const bool mine = lo + lane < hi;
            if (mine) e = a.wg.index_sorted[lo + lane];
            const unsigned long long hit = __ballot(mine && e.x == h.y);
            if (hit == 0ull) res = BNK_WG_UNKNOWN_INDEX;
            else pr = (uint32_t)__shfl((int)e.y, __ffsll((long long)hit) - 1, 64);
        }
        if (res != BNK_WG_OK) {
            if (lane == 0) {
                a.wg.result[i] = res;
                a.wg.out_len[i] = 0;
                a.wg.peer_out[i] = 0xFFFFFFFFu;
                a.wg.counter_out[i] = 0;
            }
            return;
        }
        ctr = (uint64_t)h.z | (uint64_t)h.w << 32;
        len -= 32u; // header and tag
        src += 16;
    }
    uint32_t k[8];
    {
        if (WG && OPEN) { // (the sender has only now been found)
            const uint4 *kp = reinterpret_cast<const uint4 *>(a.keys + 8u * pr);
            key_lo = kp[0];
            key_hi = kp[1];
        }
        k[0] = key_lo.x; k[1] = key_lo.y; k[2] = key_lo.z; k[3] = key_lo.w;
        k[4] = key_hi.x; k[5] = key_hi.y; k[6] = key_hi.z; k[7] = key_hi.w;
    }
    const uint32_t n1 = (uint32_t)ctr, n2 = (uint32_t)(ctr >> 32);
    uint32_t x[16];

    if (!WG && len > SPREAD_MAX_LEN) {
        const bool have = lane == 0;
        Poly32 mac;
        Head no_head;
        no_head.on = false;
        body_generic<OPEN>(tile_all[threadIdx.x >> 6], lane, have ? src : nullptr, have ? dst : nullptr,
                           have ? len : 0u, reinterpret_cast<const uint8_t *>(a.keys), k, n1, n2, mac, x, no_head);
        lane_finish<OPEN>(a, lane, have, i, len, have ? src : nullptr, have ? dst : nullptr, mac, no_head, nullptr);
        return;
    }

    // (the packet's bytes are already on their way: see the top of the kernel)
    chacha_block(k, lane, n1, n2, x);
    // Block b of the packet lies at stage + 80 b (rows padded against bank
    // conflicts): written in the order the pieces came in, read a block per lane.
    uint8_t *stage = tile_all[threadIdx.x >> 6];
    if (!tagged) want_tag = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t off = 1024u * j + 16u * lane;
        // a cell beyond the packet's whole cells is zeros, but for its last 1-15 bytes
        if (off + 16u > data_there) pre[j] = make_uint4(0, 0, 0, 0);
        if (odd_mine && (odd_at >> 10) == (uint32_t)j) pre[j] = odd_cell;
        if (1024u * j < data_there)
            *reinterpret_cast<uint4 *>(stage + (16u * j + (lane >> 2)) * LDS_ROW + 16u * (lane & 3u)) = pre[j];
    }
    wave_sync();
    uint32_t m[16];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        uint4 v = make_uint4(0, 0, 0, 0);
        // (bytes of a cell beyond the data were fetched as zeros)
        if (there > 16u * j) v = *reinterpret_cast<const uint4 *>(stage + (lane - 1u) * LDS_ROW + 16u * j);
        m[4 * j] = v.x; m[4 * j + 1] = v.y; m[4 * j + 2] = v.z; m[4 * j + 3] = v.w;
    }
    // the one-time key is lane 0's block
    const Fe26 r = fe_clamped_r((uint32_t)__builtin_amdgcn_readlane((int)x[0], 0),
                                (uint32_t)__builtin_amdgcn_readlane((int)x[1], 0),
                                (uint32_t)__builtin_amdgcn_readlane((int)x[2], 0),
                                (uint32_t)__builtin_amdgcn_readlane((int)x[3], 0));
    const uint32_t pad[4] = {(uint32_t)__builtin_amdgcn_readlane((int)x[4], 0),
                             (uint32_t)__builtin_amdgcn_readlane((int)x[5], 0),
                             (uint32_t)__builtin_amdgcn_readlane((int)x[6], 0),
                             (uint32_t)__builtin_amdgcn_readlane((int)x[7], 0)};

    // ---- crypt: o = m ^ keystream; the MAC reads the ciphertext side ----
    uint32_t o[16];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        uint4 v = make_uint4(m[4 * j] ^ x[4 * j], m[4 * j + 1] ^ x[4 * j + 1], m[4 * j + 2] ^ x[4 * j + 2],
                             m[4 * j + 3] ^ x[4 * j + 3]);
        const uint32_t have_b = mine > 16u * j ? min(mine - 16u * j, 16u) : 0u;
        v = keep_bytes(v, have_b);
        o[4 * j] = v.x; o[4 * j + 1] = v.y; o[4 * j + 2] = v.z; o[4 * j + 3] = v.w;
    }
    if (lane == 0) {
        // LE64(len(aad) = 0) || LE64(len(ciphertext)) as my only cell
        m[0] = 0; m[1] = 0; m[2] = len; m[3] = 0;
        o[0] = 0; o[1] = 0; o[2] = len; o[3] = 0;
    }
    const SpreadShare sh = spread_share(lane, len);
    const Fe26 term = spread_term(r, OPEN ? m : o, sh.k, sh.e, spread_e_max(len));

    // ---- add the 64 terms: 32 lanes fit 32 bits per limb, the last step is wider ----
    uint32_t t32[5] = {term.v0, term.v1, term.v2, term.v3, term.v4};
#pragma unroll
    for (int step = 1; step < 32; step <<= 1)
#pragma unroll
        for (int q = 0; q < 5; q++) t32[q] += (uint32_t)__shfl_xor((int)t32[q], step, 64);
    uint64_t sum[5];
#pragma unroll
    for (int q = 0; q < 5; q++) sum[q] = (uint64_t)t32[q] + (uint32_t)__shfl_xor((int)t32[q], 32, 64);
    uint32_t tag[4];
    spread_finish(sum, pad, tag);

    bool reject = false;
    if (!OPEN) {
        if (lane == 0) st16(dst + len, make_uint4(tag[0], tag[1], tag[2], tag[3]));
    } else {
        // all 16 bytes are compared, no early exit
        reject = ((want_tag.x ^ tag[0]) | (want_tag.y ^ tag[1]) | (want_tag.z ^ tag[2]) |
                  (want_tag.w ^ tag[3])) != 0;
        if (!WG && lane == 0) a.verdict[i] = reject ? 0 : 1;
    }
    if (WG && OPEN) {
        // ---- what wireguard-go checks once a packet is authentic: keepalive, IP
        // version, length fields, source inside the sender's allowed prefix.  The
        // first 16 plaintext bytes (lane 1's first cell) hold every field used.
        const uint32_t w0 = (uint32_t)__builtin_amdgcn_readlane((int)o[0], 1);
        const uint32_t w1 = (uint32_t)__builtin_amdgcn_readlane((int)o[1], 1);
        const uint32_t w3 = (uint32_t)__builtin_amdgcn_readlane((int)o[3], 1);
        uint8_t res = BNK_WG_OK;
        uint32_t inner = 0;
        const uint32_t version = (w0 >> 4) & 0xFu;
        if (reject) res = BNK_WG_AUTH_FAIL;
        else if (len == 0u) res = BNK_WG_KEEPALIVE;
        else if (len < 16u) res = BNK_WG_BAD_IP;
        else if (version == 4u) {
            const uint32_t total = __builtin_bswap32(w0) & 0xFFFFu;
            const uint2 al = a.wg.allowed[pr];
            if (len < 20u || total > len || total < 20u) res = BNK_WG_BAD_IP;
            else if ((__builtin_bswap32(w3) & al.y) != (al.x & al.y)) res = BNK_WG_NOT_ALLOWED;
            else inner = total;
        } else if (version == 6u) {
            // peers own IPv4 addresses only
            const uint32_t total = (__builtin_bswap32(w1) >> 16) + 40u;
            res = (len < 40u || total > len) ? BNK_WG_BAD_IP : BNK_WG_NOT_ALLOWED;
        } else {
            res = BNK_WG_BAD_IP;
        }
        if (lane == 0) {
            a.wg.result[i] = res;
            a.wg.out_len[i] = inner;
            a.wg.peer_out[i] = pr;
            a.wg.counter_out[i] = ctr;
        }
    }
    // ---- the bytes out, the way they came in: blocks into LDS, pieces of 1 KB in
    // a row out of it; a rejected packet leaves zeros (chacha20poly1305.Open) ----
    wave_sync();
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint4 v = reject ? make_uint4(0, 0, 0, 0)
                               : make_uint4(o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]);
        if (mine > 16u * j) *reinterpret_cast<uint4 *>(stage + (lane - 1u) * LDS_ROW + 16u * j) = v;
    }
    wave_sync();
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t off = 1024u * j + 16u * lane;
        if (1024u * j < data_len && off < data_len) {
            const uint4 v = *reinterpret_cast<const uint4 *>(stage + (16u * j + (lane >> 2)) * LDS_ROW + 16u * (lane & 3u));
            if (off + 16u <= data_len) st16(dst + off, v);
            else st_partial(dst + off, v, data_len - off);
        }
    }
}

// A lane per packet takes about 20 us + 43 ns per byte of the longest packet
// however few packets there are, a wave per packet about 17 us + 2.7 to 3.3 ns
// per packet (200 to 1420 bytes): measured crossovers 3,000 packets of 60
// bytes, 4,800 of 200, 16,400 of 1420.  With the common length known the rule
// below stays just under them; without it the caller's threshold stands alone.
bool aead_runs_spread(const AeadArgs &a)
{
    if (a.lens) return a.n <= a.spread_max;
    const uint64_t by_len = 12ull * a.len + a.spread_max / 2;
    return a.n <= std::min<uint64_t>(4ull * a.spread_max, by_len);
}

// Can the host tell that every wave of the launch takes the short path?  One
// common length of at most SHORT_BLOCKS blocks once trimmed, framed and padded,
// uniform strides, and every packet 16-byte aligned at the same place of a
// 128-byte line in both arenas.
static bool every_wave_short(const AeadArgs &a, bool open)
{
    if (a.lens || a.order || a.in_off || a.out_off) return false;
    uint64_t len = a.len;
    if (open) {
        if (a.wg.mode == WG_FUSE_DECAP) len = len >= 16u ? len - 16u : 0u; // the header
        len = len >= 16u ? len - 16u : 0u;                                  // the tag
    } else {
        len = len >= a.trim ? len - a.trim : 0u;
        if (a.wg.mode == WG_FUSE_ENCAP) len += 15u; // at most this much padding
    }
    if (len > 64u * SHORT_BLOCKS) return false;
    const uint64_t src0 = (uint64_t)(uintptr_t)a.in + a.in_skip, dst0 = (uint64_t)(uintptr_t)a.out + a.out_skip;
    if (((src0 | dst0 | a.in_stride | a.out_stride) & 15u) != 0) return false;
    return ((src0 ^ dst0) & 127u) == 0 && ((a.in_stride ^ a.out_stride) & 127u) == 0;
}

template <bool OPEN>
static hipError_t launch_wave(const AeadArgs &a, hipStream_t s)
{
    if (every_wave_short(a, OPEN))
        hipLaunchKernelGGL(aead_short_kernel<OPEN>, dim3((a.n + LANE_BLOCK - 1u) / LANE_BLOCK), dim3(LANE_BLOCK), 0, s, a);
    else
        hipLaunchKernelGGL(aead_wave_kernel<OPEN>, dim3((a.n + LANE_BLOCK - 1u) / LANE_BLOCK), dim3(LANE_BLOCK), 0, s, a);
    return hipGetLastError();
}

hipError_t launch_aead_seal(const AeadArgs &a, hipStream_t s)
{
    if (a.n == 0) return hipSuccess;
    const dim3 waves((a.n + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK);
    // (the two framing launches differ in what a packet's offset means: see AeadArgs::wg)
    if (a.wg.mode != WG_FUSE_OFF) {
        if (a.wg.mode != WG_FUSE_ENCAP) return hipErrorInvalidValue;
        if (!aead_runs_spread(a)) return a.in_skip == 16u && a.out_skip == 16u ? launch_wave<false>(a, s) : hipErrorInvalidValue;
        if (a.in_skip != 0u) return hipErrorInvalidValue;
        hipLaunchKernelGGL((aead_spread_kernel<false, true>), waves, dim3(256), 0, s, a);
    } else if (aead_runs_spread(a))
        hipLaunchKernelGGL((aead_spread_kernel<false, false>), waves, dim3(256), 0, s, a);
    else
        return launch_wave<false>(a, s);
    return hipGetLastError();
}

hipError_t launch_aead_open(const AeadArgs &a, hipStream_t s)
{
    if (a.n == 0) return hipSuccess;
    const dim3 waves((a.n + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK);
    if (a.wg.mode != WG_FUSE_OFF) {
        if (a.wg.mode != WG_FUSE_DECAP) return hipErrorInvalidValue;
        if (!aead_runs_spread(a)) return a.in_skip == 16u && a.out_skip == 0u ? launch_wave<true>(a, s) : hipErrorInvalidValue;
        if (a.in_skip != 0u) return hipErrorInvalidValue;
        hipLaunchKernelGGL((aead_spread_kernel<true, true>), waves, dim3(256), 0, s, a);
    } else if (aead_runs_spread(a))
        hipLaunchKernelGGL((aead_spread_kernel<true, false>), waves, dim3(256), 0, s, a);
    else
        return launch_wave<true>(a, s);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Group packets by ChaCha20 block count (longest first).
// ---------------------------------------------------------------------------

BNK_DEV uint32_t len_bin(uint32_t len, uint32_t tag_bytes)
{
    const uint32_t pl = len >= tag_bytes ? len - tag_bytes : 0u;
    const uint32_t nb = (pl + 63u) >> 6;
    // longest first: bin 0 holds the largest block counts
    return nb >= LEN_BINS - 1 ? 0u : (LEN_BINS - 1 - nb);
}

// Adds one to bins[b] for every participating lane and returns what the
// lane's own atomicAdd would have returned, with one LDS atomic per distinct
// bin of the wave instead of one per lane: traffic is a handful of sizes, so
// most lanes of a wave hit the same bin and would serialise on it.  The
// leader's values travel through scalar registers (v_readlane), not through
// LDS.  After eight rounds the remaining lanes (a wave with many distinct
// sizes) go one by one.
BNK_DEV uint32_t wave_bin_add(uint32_t *bins, uint32_t b, bool active)
{
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t result = 0;
    bool todo = active;
    for (int round = 0; round < 8; round++) {
        const unsigned long long left = __ballot(todo);
        if (left == 0ull) return result;
        const int leader = __ffsll((long long)left) - 1;
        const uint32_t lb = (uint32_t)__builtin_amdgcn_readlane((int)b, leader);
        const bool mine = todo && b == lb;
        const unsigned long long same = __ballot(mine);
        uint32_t old = 0;
        if ((int)lane == leader) old = atomicAdd(&bins[lb], (uint32_t)__popcll(same));
        old = (uint32_t)__builtin_amdgcn_readlane((int)old, leader);
        if (mine) {
            result = old + (uint32_t)__popcll(same & ((1ull << lane) - 1ull));
            todo = false;
        }
    }
    if (todo) result = atomicAdd(&bins[b], 1u);
    return result;
}

// A block of GROUP_THREADS threads takes GROUP_CHUNK consecutive packets, four
// per thread, loaded together so that their latencies overlap.
constexpr uint32_t GROUP_THREADS = 1024;
constexpr uint32_t GROUP_PER_THREAD = 4;
constexpr uint32_t GROUP_CHUNK = GROUP_THREADS * GROUP_PER_THREAD;

__global__ __launch_bounds__(GROUP_THREADS) void len_hist_kernel(const uint32_t *lens, uint32_t n,
                                                                 uint32_t tag_bytes, uint32_t *hist,
                                                                 uint32_t *cursor, bool clear_cursor)
{
    __shared__ uint32_t lh[LEN_BINS];
    for (uint32_t b = threadIdx.x; b < LEN_BINS; b += GROUP_THREADS) lh[b] = 0;
    // a scatter launch that scans for itself counts from zero in cursor[]
    if (clear_cursor && blockIdx.x == 0)
        for (uint32_t b = threadIdx.x; b < LEN_CURSOR_WORDS; b += GROUP_THREADS) cursor[b] = 0;
    const uint32_t base = blockIdx.x * GROUP_CHUNK + threadIdx.x;
    uint32_t len[GROUP_PER_THREAD];
#pragma unroll
    for (uint32_t j = 0; j < GROUP_PER_THREAD; j++) {
        const uint32_t i = base + j * GROUP_THREADS;
        len[j] = i < n ? lens[i] : 0u;
    }
    __syncthreads();
    // whole waves call the helper together (it uses wave-wide votes)
#pragma unroll
    for (uint32_t j = 0; j < GROUP_PER_THREAD; j++)
        (void)wave_bin_add(lh, len_bin(len[j], tag_bytes), base + j * GROUP_THREADS < n);
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < LEN_BINS; b += GROUP_THREADS)
        if (lh[b]) atomicAdd(&hist[b], lh[b]);
}

// Exclusive scan of hist into cursor (one block of LEN_SCAN_THREADS), leaving
// hist all zeros for the next grouping.  For batches of many blocks: there the
// scan inside every scatter block (below) costs more than this launch, the
// blocks of an XCD all fetching the same few lines.
constexpr uint32_t LEN_SCAN_THREADS = 1024;
__global__ __launch_bounds__(LEN_SCAN_THREADS) void len_scan_kernel(uint32_t *hist, uint32_t *cursor)
{
    __shared__ uint32_t wave_sum[LEN_SCAN_THREADS / 64];
    constexpr uint32_t PER = (LEN_BINS + LEN_SCAN_THREADS - 1) / LEN_SCAN_THREADS;
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;
    uint32_t loc[PER];
    uint32_t sum = 0;
#pragma unroll
    for (uint32_t q = 0; q < PER; q++) {
        const uint32_t b = threadIdx.x * PER + q;
        loc[q] = b < LEN_BINS ? hist[b] : 0u;
        if (b < LEN_BINS) hist[b] = 0u;
        sum += loc[q];
    }
    // inclusive scan within the wave, then across the waves
    uint32_t inc = sum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t o = (uint32_t)__shfl_up((int)inc, off, 64);
        if ((int)lane >= off) inc += o;
    }
    if (lane == 63u) wave_sum[wv] = inc;
    __syncthreads();
    uint32_t before = 0;
    for (uint32_t w = 0; w < wv; w++) before += wave_sum[w];
    uint32_t run = before + inc - sum;
#pragma unroll
    for (uint32_t q = 0; q < PER; q++) {
        const uint32_t b = threadIdx.x * PER + q;
        if (b < LEN_BINS) cursor[b] = run;
        run += loc[q];
    }
}

// Places the packets.  SCAN false: cursor[b] holds where bin b starts
// (len_scan_kernel) and a block reserves its share of the bin there.  SCAN
// true (batches of few blocks, no len_scan_kernel launch): every block scans
// the whole histogram for itself (1032 words from L2, one scan by the first
// waves of the block) and cursor[b], zero on entry, counts within the bin; the
// block that is the last to have read hist clears it for the next grouping: a
// block counts itself in cursor[LEN_DONE_WORD] behind the barrier that follows
// its scan, whose additions consumed the loaded values, so no fence is needed.
constexpr uint32_t LEN_DONE_WORD = LEN_BINS;
// up to 2^20 packets: one block per compute unit; measured 1.6 us less than the
// scan launch per grouping there, 3.6 us more at 2^22 packets
constexpr uint32_t LEN_FUSED_SCAN_MAX_BLOCKS = 256;
static_assert(LEN_CURSOR_WORDS > LEN_DONE_WORD, "cursor[] holds the count of blocks that have read hist");
template <bool SCAN>
__global__ __launch_bounds__(GROUP_THREADS) void len_scatter_kernel(const uint32_t *lens, uint32_t n,
                                                                    uint32_t tag_bytes, uint32_t *hist,
                                                                    uint32_t *cursor, uint32_t *order)
{
    constexpr uint32_t PER = (LEN_BINS + GROUP_THREADS - 1) / GROUP_THREADS;
    constexpr uint32_t SCAN_WAVES = ((LEN_BINS + PER - 1) / PER + 63) / 64;
    __shared__ uint32_t cnt[LEN_BINS];
    __shared__ uint32_t base[LEN_BINS];
    __shared__ uint32_t wave_sum[SCAN_WAVES];
    const uint32_t lane = threadIdx.x & 63u, wv = threadIdx.x >> 6;
    for (uint32_t b = threadIdx.x; b < LEN_BINS; b += GROUP_THREADS) cnt[b] = 0;
    const uint32_t first = blockIdx.x * GROUP_CHUNK + threadIdx.x;
    uint32_t bin[GROUP_PER_THREAD], at[GROUP_PER_THREAD];
#pragma unroll
    for (uint32_t j = 0; j < GROUP_PER_THREAD; j++) {
        const uint32_t i = first + j * GROUP_THREADS;
        bin[j] = len_bin(i < n ? lens[i] : 0u, tag_bytes);
    }
    // exclusive scan of hist into base[]: PER consecutive bins per thread,
    // inclusive scan within the wave, then across the waves
    uint32_t loc[PER];
    uint32_t sum = 0, inc = 0;
    if (SCAN && wv < SCAN_WAVES) {
#pragma unroll
        for (uint32_t q = 0; q < PER; q++) {
            const uint32_t b = threadIdx.x * PER + q;
            loc[q] = b < LEN_BINS ? hist[b] : 0u;
            sum += loc[q];
        }
        inc = sum;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t o = (uint32_t)__shfl_up((int)inc, off, 64);
            if ((int)lane >= off) inc += o;
        }
        if (lane == 63u) wave_sum[wv] = inc;
    }
    __syncthreads();
    uint32_t seen = 0;
    if (SCAN && threadIdx.x == 0) seen = atomicAdd(&cursor[LEN_DONE_WORD], 1u);
    if (SCAN && wv < SCAN_WAVES) {
        uint32_t run = inc - sum;
        for (uint32_t w = 0; w < wv; w++) run += wave_sum[w];
#pragma unroll
        for (uint32_t q = 0; q < PER; q++) {
            const uint32_t b = threadIdx.x * PER + q;
            if (b < LEN_BINS) base[b] = run;
            run += loc[q];
        }
    }
    // a packet's place within its block's share of the bin, then one
    // reservation per bin for the whole block
#pragma unroll
    for (uint32_t j = 0; j < GROUP_PER_THREAD; j++)
        at[j] = wave_bin_add(cnt, bin[j], first + j * GROUP_THREADS < n);
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < LEN_BINS; b += GROUP_THREADS) {
        const uint32_t c = cnt[b];
        if (c) base[b] = (SCAN ? base[b] : 0u) + atomicAdd(&cursor[b], c);
    }
    __syncthreads();
#pragma unroll
    for (uint32_t j = 0; j < GROUP_PER_THREAD; j++) {
        const uint32_t i = first + j * GROUP_THREADS;
        if (i < n) order[base[bin[j]] + at[j]] = i;
    }
    if (SCAN && wv == 0 && (uint32_t)__builtin_amdgcn_readfirstlane((int)seen) + 1u == gridDim.x)
        for (uint32_t b = lane; b < LEN_BINS; b += 64u) hist[b] = 0;
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t *p, uint32_t n, uint32_t v)
{
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < n) p[i] = v;
}

hipError_t launch_fill_u32(uint32_t *p, uint32_t n, uint32_t v, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((n + 255u) / 256u), dim3(256), 0, s, p, n, v);
    return hipGetLastError();
}

// The last launch of a host call that waits by watching a word in pinned host
// memory: everything the stream ran before this kernel has completed when it
// starts (kernels of one stream do not overlap, and a kernel's end makes its
// stores visible at system scope); the fence and the release store at system
// scope state that order for this store as well, so a host that sees `v` in the
// word also sees every result the earlier kernels wrote to host memory.
__global__ void done_word_kernel(uint32_t *word, uint32_t v)
{
    __threadfence_system();
    __hip_atomic_store(word, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

hipError_t launch_done_word(uint32_t *word, uint32_t v, hipStream_t s)
{
    hipLaunchKernelGGL(done_word_kernel, dim3(1), dim3(1), 0, s, word, v);
    return hipGetLastError();
}

// Copies `bytes` bytes from src to dst, which must share their alignment
// within 16 bytes: every lane moves one aligned 16-byte piece, so a span in
// pinned host memory crosses the link in one round trip instead of one per
// ChaCha20 line.  The ragged ends go byte by byte.
__global__ __launch_bounds__(256) void pull_kernel(const uint8_t *src, uint8_t *dst, uint64_t bytes)
{
    const uint64_t head = min((uint64_t)((16u - (uint32_t)((uintptr_t)src & 15u)) & 15u), bytes);
    const uint64_t n16 = (bytes - head) >> 4;
    const uint64_t tail = head + (n16 << 4);
    const uint64_t stride = (uint64_t)gridDim.x * 256u;
    for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < n16; i += stride)
        st16a(dst + head + (i << 4), ld16a(src + head + (i << 4)));
    if (blockIdx.x == 0) {
        if (threadIdx.x < head) st8(dst + threadIdx.x, ld8(src + threadIdx.x));
        const uint32_t t = threadIdx.x - 64u;
        if (threadIdx.x >= 64u && tail + t < bytes) st8(dst + tail + t, ld8(src + tail + t));
    }
}

hipError_t launch_pull(const void *src, void *dst, uint64_t bytes, hipStream_t s)
{
    if (bytes == 0) return hipSuccess;
    if ((((uintptr_t)src ^ (uintptr_t)dst) & 15u) != 0) return hipErrorInvalidValue;
    const uint64_t blocks = std::min<uint64_t>((bytes / 16 + 255) / 256 + 1, 2048);
    hipLaunchKernelGGL(pull_kernel, dim3((uint32_t)blocks), dim3(256), 0, s, (const uint8_t *)src,
                       (uint8_t *)dst, bytes);
    return hipGetLastError();
}

hipError_t launch_length_sort(const uint32_t *lens, uint32_t n, uint32_t tag_bytes,
                              uint32_t *order, uint32_t *hist, uint32_t *cursor,
                              hipStream_t s)
{
    if (n == 0) return hipSuccess;
    // hist is all zeros on entry: its owner clears it once when it is allocated
    // and every grouping leaves it cleared (len_scan_kernel, or the scatter
    // launch that scans for itself)
    const uint32_t blocks = (n + GROUP_CHUNK - 1u) / GROUP_CHUNK;
    const bool fused = blocks <= LEN_FUSED_SCAN_MAX_BLOCKS;
    hipLaunchKernelGGL(len_hist_kernel, dim3(blocks), dim3(GROUP_THREADS), 0, s, lens, n, tag_bytes, hist,
                       cursor, fused);
    if (fused) {
        hipLaunchKernelGGL(len_scatter_kernel<true>, dim3(blocks), dim3(GROUP_THREADS), 0, s, lens, n,
                           tag_bytes, hist, cursor, order);
    } else {
        hipLaunchKernelGGL(len_scan_kernel, dim3(1), dim3(LEN_SCAN_THREADS), 0, s, hist, cursor);
        hipLaunchKernelGGL(len_scatter_kernel<false>, dim3(blocks), dim3(GROUP_THREADS), 0, s, lens, n,
                           tag_bytes, hist, cursor, order);
    }
    return hipGetLastError();
}

} // namespace bnk
