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
#include "kernels.hpp"

namespace bnk {

// Global memory accesses of 16 bytes at any byte alignment (the hardware
// handles misaligned dwordx4 accesses; aligned ones cost nothing extra).
BNK_DEV uint4 ld16(const uint8_t *p)
{
    uint4 v;
    __builtin_memcpy(&v, p, 16);
    return v;
}

BNK_DEV void st16(uint8_t *p, uint4 v) { __builtin_memcpy(p, &v, 16); }

// m in 1..15 bytes at p, zero-extended to 16.
BNK_DEV uint4 ld_partial(const uint8_t *p, uint32_t m)
{
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 15; i++)
        if ((uint32_t)i < m) w[i >> 2] |= (uint32_t)p[i] << (8 * (i & 3));
    return make_uint4(w[0], w[1], w[2], w[3]);
}

BNK_DEV void st_partial(uint8_t *p, uint4 v, uint32_t m)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 15; i++)
        if ((uint32_t)i < m) p[i] = (uint8_t)(w[i >> 2] >> (8 * (i & 3)));
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

BNK_DEV void zero_fill(uint8_t *dst, uint32_t len)
{
    uint32_t pos = 0;
    for (; pos + 16 <= len; pos += 16) st16(dst + pos, make_uint4(0, 0, 0, 0));
    for (; pos < len; pos++) dst[pos] = 0;
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
// touched cooperatively: in step b the wave moves bytes [64b, 64b+64) of all
// its 64 packets with four 16-byte accesses per lane, four adjacent lanes
// covering one packet's 64 contiguous bytes, and a 64 x 80-byte LDS tile
// (64 data bytes + 16 bytes of padding per row, which keeps the per-lane row
// reads free of bank conflicts) turns that layout into one row per lane.
constexpr uint32_t LDS_ROW = 80;
constexpr uint32_t WAVES_PER_BLOCK = 4;

template <bool OPEN>
__global__ __launch_bounds__(256) void aead_wave_kernel(AeadArgs a)
{
    __shared__ __attribute__((aligned(16))) uint8_t tile_all[WAVES_PER_BLOCK][64 * LDS_ROW];
    const uint32_t lane = threadIdx.x & 63u;
    uint8_t *tile = tile_all[threadIdx.x >> 6];
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;

    // ---- this lane's packet ----
    bool have = t < a.n;
    uint32_t i = 0, len = 0;
    const uint8_t *src = nullptr;
    uint8_t *dst = nullptr;
    uint32_t k[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    uint64_t ctr = 0;
    if (have) {
        i = a.order ? a.order[t] : t;
        len = a.lens ? a.lens[i] : a.len;
        if (!OPEN) len = len >= a.trim ? len - a.trim : 0u;
        const uint32_t pr = a.peer ? a.peer[i] : 0u;
        if (a.skip && a.skip[i] != 0) {
            have = false;
        } else if (pr >= a.n_peers) {
            atomicOr(a.status, STATUS_PEER_RANGE);
            if (OPEN) a.verdict[i] = 0;
            have = false;
        } else if (OPEN && len < 16u) {
            a.verdict[i] = 0;
            have = false;
        } else {
            if (OPEN) len -= 16u;
            src = a.in + (a.in_off ? a.in_off[i] : (uint64_t)i * a.in_stride);
            dst = a.out + (a.out_off ? a.out_off[i] : (uint64_t)i * a.out_stride);
            const uint4 *kp = reinterpret_cast<const uint4 *>(a.keys + 8u * pr);
            const uint4 k0 = kp[0], k1 = kp[1];
            k[0] = k0.x; k[1] = k0.y; k[2] = k0.z; k[3] = k0.w;
            k[4] = k1.x; k[5] = k1.y; k[6] = k1.z; k[7] = k1.w;
            ctr = a.counters ? a.counters[i] : a.counter0 + i;
        }
    }
    if (!have) len = 0;
    const uint32_t nfull = len >> 6, rem = len & 63u;
    const uint32_t steps = nfull + (rem ? 1u : 0u);

    // ---- the four (packet, 16-byte column) cells this lane moves per step ----
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

    const uint32_t n1 = (uint32_t)ctr, n2 = (uint32_t)(ctr >> 32);
    uint32_t x[16];
    chacha_block(k, 0, n1, n2, x);
    Poly26 mac;
    mac.init(x);

    for (uint32_t b = 0; __ballot(b < steps) != 0ull; b++) {
        const uint32_t pos = 64u * b + 16u * col;
        // global -> LDS, all 64 lanes, only 16-byte cells that lie fully inside a packet
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (pos + 16u <= clen[j]) {
                const uint4 v = ld16(csrc[j] + 64u * b);
                *reinterpret_cast<uint4 *>(tile + (16u * j + (lane >> 2)) * LDS_ROW + 16u * col) = v;
            }
        }
        wave_sync();
        if (b < steps) {
            chacha_block(k, b + 1, n1, n2, x);
            uint8_t *row = tile + lane * LDS_ROW;
            if (b < nfull) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint4 v = *reinterpret_cast<const uint4 *>(row + 16 * j);
                    const uint4 o = make_uint4(v.x ^ x[4 * j], v.y ^ x[4 * j + 1],
                                               v.z ^ x[4 * j + 2], v.w ^ x[4 * j + 3]);
                    if (OPEN) mac.block(v.x, v.y, v.z, v.w);
                    else mac.block(o.x, o.y, o.z, o.w);
                    *reinterpret_cast<uint4 *>(row + 16 * j) = o;
                }
            } else {
                // last, partial block: whole cells through the tile, the
                // final 1..15 bytes straight from and to global memory
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if (rem >= 16u * (j + 1)) {
                        const uint4 v = *reinterpret_cast<const uint4 *>(row + 16 * j);
                        const uint4 o = make_uint4(v.x ^ x[4 * j], v.y ^ x[4 * j + 1],
                                                   v.z ^ x[4 * j + 2], v.w ^ x[4 * j + 3]);
                        if (OPEN) mac.block(v.x, v.y, v.z, v.w);
                        else mac.block(o.x, o.y, o.z, o.w);
                        *reinterpret_cast<uint4 *>(row + 16 * j) = o;
                    } else if (rem > 16u * j) {
                        const uint32_t m = rem - 16u * j;
                        const uint4 v = ld_partial(src + 64u * b + 16 * j, m);
                        const uint4 o = keep_bytes(
                            make_uint4(v.x ^ x[4 * j], v.y ^ x[4 * j + 1],
                                       v.z ^ x[4 * j + 2], v.w ^ x[4 * j + 3]), m);
                        // the MAC sees the ciphertext zero-padded to 16 bytes
                        if (OPEN) mac.block(v.x, v.y, v.z, v.w);
                        else mac.block(o.x, o.y, o.z, o.w);
                        st_partial(dst + 64u * b + 16 * j, o, m);
                    }
                }
            }
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
            a.verdict[i] = reject ? 0 : 1;
        }
    }
    if (OPEN && __ballot(reject) != 0ull) {
        // the plaintext cells were stored by other lanes of this wave: make
        // those stores land before this lane overwrites them with zeros
        __threadfence();
        if (reject) zero_fill(dst, len);
    }
}

hipError_t launch_aead_seal(const AeadArgs &a, hipStream_t s)
{
    if (a.n == 0) return hipSuccess;
    hipLaunchKernelGGL(aead_wave_kernel<false>, dim3((a.n + 255u) / 256u), dim3(256), 0, s, a);
    return hipGetLastError();
}

hipError_t launch_aead_open(const AeadArgs &a, hipStream_t s)
{
    if (a.n == 0) return hipSuccess;
    hipLaunchKernelGGL(aead_wave_kernel<true>, dim3((a.n + 255u) / 256u), dim3(256), 0, s, a);
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

__global__ __launch_bounds__(256) void len_hist_kernel(const uint32_t *lens, uint32_t n,
                                                       uint32_t tag_bytes, uint32_t *hist)
{
    __shared__ uint32_t lh[LEN_BINS];
    for (uint32_t b = threadIdx.x; b < LEN_BINS; b += 256) lh[b] = 0;
    __syncthreads();
    const uint32_t stride = gridDim.x * 256u;
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += stride)
        atomicAdd(&lh[len_bin(lens[i], tag_bytes)], 1u);
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < LEN_BINS; b += 256)
        if (lh[b]) atomicAdd(&hist[b], lh[b]);
}

// Exclusive scan of hist into cursor (one block).
__global__ __launch_bounds__(256) void len_scan_kernel(const uint32_t *hist, uint32_t *cursor)
{
    __shared__ uint32_t part[256];
    constexpr uint32_t PER = (LEN_BINS + 255) / 256;
    uint32_t loc[PER];
    uint32_t sum = 0;
#pragma unroll
    for (uint32_t q = 0; q < PER; q++) {
        const uint32_t b = threadIdx.x * PER + q;
        loc[q] = b < LEN_BINS ? hist[b] : 0u;
        sum += loc[q];
    }
    part[threadIdx.x] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t run = 0;
        for (int t = 0; t < 256; t++) {
            const uint32_t v = part[t];
            part[t] = run;
            run += v;
        }
    }
    __syncthreads();
    uint32_t run = part[threadIdx.x];
#pragma unroll
    for (uint32_t q = 0; q < PER; q++) {
        const uint32_t b = threadIdx.x * PER + q;
        if (b < LEN_BINS) cursor[b] = run;
        run += loc[q];
    }
}

__global__ __launch_bounds__(256) void len_scatter_kernel(const uint32_t *lens, uint32_t n,
                                                          uint32_t tag_bytes, uint32_t *cursor,
                                                          uint32_t *order)
{
    __shared__ uint32_t cnt[LEN_BINS];
    __shared__ uint32_t base[LEN_BINS];
    for (uint32_t b = threadIdx.x; b < LEN_BINS; b += 256) cnt[b] = 0;
    __syncthreads();
    const uint32_t stride = gridDim.x * 256u;
    // every block walks its strided share twice: count, reserve, place
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += stride)
        atomicAdd(&cnt[len_bin(lens[i], tag_bytes)], 1u);
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < LEN_BINS; b += 256) {
        const uint32_t c = cnt[b];
        base[b] = c ? atomicAdd(&cursor[b], c) : 0u;
        cnt[b] = 0;
    }
    __syncthreads();
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += stride) {
        const uint32_t b = len_bin(lens[i], tag_bytes);
        order[base[b] + atomicAdd(&cnt[b], 1u)] = i;
    }
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

hipError_t launch_length_sort(const uint32_t *lens, uint32_t n, uint32_t tag_bytes,
                              uint32_t *order, uint32_t *hist, uint32_t *cursor,
                              hipStream_t s)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((LEN_BINS + 255u) / 256u), dim3(256), 0, s, hist,
                       LEN_BINS, 0u);
    uint32_t blocks = (n + 255u) / 256u;
    if (blocks > 1024u) blocks = 1024u;
    hipLaunchKernelGGL(len_hist_kernel, dim3(blocks), dim3(256), 0, s, lens, n, tag_bytes, hist);
    hipLaunchKernelGGL(len_scan_kernel, dim3(1), dim3(256), 0, s, hist, cursor);
    hipLaunchKernelGGL(len_scatter_kernel, dim3(blocks), dim3(256), 0, s, lens, n, tag_bytes,
                       cursor, order);
    return hipGetLastError();
}

} // namespace bnk
