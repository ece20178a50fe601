// Batched WireGuard transport seal/open for gfx950: one lane per packet.
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

template <bool AL>
BNK_DEV uint4 ld16(const uint8_t *p)
{
    if (AL) return *reinterpret_cast<const uint4 *>(p);
    uint4 v;
    __builtin_memcpy(&v, p, 16);
    return v;
}

template <bool AL>
BNK_DEV void st16(uint8_t *p, uint4 v)
{
    if (AL) {
        *reinterpret_cast<uint4 *>(p) = v;
    } else {
        __builtin_memcpy(p, &v, 16);
    }
}

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

template <bool AL>
BNK_DEV void zero_fill(uint8_t *dst, uint32_t len)
{
    uint32_t pos = 0;
    for (; pos + 16 <= len; pos += 16) st16<AL>(dst + pos, make_uint4(0, 0, 0, 0));
    for (; pos < len; pos++) dst[pos] = 0;
}

// len is the plaintext length.  Seal reads len bytes at src and writes
// len + 16 at dst; open reads len + 16 at src and writes len at dst.
template <bool OPEN, bool AL>
BNK_DEV void aead_packet(const uint32_t (&k)[8], uint64_t counter,
                         const uint8_t *src, uint8_t *dst, uint32_t len,
                         uint8_t *verdict)
{
    const uint32_t n1 = (uint32_t)counter, n2 = (uint32_t)(counter >> 32);
    uint32_t x[16];
    chacha_block(k, 0, n1, n2, x);
    Poly26 mac;
    mac.init(x);

    const uint32_t nfull = len >> 6;
    for (uint32_t b = 0; b < nfull; b++) {
        chacha_block(k, b + 1, n1, n2, x);
        const uint8_t *s = src + 64u * b;
        uint8_t *d = dst + 64u * b;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint4 v = ld16<AL>(s + 16 * j);
            const uint4 o = make_uint4(v.x ^ x[4 * j], v.y ^ x[4 * j + 1],
                                       v.z ^ x[4 * j + 2], v.w ^ x[4 * j + 3]);
            if (OPEN) mac.block(v.x, v.y, v.z, v.w);
            else mac.block(o.x, o.y, o.z, o.w);
            st16<AL>(d + 16 * j, o);
        }
    }
    const uint32_t rem = len & 63u;
    if (rem) {
        chacha_block(k, nfull + 1, n1, n2, x);
        const uint8_t *s = src + 64u * nfull;
        uint8_t *d = dst + 64u * nfull;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (rem >= 16u * (j + 1)) {
                const uint4 v = ld16<AL>(s + 16 * j);
                const uint4 o = make_uint4(v.x ^ x[4 * j], v.y ^ x[4 * j + 1],
                                           v.z ^ x[4 * j + 2], v.w ^ x[4 * j + 3]);
                if (OPEN) mac.block(v.x, v.y, v.z, v.w);
                else mac.block(o.x, o.y, o.z, o.w);
                st16<AL>(d + 16 * j, o);
            } else if (rem > 16u * j) {
                const uint32_t m = rem - 16u * j;
                const uint4 v = ld_partial(s + 16 * j, m);
                const uint4 o = keep_bytes(
                    make_uint4(v.x ^ x[4 * j], v.y ^ x[4 * j + 1],
                               v.z ^ x[4 * j + 2], v.w ^ x[4 * j + 3]), m);
                // the MAC sees the ciphertext zero-padded to 16 bytes
                if (OPEN) mac.block(v.x, v.y, v.z, v.w);
                else mac.block(o.x, o.y, o.z, o.w);
                st_partial(d + 16 * j, o, m);
            }
        }
    }
    // LE64(len(aad) = 0) || LE64(len(ciphertext))
    mac.block(0, 0, len, 0);
    uint32_t tag[4];
    mac.finish(tag);

    if (!OPEN) {
        st16<false>(dst + len, make_uint4(tag[0], tag[1], tag[2], tag[3]));
    } else {
        const uint4 t = ld16<false>(src + len);
        // all 16 bytes are compared, no early exit
        const uint32_t diff = (t.x ^ tag[0]) | (t.y ^ tag[1]) | (t.z ^ tag[2]) |
                              (t.w ^ tag[3]);
        const bool ok = diff == 0;
        *verdict = ok ? 1 : 0;
        if (!ok) zero_fill<AL>(dst, len);
    }
}

template <bool OPEN>
__global__ __launch_bounds__(256) void aead_lane_kernel(AeadArgs a)
{
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    if (t >= a.n) return;
    const uint32_t i = a.order ? a.order[t] : t;
    uint32_t len = a.lens ? a.lens[i] : a.len;
    const uint64_t ioff = a.in_off ? a.in_off[i] : (uint64_t)i * a.in_stride;
    const uint64_t ooff = a.out_off ? a.out_off[i] : (uint64_t)i * a.out_stride;
    const uint32_t pr = a.peer ? a.peer[i] : 0u;
    if (pr >= a.n_peers) {
        atomicOr(a.status, STATUS_PEER_RANGE);
        if (OPEN) a.verdict[i] = 0;
        return;
    }
    if (OPEN) {
        if (len < 16u) {
            a.verdict[i] = 0;
            return;
        }
        len -= 16u;
    }
    const uint4 *kp = reinterpret_cast<const uint4 *>(a.keys + 8u * pr);
    const uint4 k0 = kp[0], k1 = kp[1];
    const uint32_t k[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
    const uint64_t ctr = a.counters ? a.counters[i] : a.counter0 + i;
    const uint8_t *src = a.in + ioff;
    uint8_t *dst = a.out + ooff;
    uint8_t *vd = OPEN ? a.verdict + i : nullptr;
    const bool al = (((uintptr_t)src | (uintptr_t)dst) & 15u) == 0;
    if (al) aead_packet<OPEN, true>(k, ctr, src, dst, len, vd);
    else aead_packet<OPEN, false>(k, ctr, src, dst, len, vd);
}

hipError_t launch_aead_seal(const AeadArgs &a, hipStream_t s)
{
    if (a.n == 0) return hipSuccess;
    hipLaunchKernelGGL(aead_lane_kernel<false>, dim3((a.n + 255u) / 256u), dim3(256), 0, s, a);
    return hipGetLastError();
}

hipError_t launch_aead_open(const AeadArgs &a, hipStream_t s)
{
    if (a.n == 0) return hipSuccess;
    hipLaunchKernelGGL(aead_lane_kernel<true>, dim3((a.n + 255u) / 256u), dim3(256), 0, s, a);
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
