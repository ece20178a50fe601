// libbnkprobe.so: measurement probes for the benchmark, kept apart from the
// product library.  Dependency-free VALU instruction streams (the measured
// per-instruction ceilings the AEAD roofline is read against; every lane runs
// PROBE_CHAINS independent chains so no instruction waits on the previous one)
// and a plain streaming copy (the measured HBM ceiling, and the known-size
// launch that memory-traffic counters are scaled against).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

#include "bnkprobe.h"
#include "../csrc/aead_lane.hpp"

namespace {

constexpr int PROBE_OPS = 24;
constexpr uint32_t PROBE_THREADS = 256;
constexpr uint32_t PROBE_CHAINS = 8;   // independent dependency chains per lane
constexpr uint32_t PROBE_UNROLL = 16;  // instructions per chain per iteration

template <int OP>
__global__ __launch_bounds__(256) void probe_kernel(uint32_t iters, uint32_t *out)
{
    const uint32_t tid = blockIdx.x * 256u + threadIdx.x;
    uint32_t a[PROBE_CHAINS];
    uint64_t q[PROBE_CHAINS];
    double d[PROBE_CHAINS];
#pragma unroll
    for (uint32_t c = 0; c < PROBE_CHAINS; c++) {
        a[c] = tid * 2654435761u + c;
        q[c] = a[c];
        d[c] = 1.0 + (double)c;
    }
    uint32_t b = tid | 1u, m = 0x9e3779b9u;
    double one = 1.0, zero = 0.0;
    asm volatile("" : "+v"(b), "+v"(m), "+v"(one), "+v"(zero));
    for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
        for (uint32_t u = 0; u < PROBE_UNROLL; u++) {
#pragma unroll
            for (uint32_t c = 0; c < PROBE_CHAINS; c++) {
                if (OP == 0) asm volatile("v_add_u32 %0, %0, %1" : "+v"(a[c]) : "v"(b));
                if (OP == 1) asm volatile("v_xor_b32 %0, %0, %1" : "+v"(a[c]) : "v"(b));
                if (OP == 2) asm volatile("v_alignbit_b32 %0, %0, %0, 7" : "+v"(a[c]));
                if (OP == 3)
                    asm volatile("v_mad_u64_u32 %0, vcc, %1, %2, %0"
                                 : "+v"(q[c]) : "v"(b), "v"(m) : "vcc");
                if (OP == 4) asm volatile("v_fma_f64 %0, %0, %1, %2" : "+v"(d[c]) : "v"(one), "v"(zero));
                if (OP == 5) asm volatile("v_mul_lo_u32 %0, %0, %1" : "+v"(a[c]) : "v"(b));
                if (OP == 6) asm volatile("v_add_f64 %0, %0, %1" : "+v"(d[c]) : "v"(zero));
                if (OP == 7) asm volatile("v_add_u32_e64 %0, %0, %1" : "+v"(a[c]) : "v"(b));
                if (OP == 8) asm volatile("v_xad_u32 %0, %0, %1, %2" : "+v"(a[c]) : "v"(b), "v"(m));
                if (OP == 9) asm volatile("v_add3_u32 %0, %0, %1, %2" : "+v"(a[c]) : "v"(b), "v"(m));
                if (OP == 10) asm volatile("v_perm_b32 %0, %0, %0, %1" : "+v"(a[c]) : "v"(m));
                if (OP == 11) asm volatile("v_lshl_or_b32 %0, %0, 7, %1" : "+v"(a[c]) : "v"(b));
                if (OP == 12)
                    asm volatile("v_xor_b32_sdwa %0, %0, %1 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE "
                                 "src0_sel:WORD_0 src1_sel:WORD_0" : "+v"(a[c]) : "v"(b));
                if (OP == 13)
                    asm volatile("v_mov_b32_dpp %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf"
                                 : "+v"(a[c]));
                if (OP == 14) asm volatile("v_lshlrev_b32 %0, 7, %0" : "+v"(a[c]));
                if (OP == 15) asm volatile("v_and_or_b32 %0, %0, %1, %2" : "+v"(a[c]) : "v"(b), "v"(m));
                if (OP == 16) asm volatile("v_bfe_u32 %0, %0, 3, 22" : "+v"(a[c]));
                if (OP == 17) asm volatile("v_mad_u32_u24 %0, %0, %1, %2" : "+v"(a[c]) : "v"(b), "v"(m));
                if (OP == 18) asm volatile("v_pk_add_u16 %0, %0, %1" : "+v"(a[c]) : "v"(b));
                if (OP == 19) asm volatile("v_alignbit_b32 %0, %0, %1, 7" : "+v"(a[c]) : "v"(b));
                if (OP == 20) asm volatile("v_mul_u32_u24 %0, %0, %1" : "+v"(a[c]) : "v"(b));
                if (OP == 21) asm volatile("v_mul_f64 %0, %0, %1" : "+v"(d[c]) : "v"(one));
                if (OP == 22) asm volatile("v_add_f32 %0, %0, %1" : "+v"(a[c]) : "v"(b));
                if (OP == 23) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(a[c]) : "v"(b), "v"(m));
            }
        }
    }
    uint32_t acc = 0;
#pragma unroll
    for (uint32_t c = 0; c < PROBE_CHAINS; c++)
        acc ^= a[c] ^ (uint32_t)q[c] ^ (uint32_t)(q[c] >> 32) ^ (uint32_t)d[c];
    out[tid] = acc;
}

// Plain streaming copy: the measured HBM ceiling, and the known-size kernel
// the FETCH_SIZE / WRITE_SIZE counters are scaled against.
__global__ __launch_bounds__(256) void copy_kernel(const uint4 *src, uint4 *dst, size_t n16)
{
    const size_t stride = (size_t)gridDim.x * 256u;
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

static hipError_t launch_copy(const void *src, void *dst, size_t bytes, uint32_t blocks, hipStream_t s)
{
    hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, s, (const uint4 *)src, (uint4 *)dst,
                       bytes / 16);
    return hipGetLastError();
}

// The AEAD kernel's way of moving packets, with nothing to compute: a lane per
// packet for the bookkeeping, eight adjacent lanes per aligned 128-byte line, so
// that one load instruction of a wave fetches one line from each of eight
// packets (`stride` bytes apart) and a wave walks its 64 packets line by line,
// each line held in registers for `depth` steps before it is stored to the same
// place of the other arena.  `spin` dependent VALU instructions per step stand
// for the arithmetic (0: none).  Dynamic LDS sets how many waves a SIMD holds.
template <int DEPTH>
__global__ __launch_bounds__(256) void line_copy_kernel(const uint8_t *src, uint8_t *dst, uint32_t packets,
                                                        uint32_t stride, uint32_t len, uint32_t spin, uint32_t *sink)
{
    extern __shared__ uint32_t occupancy_pad[];
    const uint32_t lane = threadIdx.x & 63u, sub = lane & 7u, g = lane >> 3;
    const uint32_t wave_first = (blockIdx.x * 256u + (threadIdx.x & ~63u));
    if (wave_first >= packets) return;
    // the (packet, cell-of-line) positions this lane moves per line: packet 8 q + g of the wave
    uint64_t at[8];
    uint32_t lines = 0;
#pragma unroll
    for (int q = 0; q < 8; q++) {
        const uint32_t p = min(wave_first + 8u * q + g, packets - 1u);
        const uint64_t start = (uint64_t)p * stride;
        at[q] = (start & ~127ull) + 16u * sub;
        const uint32_t n = (uint32_t)((start & 127u) + len + 127u) >> 7;
        lines = n > lines ? n : lines;
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)lines, off, 64);
        lines = o > lines ? o : lines;
    }
    lines = __builtin_amdgcn_readfirstlane(lines);
    uint4 buf[DEPTH][8];
    uint32_t acc = lane;
    for (int d = 0; d < DEPTH; d++) {
#pragma unroll
        for (int q = 0; q < 8; q++) buf[d][q] = make_uint4(0, 0, 0, 0);
    }
    // step m: line m comes in, line m - DEPTH goes out
    for (uint32_t m = 0; m < lines + DEPTH; m++) {
        uint4 out[8];
#pragma unroll
        for (int q = 0; q < 8; q++) out[q] = buf[DEPTH - 1][q];
#pragma unroll
        for (int d = DEPTH - 1; d > 0; d--) {
#pragma unroll
            for (int q = 0; q < 8; q++) buf[d][q] = buf[d - 1][q];
        }
        if (m < lines) {
#pragma unroll
            for (int q = 0; q < 8; q++)
                buf[0][q] = *reinterpret_cast<const uint4 *>(src + at[q] + 128ull * m);
        }
        if (m >= (uint32_t)DEPTH) {
#pragma unroll
            for (int q = 0; q < 8; q++)
                *reinterpret_cast<uint4 *>(dst + at[q] + 128ull * (m - DEPTH)) = out[q];
        }
        for (uint32_t k = 0; k < spin; k++) asm volatile("v_add_u32 %0, %0, %0" : "+v"(acc));
    }
    if (acc == 0x12345u) sink[0] = acc; // keeps the spin alive
}

// ---------------------------------------------------------------------------
// How a SIMD shares its issue between two waves.
//
// pair_kernel: one workgroup of eight waves per CU, so that waves w and w + 4
// share a SIMD; the first four run one instruction kind, the second four
// another, and each group reports how long its own stream took.
// mix_kernel: the ChaCha20 quarter-round stream (four adds, four xors, four
// rotates, each group depending on the one before) in many short-lived
// workgroups, a chosen number resident per CU, with or without raised wave
// priority around the rotates.
// ---------------------------------------------------------------------------
#define P_ADD(a, b) asm volatile("v_add_u32 %0, %0, %1" : "+v"(a) : "v"(b))
#define P_XOR(a, b) asm volatile("v_xor_b32 %0, %0, %1" : "+v"(a) : "v"(b))
#define P_ROT(a, n) asm volatile("v_alignbit_b32 %0, %0, %0, " #n : "+v"(a))

constexpr int PAIR_KINDS = 8;
template <int K>
__device__ __forceinline__ void pair_stream(uint32_t iters, uint32_t (&x)[8], uint32_t b, uint32_t m, uint64_t (&q)[8])
{
    for (uint32_t it = 0; it < iters; it++) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
#pragma unroll
            for (int c = 0; c < 8; c++) {
                if (K == 0) P_ADD(x[c], b);
                if (K == 1) P_XOR(x[c], b);
                if (K == 2) P_ROT(x[c], 7);
                if (K == 3) asm volatile("v_mad_u64_u32 %0, vcc, %1, %2, %0" : "+v"(q[c]) : "v"(b), "v"(m) : "vcc");
                if (K == 4) asm volatile("v_addc_co_u32 %0, vcc, %0, %1, vcc" : "+v"(x[c]) : "v"(b) : "vcc");
                if (K == 5) asm volatile("v_lshlrev_b32 %0, 7, %0" : "+v"(x[c]));
                if (K == 6) asm volatile("v_lshrrev_b32 %0, 7, %0" : "+v"(x[c]));
                if (K == 7) asm volatile("v_mov_b32 %0, %1" : "+v"(x[c]) : "v"(b));
            }
        }
    }
}

template <int KA, int KB>
__global__ __launch_bounds__(512) void pair_kernel(uint32_t iters, uint32_t *out, uint64_t *ticks)
{
    extern __shared__ uint32_t pair_lds[];
    const uint32_t tid = blockIdx.x * 512u + threadIdx.x;
    uint32_t x[8];
    uint64_t q[8];
#pragma unroll
    for (int i = 0; i < 8; i++) { x[i] = tid * 2654435761u + i; q[i] = x[i]; }
    uint32_t b = tid | 1u, m = 0x9e3779b9u;
    asm volatile("" : "+v"(b), "+v"(m));
    const bool second = threadIdx.x >= 256;
    __syncthreads();
    const uint64_t t0 = wall_clock64();
    if (!second) pair_stream<KA>(iters, x, b, m, q);
    else if (KB >= 0) pair_stream<(KB >= 0 ? KB : 0)>(iters, x, b, m, q);
    const uint64_t t1 = wall_clock64();
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) acc ^= x[i] ^ (uint32_t)q[i] ^ (uint32_t)(q[i] >> 32);
    out[tid] = acc + pair_lds[threadIdx.x & 1u];
    if (blockIdx.x == 0 && (threadIdx.x == 0 || threadIdx.x == 256)) ticks[second ? 1 : 0] = t1 - t0;
}

template <int KA, int KB>
static hipError_t pair_dispatch(int ka, int kb, uint32_t iters, uint32_t blocks, uint32_t *out, uint64_t *ticks, hipStream_t s)
{
    if (ka == KA && kb == KB) {
        // more than half a CU's LDS: one workgroup per CU
        const uint32_t lds_bytes = 96u * 1024u;
        hipError_t e = hipFuncSetAttribute((const void *)pair_kernel<KA, KB>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL((pair_kernel<KA, KB>), dim3(blocks), dim3(512), lds_bytes, s, iters, out, ticks);
        return hipGetLastError();
    }
    if constexpr (KB + 1 < PAIR_KINDS) return pair_dispatch<KA, KB + 1>(ka, kb, iters, blocks, out, ticks, s);
    else if constexpr (KA + 1 < PAIR_KINDS) return pair_dispatch<KA + 1, -1>(ka, kb, iters, blocks, out, ticks, s);
    return hipErrorInvalidValue;
}

template <int PRIO>
__global__ __launch_bounds__(256) void mix_kernel(uint32_t iters, uint32_t *out)
{
    extern __shared__ uint32_t mix_lds[];
    const uint32_t tid = blockIdx.x * 256u + threadIdx.x;
    uint32_t x[16];
#pragma unroll
    for (int i = 0; i < 16; i++) x[i] = tid * 2654435761u + i;
#define P_STEP(a0, a1, a2, a3, b0, b1, b2, b3, d0, d1, d2, d3, n)                                \
    P_ADD(x[a0], x[b0]); P_ADD(x[a1], x[b1]); P_ADD(x[a2], x[b2]); P_ADD(x[a3], x[b3]);         \
    P_XOR(x[d0], x[a0]); P_XOR(x[d1], x[a1]); P_XOR(x[d2], x[a2]); P_XOR(x[d3], x[a3]);         \
    if (PRIO) asm volatile("s_setprio 1");                                                      \
    P_ROT(x[d0], n); P_ROT(x[d1], n); P_ROT(x[d2], n); P_ROT(x[d3], n);                         \
    if (PRIO) asm volatile("s_setprio 0");
    for (uint32_t it = 0; it < iters; it++) {
        P_STEP(0, 1, 2, 3, 4, 5, 6, 7, 12, 13, 14, 15, 16)
        P_STEP(8, 9, 10, 11, 12, 13, 14, 15, 4, 5, 6, 7, 20)
        P_STEP(0, 1, 2, 3, 4, 5, 6, 7, 12, 13, 14, 15, 24)
        P_STEP(8, 9, 10, 11, 12, 13, 14, 15, 4, 5, 6, 7, 25)
        P_STEP(0, 1, 2, 3, 5, 6, 7, 4, 15, 12, 13, 14, 16)
        P_STEP(10, 11, 8, 9, 15, 12, 13, 14, 5, 6, 7, 4, 20)
        P_STEP(0, 1, 2, 3, 5, 6, 7, 4, 15, 12, 13, 14, 24)
        P_STEP(10, 11, 8, 9, 15, 12, 13, 14, 5, 6, 7, 4, 25)
    }
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) acc ^= x[i];
    out[tid & 0xFFFFFu] = acc + mix_lds[threadIdx.x & 1u];
}
constexpr uint32_t MIX_INSTR_PER_ITER = 96;

// The AEAD kernel's arithmetic with nothing else: a packet per lane, per 64
// bytes one ChaCha20 block, the xor with the data and four Poly1305 blocks,
// the product's own lane code (aead_lane.hpp), the data a constant in
// registers.  PAIRED: two keystream blocks side by side with the part of the
// first round that a packet's blocks share computed once, as the kernel's
// 128-byte steps do.  What it reaches with w waves per SIMD is what the kernel
// could reach if moving the packets cost nothing.
template <bool PAIRED>
__global__ __launch_bounds__(256) void aead_compute_kernel(uint32_t data_blocks, uint32_t *out)
{
    extern __shared__ uint32_t compute_lds[];
    const uint32_t tid = blockIdx.x * 256u + threadIdx.x;
    uint32_t k[8];
#pragma unroll
    for (int i = 0; i < 8; i++) k[i] = tid * 2654435761u + (uint32_t)i;
    const uint32_t n1 = tid, n2 = 7;
    const uint32_t d0 = tid, d1 = tid ^ 0x55u, d2 = tid + 3u, d3 = ~tid;
    uint32_t x[16];
    bnk::chacha_block(k, 0, n1, n2, x);
    bnk::Poly32 mac;
    mac.init(x);
    if (!PAIRED) {
        for (uint32_t b = 0; b < data_blocks; b++) {
            bnk::chacha_block(k, b + 1, n1, n2, x);
#pragma unroll
            for (int j = 0; j < 4; j++) mac.block(x[4 * j] ^ d0, x[4 * j + 1] ^ d1, x[4 * j + 2] ^ d2, x[4 * j + 3] ^ d3);
        }
    } else {
        uint32_t y[16];
        bnk::ChachaShared shared;
        bnk::chacha_shared(k, n1, n2, shared);
        for (uint32_t b = 0; b < data_blocks; b += 2) {
            bnk::chacha_block2_shared(k, shared, b + 1, n1, n2, x, y);
#pragma unroll
            for (int j = 0; j < 4; j++) mac.block(x[4 * j] ^ d0, x[4 * j + 1] ^ d1, x[4 * j + 2] ^ d2, x[4 * j + 3] ^ d3);
#pragma unroll
            for (int j = 0; j < 4; j++) mac.block(y[4 * j] ^ d0, y[4 * j + 1] ^ d1, y[4 * j + 2] ^ d2, y[4 * j + 3] ^ d3);
        }
    }
    uint32_t tag[4];
    mac.finish(tag);
    out[tid & 0xFFFFFu] = (tag[0] ^ tag[1] ^ tag[2] ^ tag[3]) + compute_lds[threadIdx.x & 1u];
}

template <int OP>
static hipError_t probe_dispatch(int op, uint32_t iters, uint32_t blocks, uint32_t *out, hipStream_t s)
{
    if (op == OP) {
        hipLaunchKernelGGL(probe_kernel<OP>, dim3(blocks), dim3(256), 0, s, iters, out);
        return hipGetLastError();
    }
    if constexpr (OP + 1 < PROBE_OPS) return probe_dispatch<OP + 1>(op, iters, blocks, out, s);
    return hipErrorInvalidValue;
}

static hipError_t launch_probe(int op, uint32_t iters, uint32_t blocks, uint32_t *out, hipStream_t s)
{
    return probe_dispatch<0>(op, iters, blocks, out, s);
}

} // namespace

#define PROBE_CHK(expr)                       \
    do {                                      \
        if ((expr) != hipSuccess) goto fail;  \
    } while (0)

extern "C" int bnkp_valu(int device, int op, uint32_t iters, double *ops_per_sec)
{
    if (!ops_per_sec || iters == 0 || op < 0 || op >= PROBE_OPS) return -1;
    hipDeviceProp_t prop;
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    uint32_t *out = nullptr;
    float ms = 0;
    int rc = -3;
    uint32_t blocks = 0;
    PROBE_CHK(hipSetDevice(device));
    PROBE_CHK(hipGetDeviceProperties(&prop, device));
    // 8 workgroups of 4 waves per CU: every SIMD holds 8 waves
    blocks = (uint32_t)prop.multiProcessorCount * 8u;
    PROBE_CHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    PROBE_CHK(hipEventCreate(&e0));
    PROBE_CHK(hipEventCreate(&e1));
    PROBE_CHK(hipMalloc((void **)&out, (size_t)blocks * PROBE_THREADS * 4));
    PROBE_CHK(launch_probe(op, 4, blocks, out, s)); // warm-up
    PROBE_CHK(hipEventRecord(e0, s));
    PROBE_CHK(launch_probe(op, iters, blocks, out, s));
    PROBE_CHK(hipEventRecord(e1, s));
    PROBE_CHK(hipEventSynchronize(e1));
    PROBE_CHK(hipEventElapsedTime(&ms, e0, e1));
    *ops_per_sec = (double)blocks * PROBE_THREADS * (double)iters * PROBE_CHAINS * PROBE_UNROLL / ((double)ms * 1e-3);
    rc = 0;
fail:
    if (out) (void)hipFree(out);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (s) (void)hipStreamDestroy(s);
    return rc;
}

extern "C" int bnkp_copy(int device, size_t bytes, uint32_t iters, double *bytes_per_sec)
{
    if (!bytes_per_sec || iters == 0 || bytes < 4096 || (bytes & 15)) return -1;
    hipDeviceProp_t prop;
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    void *src = nullptr, *dst = nullptr;
    float ms = 0;
    int rc = -3;
    uint32_t blocks = 0;
    PROBE_CHK(hipSetDevice(device));
    PROBE_CHK(hipGetDeviceProperties(&prop, device));
    // four pieces per thread: many short workgroups stream faster than few long ones
    // (5.4 TB/s against 4.6 with 16 workgroups per CU, 1 GiB)
    blocks = (uint32_t)std::min<size_t>(std::max<size_t>(bytes / 16 / 256 / 4, (size_t)prop.multiProcessorCount), 1u << 20);
    PROBE_CHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    PROBE_CHK(hipEventCreate(&e0));
    PROBE_CHK(hipEventCreate(&e1));
    PROBE_CHK(hipMalloc(&src, bytes));
    PROBE_CHK(hipMalloc(&dst, bytes));
    PROBE_CHK(hipMemsetAsync(src, 0x5a, bytes, s));
    PROBE_CHK(launch_copy(src, dst, bytes, blocks, s)); // warm-up
    PROBE_CHK(hipEventRecord(e0, s));
    for (uint32_t i = 0; i < iters; i++) PROBE_CHK(launch_copy(src, dst, bytes, blocks, s));
    PROBE_CHK(hipEventRecord(e1, s));
    PROBE_CHK(hipEventSynchronize(e1));
    PROBE_CHK(hipEventElapsedTime(&ms, e0, e1));
    // bytes read plus bytes written
    *bytes_per_sec = 2.0 * (double)bytes * iters / ((double)ms * 1e-3);
    rc = 0;
fail:
    if (src) (void)hipFree(src);
    if (dst) (void)hipFree(dst);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (s) (void)hipStreamDestroy(s);
    return rc;
}

extern "C" int bnkp_line_copy(int device, uint32_t packets, uint32_t stride, uint32_t len, int waves_per_simd,
                              int depth, uint32_t spin, uint32_t iters, double *ms_per_launch)
{
    if (!ms_per_launch || iters == 0 || packets == 0 || (stride & 15u) || len == 0 || len > stride ||
        waves_per_simd < 1 || waves_per_simd > 4 || depth < 1 || depth > 2)
        return -1;
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    uint8_t *src = nullptr, *dst = nullptr;
    uint32_t *sink = nullptr;
    float ms = 0;
    int rc = -3;
    const size_t bytes = (size_t)packets * stride + 256;
    // a workgroup is four waves, one per SIMD: 160 KB of LDS / waves_per_simd workgroups
    const size_t lds = (size_t)(160u * 1024u) / (size_t)waves_per_simd - 1024u;
    const dim3 grid((packets + 255u) / 256u);
    auto launch = [&]() -> hipError_t {
        if (depth == 1)
            hipLaunchKernelGGL(line_copy_kernel<1>, grid, dim3(256), lds, s, src, dst, packets, stride, len, spin, sink);
        else
            hipLaunchKernelGGL(line_copy_kernel<2>, grid, dim3(256), lds, s, src, dst, packets, stride, len, spin, sink);
        return hipGetLastError();
    };
    PROBE_CHK(hipSetDevice(device));
    PROBE_CHK(hipFuncSetAttribute(reinterpret_cast<const void *>(line_copy_kernel<1>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    PROBE_CHK(hipFuncSetAttribute(reinterpret_cast<const void *>(line_copy_kernel<2>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    PROBE_CHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    PROBE_CHK(hipEventCreate(&e0));
    PROBE_CHK(hipEventCreate(&e1));
    PROBE_CHK(hipMalloc((void **)&src, bytes));
    PROBE_CHK(hipMalloc((void **)&dst, bytes));
    PROBE_CHK(hipMalloc((void **)&sink, 64));
    PROBE_CHK(hipMemsetAsync(src, 0x5a, bytes, s));
    for (int w = 0; w < 3; w++) PROBE_CHK(launch()); // warm-up
    PROBE_CHK(hipEventRecord(e0, s));
    for (uint32_t i = 0; i < iters; i++) PROBE_CHK(launch());
    PROBE_CHK(hipEventRecord(e1, s));
    PROBE_CHK(hipEventSynchronize(e1));
    PROBE_CHK(hipEventElapsedTime(&ms, e0, e1));
    *ms_per_launch = (double)ms / iters;
    rc = 0;
fail:
    if (src) (void)hipFree(src);
    if (dst) (void)hipFree(dst);
    if (sink) (void)hipFree(sink);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (s) (void)hipStreamDestroy(s);
    return rc;
}

extern "C" int bnkp_pair(int device, int kind_a, int kind_b, uint32_t iters, double *ns_a, double *ns_b)
{
    if (!ns_a || !ns_b || iters == 0 || kind_a < 0 || kind_a >= PAIR_KINDS || kind_b < -1 || kind_b >= PAIR_KINDS) return -1;
    hipDeviceProp_t prop;
    hipStream_t s = nullptr;
    uint32_t *out = nullptr;
    uint64_t *ticks = nullptr;
    uint64_t h[2] = {0, 0};
    int rc = -3;
    uint32_t blocks = 0;
    PROBE_CHK(hipSetDevice(device));
    PROBE_CHK(hipGetDeviceProperties(&prop, device));
    blocks = (uint32_t)prop.multiProcessorCount;
    PROBE_CHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    PROBE_CHK(hipMalloc((void **)&out, (size_t)blocks * 512 * 4));
    PROBE_CHK(hipMalloc((void **)&ticks, 16));
    PROBE_CHK(hipMemsetAsync(ticks, 0, 16, s));
    PROBE_CHK((pair_dispatch<0, -1>(kind_a, kind_b, 64, blocks, out, ticks, s))); // warm-up
    PROBE_CHK((pair_dispatch<0, -1>(kind_a, kind_b, iters, blocks, out, ticks, s)));
    PROBE_CHK(hipStreamSynchronize(s));
    PROBE_CHK(hipMemcpy(h, ticks, 16, hipMemcpyDeviceToHost));
    // the realtime counter runs at 100 MHz; 64 instructions per pass of the stream
    *ns_a = (double)h[0] * 10.0 / ((double)iters * 64.0);
    *ns_b = kind_b >= 0 ? (double)h[1] * 10.0 / ((double)iters * 64.0) : 0.0;
    rc = 0;
fail:
    if (out) (void)hipFree(out);
    if (ticks) (void)hipFree(ticks);
    if (s) (void)hipStreamDestroy(s);
    return rc;
}

extern "C" int bnkp_mix(int device, int raised_priority, int waves_per_simd, uint32_t iters, double *ops_per_sec)
{
    if (!ops_per_sec || iters == 0 || waves_per_simd < 1 || waves_per_simd > 8) return -1;
    hipDeviceProp_t prop;
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    uint32_t *out = nullptr;
    float ms = 0;
    int rc = -3;
    uint32_t blocks = 0, lds_bytes = 0;
    const void *fn = raised_priority ? (const void *)mix_kernel<1> : (const void *)mix_kernel<0>;
    PROBE_CHK(hipSetDevice(device));
    PROBE_CHK(hipGetDeviceProperties(&prop, device));
    // workgroups of four waves, one per SIMD; their LDS allocation limits how many a CU
    // holds at a time; 32 rounds of them, so that waves come and go as in a long launch
    lds_bytes = ((uint32_t)prop.maxSharedMemoryPerMultiProcessor / (uint32_t)waves_per_simd) & ~1023u;
    if (lds_bytes > 160u * 1024u) lds_bytes = 160u * 1024u;
    blocks = (uint32_t)prop.multiProcessorCount * (uint32_t)waves_per_simd * 32u;
    PROBE_CHK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    PROBE_CHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    PROBE_CHK(hipEventCreate(&e0));
    PROBE_CHK(hipEventCreate(&e1));
    PROBE_CHK(hipMalloc((void **)&out, (size_t)(1u << 20) * 4));
    for (int pass = 0; pass < 2; pass++) { // the first pass warms up
        PROBE_CHK(hipEventRecord(e0, s));
        if (raised_priority) hipLaunchKernelGGL(mix_kernel<1>, dim3(blocks), dim3(256), lds_bytes, s, iters, out);
        else hipLaunchKernelGGL(mix_kernel<0>, dim3(blocks), dim3(256), lds_bytes, s, iters, out);
        PROBE_CHK(hipGetLastError());
        PROBE_CHK(hipEventRecord(e1, s));
        PROBE_CHK(hipEventSynchronize(e1));
    }
    PROBE_CHK(hipEventElapsedTime(&ms, e0, e1));
    *ops_per_sec = (double)blocks * 256.0 * (double)iters * MIX_INSTR_PER_ITER / ((double)ms * 1e-3);
    rc = 0;
fail:
    if (out) (void)hipFree(out);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (s) (void)hipStreamDestroy(s);
    return rc;
}

extern "C" int bnkp_aead_compute(int device, int paired, int waves_per_simd, uint32_t data_blocks, double *blocks_per_sec)
{
    if (!blocks_per_sec || data_blocks == 0 || (data_blocks & 1u) || waves_per_simd < 1 || waves_per_simd > 4) return -1;
    hipDeviceProp_t prop;
    hipStream_t s = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    uint32_t *out = nullptr;
    float ms = 0;
    int rc = -3;
    uint32_t blocks = 0, lds_bytes = 0;
    const void *fn = paired ? (const void *)aead_compute_kernel<true> : (const void *)aead_compute_kernel<false>;
    PROBE_CHK(hipSetDevice(device));
    PROBE_CHK(hipGetDeviceProperties(&prop, device));
    // workgroups of four waves, one per SIMD; their LDS allocation limits how many a CU
    // holds at a time (the kernels need at most 83 registers: four waves fit a SIMD)
    lds_bytes = (((uint32_t)prop.maxSharedMemoryPerMultiProcessor / (uint32_t)waves_per_simd) & ~1023u) - 1024u;
    blocks = (uint32_t)prop.multiProcessorCount * (uint32_t)waves_per_simd * 8u;
    PROBE_CHK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
    PROBE_CHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    PROBE_CHK(hipEventCreate(&e0));
    PROBE_CHK(hipEventCreate(&e1));
    PROBE_CHK(hipMalloc((void **)&out, (size_t)(1u << 20) * 4));
    for (int pass = 0; pass < 3; pass++) { // the first passes warm up
        PROBE_CHK(hipEventRecord(e0, s));
        if (paired) hipLaunchKernelGGL(aead_compute_kernel<true>, dim3(blocks), dim3(256), lds_bytes, s, data_blocks, out);
        else hipLaunchKernelGGL(aead_compute_kernel<false>, dim3(blocks), dim3(256), lds_bytes, s, data_blocks, out);
        PROBE_CHK(hipGetLastError());
        PROBE_CHK(hipEventRecord(e1, s));
        PROBE_CHK(hipEventSynchronize(e1));
    }
    PROBE_CHK(hipEventElapsedTime(&ms, e0, e1));
    // the key block counts too
    *blocks_per_sec = (double)blocks * 256.0 * (double)(data_blocks + 1u) / ((double)ms * 1e-3);
    rc = 0;
fail:
    if (out) (void)hipFree(out);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (s) (void)hipStreamDestroy(s);
    return rc;
}
