// libbnkprobe.so: measurement probes for the benchmark, kept apart from the
// product library.  Dependency-free VALU instruction streams (the measured
// per-instruction ceilings the AEAD roofline is read against; every lane runs
// PROBE_CHAINS independent chains so no instruction waits on the previous one)
// and a plain streaming copy (the measured HBM ceiling, and the known-size
// launch that memory-traffic counters are scaled against).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bnkprobe.h"

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
    blocks = (uint32_t)prop.multiProcessorCount * 16u;
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
