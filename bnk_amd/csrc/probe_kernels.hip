// Dependency-free VALU instruction streams: the measured per-op ceilings the
// AEAD roofline fractions are quoted against.  Every lane runs PROBE_CHAINS
// independent chains so no instruction waits on the previous one.
#include "kernels.hpp"

namespace bnk {

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

hipError_t launch_copy(const void *src, void *dst, size_t bytes, uint32_t blocks, hipStream_t s)
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

hipError_t launch_probe(int op, uint32_t iters, uint32_t blocks, uint32_t *out, hipStream_t s)
{
    return probe_dispatch<0>(op, iters, blocks, out, s);
}

} // namespace bnk
