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
            }
        }
    }
    uint32_t acc = 0;
#pragma unroll
    for (uint32_t c = 0; c < PROBE_CHAINS; c++)
        acc ^= a[c] ^ (uint32_t)q[c] ^ (uint32_t)(q[c] >> 32) ^ (uint32_t)d[c];
    out[tid] = acc;
}

hipError_t launch_probe(int op, uint32_t iters, uint32_t blocks, uint32_t *out, hipStream_t s)
{
    switch (op) {
    case 0: hipLaunchKernelGGL(probe_kernel<0>, dim3(blocks), dim3(256), 0, s, iters, out); break;
    case 1: hipLaunchKernelGGL(probe_kernel<1>, dim3(blocks), dim3(256), 0, s, iters, out); break;
    case 2: hipLaunchKernelGGL(probe_kernel<2>, dim3(blocks), dim3(256), 0, s, iters, out); break;
    case 3: hipLaunchKernelGGL(probe_kernel<3>, dim3(blocks), dim3(256), 0, s, iters, out); break;
    case 4: hipLaunchKernelGGL(probe_kernel<4>, dim3(blocks), dim3(256), 0, s, iters, out); break;
    case 5: hipLaunchKernelGGL(probe_kernel<5>, dim3(blocks), dim3(256), 0, s, iters, out); break;
    case 6: hipLaunchKernelGGL(probe_kernel<6>, dim3(blocks), dim3(256), 0, s, iters, out); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

} // namespace bnk
