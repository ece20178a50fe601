/*
 * bnkprobe.h -- C ABI of libbnkprobe.so: measurement probes used by the
 * benchmark only.  Not part of the product library (libbnkhip.so) and with no
 * counterpart in the reference.  Return 0 on success, -1 for a bad argument,
 * -3 for a HIP failure.
 */
#ifndef BNKPROBE_H
#define BNKPROBE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Runs a dependency-free VALU instruction stream on `device` and reports
 * lane-ops per second.  op: 0 v_add_u32, 1 v_xor_b32, 2 v_alignbit_b32,
 * 3 v_mad_u64_u32, 4 v_fma_f64, 5 v_mul_lo_u32, 6 v_add_f64, 7.. further
 * instruction kinds (see probe_kernels.hip). */
int bnkp_valu(int device, int op, uint32_t iters, double *ops_per_sec);

/* Streams `bytes` (a multiple of 16) from one device buffer to another `iters`
 * times (copy_kernel) and reports bytes read plus bytes written per second. */
int bnkp_copy(int device, size_t bytes, uint32_t iters, double *bytes_per_sec);

#ifdef __cplusplus
}
#endif
#endif
