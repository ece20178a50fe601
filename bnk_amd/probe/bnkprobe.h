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

/* The AEAD kernel's way of moving packets with nothing (or a stand-in) to
 * compute: `packets` slots `stride` bytes apart (a multiple of 16), `len` bytes
 * each, copied from one device arena to the same place of another, a lane per
 * packet, eight adjacent lanes per aligned 128-byte line, a wave walking its 64
 * packets line by line with each line held in registers for `depth` (1 or 2)
 * steps; `spin` dependent VALU instructions per line stand for the arithmetic;
 * `waves_per_simd` (1..4) waves resident per SIMD.  Reports milliseconds per
 * launch. */
int bnkp_line_copy(int device, uint32_t packets, uint32_t stride, uint32_t len, int waves_per_simd,
                   int depth, uint32_t spin, uint32_t iters, double *ms_per_launch);

/* Two instruction streams sharing each SIMD: one workgroup of eight waves per
 * CU, waves 0-3 run kind_a and waves 4-7 (one on each SIMD beside the first
 * four) kind_b, or nothing with kind_b = -1.  Kinds: 0 v_add_u32, 1 v_xor_b32,
 * 2 v_alignbit_b32, 3 v_mad_u64_u32, 4 v_addc_co_u32, 5 v_lshlrev_b32,
 * 6 v_lshrrev_b32, 7 v_mov_b32.  Reports each group's nanoseconds per
 * instruction over its own stream (the second group's figure includes the
 * time it runs alone after the first has finished, if it is the slower). */
int bnkp_pair(int device, int kind_a, int kind_b, uint32_t iters, double *ns_a, double *ns_b);

/* The ChaCha20 quarter-round stream (adds, xors and rotates 1:1:1 in groups of
 * four) with `waves_per_simd` waves resident per SIMD, waves coming and going
 * as in a long launch; with raised_priority the four rotates of a group run
 * between s_setprio 1 and s_setprio 0.  Reports VALU lane-ops per second. */
int bnkp_mix(int device, int raised_priority, int waves_per_simd, uint32_t iters, double *ops_per_sec);

/* The AEAD kernel's arithmetic alone (the product's lane code: per 64 bytes a
 * ChaCha20 block, the xor and four Poly1305 blocks, a packet per lane, the
 * data a constant in registers) with `waves_per_simd` (1..4) waves resident
 * per SIMD; paired: two keystream blocks side by side as in the kernel's
 * 128-byte steps.  data_blocks (even) per lane.  Reports 64-byte blocks per
 * second, the packet's key block included: the kernel's rate if moving the
 * packets cost nothing. */
int bnkp_aead_compute(int device, int paired, int waves_per_simd, uint32_t data_blocks, double *blocks_per_sec);

#ifdef __cplusplus
}
#endif
#endif
