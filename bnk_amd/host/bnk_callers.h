/* Load generator with wireguard-go's calling pattern (bnk_callers.cpp,
 * libbnkcallers.so): T threads, each one per-peer goroutine's worth of calls of
 * at most 128 packets from its own part of a pinned ring
 * (internal/filter/filter.go:160-186, internal/magicsock/bind.go:326-328,
 * 372-377).  For the benchmark and the many-callers test; not part of the
 * product library. */
#ifndef BNK_CALLERS_H
#define BNK_CALLERS_H

#include "../../include/bnkhip.h"

#ifdef __cplusplus
extern "C" {
#endif

enum { BNKC_AEAD = 0, BNKC_TUNNEL = 1 };

typedef struct bnkc_result {
    double seconds;           /* wall time of the timed rounds, all threads */
    uint64_t calls;           /* calls made in that time (two per thread and round) */
    uint64_t packets;         /* packets through a round trip */
    uint64_t plaintext_bytes; /* their plaintext bytes (counted once per round trip) */
    double out_p50_us, out_p99_us, out_max_us; /* per-call latency: seal / NoteOutbound+encapsulate */
    double in_p50_us, in_p99_us, in_max_us;    /* per-call latency: open / decapsulate+CheckInbound */
    int rc;                   /* first failing return code of any call, 0 if none */
    uint64_t mismatches;      /* packets whose round trip did not give the expected result or bytes */
    uint64_t filtered;        /* tunnel: packets the inbound filter dropped (by construction: dst port 23) */
} bnkc_result;

/* Runs `warmup` untimed and `rounds` timed round trips on each of `threads`
 * threads; thread t uses peer t.  BNKC_AEAD: seal then open of
 * packets_per_call x payload bytes.  BNKC_TUNNEL: NoteOutbound + encapsulate,
 * then decapsulate + CheckInbound at now_ns; the context needs a peer table
 * that loops back (peer t: remote index = local index, send key = receive key,
 * allowed address 100.64.(t >> 8).(t & 255)) and rules that pass tcp port 8000
 * and not port 23.  Every round's results are checked (mismatches). */
int bnkc_run(bnk_ctx *ctx, int workload, uint32_t threads, uint32_t packets_per_call, uint32_t payload,
             uint32_t rounds, uint32_t warmup, int64_t now_ns, bnkc_result *out);

/* The same under an offered load instead of back-to-back calls: the threads
 * together offer gbit_per_s_per_direction of plaintext each way, every thread
 * starting its timed rounds at fixed intervals (first rounds spread evenly over
 * one interval) whether or not the round before has returned.  The outbound
 * call's time counts from when its round was due, so a thread that has fallen
 * behind shows it; `seconds` against the offered rate tells whether the load
 * was carried. */
int bnkc_run_paced(bnk_ctx *ctx, int workload, uint32_t threads, uint32_t packets_per_call, uint32_t payload,
                   uint32_t rounds, uint32_t warmup, int64_t now_ns, double gbit_per_s_per_direction,
                   bnkc_result *out);

#ifdef __cplusplus
}
#endif
#endif
