#!/usr/bin/env python3
"""Headline benchmark: batched WireGuard transport seal+open at 1420 B.

One step = one pass of the hot path over one batch: seal then open of
2^20 packets x 1420 B (one peer key, sequential 64-bit counters, packet slots
at a 1440-byte stride), inputs resident in HBM before the timed region.  The
value is plaintext Gbit/s through the seal+open pair on one MI355X.

Prints ONE JSON line.  Besides the contract fields it carries
  roofline       HBM view of the dominant kernel (aead_wave_kernel)
  roofline_valu  the same launches priced in int32 op-equivalents
  cpu_baseline   the CPU oracle timed on this box's host cores (bounded sample)
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

L = 1420
STRIDE = 1440
HBM_PEAK_GBS = 8000.0
VALU_PEAK_TOPS = 39.3  # 256 CU x 64 lanes x 2.4 GHz, one int32 op per lane per clock


def ops_chacha(length: int) -> int:
    nb = (length + 63) // 64
    return 976 * (nb + 1) + 16 * nb


def ops_poly(length: int) -> int:
    return 142 * ((length + 15) // 16 + 1) + 40


def ops_aead(length: int) -> int:
    """int32 op-equivalents of one seal (or open): 80 quarter-rounds x 12 + 16
    feed-forward adds per ChaCha20 block, 16 XORs per data block; per Poly1305
    block 25 multiply-accumulates at 4 op-equivalents + 42 simple ops, + 40 to
    finish."""
    return ops_chacha(length) + ops_poly(length)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--packets", type=int, default=1 << 20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample", type=int, default=0,
                    help="packets in the CPU baseline sample (0 = sized for ~10 s)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no cross-GPU step and every box "
              "here has one GPU; run with --gpus 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch
    from bnk_amd import lib, workloads as W

    if not torch.cuda.is_available():
        print("no GPU visible: bench.py needs an MI355X", file=sys.stderr)
        return 2
    n = args.packets
    ctx = lib.Context(0)
    key = W.rand_bytes(W.stream_seed(2, 0), 32).reshape(1, 32)
    ctx.keys_set(lib.KEYS_SEND, key)
    ctx.keys_set(lib.KEYS_RECV, key)

    dev = torch.device("cuda:0")
    plain = W.aead_uniform_torch(2, n, L, STRIDE, dev)
    sealed = torch.zeros_like(plain)
    opened = torch.zeros_like(plain)
    verdict = torch.zeros(n, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    nbytes = n * STRIDE
    b_plain = lib.make_batch(plain, nbytes, n, lib.MEM_DEVICE, stride=STRIDE, length=L)
    b_sealed_out = lib.make_batch(sealed, nbytes, n, lib.MEM_DEVICE, stride=STRIDE)
    b_sealed_in = lib.make_batch(sealed, nbytes, n, lib.MEM_DEVICE, stride=STRIDE, length=L + 16)
    b_opened = lib.make_batch(opened, nbytes, n, lib.MEM_DEVICE, stride=STRIDE)

    def step():
        ctx.seal(b_plain, b_sealed_out)
        ctx.open(b_sealed_in, b_opened, verdict)

    for _ in range(args.warmup):
        step()
    ctx.sync()
    torch.cuda.synchronize()

    # HIP events on the library's own stream bracket every launch
    stream = torch.cuda.ExternalStream(ctx.stream, device=dev)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for s in range(args.steps):
        ev[s][0].record(stream)
        ctx.seal(b_plain, b_sealed_out)
        ev[s][1].record(stream)
        ctx.open(b_sealed_in, b_opened, verdict)
        ev[s][2].record(stream)
    ctx.sync()
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    ms_per_step = (t1 - t0) * 1e3 / args.steps
    seal_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    open_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
    gbps = n * L * 8 / (ms_per_step * 1e-3) / 1e9

    # correctness of what was timed: round trip is the identity, all tags verify
    ok = bool(verdict.all()) and bool(torch.equal(opened[:, :L], plain[:, :L]))
    if not ok:
        print("seal->open round trip failed", file=sys.stderr)
        return 1

    # the dominant kernel is aead_wave_kernel; a step holds two launches of it
    # (seal and open) with the same algorithmic traffic: L in + (L + 16) out
    # (+1 verdict byte on open); counters and peers are implicit here
    alg_bytes = n * (2 * L + 16)
    kern_ms = 0.5 * (seal_ms + open_ms)
    achieved_gbs = alg_bytes / (kern_ms * 1e-3) / 1e9
    ops = n * ops_aead(L)
    achieved_tops = ops / (kern_ms * 1e-3) / 1e12

    probes = {}
    for name in ("v_add_u32", "v_xor_b32", "v_alignbit_b32", "v_mad_u64_u32"):
        probes[name] = round(ctx.probe_valu(name, 2000) / 1e12, 2)

    out = {
        "metric": "aead_seal_open_gbit_per_s_1420B",
        "value": round(gbps, 1),
        "unit": "Gbit/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u32",
        "data": "synthetic",
        "config": {
            "workload": "cfg2: seal+open of %d packets x %d B, one peer key, sequential "
                        "counters, %d-byte slots, device resident" % (n, L, STRIDE),
            "packets": n, "payload_bytes": L, "slot_stride": STRIDE,
        },
        "seal_ms": round(seal_ms, 4),
        "open_ms": round(open_ms, 4),
        "mpkt_per_s_pair": round(n / (ms_per_step * 1e-3) / 1e6, 1),
        "roofline": {
            "bound": "hbm", "kernel": "aead_wave_kernel",
            "achieved": round(achieved_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved_gbs / HBM_PEAK_GBS, 4),
            "traffic": None,
            "bytes_per_launch": alg_bytes, "avg_launch_ms": round(kern_ms, 4),
        },
        "roofline_valu": {
            "bound": "valu_int32", "achieved": round(achieved_tops, 2),
            "peak": VALU_PEAK_TOPS, "unit": "Top/s (int32 op-equivalents)",
            "frac": round(achieved_tops / VALU_PEAK_TOPS, 4),
            "ops_per_packet": ops_aead(L),
            "measured_ceilings_tops": probes,
        },
    }

    if not args.no_cpu_baseline:
        from oracle import binding as O
        threads = min(16, os.cpu_count() or 1)
        # size the sample from a short single-thread probe so the leg takes ~10 s
        probe_n = 2048
        hb = W.aead_uniform(2, probe_n, L, STRIDE)
        ho = np.zeros_like(hb.plain)
        hv = np.zeros_like(hb.plain)
        keys = np.ascontiguousarray(hb.keys)
        tp = time.perf_counter()
        O.seal_batch(keys, hb.peer, hb.counters, hb.plain, hb.off, hb.lens, ho, hb.off, 1)
        O.open_batch(keys, hb.peer, hb.counters, ho, hb.off, hb.lens + 16, hv, hb.off, 1)
        per_pkt = (time.perf_counter() - tp) / probe_n
        sample = args.cpu_sample or int(max(4096, min(1 << 18, 10.0 * threads / per_pkt)))
        sample = (sample // 1024) * 1024
        hb = W.aead_uniform(2, sample, L, STRIDE)
        ho = np.zeros_like(hb.plain)
        hv = np.zeros_like(hb.plain)
        tp = time.perf_counter()
        O.seal_batch(keys, hb.peer, hb.counters, hb.plain, hb.off, hb.lens, ho, hb.off, threads)
        v = O.open_batch(keys, hb.peer, hb.counters, ho, hb.off, hb.lens + 16, hv, hb.off, threads)
        dt = time.perf_counter() - tp
        assert v.all() and np.array_equal(hv, hb.plain)
        # the GPU's first `sample` packets are the same bytes: compare them
        same = bool(np.array_equal(sealed[:sample].cpu().numpy().reshape(-1), ho))
        out["cpu_baseline"] = {
            "value": round(sample * L * 8 / dt / 1e9, 3), "unit": "Gbit/s",
            "cores": threads, "kind": "port",
            "sample": "seal+open of the first %d packets of the same workload, scalar C "
                      "restatement of RFC 8439 (oracle/aead.c), %d pthreads; the Go reference "
                      "cannot be built offline (no Go toolchain)" % (sample, threads),
            "gpu_output_matches": same,
        }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
