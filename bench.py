#!/usr/bin/env python3
"""Headline benchmark: batched WireGuard transport seal+open at 1420 B.

One step = one pass of the hot path over one batch: seal then open of
2^20 packets x 1420 B (one peer key, sequential 64-bit counters, packet slots
at a 1440-byte stride), inputs resident in HBM before the timed region.  The
value is plaintext Gbit/s through the seal+open pair on one MI355X.

Prints ONE JSON line.  Besides the contract fields it carries
  roofline       the binding one: int32 VALU instructions issued by the dominant kernel
                 (aead_wave_kernel) against the rate at which the SIMDs can take them, with an
                 op-equivalent model beside it
  roofline_hbm   the same launches as algorithmic bytes against the HBM peak
  cpu_baseline   the CPU oracle timed on this box's host cores (bounded sample)
  cpu_baseline_openssl  the same sample through OpenSSL's assembly, when libcrypto is there
  packed_layout  the same packets back to back (no slot 16-byte aligned)
  extra          the ACL filter rate (configuration 4) with its own roofline and CPU
                 baseline, what one call costs on 128 packets in pinned host rings, and the
                 rates of configurations 3 and 5 and of the transport framing

--workload filter | imix | relay | wg | host | latency | callers | copy | sizes | issue print one line for that
workload alone; --no-extras leaves out everything but the timed launches (for traces).
"""
from __future__ import annotations

import argparse
import json
import os
import shutil
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

L = 1420
STRIDE = 1440
HBM_PEAK_GBS = 8000.0
# VALU issue: a SIMD (16 lanes wide) takes a 64-lane instruction in four cycles, and two of
# them together when both are of the plain kind (add, xor, and, or, move, select, fused
# multiply-add in fp32: the rate behind the published 157.3 TFLOP/s fp32 vector figure, two
# FLOP per lane-op) and come from different waves; rotates, shifts left, multiplies and
# add-with-carry go one at a time.  1024 SIMDs x 16 lanes x 2.4 GHz = 39.3 T lane-op/s for
# the second kind, twice that for the first.
VALU_PEAK_TOPS = 78.6
VALU_SINGLE_ISSUE_TOPS = 39.3
# Counter readings for one launch of aead_wave_kernel over 2^20 packets x 1420 B (mean of
# seal and open), taken with rocprofv3 --pmc and kept in profiles/aead_wave_kernel_cfg2.md;
# they change only when the kernel does.
VALU_LANE_INSTR_PER_PACKET = 27697   # SQ_INSTS_VALU x 64 / 2^20
VALU_SINGLE_ISSUE_SHARE = 0.40       # of them: v_alignbit_b32, v_mad_u64_u32, v_add_co/v_addc_co (counted in the kernel's loops)
TRAFFIC_BYTES_PER_LAUNCH = 3.1783e9   # FETCH_SIZE + WRITE_SIZE, scaled by copy_kernel
# the same for filter_check_kernel over 2^22 headers (profiles/filter_check_kernel_cfg4.md)
FILTER_TRAFFIC_BYTES_PER_LAUNCH = 192.0e6
# The counter readings above describe the kernel sources as they were when the readings
# were taken: sha256 (first 16 hex digits) over the files named, in order.  When a file has
# changed since, the JSON line says "counters_stale": true beside the figures derived from
# them, until the profile is taken again and the hash here replaced
# (`python bench.py --source-hashes` prints the current ones).
AEAD_COUNTER_SOURCES = ("bnk_amd/csrc/aead_kernels.hip", "bnk_amd/csrc/aead_lane.hpp", "bnk_amd/csrc/kernels.hpp")
AEAD_COUNTERS_TAKEN_ON = "1f5676f98fa92181"
FILTER_COUNTER_SOURCES = ("bnk_amd/csrc/filter_kernels.hip", "bnk_amd/csrc/filter_dev.hpp")
FILTER_COUNTERS_TAKEN_ON = "f5d0b5f0eddaea31"


def source_hash(files) -> str:
    import hashlib
    h = hashlib.sha256()
    for f in files:
        with open(os.path.join(ROOT, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


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


def _events(torch, stream, k):
    return [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(k)]


def bench_filter(args) -> dict:
    """Configuration 4: 2^22 IPv4 headers (28-byte records back to back) against
    4096 rules and a flow table built from 65,536 noted outbound packets; one
    step = one CheckInbound batch."""
    import numpy as np
    import torch
    from bnk_amd import lib, workloads as W
    n = 1 << 22
    w = W.acl_workload(n=n)
    ctx = lib.Context(0)
    ctx.filter_set_rules(w.rules_ref)
    for now, rec in w.note_batches:
        buf = np.ascontiguousarray(rec).reshape(-1)
        ctx.filter_note_outbound(
            lib.make_batch(buf, buf.nbytes, rec.shape[0], lib.MEM_HOST, stride=32, length=28), now)
    dev = torch.device("cuda:0")
    # the headers back to back: 20 bytes of IPv4 + 8 of L4, nothing between them
    d_rec = torch.from_numpy(np.ascontiguousarray(w.check[:, :28])).to(dev)
    d_v = torch.zeros(n, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    batch = lib.make_batch(d_rec, n * 28, n, lib.MEM_DEVICE, stride=28, length=28)
    for _ in range(args.warmup):
        ctx.filter_check_inbound(batch, w.now_ns, d_v)
    ctx.sync()
    stream = torch.cuda.ExternalStream(ctx.stream, device=dev)
    ev = _events(torch, stream, args.steps)
    t0 = time.perf_counter()
    for s in range(args.steps):
        ev[s][0].record(stream)
        ctx.filter_check_inbound(batch, w.now_ns, d_v)
        ev[s][1].record(stream)
    ctx.sync()
    t1 = time.perf_counter()
    ms = (t1 - t0) * 1e3 / args.steps
    kern_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    v = d_v.cpu().numpy()
    allowed = float(v.mean())
    # algorithmic bytes: 20-byte header + 4 port bytes in, 1 verdict byte out, and one 16-byte
    # flow slot for every packet no rule admits (the reference probes its map for those)
    alg_bytes = n * 25 + int((1.0 - allowed) * n) * 16
    gbs = alg_bytes / (kern_ms * 1e-3) / 1e9
    out = {
        "metric": "acl_filter_mpkt_per_s", "value": round(n / (ms * 1e-3) / 1e6, 1),
        "unit": "Mpkt/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u32", "data": "synthetic",
        "config": {"workload": "cfg4: CheckInbound of %d IPv4 headers (28-byte records back to back), 4096 "
                               "rules, flow table from 65536 noted packets, device resident" % n,
                   "packets": n, "rules": 4096, "allowed_fraction": round(allowed, 4)},
        "roofline": {"bound": "hbm", "kernel": "filter_check_kernel", "achieved": round(gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "counters_stale": source_hash(FILTER_COUNTER_SOURCES) != FILTER_COUNTERS_TAKEN_ON,
                     "traffic": FILTER_TRAFFIC_BYTES_PER_LAUNCH if n == 1 << 22 else None,
                     "traffic_source": "profiles/filter_check_kernel_cfg4.md (FETCH_SIZE and WRITE_SIZE under "
                                       "rocprofv3 --pmc, scaled by copy_kernel; not re-measured in this run)",
                     "bytes_per_launch": alg_bytes,
                     "avg_launch_ms": round(kern_ms, 4)},
    }
    if not args.no_cpu_baseline:
        from oracle import binding as O
        ora = O.Filter()
        ora.set_rules(w.rules_ref)
        for now, rec in w.note_batches:
            m = rec.shape[0]
            ora.note_outbound_batch(np.ascontiguousarray(rec).reshape(-1),
                                    np.arange(m, dtype=np.uint64) * 32, np.full(m, 28, np.uint32), now)
        sample = args.cpu_sample or 1 << 18  # about five seconds of one core
        buf = np.ascontiguousarray(w.check[:sample]).reshape(-1)
        tp = time.perf_counter()
        ov = ora.check_inbound_batch(buf, np.arange(sample, dtype=np.uint64) * 32,
                                     np.full(sample, 28, np.uint32), w.now_ns)
        dt = time.perf_counter() - tp
        out["cpu_baseline"] = {
            "value": round(sample / dt / 1e6, 4), "unit": "Mpkt/s", "cores": 1, "kind": "port",
            "sample": "CheckInbound of the first %d headers of the same workload, C restatement "
                      "of filter.go/acl.go (linear rule scan under one lock, as the reference), "
                      "1 thread" % sample,
            "gpu_output_matches": bool(np.array_equal(ov, v[:sample])),
        }
        # All cores: the reference serialises CheckInbound behind one mutex
        # (filter.go:122), so more cores do not help it; this is what the same
        # algorithm gives with one private filter (rules and flows) per core.
        import threading
        threads = min(16, os.cpu_count() or 1)
        per = 1 << 15
        filters = []
        for _ in range(threads):
            f = O.Filter()
            f.set_rules(w.rules_ref)
            for now, rec in w.note_batches:
                m = rec.shape[0]
                f.note_outbound_batch(np.ascontiguousarray(rec).reshape(-1),
                                      np.arange(m, dtype=np.uint64) * 32, np.full(m, 28, np.uint32), now)
            filters.append(f)
        outs = [None] * threads

        def work(t):
            part = np.ascontiguousarray(w.check[t * per:(t + 1) * per]).reshape(-1)
            outs[t] = filters[t].check_inbound_batch(part, np.arange(per, dtype=np.uint64) * 32,
                                                     np.full(per, 28, np.uint32), w.now_ns)

        ths = [threading.Thread(target=work, args=(t,)) for t in range(threads)]
        tp = time.perf_counter()
        for th in ths:
            th.start()
        for th in ths:
            th.join()
        dt = time.perf_counter() - tp
        out["cpu_baseline_all_cores"] = {
            "value": round(threads * per / dt / 1e6, 4), "unit": "Mpkt/s", "cores": threads, "kind": "port",
            "sample": "%d threads x %d headers of the same workload, one private filter per thread (the "
                      "reference's single mutex would serialise them)" % (threads, per),
            "gpu_output_matches": bool(np.array_equal(np.concatenate(outs), v[:threads * per])),
        }
    ctx.close()
    return out


def _imix_device(torch, np, W, b, dev):
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    return (d(b.off.astype(np.int64)), d(b.peer.astype(np.int32)), d(b.counters.astype(np.int64)),
            d(b.lens.astype(np.int32)), d((b.lens + 16).astype(np.int32)))


def bench_imix(args) -> dict:
    """Configuration 3: 2^20 IMIX packets (60/576/1420 B, 7:4:1), 256 peers;
    seal, then open with 1 % of the tags forged."""
    import numpy as np
    import torch
    from bnk_amd import lib, workloads as W
    n = 1 << 20
    b = W.aead_imix(3, n, n_peers=256, payload=False, align=args.slot_align)
    dev = torch.device("cuda:0")
    total = b.meta["total"]
    plain = W.imix_plain_torch(b, dev)
    d_off, d_peer, d_ctr, d_lens, d_ctl = _imix_device(torch, np, W, b, dev)
    sealed = torch.zeros(total, dtype=torch.uint8, device=dev)
    forged_copy = torch.zeros(total, dtype=torch.uint8, device=dev)
    back = torch.zeros(total, dtype=torch.uint8, device=dev)
    v = torch.zeros(n, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    ctx = lib.Context(0)
    ctx.keys_set(lib.KEYS_SEND, b.keys)
    ctx.keys_set(lib.KEYS_RECV, b.keys)
    sb = lib.make_batch(plain, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens, peer=d_peer,
                        counters=d_ctr)
    so = lib.make_batch(sealed, total, n, lib.MEM_DEVICE, offsets=d_off)
    ctx.seal(sb, so)
    ctx.sync()
    forged_copy.copy_(sealed)
    k = int(0.01 * n)
    which = W.permutation(W.stream_seed(3, 5), n)[:k].astype(np.int64)
    bit = W.rand_below(W.stream_seed(3, 6), k, 128)
    pos = b.off[which].astype(np.int64) + b.lens[which].astype(np.int64) + (bit >> 3).astype(np.int64)
    forged_copy[torch.from_numpy(pos).to(dev)] ^= torch.from_numpy((1 << (bit & 7)).astype(np.uint8)).to(dev)
    torch.cuda.synchronize()
    ob = lib.make_batch(forged_copy, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_ctl, peer=d_peer,
                        counters=d_ctr)
    oo = lib.make_batch(back, total, n, lib.MEM_DEVICE, offsets=d_off)
    for _ in range(args.warmup):
        ctx.seal(sb, so)
        ctx.open(ob, oo, v)
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ctx.seal(sb, so)
        ctx.open(ob, oo, v)
    ctx.sync()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    vv = v.cpu().numpy()
    forged = np.zeros(n, bool)
    forged[which] = True
    assert np.array_equal(vv == 0, forged), "forged tags and rejects differ"
    payload = int(b.lens.sum())
    ops = sum(int((b.lens == L_).sum()) * ops_aead(L_) for L_ in (60, 576, 1420))
    # The two directions do not depend on each other here (open reads its own arena), as
    # inbound and outbound traffic of a relay do not: the same steps with the opens on a
    # second context, whose stream runs beside the first one's.
    two = None
    if not args.no_extras:
        ctx2 = lib.Context(0)
        ctx2.keys_set(lib.KEYS_RECV, b.keys)
        for _ in range(args.warmup):
            ctx.seal(sb, so)
            ctx2.open(ob, oo, v)
        ctx.sync()
        ctx2.sync()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            ctx.seal(sb, so)
            ctx2.open(ob, oo, v)
        ctx.sync()
        ctx2.sync()
        ms2 = (time.perf_counter() - t0) * 1e3 / args.steps
        assert np.array_equal(v.cpu().numpy() == 0, forged), "forged tags and rejects differ (two contexts)"
        two = {"value": round(payload * 8 / (ms2 * 1e-3) / 1e9, 1), "unit": "Gbit/s", "ms_per_step": round(ms2, 4),
               "workload": "the same seals and opens, the opens on a second context (its own stream)"}
        ctx2.close()
    ctx.close()
    return {
        "metric": "aead_seal_open_gbit_per_s_imix", "value": round(payload * 8 / (ms * 1e-3) / 1e9, 1),
        "unit": "Gbit/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u32", "data": "synthetic",
        "config": {"workload": "cfg3: seal+open of %d IMIX packets (60/576/1420 B 7:4:1), 256 peers, "
                               "1%% forged tags on open, device resident, slots back to back at "
                               "%d-byte alignment" % (n, args.slot_align), "packets": n},
        "mpkt_per_s_pair": round(n / (ms * 1e-3) / 1e6, 1),
        "rejected": int((vv == 0).sum()),
        "two_contexts": two,
        "op_equivalent_model": {"achieved": round(2 * ops / (ms * 1e-3) / 1e12, 2),
                                "unit": "Top/s (int32 op-equivalents)",
                                "ratio_to_single_issue_rate": round(2 * ops / (ms * 1e-3) / 1e12 / VALU_SINGLE_ISSUE_TOPS, 4)},
    }


def bench_relay(args) -> dict:
    """Configuration 5: open -> filter -> re-seal of 2^22 IMIX packets across
    4096 peers, 0.5 % forged tags, 5 % denied by the ACL."""
    import numpy as np
    import torch
    from bnk_amd import lib, workloads as W
    n = 1 << 22
    w = W.relay_workload(n=n, payload=False, align=args.slot_align)
    b = w.batch
    dev = torch.device("cuda:0")
    total = b.meta["total"]
    plain = W.relay_plain_torch(w, dev)
    d_off, d_peer, d_ctr, d_lens, d_ctl = _imix_device(torch, np, W, b, dev)
    d_peer_out = torch.from_numpy(w.peer_out.astype(np.int32)).to(dev)
    d_base = torch.from_numpy(w.ctr_base_out.astype(np.int64)).to(dev)
    sealed = torch.zeros(total, dtype=torch.uint8, device=dev)
    out = torch.zeros(total, dtype=torch.uint8, device=dev)
    verdict = torch.zeros(n, dtype=torch.uint8, device=dev)
    ctr_out = torch.zeros(n, dtype=torch.int64, device=dev)
    torch.cuda.synchronize()
    ctx = lib.Context(0)
    ctx.filter_set_rules(w.rules_ref)
    now, rec = w.note_batch
    buf = np.ascontiguousarray(rec).reshape(-1)
    ctx.filter_note_outbound(lib.make_batch(buf, buf.nbytes, rec.shape[0], lib.MEM_HOST, stride=32,
                                            length=28), now)
    ctx.keys_set(lib.KEYS_SEND, b.keys)
    ctx.seal(lib.make_batch(plain, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens, peer=d_peer,
                            counters=d_ctr),
             lib.make_batch(sealed, total, n, lib.MEM_DEVICE, offsets=d_off))
    ctx.sync()
    k = int(w.forged_fraction * n)
    which = W.permutation(W.stream_seed(5, 5), n)[:k].astype(np.int64)
    bit = W.rand_below(W.stream_seed(5, 6), k, 128)
    pos = b.off[which].astype(np.int64) + b.lens[which].astype(np.int64) + (bit >> 3).astype(np.int64)
    sealed[torch.from_numpy(pos).to(dev)] ^= torch.from_numpy((1 << (bit & 7)).astype(np.uint8)).to(dev)
    torch.cuda.synchronize()
    ctx.keys_set(lib.KEYS_RECV, b.keys)
    ctx.keys_set(lib.KEYS_SEND, w.keys_out)
    ib = lib.make_batch(sealed, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_ctl, peer=d_peer,
                        counters=d_ctr)
    ob = lib.make_batch(out, total, n, lib.MEM_DEVICE, offsets=d_off)

    def step():
        ctx.relay_fused(ib, d_peer_out, d_base, len(w.ctr_base_out), w.now_ns, ob, verdict, ctr_out)

    for _ in range(args.warmup):
        step()
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    ctx.sync()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    v = verdict.cpu().numpy()
    forged = np.zeros(n, bool)
    forged[which] = True
    assert np.array_equal(v, np.where(forged, 1, np.where(w.denied, 2, 0))), "verdicts differ"
    payload = int(b.lens.sum())
    ctx.close()
    return {
        "metric": "relay_open_filter_reseal_mpkt_per_s", "value": round(n / (ms * 1e-3) / 1e6, 1),
        "unit": "Mpkt/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u32", "data": "synthetic",
        "config": {"workload": "cfg5: open->filter->re-seal of %d IMIX packets, 4096 peers, 4096 rules, "
                               "0.5%% forged, 5%% denied, device resident, slots back to back at %d-byte "
                               "alignment" % (n, args.slot_align), "packets": n},
        "gbit_per_s_plaintext": round(payload * 8 / (ms * 1e-3) / 1e9, 1),
        "verdicts": {"ok": int((v == 0).sum()), "forged": int((v == 1).sum()),
                     "denied": int((v == 2).sum())},
    }


def bench_wg(args) -> dict:
    """Transport framing around the AEAD: encapsulate (header, padding, per-peer
    counters, seal in place) and decapsulate (header checks, index lookup, open,
    anti-replay windows, IPv4 trim, allowed-IP check) 2^20 MTU-sized packets
    across 1024 peers.  One step = encapsulate an arena in place, decapsulate
    it into a second arena; the next step sends what was just received, so
    every step carries fresh counters through the windows."""
    import numpy as np
    import torch
    from bnk_amd import lib, workloads as W
    dev = torch.device("cuda:0")
    n, n_peers, plen, mtu, stride = 1 << 20, 1024, 1420, 1420, 1456
    wire_len = 16 + plen + 16
    keys = W.rand_bytes(W.stream_seed(2, 40), n_peers * 32).reshape(n_peers, 32)
    # both ends in one context: each peer's two indices are the same number
    idx = (np.arange(n_peers, dtype=np.uint32) * 7919 + 3).astype(np.uint32)
    addr = (0x64400000 + np.arange(n_peers, dtype=np.uint32)).astype(np.uint32)
    full = np.full(n_peers, 0xFFFFFFFF, np.uint32)
    peer = W.rand_below(W.stream_seed(2, 41), n, n_peers).astype(np.uint32)
    d_peer = torch.from_numpy(peer.astype(np.int32)).to(dev)

    a = torch.zeros(n * stride + 16, dtype=torch.uint8, device=dev)
    b = torch.zeros(n * stride + 16, dtype=torch.uint8, device=dev)
    slots = a[:n * stride].view(n, stride)
    slots.copy_(W.rand_bytes_torch(W.stream_seed(2, 42), n * stride, dev).view(n, stride))
    slots[:, 16] = 0x45
    slots[:, 18] = plen >> 8
    slots[:, 19] = plen & 0xFF
    src = torch.from_numpy(addr.astype(np.int64)).to(dev)[d_peer.long()]
    for k in range(4):
        slots[:, 28 + k] = ((src >> (24 - 8 * k)) & 0xFF).to(torch.uint8)
    first_plain = slots[:, 16:16 + plen].clone()
    d_wl = torch.zeros(n, dtype=torch.int32, device=dev)
    d_res = torch.zeros(n, dtype=torch.uint8, device=dev)
    d_olen = torch.zeros(n, dtype=torch.int32, device=dev)
    d_gp = torch.zeros(n, dtype=torch.int32, device=dev)
    d_gc = torch.zeros(n, dtype=torch.int64, device=dev)
    torch.cuda.synchronize()
    ctx = lib.Context(0)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    ctx.wg_peers_set(np.stack([idx, idx, addr, full], 1))
    nbytes = n * stride
    arenas = (a, b)

    def step(k):
        cur, nxt = arenas[k & 1], arenas[1 - (k & 1)]
        ctx.wg_encap(lib.make_batch(cur, nbytes, n, lib.MEM_DEVICE, stride=stride, length=plen, peer=d_peer),
                     mtu, d_wl)
        # the plaintext lands 16 bytes into the other arena's slots: headroom for the next header
        ctx.wg_decap(lib.make_batch(cur, nbytes, n, lib.MEM_DEVICE, stride=stride, length=wire_len),
                     lib.make_batch(nxt[16:], nbytes, n, lib.MEM_DEVICE, stride=stride), d_res, d_olen, d_gp, d_gc)

    done = 0

    def timed(steps):
        nonlocal done
        ctx.sync()
        t0 = time.perf_counter()
        for k in range(done, done + steps):
            step(k)
        ctx.sync()
        done += steps
        return (time.perf_counter() - t0) * 1e3 / steps

    timed(args.warmup)
    ms = timed(args.steps)
    # the same steps with the framing in kernels of its own, and without the windows
    variants = None
    if not args.no_extras:
        ctx.wg_set_fused(False)
        timed(1)
        ms_separate = timed(args.steps)
        ctx.wg_set_fused(True)
        timed(1)
        ms_again = timed(args.steps)  # clocks drift over a run: the first figure once more
        ctx.wg_set_replay(False)
        timed(1)
        ms_no_windows = timed(args.steps)
        variants = {"framing_in_kernels_of_its_own": round(ms_separate, 4),
                    "as_value_measured_again": round(ms_again, 4),
                    "anti_replay_windows_off": round(ms_no_windows, 4)}
    last = arenas[done & 1][:n * stride].view(n, stride)[:, 16:16 + plen]
    assert bool((d_res == 0).all()) and bool((d_olen == plen).all()) and bool((d_gp == d_peer).all())
    assert bool((d_wl == wire_len).all()) and torch.equal(last, first_plain), "the packets did not survive the trips"
    want_ctr = W.per_peer_sequence(peer, n_peers) + np.bincount(peer, minlength=n_peers)[peer].astype(np.uint64) * \
        np.uint64(done - 1)
    assert np.array_equal(d_gc.cpu().numpy().astype(np.uint64), want_ctr), "counters do not follow the send order"
    ops = n * ops_aead(plen)
    ctx.close()
    return {
        "metric": "wg_encap_decap_gbit_per_s", "value": round(n * plen * 8 / (ms * 1e-3) / 1e9, 1),
        "unit": "Gbit/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u32", "data": "synthetic",
        "config": {"workload": "transport framing: encapsulate in place + decapsulate (anti-replay windows "
                               "included) %d packets x %d B (wire %d B, slot stride %d), %d peers, device "
                               "resident; every step sends what the step before received"
                               % (n, plen, wire_len, stride, n_peers), "packets": n},
        "mpkt_per_s_pair": round(n / (ms * 1e-3) / 1e6, 1),
        "same_run_ms_per_step": variants,
        "op_equivalent_model": {"achieved": round(2 * ops / (ms * 1e-3) / 1e12, 2),
                                "unit": "Top/s (int32 op-equivalents)",
                                "ratio_to_single_issue_rate": round(2 * ops / (ms * 1e-3) / 1e12 / VALU_SINGLE_ISSUE_TOPS, 4)},
    }


def bench_host(args) -> dict:
    """Configuration 2 handed over as BNK_MEM_HOST batches in a pinned ring:
    every call uploads the arena, runs the kernel and downloads the result, so
    the rate is bound by the host link, not by the kernel."""
    import numpy as np
    from bnk_amd import lib, workloads as W
    n = min(args.packets, 1 << 18)
    ctx = lib.Context(0)
    key = W.rand_bytes(W.stream_seed(2, 0), 32).reshape(1, 32)
    ctx.keys_set(lib.KEYS_SEND, key)
    ctx.keys_set(lib.KEYS_RECV, key)
    nbytes = n * STRIDE
    plain, sealed, opened = (ctx.ring_alloc(nbytes) for _ in range(3))
    plain_copy = W.rand_bytes(W.stream_seed(2, 1), n * L).reshape(n, L)
    plain.reshape(n, STRIDE)[:, :L] = plain_copy
    verdict = np.zeros(n, np.uint8)
    b_plain = lib.make_batch(plain, nbytes, n, lib.MEM_HOST, stride=STRIDE, length=L)
    b_sealed_out = lib.make_batch(sealed, nbytes, n, lib.MEM_HOST, stride=STRIDE)
    b_sealed_in = lib.make_batch(sealed, nbytes, n, lib.MEM_HOST, stride=STRIDE, length=L + 16)
    b_opened = lib.make_batch(opened, nbytes, n, lib.MEM_HOST, stride=STRIDE)

    def step():
        ctx.seal(b_plain, b_sealed_out)
        ctx.open(b_sealed_in, b_opened, verdict)

    for _ in range(args.warmup):
        step()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    assert verdict.all() and np.array_equal(opened.reshape(n, STRIDE)[:, :L], plain.reshape(n, STRIDE)[:, :L])
    for r in (plain, sealed, opened):
        ctx.ring_free(r)
    # the same through the framing entry points: encapsulate in place, decapsulate into a second ring
    n_peers, wstride = 256, 1456
    keys = W.rand_bytes(W.stream_seed(2, 40), n_peers * 32).reshape(n_peers, 32)
    ia = (np.arange(n_peers, dtype=np.uint32) * 7919 + 3).astype(np.uint32)
    ib = (np.arange(n_peers, dtype=np.uint32) * 104729 + 11).astype(np.uint32)
    addr = (0x64400000 + np.arange(n_peers, dtype=np.uint32)).astype(np.uint32)
    full = np.full(n_peers, 0xFFFFFFFF, np.uint32)
    peer = W.rand_below(W.stream_seed(2, 41), n, n_peers).astype(np.uint32)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.wg_peers_set(np.stack([ia, ib, addr, full], 1))
    rx = lib.Context(0)
    rx.keys_set(lib.KEYS_RECV, keys)
    rx.wg_peers_set(np.stack([ib, ia, addr, full], 1))
    ring, out = ctx.ring_alloc(n * wstride), rx.ring_alloc(n * wstride + 16)
    slots = ring.reshape(n, wstride)
    slots[:, 16:16 + L] = plain_copy
    slots[:, 16] = 0x45
    slots[:, 18] = L >> 8
    slots[:, 19] = L & 0xFF
    for k in range(4):
        slots[:, 28 + k] = ((addr[peer] >> (24 - 8 * k)) & 0xFF).astype(np.uint8)
    wl = np.zeros(n, np.uint32)
    res = np.zeros(n, np.uint8)
    olen = np.zeros(n, np.uint32)
    gp = np.zeros(n, np.uint32)
    gc = np.zeros(n, np.uint64)
    b_slots = lib.make_batch(ring, n * wstride, n, lib.MEM_HOST, stride=wstride, length=L, peer=peer)
    b_wire = lib.make_batch(ring, n * wstride, n, lib.MEM_HOST, stride=wstride, length=L + 32)
    b_out = lib.make_batch(out[16:], n * wstride, n, lib.MEM_HOST, stride=wstride)
    wg_ms = []
    for it in range(args.warmup + args.steps):
        # the header fields the receive side checks were encrypted by the last round (untimed)
        slots[:, 16] = 0x45
        slots[:, 18] = L >> 8
        slots[:, 19] = L & 0xFF
        for k in range(4):
            slots[:, 28 + k] = ((addr[peer] >> (24 - 8 * k)) & 0xFF).astype(np.uint8)
        t0 = time.perf_counter()
        ctx.wg_encap(b_slots, L, wl)
        rx.wg_decap(b_wire, b_out, res, olen, gp, gc)
        wg_ms.append((time.perf_counter() - t0) * 1e3)
    assert (res == 0).all() and (olen == L).all() and np.array_equal(gp, peer)
    wg = sum(wg_ms[args.warmup:]) / args.steps
    ctx.ring_free(ring)
    rx.ring_free(out)
    rx.close()
    ctx.close()
    moved = 2 * (n * STRIDE + n * STRIDE)  # per step: arena up and arena down, twice
    return {
        "metric": "aead_seal_open_gbit_per_s_1420B_host_memory", "value": round(n * L * 8 / (ms * 1e-3) / 1e9, 1),
        "unit": "Gbit/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u32", "data": "synthetic",
        "config": {"workload": "cfg2 through BNK_MEM_HOST: seal+open of %d packets x %d B from pinned host "
                               "rings, upload and download inside every call" % (n, L), "packets": n},
        "host_link_gb_per_s": round(moved / (ms * 1e-3) / 1e9, 1),
        "framing": {"metric": "wg_encap_decap_gbit_per_s_host_memory",
                    "value": round(n * L * 8 / (wg * 1e-3) / 1e9, 1), "ms_per_step": round(wg, 3),
                    "workload": "encapsulate in place + decapsulate of the same packets through pinned "
                                "rings, %d peers" % n_peers},
    }


def bench_latency(args) -> dict:
    """What one call costs at the batch sizes the reference's interfaces hand over
    (wireguard-go passes at most 128 packets per Read/Write): host-memory seal,
    open and filter check, one call at a time, median of many."""
    import numpy as np
    from bnk_amd import lib, workloads as W
    ctx = lib.Context(0)
    key = W.rand_bytes(W.stream_seed(2, 0), 32).reshape(1, 32)
    ctx.keys_set(lib.KEYS_SEND, key)
    ctx.keys_set(lib.KEYS_RECV, key)
    ctx.filter_set_rules([([(W.CGNAT_BASE | 7, 32)], "tcp", [(22, 22)])])
    out = {}
    reps = max(args.steps, 5) * 10
    for n in (1, 128, 1024, 8192):
        nbytes = n * STRIDE
        plain, sealed, opened = (ctx.ring_alloc(nbytes) for _ in range(3))
        plain.reshape(n, STRIDE)[:, :L] = W.rand_bytes(W.stream_seed(2, 1), n * L).reshape(n, L)
        plain.reshape(n, STRIDE)[:, 0] = 0x45
        plain.reshape(n, STRIDE)[:, 9] = 6
        v = np.zeros(n, np.uint8)
        b_plain = lib.make_batch(plain, nbytes, n, lib.MEM_HOST, stride=STRIDE, length=L)
        b_so = lib.make_batch(sealed, nbytes, n, lib.MEM_HOST, stride=STRIDE)
        b_si = lib.make_batch(sealed, nbytes, n, lib.MEM_HOST, stride=STRIDE, length=L + 16)
        b_op = lib.make_batch(opened, nbytes, n, lib.MEM_HOST, stride=STRIDE)
        t = {"seal": [], "open": [], "filter": [], "note": []}
        for it in range(reps + 5):
            t0 = time.perf_counter()
            ctx.seal(b_plain, b_so)
            t1 = time.perf_counter()
            ctx.open(b_si, b_op, v)
            t2 = time.perf_counter()
            ctx.filter_check_inbound(b_plain, 1_700_000_000_000_000_000, v)
            t3 = time.perf_counter()
            ctx.filter_note_outbound(b_plain, 1_700_000_000_000_000_000)
            t4 = time.perf_counter()
            if it >= 5:
                t["seal"].append(t1 - t0)
                t["open"].append(t2 - t1)
                t["filter"].append(t3 - t2)
                t["note"].append(t4 - t3)
        out[str(n)] = {k: round(float(np.median(x)) * 1e6, 1) for k, x in t.items()}
        for r in (plain, sealed, opened):
            ctx.ring_free(r)
    # WireGuard framing around the AEAD, the calls a wireguard-go bind would make
    P = 16
    keys = W.rand_bytes(W.stream_seed(2, 3), 32 * P).reshape(P, 32)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    ctx.wg_peers_set([(100 + i, 100 + i, W.CGNAT_BASE | (i + 1), 0xFFFFFFFF) for i in range(P)])
    slot, inner = 1504, 1400
    for n in (1, 128, 1024):
        ring, back = ctx.ring_alloc(n * slot), ctx.ring_alloc(n * slot)
        off = np.arange(n, dtype=np.uint64) * slot
        lens = np.full(n, inner, np.uint32)
        peer = (np.arange(n) % P).astype(np.uint32)
        src = (W.CGNAT_BASE | (peer + 1)).astype(np.uint32)
        rows = ring.reshape(n, slot)
        wl, res, ol = np.zeros(n, np.uint32), np.zeros(n, np.uint8), np.zeros(n, np.uint32)
        gp, gc = np.zeros(n, np.uint32), np.zeros(n, np.uint64)
        te, td, tne, tdf = [], [], [], []
        for it in range(reps + 5):
            rows[:, 16:36] = 0
            rows[:, 16] = 0x45
            rows[:, 18] = inner >> 8
            rows[:, 19] = inner & 255
            for k in range(4):
                rows[:, 28 + k] = (src >> (24 - 8 * k)) & 255
            t0 = time.perf_counter()
            ctx.wg_encap(lib.make_batch(ring, n * slot, n, lib.MEM_HOST, offsets=off, lens=lens, peer=peer),
                         1420, wl)
            t1 = time.perf_counter()
            ctx.wg_decap(lib.make_batch(ring, n * slot, n, lib.MEM_HOST, offsets=off, lens=wl),
                         lib.make_batch(back, n * slot, n, lib.MEM_HOST, offsets=off), res, ol, gp, gc)
            t2 = time.perf_counter()
            if int((res != 0).sum()) != 0:
                raise SystemExit("framing round trip rejected packets")
            # the same with the filter inside the call: NoteOutbound before the
            # encapsulation, CheckInbound after the decapsulation
            rows[:, 16:36] = 0
            rows[:, 16] = 0x45
            rows[:, 18] = inner >> 8
            rows[:, 19] = inner & 255
            rows[:, 25] = 17
            for k in range(4):
                rows[:, 28 + k] = (src >> (24 - 8 * k)) & 255
            t3 = time.perf_counter()
            ctx.wg_note_encap(lib.make_batch(ring, n * slot, n, lib.MEM_HOST, offsets=off, lens=lens, peer=peer),
                              1420, 1_700_000_000_000_000_000, wl)
            t4 = time.perf_counter()
            ctx.wg_decap_filter(lib.make_batch(ring, n * slot, n, lib.MEM_HOST, offsets=off, lens=wl),
                                lib.make_batch(back, n * slot, n, lib.MEM_HOST, offsets=off),
                                1_700_000_000_000_000_000, res, ol, gp, gc)
            t5 = time.perf_counter()
            if it >= 5:
                te.append(t1 - t0)
                td.append(t2 - t1)
                tne.append(t4 - t3)
                tdf.append(t5 - t4)
        out[str(n)]["wg_encap"] = round(float(np.median(te)) * 1e6, 1)
        out[str(n)]["wg_decap"] = round(float(np.median(td)) * 1e6, 1)
        out[str(n)]["wg_note_encap"] = round(float(np.median(tne)) * 1e6, 1)
        out[str(n)]["wg_decap_filter"] = round(float(np.median(tdf)) * 1e6, 1)
        ctx.ring_free(ring)
        ctx.ring_free(back)
    ctx.close()
    return {
        "metric": "call_latency_us_host_memory", "value": out["128"]["seal"], "unit": "us", "n_gpus": 1,
        "steps": reps, "warmup": 5, "ms_per_step": round(out["128"]["seal"] / 1e3, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "u32",
        "data": "synthetic",
        "config": {"workload": "median microseconds per call (upload + kernel + download + wait) for "
                               "batches of 1 / 128 / 1024 / 8192 packets x %d B in pinned rings, and for "
                               "WireGuard encapsulation / decapsulation of 1400-byte inner packets; value "
                               "is seal at 128 packets" % L},
        "per_batch_size_us": out,
    }


def bench_callers(args) -> dict:
    """The reference's calling pattern: T threads, each one per-peer goroutine's worth of
    blocking calls of 128 packets x 1420 B from its own part of a pinned ring
    (internal/filter/filter.go:160-186, internal/magicsock/bind.go:326-328, 372-377), through
    the library as it is (one call at a time behind the context lock) and with the library
    merging them (bnk_set_coalesce).  The load generator is native code over the C ABI
    (bnk_amd/host/bnk_callers.cpp): Python threads would measure the interpreter lock."""
    import ctypes as C
    import numpy as np
    from bnk_amd import lib, workloads as W
    so = C.CDLL(os.path.join(ROOT, "bnk_amd", "libbnkcallers.so"))

    class Result(C.Structure):
        _fields_ = [("seconds", C.c_double), ("calls", C.c_uint64), ("packets", C.c_uint64),
                    ("plaintext_bytes", C.c_uint64), ("out_p50_us", C.c_double), ("out_p99_us", C.c_double),
                    ("out_max_us", C.c_double), ("in_p50_us", C.c_double), ("in_p99_us", C.c_double),
                    ("in_max_us", C.c_double), ("rc", C.c_int), ("mismatches", C.c_uint64),
                    ("filtered", C.c_uint64)]

    t_max, per_call, rounds, warm = 16, 128, max(args.steps, 20) * 4, 10
    window_packets, wait_us = 4096, 30
    ctx = lib.Context(0)
    keys = W.rand_bytes(W.stream_seed(2, 7), t_max * 32).reshape(t_max, 32)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    # a peer table that loops back: what a peer sends is addressed to itself
    ctx.wg_peers_set([(0x1000 + 37 * t, 0x1000 + 37 * t, W.CGNAT_BASE + t, 0xFFFFFFFF) for t in range(t_max)])
    ctx.filter_set_rules([([(W.CGNAT_BASE, 10)], "tcp", [(8000, 8000)])])
    now = 1_700_000_000 * 10**9
    rows = []
    for workload, name, legs in ((0, "seal + open", ("seal", "open")),
                                 (1, "NoteOutbound + encapsulate, decapsulate + CheckInbound",
                                  ("note_encap", "decap_filter"))):
        for threads in (1, 4, 16):
            for merged in (False, True):
                ctx.set_coalesce(window_packets if merged else 0, wait_us)
                s0 = ctx.coalesce_stats()
                r = Result()
                rc = so.bnkc_run(C.c_void_p(ctx._h.value), C.c_int(workload), C.c_uint32(threads),
                                 C.c_uint32(per_call), C.c_uint32(L), C.c_uint32(rounds), C.c_uint32(warm),
                                 C.c_int64(now), C.byref(r))
                if rc != 0 or r.mismatches:
                    raise RuntimeError("callers workload failed: rc %d, %d mismatches" % (rc, r.mismatches))
                s1 = ctx.coalesce_stats()
                calls, batches = s1["calls"] - s0["calls"], s1["batches"] - s0["batches"]
                rows.append({
                    "calls": name, "threads": threads, "mode": "merged" if merged else "direct",
                    "gbit_per_s_round_trip": round(r.plaintext_bytes * 8e-9 / r.seconds, 1),
                    "gbit_per_s_per_direction": round(2 * r.plaintext_bytes * 8e-9 / r.seconds, 1),
                    "us_per_call": {legs[0]: {"p50": round(r.out_p50_us, 1), "p99": round(r.out_p99_us, 1)},
                                    legs[1]: {"p50": round(r.in_p50_us, 1), "p99": round(r.in_p99_us, 1)}},
                    "calls_per_launch": round(calls / batches, 2) if batches else 1.0,
                    "windows": batches,
                    "windows_that_waited_in_vain": s1["timed_out"] - s0["timed_out"],
                })
    # The same 16 callers under an offered load (every caller's rounds due at fixed intervals,
    # the callers' phases spread over an interval) instead of back to back: what a call costs
    # when the library is not saturated.  Offered: a quarter, half and three quarters of what
    # the merged calls carried above.  The outbound call's time counts from when it was due.
    so.bnkc_run_paced.restype = C.c_int
    for workload, name, legs in ((0, "seal + open", ("seal", "open")),
                                 (1, "NoteOutbound + encapsulate, decapsulate + CheckInbound",
                                  ("note_encap", "decap_filter"))):
        full = max(x["gbit_per_s_per_direction"] for x in rows
                   if x["calls"] == name and x["threads"] == t_max and x["mode"] == "merged") / 2.0
        for share in (0.25, 0.5, 0.75):
            for merged in (False, True):
                ctx.set_coalesce(window_packets if merged else 0, wait_us)
                s0 = ctx.coalesce_stats()
                r = Result()
                rc = so.bnkc_run_paced(C.c_void_p(ctx._h.value), C.c_int(workload), C.c_uint32(t_max),
                                       C.c_uint32(per_call), C.c_uint32(L), C.c_uint32(rounds), C.c_uint32(warm),
                                       C.c_int64(now), C.c_double(share * full), C.byref(r))
                if rc != 0 or r.mismatches:
                    raise RuntimeError("paced callers workload failed: rc %d, %d mismatches" % (rc, r.mismatches))
                s1 = ctx.coalesce_stats()
                calls, batches = s1["calls"] - s0["calls"], s1["batches"] - s0["batches"]
                rows.append({
                    "calls": name, "threads": t_max, "mode": ("merged" if merged else "direct") + ", offered load",
                    "offered_gbit_per_s_each_way": round(share * full, 1),
                    "carried_gbit_per_s_each_way": round(r.plaintext_bytes * 8e-9 / r.seconds, 1),
                    "us_per_call": {legs[0]: {"p50": round(r.out_p50_us, 1), "p99": round(r.out_p99_us, 1)},
                                    legs[1]: {"p50": round(r.in_p50_us, 1), "p99": round(r.in_p99_us, 1)}},
                    "calls_per_launch": round(calls / batches, 2) if batches else 1.0,
                })
    # Peers are independent of each other (keys, counters, windows, and a peer's flows are its
    # own), so they can be sharded over contexts: the same 16 callers, eight on each of two
    # contexts, whose streams run beside each other.
    import threading
    ctx2 = lib.Context(0)
    ctx2.keys_set(lib.KEYS_SEND, keys)
    ctx2.keys_set(lib.KEYS_RECV, keys)
    ctx2.wg_peers_set([(0x1000 + 37 * t, 0x1000 + 37 * t, W.CGNAT_BASE + t, 0xFFFFFFFF) for t in range(t_max)])
    ctx2.filter_set_rules([([(W.CGNAT_BASE, 10)], "tcp", [(8000, 8000)])])
    for c in (ctx, ctx2):
        c.set_coalesce(window_packets, wait_us)
    for workload, name, legs in ((0, "seal + open", ("seal", "open")),
                                 (1, "NoteOutbound + encapsulate, decapsulate + CheckInbound",
                                  ("note_encap", "decap_filter"))):
        res = [Result(), Result()]
        rcs = [0, 0]

        def half(k, c):
            rcs[k] = so.bnkc_run(C.c_void_p(c._h.value), C.c_int(workload), C.c_uint32(t_max // 2),
                                 C.c_uint32(per_call), C.c_uint32(L), C.c_uint32(rounds), C.c_uint32(warm),
                                 C.c_int64(now), C.byref(res[k]))

        th = [threading.Thread(target=half, args=(k, c)) for k, c in enumerate((ctx, ctx2))]
        for t in th:
            t.start()
        for t in th:
            t.join()
        if any(rcs) or any(r.mismatches for r in res):
            raise RuntimeError("callers workload on two contexts failed: %r" % (rcs,))
        rate = sum(r.plaintext_bytes * 8e-9 / r.seconds for r in res)
        rows.append({
            "calls": name, "threads": t_max, "mode": "merged, two contexts of 8 callers each",
            "gbit_per_s_round_trip": round(rate, 1), "gbit_per_s_per_direction": round(2 * rate, 1),
            "us_per_call": {legs[0]: {"p50": round(max(r.out_p50_us for r in res), 1),
                                      "p99": round(max(r.out_p99_us for r in res), 1)},
                            legs[1]: {"p50": round(max(r.in_p50_us for r in res), 1),
                                      "p99": round(max(r.in_p99_us for r in res), 1)}},
        })
    ctx2.set_coalesce(0)
    ctx2.close()
    ctx.set_coalesce(0)
    ctx.close()
    best = max((x for x in rows if x["threads"] == 16 and x["mode"] == "merged" and x["calls"] == "seal + open"),
               key=lambda x: x["gbit_per_s_round_trip"])
    # value: the plaintext the calls carried, every call's packets counted (a thread's seal and its
    # open each carry its 128 packets); gbit_per_s_round_trip counts a pair of calls once
    return {"metric": "callers_seal_open_gbit_per_s_16_threads_merged", "value": best["gbit_per_s_per_direction"],
            "unit": "Gbit/s of plaintext through the calls", "n_gpus": 1, "higher_is_better": True,
            "data": "synthetic", "dtype": "u32",
            "gbit_per_s_round_trip": best["gbit_per_s_round_trip"],
            "config": {"workload": "T threads x blocking calls of %d packets x %d B in one pinned ring, each thread "
                                   "a round trip (two calls) per round; direct = one "
                                   "call at a time behind the context lock, merged = bnk_set_coalesce(%d packets, "
                                   "%d us)" % (per_call, L, window_packets, wait_us),
                       "rounds": rounds, "host_cpus": os.cpu_count()},
            "rows": rows}


def bench_sizes(args) -> dict:
    """Seal and open of 2^20 packets of one common length, for each of a list
    of lengths (--sizes, default the three IMIX sizes): how far short packets
    are from the long ones.  Slots at the next multiple of 16 above length + 16."""
    import torch
    from bnk_amd import lib, workloads as W
    n = 1 << 20
    dev = torch.device("cuda:0")
    ctx = lib.Context(0)
    key = W.rand_bytes(W.stream_seed(2, 0), 32).reshape(1, 32)
    ctx.keys_set(lib.KEYS_SEND, key)
    ctx.keys_set(lib.KEYS_RECV, key)
    stream = torch.cuda.ExternalStream(ctx.stream, device=dev)
    per = {}
    for length in [int(x) for x in args.sizes.split(",")]:
        stride = (length + 16 + 15) // 16 * 16
        # --packed: the packets back to back on either side, no slot aligned
        ps, ss = (length, length + 16) if args.packed else (stride, stride)
        plain = W.rand_bytes_torch(W.stream_seed(2, 50), n * ps, dev).clone()
        sealed = torch.zeros(n * ss, dtype=torch.uint8, device=dev)
        back = torch.zeros_like(plain)
        v = torch.zeros(n, dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        bi = lib.make_batch(plain, n * ps, n, lib.MEM_DEVICE, stride=ps, length=length)
        bs = lib.make_batch(sealed, n * ss, n, lib.MEM_DEVICE, stride=ss)
        bc = lib.make_batch(sealed, n * ss, n, lib.MEM_DEVICE, stride=ss, length=length + 16)
        bb = lib.make_batch(back, n * ps, n, lib.MEM_DEVICE, stride=ps)
        for _ in range(args.warmup):
            ctx.seal(bi, bs)
            ctx.open(bc, bb, v)
        ctx.sync()
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
        for k in range(args.steps):
            ev[k][0].record(stream)
            ctx.seal(bi, bs)
            ev[k][1].record(stream)
            ctx.open(bc, bb, v)
            ev[k][2].record(stream)
        ctx.sync()
        torch.cuda.synchronize()
        seal_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
        open_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
        assert bool(v.all()) and torch.equal(back.view(n, ps)[:, :length], plain.view(n, ps)[:, :length])
        ops = n * ops_aead(length)
        per[str(length)] = {
            "seal_us": round(seal_ms * 1e3, 1), "open_us": round(open_ms * 1e3, 1),
            "gbit_per_s_pair": round(n * length * 8 / ((seal_ms + open_ms) * 1e-3) / 1e9, 1),
            "op_equivalent_ratio_to_single_issue_rate": round(2 * ops / ((seal_ms + open_ms) * 1e-3) / 1e12 / VALU_SINGLE_ISSUE_TOPS, 4),
        }
        del plain, sealed, back
    ctx.close()
    first = per[args.sizes.split(",")[0]]
    return {"metric": "aead_seal_open_us_by_length", "value": first["seal_us"], "unit": "us per seal launch, first length",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": False,
            "dtype": "u32", "data": "synthetic",
            "config": {"workload": "seal and open of %d packets of one common length, device resident, "
                                   "HIP events around each launch" % n, "lengths": args.sizes,
                       "layout": "back to back (plaintext stride = length, sealed stride = length + 16)"
                       if args.packed else "slots of the next multiple of 16 above length + 16"},
            "per_length": per}


def bench_copy(args) -> dict:
    """Plain device-to-device copy of 1 GiB: the measured HBM ceiling and the
    known-size launch the FETCH_SIZE / WRITE_SIZE counters are scaled by."""
    from bnk_amd import probe
    nbytes = 1 << 30
    rate = probe.copy(nbytes, max(args.steps, 1))
    return {"metric": "hbm_copy_gb_per_s", "value": round(rate / 1e9, 1), "unit": "GB/s",
            "n_gpus": 1, "steps": args.steps, "warmup": 1, "higher_is_better": True,
            "config": {"workload": "copy_kernel: %d bytes read + %d bytes written per launch"
                                   % (nbytes, nbytes)}}


def bench_issue(args) -> dict:
    """How a SIMD shares its issue between two waves (the rates the AEAD roofline is read
    against): pairs of instruction streams on one SIMD, and the ChaCha20 quarter-round
    stream by waves per SIMD with and without raised priority around its rotates."""
    from bnk_amd import probe
    pairs = {}
    for a, b in (("v_add_u32", None), ("v_alignbit_b32", None), ("v_mad_u64_u32", None),
                 ("v_add_u32", "v_add_u32"), ("v_add_u32", "v_xor_b32"), ("v_add_u32", "v_mov_b32"),
                 ("v_add_u32", "v_lshrrev_b32"), ("v_alignbit_b32", "v_add_u32"),
                 ("v_add_u32", "v_alignbit_b32"), ("v_alignbit_b32", "v_alignbit_b32"),
                 ("v_add_u32", "v_mad_u64_u32"), ("v_add_u32", "v_addc_co_u32"),
                 ("v_add_u32", "v_lshlrev_b32"), ("v_mad_u64_u32", "v_mad_u64_u32")):
        na, nb = probe.pair(a, b)
        pairs["%s | %s" % (a, b or "-")] = [round(na, 3), round(nb, 3)]
    mixes = {}
    for w in (1, 2, 3, 4):
        mixes[str(w)] = {"plain": round(probe.mix(False, w) / 1e12, 2),
                         "rotates_at_raised_priority": round(probe.mix(True, w) / 1e12, 2)}
    return {"metric": "valu_issue_probes", "value": mixes["2"]["rotates_at_raised_priority"],
            "unit": "T lane-op/s (quarter-round stream, two waves per SIMD, rotates at raised priority)",
            "n_gpus": 1, "steps": 1, "warmup": 1, "higher_is_better": True,
            "config": {"workload": "libbnkprobe.so: bnkp_pair and bnkp_mix"},
            "ns_per_instruction_first_and_second_wave": pairs,
            "quarter_round_stream_tops_by_waves_per_simd": mixes}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps first: a chip that was idle needs some 50 ms of work to reach the "
                         "clocks it then holds (the first 20 steps run about 5 %% slower); default 30, "
                         "110 for imix and 35 for wg, whose steps are shorter")
    ap.add_argument("--packets", type=int, default=1 << 20)
    ap.add_argument("--workload", default="aead", choices=["aead", "filter", "imix", "relay", "wg", "host", "latency", "callers", "copy", "sizes", "issue"],
                    help="aead (default, the headline line, with the ACL filter rate as an extra); "
                         "filter / imix / relay / wg / host / latency / copy print one line for that workload alone")
    ap.add_argument("--sizes", default="60,576,1420", help="sizes: packet lengths, comma separated")
    ap.add_argument("--packed", action="store_true",
                    help="sizes: packets back to back on either side (no slot aligned) instead of 16-byte aligned slots")
    ap.add_argument("--slot-align", type=int, default=128, choices=[16, 32, 64, 128],
                    help="imix, relay: packets lie back to back, each starting at a multiple of this "
                         "(128: every packet in 128-byte lines of its own, as in a ring of buffers; "
                         "16: packets share lines)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="aead: leave out the packed-layout leg and the ACL filter extra, so that a "
                         "kernel trace of the run holds the timed launches only")
    ap.add_argument("--cpu-sample", type=int, default=0,
                    help="packets in the CPU baseline sample (0 = sized for ~10 s)")
    ap.add_argument("--source-hashes", action="store_true",
                    help="print the hashes of the kernel sources the pasted counter readings belong to, and exit")
    args = ap.parse_args()
    if args.warmup is None:
        args.warmup = {"imix": 110, "wg": 35}.get(args.workload, 30)
    if args.source_hashes:
        print(json.dumps({"AEAD_COUNTERS_TAKEN_ON": source_hash(AEAD_COUNTER_SOURCES),
                          "FILTER_COUNTERS_TAKEN_ON": source_hash(FILTER_COUNTER_SOURCES)}))
        return 0
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
    if args.workload != "aead":
        out = {"filter": bench_filter, "imix": bench_imix, "relay": bench_relay,
               "wg": bench_wg, "host": bench_host, "latency": bench_latency, "callers": bench_callers,
               "copy": bench_copy, "issue": bench_issue,
               "sizes": bench_sizes}[args.workload](args)
        print(json.dumps(out))
        return 0
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

    from bnk_amd import probe
    probes = {}
    for name in ("v_add_u32", "v_xor_b32", "v_alignbit_b32", "v_mad_u64_u32"):
        probes[name] = round(probe.valu(name, 2000) / 1e12, 2)
    lane_instr = n * VALU_LANE_INSTR_PER_PACKET
    achieved_lane_tops = lane_instr / (kern_ms * 1e-3) / 1e12
    counters_apply = n == 1 << 20
    # Two measured ceilings beside the nominal ones: the kernel's arithmetic with no
    # packet movement (the product's lane code on constants in registers) at 1-4 waves
    # per SIMD, and a plain copy.  The kernel runs two waves per SIMD.
    blocks_per_packet = (L + 63) // 64 + 1
    kernel_gblocks = n * blocks_per_packet / (kern_ms * 1e-3) / 1e9
    arithmetic_alone = copy_gbs = None
    if not args.no_extras:
        arithmetic_alone = {str(w): round(probe.aead_compute(True, w) / 1e9, 1) for w in (1, 2, 3, 4)}
        copy_gbs = probe.copy(1 << 30, 10) / 1e9
    traffic_gbs = TRAFFIC_BYTES_PER_LAUNCH / (kern_ms * 1e-3) / 1e9 if counters_apply else None

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
        # The kernel is bound by VALU issue, not by memory: the binding roofline is
        # instructions actually issued against the rate at which the SIMDs can take them.
        "roofline": {
            "bound": "valu_int32", "kernel": "aead_wave_kernel",
            "achieved": round(achieved_lane_tops, 2), "peak": VALU_PEAK_TOPS,
            "unit": "T int32 lane-op/s (VALU instructions issued x 64 lanes)",
            "frac": round(achieved_lane_tops / VALU_PEAK_TOPS, 4),
            "peak_source": "two 64-lane VALU instructions per SIMD per four cycles x 1024 SIMDs x 2.4 GHz "
                           "(the issue rate behind the published 157.3 TFLOP/s fp32 vector figure); "
                           "reached only by pairs of plain instructions from two waves",
            # what earlier revisions of this line reported as frac: against one instruction
            # per SIMD per four cycles, the rate of the rotates, multiplies and carries
            "frac_of_single_issue_rate": round(achieved_lane_tops / VALU_SINGLE_ISSUE_TOPS, 4),
            "single_issue_share_of_instructions": VALU_SINGLE_ISSUE_SHARE,
            "counters_stale": source_hash(AEAD_COUNTER_SOURCES) != AEAD_COUNTERS_TAKEN_ON,
            "instructions_per_packet": VALU_LANE_INSTR_PER_PACKET,
            "instructions_source": "SQ_INSTS_VALU per launch x 64 / packets, rocprofv3 --pmc, mean of the "
                                   "seal and the open launch (profiles/aead_wave_kernel_cfg2.md); "
                                   "not re-measured in this run",
            "avg_launch_ms": round(kern_ms, 4),
            "traffic": TRAFFIC_BYTES_PER_LAUNCH if counters_apply else None,
            "traffic_source": "profiles/aead_wave_kernel_cfg2.md (FETCH_SIZE and WRITE_SIZE under "
                              "rocprofv3 --pmc, scaled by copy_kernel; not re-measured in this run)",
            # an op-equivalent model beside it (976 per ChaCha20 block + 16 per data block, 142 per Poly1305 block + 40): it prices a 64-bit multiply-add at 4 and
            # assumes 25 of them per Poly1305 block (radix 2^26), the kernel issues 20
            # (radix 2^32), so this ratio is not bounded by 1 and is no roofline fraction
            "op_equivalent_model": {
                "ops_per_packet": ops_aead(L), "achieved": round(achieved_tops, 2),
                "unit": "Top/s (int32 op-equivalents)",
                "ratio_to_single_issue_rate": round(achieved_tops / VALU_SINGLE_ISSUE_TOPS, 4),
                "ratio_to_peak": round(achieved_tops / VALU_PEAK_TOPS, 4),
            },
            "measured_ceilings_tops": probes,
            # 64-byte blocks (ChaCha20 block + xor + four Poly1305 blocks) per second: the
            # kernel, and the same arithmetic alone by waves resident per SIMD
            "arithmetic_alone": None if arithmetic_alone is None else {
                "unit": "G 64-byte blocks/s", "kernel": round(kernel_gblocks, 1),
                "by_waves_per_simd": arithmetic_alone,
                "kernel_over_two_waves_per_simd": round(kernel_gblocks / arithmetic_alone["2"], 4),
            },
        },
        "roofline_hbm": {
            "bound": "hbm", "kernel": "aead_wave_kernel",
            "achieved": round(achieved_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved_gbs / HBM_PEAK_GBS, 4),
            "counters_stale": source_hash(AEAD_COUNTER_SOURCES) != AEAD_COUNTERS_TAKEN_ON,
            "traffic": TRAFFIC_BYTES_PER_LAUNCH if counters_apply else None,
            "traffic_source": "profiles/aead_wave_kernel_cfg2.md (not re-measured in this run)",
            "bytes_per_launch": alg_bytes, "avg_launch_ms": round(kern_ms, 4),
            # what a plain copy of 1 GiB reaches on this box (bytes read + written), and the
            # kernel's counter traffic per second against it
            "measured_copy_gb_per_s": None if copy_gbs is None else round(copy_gbs, 1),
            "traffic_gb_per_s": None if traffic_gbs is None else round(traffic_gbs, 1),
            "traffic_over_measured_copy": None if copy_gbs is None or traffic_gbs is None
            else round(traffic_gbs / copy_gbs, 4),
        },
    }

    # the same packets packed back to back (plaintexts at a 1420-byte stride,
    # sealed packets at 1436): no slot is 16-byte aligned, so the kernel moves
    # them 64 bytes at a time at any alignment instead of whole 128-byte lines
    if args.no_extras:
        ctx.close()
        print(json.dumps(out))
        return 0
    pk_plain = plain[:, :L].contiguous().view(-1)
    pk_sealed = torch.zeros(n * (L + 16), dtype=torch.uint8, device=dev)
    pk_opened = torch.zeros(n * L, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    pb_plain = lib.make_batch(pk_plain, n * L, n, lib.MEM_DEVICE, stride=L, length=L)
    pb_sealed_out = lib.make_batch(pk_sealed, n * (L + 16), n, lib.MEM_DEVICE, stride=L + 16)
    pb_sealed_in = lib.make_batch(pk_sealed, n * (L + 16), n, lib.MEM_DEVICE, stride=L + 16, length=L + 16)
    pb_opened = lib.make_batch(pk_opened, n * L, n, lib.MEM_DEVICE, stride=L)
    verdict.zero_()
    # (warmed up like the main loop: a chip that has idled runs its first steps slower)
    psteps, pwarm = max(3, args.steps // 2), max(1, args.warmup // 2)
    for it in range(psteps + pwarm):
        if it == pwarm:
            ctx.sync()
            tp0 = time.perf_counter()
        ctx.seal(pb_plain, pb_sealed_out)
        ctx.open(pb_sealed_in, pb_opened, verdict)
    ctx.sync()
    torch.cuda.synchronize()
    packed_ms = (time.perf_counter() - tp0) * 1e3 / psteps
    if not (bool(verdict.all()) and bool(torch.equal(pk_opened, pk_plain)) and
            bool(torch.equal(pk_sealed.view(n, L + 16), sealed[:, :L + 16]))):
        print("packed layout: results differ from the slotted layout", file=sys.stderr)
        return 1
    out["packed_layout"] = {
        "value": round(n * L * 8 / (packed_ms * 1e-3) / 1e9, 1), "unit": "Gbit/s",
        "ms_per_step": round(packed_ms, 4), "steps": psteps, "warmup": pwarm,
        "ratio_to_slotted": round(ms_per_step / packed_ms, 4),
        "workload": "the same packets back to back: plaintext stride %d, sealed stride %d" % (L, L + 16),
    }
    del pk_plain, pk_sealed, pk_opened

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
        # passes over the sample until about ten seconds have gone by
        dt, passes = 0.0, 0
        while passes == 0 or (dt < 10.0 and passes < 200):
            tp = time.perf_counter()
            O.seal_batch(keys, hb.peer, hb.counters, hb.plain, hb.off, hb.lens, ho, hb.off, threads)
            v = O.open_batch(keys, hb.peer, hb.counters, ho, hb.off, hb.lens + 16, hv, hb.off, threads)
            dt += time.perf_counter() - tp
            passes += 1
        assert v.all() and np.array_equal(hv, hb.plain)
        # the GPU's first `sample` packets are the same bytes: compare them
        same = bool(np.array_equal(sealed[:sample].cpu().numpy().reshape(-1), ho))
        out["cpu_baseline"] = {
            "value": round(passes * sample * L * 8 / dt / 1e9, 3), "unit": "Gbit/s",
            "cores": threads, "kind": "port",
            "sample": "seal+open of the first %d packets of the same workload, %d passes in "
                      "%.1f s, scalar C restatement of RFC 8439 (oracle/aead.c), %d pthreads; the "
                      "Go reference cannot be built offline (no Go toolchain)"
                      % (sample, passes, dt, threads),
            "gpu_output_matches": same,
            # the reference's own Go path (x/crypto via wireguard-go) would be timed here with
            # GOMAXPROCS stated; it needs a Go toolchain and the module cache on this box
            "go_toolchain_on_box": shutil.which("go") is not None,
            "host_cpus": os.cpu_count(),
        }
        if O.ossl_available():
            # the same sample through OpenSSL's assembly implementation, the nearest
            # stand-in on this box for the assembly the Go reference runs
            so = np.zeros_like(hb.plain)
            sv = np.zeros_like(hb.plain)
            res = {}
            for nt in (1, threads):
                # about three seconds each
                tot, np_ = 0.0, 0
                while np_ == 0 or (tot < 3.0 and np_ < 200):
                    tp = time.perf_counter()
                    okc = O.ossl_seal_open_batch(keys, hb.peer, hb.counters, hb.plain, hb.off, hb.lens,
                                                 so, sv, nt)
                    tot += time.perf_counter() - tp
                    np_ += 1
                    assert okc == sample
                res[nt] = tot / np_
            out["cpu_baseline_openssl"] = {
                "value": round(sample * L * 8 / res[threads] / 1e9, 3), "unit": "Gbit/s",
                "cores": threads, "one_thread": round(sample * L * 8 / res[1] / 1e9, 3),
                "kind": "library",
                "sample": "the same %d packets, EVP_chacha20_poly1305 seal+open, %d pthreads"
                          % (sample, threads),
                "matches_oracle": bool(np.array_equal(so, ho)),
            }
    ctx.close()
    acl = bench_filter(args)
    out["extra"] = {"acl_filter": {k: acl[k] for k in ("metric", "value", "unit", "ms_per_step",
                                                       "config", "roofline", "cpu_baseline",
                                                       "cpu_baseline_all_cores")
                                   if k in acl}}
    # what one call costs at wireguard-go's own batch size (128 packets in pinned rings)
    largs = argparse.Namespace(**vars(args))
    largs.steps = 5
    lat = bench_latency(largs)
    out["extra"]["call_latency_us_128_packets"] = {
        "unit": "us per call, median, upload and download included",
        "workload": lat["config"]["workload"],
        **lat["per_batch_size_us"]["128"],
    }
    # the same calls from 16 threads at once, the way wireguard-go's per-peer goroutines
    # make them, one at a time behind the context lock and merged by the library
    try:
        cargs = argparse.Namespace(**vars(args))
        cargs.steps = 20
        cal = bench_callers(cargs)
        out["extra"]["callers_16_threads_x_128_packets"] = {
            "unit": "Gbit/s of plaintext: gbit_per_s_per_direction counts every call's packets, "
                    "gbit_per_s_round_trip a pair of calls once; us per call",
            "workload": cal["config"]["workload"],
            "rows": [r for r in cal["rows"] if r["threads"] == 16],
        }
    except Exception as e:  # a side measurement must not take the headline line with it
        out["extra"]["callers_16_threads_x_128_packets"] = {"error": "%s: %s" % (type(e).__name__, e)}
    # the other configurations the path is specified on, each a short run of its own
    # workload (their full lines: --workload imix | relay | wg)
    others = {}
    oargs = argparse.Namespace(**vars(args))
    oargs.no_cpu_baseline, oargs.no_extras = True, True
    # (warm-up by time rather than by count: some 60 ms of work, which is what a chip that has
    # idled through the host-side legs above needs to reach the clocks it then holds)
    for name, fn, steps, warm in (("cfg3_imix", bench_imix, 40, 110), ("cfg5_relay", bench_relay, 20, 30),
                                  ("transport_framing", bench_wg, 20, 35)):
        try:
            oargs.steps, oargs.warmup = steps, warm
            r = fn(oargs)
            others[name] = {"metric": r["metric"], "value": r["value"], "unit": r["unit"],
                            "ms_per_step": r["ms_per_step"], "steps": steps, "warmup": warm,
                            "workload": r["config"]["workload"]}
        except Exception as e:  # a side measurement must not take the headline line with it
            others[name] = {"error": "%s: %s" % (type(e).__name__, e)}
    out["extra"]["other_configurations"] = others
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
