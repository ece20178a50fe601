"""Writes tests/golden/filter_relay_digests.json.

SHA-256 digests of what the CPU oracle (oracle/filter.c, oracle/relay.c,
oracle/aead.c: the line-by-line restatement of internal/filter/filter.go and
internal/acl/acl.go, one packet after the other in batch order as the
reference's mutex would serialise them) computes for configurations 4 and 5 at
their full size, so that the GPU's results can be compared byte for byte where
the oracle itself is too slow to run beside a test:

  cfg4  2^22 IPv4 headers against 4096 rules and the flow table 65,536 noted
        packets leave behind, checked at t0: digest of the 2^22 verdict bytes,
        and of the flow table afterwards (entries sorted by key; a refreshed
        entry carries its new expiry, an expired one that was asked for is gone);
  cfg5  2^22 IMIX packets, 4096 peers, 0.5 % forged tags, 5 % denied: digest of
        verdicts || outbound counters (LE64), and of ciphertext || tag of every
        packet that was re-sealed, in packet order.

Takes about five minutes and 8 GB of memory.  Run from the repository root:
    python tests/golden/make_filter_relay_digests.py
"""
import hashlib
import json
import os
import struct
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from bnk_amd import workloads as W  # noqa: E402
from oracle import binding as O  # noqa: E402


def flows_digest(flows: dict) -> str:
    """SHA-256 over (remote, remote port, local port, proto, expiry ns) of every
    entry, sorted by key, each packed little-endian as I H H B q."""
    h = hashlib.sha256()
    for key in sorted(flows):
        h.update(struct.pack("<IHHBq", key[0], key[1], key[2], key[3], flows[key]))
    return h.hexdigest()


def concat_sha(arena: np.ndarray, off, lens, extra: int, only=None) -> str:
    h = hashlib.sha256()
    mv = memoryview(arena)
    idx = range(len(off)) if only is None else only.tolist()
    for i in idx:
        o = int(off[i])
        h.update(mv[o:o + int(lens[i]) + extra])
    return h.hexdigest()


def cfg4(n: int) -> dict:
    w = W.acl_workload(n=n)
    ora = O.Filter()
    ora.set_rules(w.rules_ref)
    for now, rec in w.note_batches:
        buf = np.ascontiguousarray(rec).reshape(-1)
        m = rec.shape[0]
        ora.note_outbound_batch(buf, np.arange(m, dtype=np.uint64) * 32, np.full(m, 28, np.uint32), now)
    before = ora.flows()
    t = time.time()
    buf = np.ascontiguousarray(w.check).reshape(-1)
    v = ora.check_inbound_batch(buf, np.arange(n, dtype=np.uint64) * 32, np.full(n, 28, np.uint32), w.now_ns)
    print("  cfg4: %d verdicts in %.0f s, %.4f allowed" % (n, time.time() - t, v.mean()), flush=True)
    after = ora.flows()
    return {"packets": n, "rules": len(w.rules_ref), "sha256_headers": hashlib.sha256(buf.data).hexdigest(),
            "sha256_verdicts": hashlib.sha256(np.ascontiguousarray(v).data).hexdigest(),
            "allowed": int(v.sum()), "flows_before": len(before), "sha256_flows_before": flows_digest(before),
            "flows_after": len(after), "sha256_flows_after": flows_digest(after)}


def cfg5(n: int) -> dict:
    w = W.relay_workload(n=n, payload=True, align=128)
    b = w.batch
    keys_in, keys_out = np.ascontiguousarray(b.keys), np.ascontiguousarray(w.keys_out)
    ct_lens = (b.lens + 16).astype(np.uint32)
    sealed = np.zeros_like(b.plain)
    O.seal_batch(keys_in, b.peer, b.counters, b.plain, b.off, b.lens, sealed, b.off, 8)
    which, pos, mask = W.relay_forged_bits(w)
    sealed[pos] ^= mask
    ora = O.Filter()
    ora.set_rules(w.rules_ref)
    now, rec = w.note_batch
    m = rec.shape[0]
    ora.note_outbound_batch(np.ascontiguousarray(rec).reshape(-1), np.arange(m, dtype=np.uint64) * 32,
                            np.full(m, 28, np.uint32), now)
    out = np.full_like(sealed, 0x77)
    t = time.time()
    v, c = ora.relay_fused_batch(keys_in, b.peer, b.counters, keys_out, w.peer_out, w.ctr_base_out, sealed, b.off,
                                 ct_lens, out, b.off, w.now_ns)
    print("  cfg5: %d packets in %.0f s, verdict counts %s" % (n, time.time() - t, np.bincount(v, minlength=3)),
          flush=True)
    ok = np.flatnonzero(v == 0)
    h = hashlib.sha256()
    h.update(np.ascontiguousarray(v).data)
    h.update(np.ascontiguousarray(c.astype("<u8")).data)
    some = {}
    for i in (int(ok[0]), int(ok[1]), int(ok[len(ok) // 2]), int(ok[-2]), int(ok[-1])):
        o, L = int(b.off[i]), int(b.lens[i])
        some[str(i)] = hashlib.sha256(out[o:o + L + 16].data).hexdigest()
    return {"packets": n, "peers": int(keys_in.shape[0]), "arena_bytes": int(sealed.nbytes),
            "sha256_plain": concat_sha(b.plain, b.off, b.lens, 0),
            "sha256_sealed_in": concat_sha(sealed, b.off, b.lens, 16),
            "sha256_verdicts_and_counters": h.hexdigest(),
            "verdict_counts": [int(x) for x in np.bincount(v, minlength=3)],
            "sha256_resealed": concat_sha(out, b.off, b.lens, 16, only=ok),
            "sha256_of_resealed_packet": some,
            "sha256_flows_after": flows_digest(ora.flows()), "flows_after": len(ora.flows())}


def main() -> None:
    n = int(sys.argv[1]) if len(sys.argv) > 1 else 1 << 22
    doc = {"what": "SHA-256 digests of the CPU oracle's results (sequential, batch order) for "
                   "configurations 4 and 5; see tests/golden/make_filter_relay_digests.py"}
    print("cfg4", flush=True)
    doc["cfg4"] = cfg4(n)
    print("cfg5", flush=True)
    doc["cfg5"] = cfg5(n)
    name = "filter_relay_digests.json" if n == 1 << 22 else "filter_relay_digests_%d.json" % n
    with open(os.path.join(HERE, name), "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")


if __name__ == "__main__":
    main()
