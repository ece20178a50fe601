"""Writes tests/golden/aead_cfg2_cfg3_digests.json.

SHA-256 digests of the sealed packets of configurations 2 and 3 at their full
size, produced with OpenSSL's EVP_chacha20_poly1305 (an independent
implementation of RFC 8439; neither the CPU oracle nor the HIP library takes
part):

  cfg2  2^20 payloads x 1420 seeded-random bytes, one seeded key, counters
        0 .. 2^20-1; digest over the 2^20 sealed packets (1436 bytes each)
        concatenated in packet order -- which is also the byte image of the
        packed sealed arena (stride 1436);
  cfg3  2^20 IMIX payloads (60/576/1420 bytes 7:4:1, seeded shuffle), 256
        seeded keys, counter = per-peer base + per-peer sequence; digest over
        ciphertext || tag of every packet concatenated in packet order.

Nonce = 4 zero bytes || LE64(counter), empty AAD.  Takes about two minutes and
4 GB of memory.  Run from the repository root:
    python tests/golden/make_aead_digests.py
"""
import hashlib
import json
import os
import struct
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import openssl_ref  # noqa: E402
from bnk_amd import workloads as W  # noqa: E402

N = 1 << 20


def digest(b, n):
    """(sha256 of the concatenated sealed packets, sha256 of the concatenated
    plaintexts, {index: sha256 of that sealed packet} for a few packets)."""
    hs, hp = hashlib.sha256(), hashlib.sha256()
    some = {}
    keep = {0, 1, 63, 64, n // 2, n - 2, n - 1}
    for i in range(n):
        o, L = int(b.off[i]), int(b.lens[i])
        pt = b.plain[o:o + L].tobytes()
        nonce = b"\x00" * 4 + struct.pack("<Q", int(b.counters[i]))
        ct = openssl_ref.seal(b.keys[int(b.peer[i])].tobytes(), nonce, pt)
        hs.update(ct)
        hp.update(pt)
        if i in keep:
            some[str(i)] = hashlib.sha256(ct).hexdigest()
        if i % (1 << 17) == 0:
            print("  packet", i, flush=True)
    return hs.hexdigest(), hp.hexdigest(), some


def main() -> None:
    assert openssl_ref.available(), "libcrypto is required to write the fixture"
    n = int(sys.argv[1]) if len(sys.argv) > 1 else N
    doc = {"what": "SHA-256 over the sealed packets concatenated in packet order, OpenSSL "
                   "EVP_chacha20_poly1305, WireGuard nonce, empty AAD", "packets": n}
    print("cfg2", flush=True)
    b = W.aead_uniform(2, n, 1420, 1440)
    s, p, some = digest(b, n)
    doc["cfg2"] = {"sha256_sealed": s, "sha256_plain": p, "sha256_of_packet": some,
                   "key": b.keys[0].tobytes().hex()}
    del b
    print("cfg3", flush=True)
    b = W.aead_imix(3, n, n_peers=256)
    s, p, some = digest(b, n)
    doc["cfg3"] = {"sha256_sealed": s, "sha256_plain": p, "sha256_of_packet": some,
                   "arena_bytes": int(b.meta["total"]), "payload_bytes": int(b.lens.sum())}
    name = "aead_cfg2_cfg3_digests.json" if n == N else "aead_cfg2_cfg3_digests_%d.json" % n
    with open(os.path.join(HERE, name), "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")


if __name__ == "__main__":
    main()
