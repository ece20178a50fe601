"""Writes tests/golden/aead_cfg1_openssl.json.

Configuration 1 of the benchmark (128 WireGuard transport payloads of 1420
seeded-random bytes, one seeded key, counters 0..127, nonce = 4 zero bytes ||
LE64(counter), empty AAD) sealed with OpenSSL's EVP_chacha20_poly1305 -- an
independent implementation of RFC 8439, which is also what
golang.org/x/crypto/chacha20poly1305 implements.  Neither the CPU oracle nor
the HIP library is involved in producing the fixture.

Run from the repository root:  python tests/golden/make_aead_golden.py
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


def main() -> None:
    assert openssl_ref.available(), "libcrypto is required to write the fixture"
    b = W.aead_uniform(1, 128, 1420)
    key = b.keys[0].tobytes()
    sealed = []
    for i in range(b.n):
        o = int(b.off[i])
        nonce = b"\x00" * 4 + struct.pack("<Q", int(b.counters[i]))
        sealed.append(openssl_ref.seal(key, nonce, b.plain[o:o + 1420].tobytes()))
    doc = {
        "what": "cfg1: 128 x 1420 B, WireGuard nonce, empty AAD, OpenSSL EVP_chacha20_poly1305",
        "key": key.hex(),
        "sha256_all_plain": hashlib.sha256(
            b.plain.reshape(128, b.stride)[:, :1420].tobytes()).hexdigest(),
        "sha256_all_sealed": hashlib.sha256(b"".join(sealed)).hexdigest(),
        "packets": {str(i): sealed[i].hex() for i in (0, 1, 63, 127)},
    }
    with open(os.path.join(HERE, "aead_cfg1_openssl.json"), "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")


if __name__ == "__main__":
    main()
