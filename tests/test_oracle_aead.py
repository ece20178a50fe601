"""Pins the CPU oracle's AEAD (oracle/aead.c) before anything trusts it.

Three independent anchors:
  1. RFC 8439 known-answer vectors (sections 2.3.2, 2.4.2, 2.5.2, 2.6.2,
     2.8.2 and the appendix A.3 Poly1305 carry/wrap vectors);
  2. a literal big-integer transcription of the RFC pseudocode
     (tests/rfc8439_py.py);
  3. OpenSSL's EVP_chacha20_poly1305 on the benchmark shapes.
golang.org/x/crypto's chacha20poly1305, which the reference reaches through
wireguard-go (go.mod:8,10; internal/dataplane/engine.go:51), implements the
same RFC and is tested against the same vectors.
"""
import hashlib
import json
import os

import numpy as np
import pytest

import openssl_ref
import rfc8439_py as rfc
from bnk_amd import workloads as W
from oracle import binding as O

H = bytes.fromhex
SUNSCREEN = (b"Ladies and Gentlemen of the class of '99: If I could offer you "
             b"only one tip for the future, sunscreen would be it.")


def test_chacha20_block_rfc_2_3_2():
    got = O.chacha20_block(bytes(range(32)), 1, H("000000090000004a00000000"))
    assert got == H(
        "10f1e7e4d13b5915500fdd1fa32071c4c7d1f4c733c068030422aa9ac3d46c4e"
        "d2826446079faa0914c2d705d98b02a2b5129cd1de164eb9cbd083e8a2503c4e")


def test_chacha20_block_all_zero_a1():
    # RFC 8439 A.1 vector 1: zero key, zero nonce, counter 0
    got = O.chacha20_block(bytes(32), 0, bytes(12))
    assert got == H(
        "76b8e0ada0f13d90405d6ae55386bd28bdd219b8a08ded1aa836efcc8b770dc7"
        "da41597c5157488d7724e03fb8d84a376a43b8f41518a11cc387b669b2ee6586")


def test_chacha20_encrypt_rfc_2_4_2():
    got = O.chacha20_xor(bytes(range(32)), 1, H("000000000000004a00000000"), SUNSCREEN)
    assert got == H(
        "6e2e359a2568f98041ba0728dd0d6981e97e7aec1d4360c20a27afccfd9fae0b"
        "f91b65c5524733ab8f593dabcd62b3571639d624e65152ab8f530c359f0861d8"
        "07ca0dbf500d6a6156a38e088a22b65e52bc514d16ccf806818ce91ab7793736"
        "5af90bbf74a35be6b40b8eedf2785e42874d")


def test_poly1305_rfc_2_5_2():
    key = H("85d6be7857556d337f4452fe42d506a80103808afb0db2fd4abff6af4149f51b")
    assert O.poly1305(key, b"Cryptographic Forum Research Group") == H(
        "a8061dc1305136c6c22b8baf0c0127a9")


# RFC 8439 A.3 vectors 1 and 5-11: degenerate keys and the 2^130-5 wrap cases.
A3 = [
    (bytes(32), bytes(64), bytes(16)),
    (H("02" + "00" * 31), H("ff" * 16), H("03" + "00" * 15)),
    (H("02" + "00" * 15 + "ff" * 16), H("02" + "00" * 15), H("03" + "00" * 15)),
    (H("01" + "00" * 31),
     H("ff" * 16 + "f0" + "ff" * 15 + "11" + "00" * 15), H("05" + "00" * 15)),
    (H("01" + "00" * 31),
     H("ff" * 16 + "fb" + "fe" * 15 + "01" * 16), bytes(16)),
    (H("02" + "00" * 31), H("fd" + "ff" * 15), H("fa" + "ff" * 15)),
    (H("01" + "00" * 7 + "04" + "00" * 23),
     H("e33594d7505e43b9" + "00" * 8 + "3394d7505e4379cd" + "01" + "00" * 7
       + "00" * 16 + "01" + "00" * 15),
     H("14" + "00" * 7 + "55" + "00" * 7)),
    (H("01" + "00" * 7 + "04" + "00" * 23),
     H("e33594d7505e43b9" + "00" * 8 + "3394d7505e4379cd" + "01" + "00" * 7
       + "00" * 16),
     H("13" + "00" * 15)),
]


@pytest.mark.parametrize("key,msg,tag", A3)
def test_poly1305_appendix_a3_edges(key, msg, tag):
    # the big-integer transcription fixes what the tag must be; the recalled
    # RFC value and the C oracle both have to agree with it
    assert rfc.poly1305(key, msg) == tag
    assert O.poly1305(key, msg) == tag


def test_poly1305_keygen_rfc_2_6_2():
    got = O.poly1305_keygen(bytes(range(0x80, 0xA0)), H("000000000001020304050607"))
    assert got == H("8ad5a08b905f81cc815040274ab29471a833b637e3fd0da508dbb8e2fdd1a646")


def test_aead_rfc_2_8_2():
    key = bytes(range(0x80, 0xA0))
    nonce = H("070000004041424344454647")
    aad = H("50515253c0c1c2c3c4c5c6c7")
    out = O.aead_seal(key, nonce, SUNSCREEN, aad)
    assert out[:16] == H("d31a8d34648e60db7b86afbc53ef7ec2")
    assert out[-16:] == H("1ae10b594f09e26a7e902ecbd0600691")
    assert out == rfc.aead_seal(key, nonce, SUNSCREEN, aad)
    ok, pt = O.aead_open(key, nonce, out, aad)
    assert ok and pt == SUNSCREEN


def test_aead_zero_key_empty_is_keepalive_tag():
    # empty plaintext, empty AAD: Poly1305 over the single length block of
    # zeros -- the body of a WireGuard keepalive under an all-zero key.  The
    # value is what OpenSSL (via node) produced when this vector was first recorded;
    # the big-integer transcription must agree.
    want = H("4eb972c9a8fb3a1b382bb4d36f5ffad1")
    assert rfc.aead_seal(bytes(32), bytes(12), b"") == want
    assert O.aead_seal(bytes(32), bytes(12), b"") == want


def test_wg_nonce_layout():
    assert O.wg_nonce(0) == bytes(12)
    assert O.wg_nonce(0x0102030405060708) == H("00000000" "0807060504030201")
    assert O.wg_nonce(1 << 32) == H("00000000" "0000000001000000")


LENS = [0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 576,
        1419, 1420, 1424, 1500]


@pytest.mark.parametrize("length", LENS)
def test_oracle_vs_bigint_restatement(length):
    seed = W.stream_seed(100, length)
    key = W.rand_bytes(seed, 32).tobytes()
    pt = W.rand_bytes(seed + 1, length).tobytes()
    for counter in (0, 1, 0xFFFFFFFF, 1 << 32, (1 << 64) - 1):
        nonce = O.wg_nonce(counter)
        assert nonce == rfc.wg_nonce(counter)
        sealed = O.aead_seal(key, nonce, pt)
        assert sealed == rfc.aead_seal(key, nonce, pt)
        ok, back = O.aead_open(key, nonce, sealed)
        assert ok and back == pt


def test_poly1305_random_vs_bigint():
    for i in range(200):
        seed = W.stream_seed(101, i)
        key = W.rand_bytes(seed, 32).tobytes()
        n = int(W.rand_below(seed + 1, 1, 300)[0])
        msg = W.rand_bytes(seed + 2, n).tobytes()
        assert O.poly1305(key, msg) == rfc.poly1305(key, msg)
    # all-ones r (before the clamp) and all-ones message: maximal limbs
    key = b"\xff" * 32
    for n in (16, 32, 160, 1440):
        assert O.poly1305(key, b"\xff" * n) == rfc.poly1305(key, b"\xff" * n)


@pytest.mark.skipif(not openssl_ref.available(), reason="libcrypto not present")
@pytest.mark.parametrize("length", [0, 1, 16, 60, 64, 576, 1419, 1420, 1500])
def test_oracle_vs_openssl(length):
    seed = W.stream_seed(102, length)
    key = W.rand_bytes(seed, 32).tobytes()
    pt = W.rand_bytes(seed + 1, length).tobytes()
    for counter in (0, 127, (1 << 48) + 5):
        nonce = O.wg_nonce(counter)
        sealed = O.aead_seal(key, nonce, pt)
        assert sealed == openssl_ref.seal(key, nonce, pt)
        assert openssl_ref.open_(key, nonce, sealed) == pt


def test_single_bit_flips_reject_and_zero_output():
    b = W.aead_uniform(1, 1, 100)
    key = b.keys[0].tobytes()
    nonce = O.wg_nonce(7)
    pt = b.plain[:100].tobytes()
    sealed = bytearray(O.aead_seal(key, nonce, pt))
    for pos in list(range(0, 116, 7)) + [100, 115]:
        for bit in (0, 7):
            bad = bytearray(sealed)
            bad[pos] ^= 1 << bit
            ok, out = O.aead_open(key, nonce, bytes(bad))
            assert not ok and out == bytes(100)
    # wrong counter, wrong key
    ok, _ = O.aead_open(key, O.wg_nonce(8), bytes(sealed))
    assert not ok
    k2 = bytearray(key); k2[31] ^= 0x80
    ok, _ = O.aead_open(bytes(k2), nonce, bytes(sealed))
    assert not ok
    # shorter than a tag: reject
    ok, _ = O.aead_open(key, nonce, bytes(sealed[:15]))
    assert not ok


def _seal_arena(b, nthreads=1):
    out = np.zeros_like(b.plain)
    O.seal_batch(np.ascontiguousarray(b.keys), b.peer, b.counters, b.plain, b.off,
                 b.lens, out, b.off, nthreads)
    return out


def test_batch_matches_single_and_threads():
    b = W.aead_imix(3, 600, n_peers=16)
    one = _seal_arena(b, 1)
    many = _seal_arena(b, 4)
    assert np.array_equal(one, many)
    for i in (0, 1, 17, 599):
        o, L = int(b.off[i]), int(b.lens[i])
        want = O.aead_seal(b.keys[b.peer[i]].tobytes(), O.wg_nonce(int(b.counters[i])),
                           b.plain[o:o + L].tobytes())
        assert one[o:o + L + 16].tobytes() == want
    back = np.zeros_like(b.plain)
    v = O.open_batch(np.ascontiguousarray(b.keys), b.peer, b.counters, one, b.off,
                     b.lens + 16, back, b.off, 3)
    assert v.all() and np.array_equal(back, b.plain)


GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "aead_cfg1_openssl.json")


def test_cfg1_golden_fixture():
    """Configuration 1 (128 x 1420 B, one key, counters 0..127) against the
    committed OpenSSL-generated fixture (tests/golden/make_aead_golden.py)."""
    g = json.load(open(GOLDEN))
    b = W.aead_uniform(1, 128, 1420)
    assert b.keys[0].tobytes().hex() == g["key"]
    sealed = _seal_arena(b).reshape(128, b.stride)[:, :1436]
    assert hashlib.sha256(sealed.tobytes()).hexdigest() == g["sha256_all_sealed"]
    for idx, hx in g["packets"].items():
        assert sealed[int(idx)].tobytes().hex() == hx


def test_openssl_batch_baseline_agrees_with_the_oracle():
    """The second CPU baseline bench.py reports (oracle/openssl_batch.c) seals
    to the same bytes as the restatement and opens back to the plaintext."""
    from bnk_amd import workloads as W
    if not O.ossl_available():
        pytest.skip("libcrypto not on this machine")
    b = W.aead_imix(3, 3000, n_peers=16)
    keys = np.ascontiguousarray(b.keys)
    want = np.zeros_like(b.plain)
    O.seal_batch(keys, b.peer, b.counters, b.plain, b.off, b.lens, want, b.off, 4)
    sealed = np.zeros_like(b.plain)
    opened = np.zeros_like(b.plain)
    assert O.ossl_seal_open_batch(keys, b.peer, b.counters, b.plain, b.off, b.lens, sealed, opened, 3) == b.n
    assert np.array_equal(sealed, want)
    for i in (0, 1, b.n - 1):
        o, l = int(b.off[i]), int(b.lens[i])
        assert np.array_equal(opened[o:o + l], b.plain[o:o + l])


@pytest.mark.parametrize("cfg", ["cfg2", "cfg3"])
def test_oracle_matches_the_openssl_digests_at_full_size(cfg):
    """The oracle's sealed bytes for configurations 2 and 3 at 2^20 packets,
    hashed in packet order, against the digests OpenSSL produced for the same
    seeded inputs (tests/golden/make_aead_digests.py)."""
    import hashlib
    import json
    import os
    g = json.load(open(os.path.join(os.path.dirname(__file__), "golden",
                                    "aead_cfg2_cfg3_digests.json")))
    n = g["packets"]
    b = W.aead_uniform(2, n, 1420, 1440) if cfg == "cfg2" else W.aead_imix(3, n, n_peers=256)
    out = np.zeros_like(b.plain)
    O.seal_batch(np.ascontiguousarray(b.keys), b.peer, b.counters, b.plain, b.off, b.lens, out, b.off, 8)
    h = hashlib.sha256()
    if cfg == "cfg2":
        h.update(np.ascontiguousarray(out.reshape(n, 1440)[:, :1436]).data)
    else:
        mv = memoryview(out)
        for o, L in zip(b.off.tolist(), b.lens.tolist()):
            h.update(mv[o:o + L + 16])
    assert h.hexdigest() == g[cfg]["sha256_sealed"]
