"""The oracle's WireGuard transport framing (oracle/wg.c) and replay window.

wireguard-go is not in the reference tree, so no golden vector of the
reference covers these functions (they stay "parity unpinned").  What can be
fixed without it is fixed here: the datagram layout against the protocol
paper's field list, the AEAD inside it against the independent big-integer
RFC 8439 transcription, every rejection class, and the replay window against a
brute-force model plus WireGuard's published counter self-test sequence
(tests/cpp/replay_test.cpp).
"""
import os
import struct
import subprocess

import numpy as np
import pytest

from oracle import binding as ob
from tests import rfc8439_py as rfc
from bnk_amd import workloads as wl

HERE = os.path.dirname(os.path.abspath(__file__))



def udp(src, dst, sport, dport, payload=b""):
    hdr = sport.to_bytes(2, "big") + dport.to_bytes(2, "big") + (8 + len(payload)).to_bytes(2, "big") + b"\0\0"
    return wl.ipv4(17, src, dst, hdr + payload)


KEY = bytes(range(32))
KEYS = np.frombuffer(bytes(range(32)) + bytes(range(100, 132)), np.uint8).reshape(2, 32).copy()
# (local_index, remote_index, allowed_net, allowed_mask)
PEERS = [(0x11111111, 0xAAAA0001, 0x64400001, 0xFFFFFFFF),
         (0x22222222, 0xAAAA0002, 0x64400100, 0xFFFFFF00)]


@pytest.mark.parametrize("length,mtu,pad", [
    (0, 1420, 0), (1, 1420, 15), (15, 1420, 1), (16, 1420, 0), (17, 1420, 15),
    (1408, 1420, 0), (1409, 1420, 11), (1419, 1420, 1), (1420, 1420, 0),
    (1421, 1420, 15),      # longer than the MTU: only the remainder is padded
    (2840, 1420, 0), (100, 0, 12), (1419, 0, 5), (30, 20, 6), (17, 20, 3),
])
def test_padding_table(length, mtu, pad):
    assert ob.wg_padding(length, mtu) == pad
    if mtu and length <= mtu:
        assert (length + pad) % 16 == 0 or length + pad == mtu


def test_encap_layout_and_aead():
    pt = udp(0x64400001, 0x64400002, 1000, 2000, b"hello wireguard")  # 43 bytes
    wire = ob.wg_encap(pt, 1420, KEY, 0xAAAA0001, 7)
    pad = (-len(pt)) % 16
    assert len(wire) == 16 + len(pt) + pad + 16
    assert wire[:4] == b"\x04\x00\x00\x00"
    assert wire[4:8] == struct.pack("<I", 0xAAAA0001)
    assert wire[8:16] == struct.pack("<Q", 7)
    assert wire[16:] == rfc.aead_seal(KEY, rfc.wg_nonce(7), pt + bytes(pad))


def test_keepalive_is_32_bytes():
    wire = ob.wg_encap(b"", 1420, KEY, 5, 0)
    assert len(wire) == 32
    assert wire[16:] == rfc.aead_seal(KEY, rfc.wg_nonce(0), b"")
    rc, out, peer, ctr = ob.wg_decap(wire[:4] + struct.pack("<I", PEERS[0][0]) + wire[8:], PEERS,
                                     KEYS)
    assert (rc, out, peer, ctr) == (ob.WG_KEEPALIVE, b"", 0, 0)


def _wire(pt, peer=0, counter=3, mtu=1420):
    """As the remote peer would send it to us: our local index in the header."""
    w = ob.wg_encap(pt, mtu, KEYS[peer].tobytes(), PEERS[peer][0], counter)
    return w


def test_decap_round_trip_trims_padding():
    pt = udp(0x64400001, 0x0A000001, 1, 2, b"x" * 5)  # 33 bytes -> 15 bytes of padding
    rc, out, peer, ctr = ob.wg_decap(_wire(pt, counter=99), PEERS, KEYS)
    assert (rc, out, peer, ctr) == (ob.WG_OK, pt, 0, 99)
    pt2 = wl.tcp(0x644001FE, 0x0A000001, 1, 2)  # inside peer 1's /24
    rc, out, peer, ctr = ob.wg_decap(_wire(pt2, peer=1, counter=2 ** 40), PEERS, KEYS)
    assert (rc, out, peer, ctr) == (ob.WG_OK, pt2, 1, 2 ** 40)


def test_decap_rejections():
    pt = udp(0x64400001, 0x0A000001, 1, 2, b"payload")
    good = _wire(pt)
    assert ob.wg_decap(good[:31], PEERS, KEYS)[0] == ob.WG_BAD_HEADER
    assert ob.wg_decap(b"", PEERS, KEYS)[0] == ob.WG_BAD_HEADER
    for t in (1, 2, 3, 5, 0x04000000, 0x104):
        assert ob.wg_decap(struct.pack("<I", t) + good[4:], PEERS, KEYS)[0] == ob.WG_BAD_HEADER
    rc, _, peer, _ = ob.wg_decap(good[:4] + struct.pack("<I", 0x33333333) + good[8:], PEERS, KEYS)
    assert (rc, peer) == (ob.WG_UNKNOWN_INDEX, 0xFFFFFFFF)
    # any flipped bit after the index fails authentication: counter, body, tag
    for pos in (8, 15, 16, 40, len(good) - 1):
        bad = bytearray(good)
        bad[pos] ^= 0x20
        rc, out, peer, _ = ob.wg_decap(bytes(bad), PEERS, KEYS)
        assert (rc, out, peer) == (ob.WG_AUTH_FAIL, b"", 0)
    # right peer's key, wrong peer's index
    assert ob.wg_decap(good[:4] + struct.pack("<I", PEERS[1][0]) + good[8:], PEERS, KEYS)[0] == \
        ob.WG_AUTH_FAIL
    # inner source is not the peer's allowed address
    spoof = udp(0x64400002, 0x0A000001, 1, 2, b"payload")
    assert ob.wg_decap(_wire(spoof), PEERS, KEYS)[0] == ob.WG_NOT_ALLOWED
    assert ob.wg_decap(_wire(wl.tcp(0x64400200, 1, 1, 2), peer=1), PEERS, KEYS)[0] == ob.WG_NOT_ALLOWED


def test_decap_ip_checks():
    base = bytearray(udp(0x64400001, 0x0A000001, 1, 2, b"0123456789"))
    v5 = bytearray(base); v5[0] = 0x55
    assert ob.wg_decap(_wire(bytes(v5)), PEERS, KEYS)[0] == ob.WG_BAD_IP
    long_ = bytearray(base); long_[2:4] = struct.pack(">H", len(base) + 16)  # beyond even the padding
    assert ob.wg_decap(_wire(bytes(long_)), PEERS, KEYS)[0] == ob.WG_BAD_IP
    tiny = bytearray(base); tiny[2:4] = struct.pack(">H", 19)
    assert ob.wg_decap(_wire(bytes(tiny)), PEERS, KEYS)[0] == ob.WG_BAD_IP
    assert ob.wg_decap(_wire(bytes(base[:16])), PEERS, KEYS)[0] == ob.WG_BAD_IP  # 16 < 20
    # a total length below the real one is a trim, not an error
    short = bytearray(base); short[2:4] = struct.pack(">H", 24)
    rc, out, _, _ = ob.wg_decap(_wire(bytes(short)), PEERS, KEYS)
    assert rc == ob.WG_OK and out == bytes(short[:24])
    # IPv6: well-formed is refused by the allowed-IP table, malformed as bad IP
    v6 = bytearray(48); v6[0] = 0x60; v6[4:6] = struct.pack(">H", 8)
    assert ob.wg_decap(_wire(bytes(v6)), PEERS, KEYS)[0] == ob.WG_NOT_ALLOWED
    v6[4:6] = struct.pack(">H", 9)
    assert ob.wg_decap(_wire(bytes(v6)), PEERS, KEYS)[0] == ob.WG_BAD_IP
    assert ob.wg_decap(_wire(bytes(v6[:32])), PEERS, KEYS)[0] == ob.WG_BAD_IP


def test_replay_window_python_model():
    f = ob.ReplayFilter()
    assert f.validate(5) and not f.validate(5)
    assert f.validate(5 + 8128 + 1) and not f.validate(5)  # slid out of the window
    assert f.validate(6)                                   # exactly 8128 behind: still in
    assert not f.validate(100, limit=100) and f.validate(99, limit=100)


def test_replay_window_against_model_and_selftest():
    subprocess.run(["make", "-s", "-C", os.path.join(HERE, "..", "oracle")], check=True)
    subprocess.run(["make", "-s", "-C", os.path.join(HERE, "cpp"), "replay_test"], check=True)
    r = subprocess.run([os.path.join(HERE, "cpp", "replay_test")], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
