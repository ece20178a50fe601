"""ctypes binding of the CPU oracle (oracle/libbnkoracle.so).

TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Imported only by tests/, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``,
and only as the checker.  ``bnk_amd`` never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# BNK_ORACLE_SO: another build of the same library (the sanitizer build, oracle/san/)
_SO = os.environ.get("BNK_ORACLE_SO") or os.path.join(_HERE, "libbnkoracle.so")


def build() -> str:
    """Compile the oracle with the Makefile beside this file."""
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _SO


def _load() -> C.CDLL:
    if not os.path.exists(_SO):
        build()
    return C.CDLL(_SO)


_lib = _load()

_u8p = C.POINTER(C.c_uint8)
_u32p = C.POINTER(C.c_uint32)
_u64p = C.POINTER(C.c_uint64)
_i64p = C.POINTER(C.c_int64)


def _p(a: np.ndarray | None, t):
    if a is None:
        return C.cast(None, t)
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(t)


def _b(x) -> np.ndarray:
    return np.frombuffer(bytes(x), dtype=np.uint8).copy()


# ---- RFC 8439 primitives -------------------------------------------------

def chacha20_block(key: bytes, counter: int, nonce: bytes) -> bytes:
    out = np.zeros(64, np.uint8)
    _lib.bnko_chacha20_block(_p(_b(key), _u8p), C.c_uint32(counter),
                             _p(_b(nonce), _u8p), _p(out, _u8p))
    return out.tobytes()


def chacha20_xor(key: bytes, counter: int, nonce: bytes, data: bytes) -> bytes:
    src = _b(data) if len(data) else np.zeros(1, np.uint8)
    out = np.zeros(max(len(data), 1), np.uint8)
    _lib.bnko_chacha20_xor(_p(_b(key), _u8p), C.c_uint32(counter),
                           _p(_b(nonce), _u8p), _p(src, _u8p), _p(out, _u8p),
                           C.c_size_t(len(data)))
    return out.tobytes()[:len(data)]


def poly1305(key: bytes, msg: bytes) -> bytes:
    src = _b(msg) if len(msg) else np.zeros(1, np.uint8)
    tag = np.zeros(16, np.uint8)
    _lib.bnko_poly1305(_p(_b(key), _u8p), _p(src, _u8p), C.c_size_t(len(msg)),
                       _p(tag, _u8p))
    return tag.tobytes()


def poly1305_keygen(key: bytes, nonce: bytes) -> bytes:
    out = np.zeros(32, np.uint8)
    _lib.bnko_poly1305_keygen(_p(_b(key), _u8p), _p(_b(nonce), _u8p),
                              _p(out, _u8p))
    return out.tobytes()


def aead_seal(key: bytes, nonce: bytes, pt: bytes, aad: bytes = b"") -> bytes:
    src = _b(pt) if len(pt) else np.zeros(1, np.uint8)
    a = _b(aad) if len(aad) else np.zeros(1, np.uint8)
    out = np.zeros(len(pt) + 16, np.uint8)
    _lib.bnko_aead_seal(_p(_b(key), _u8p), _p(_b(nonce), _u8p), _p(src, _u8p),
                        C.c_size_t(len(pt)), _p(a, _u8p),
                        C.c_size_t(len(aad)), _p(out, _u8p))
    return out.tobytes()


def aead_open(key: bytes, nonce: bytes, ct: bytes, aad: bytes = b""):
    """Returns (ok, plaintext bytes); plaintext is all zero when not ok."""
    src = _b(ct) if len(ct) else np.zeros(1, np.uint8)
    a = _b(aad) if len(aad) else np.zeros(1, np.uint8)
    out = np.full(max(len(ct) - 16, 1), 0xAA, np.uint8)
    _lib.bnko_aead_open.restype = C.c_int
    ok = _lib.bnko_aead_open(_p(_b(key), _u8p), _p(_b(nonce), _u8p),
                             _p(src, _u8p), C.c_size_t(len(ct)), _p(a, _u8p),
                             C.c_size_t(len(aad)), _p(out, _u8p))
    return bool(ok), out.tobytes()[:max(len(ct) - 16, 0)]


def wg_nonce(counter: int) -> bytes:
    out = np.zeros(12, np.uint8)
    _lib.bnko_wg_nonce(C.c_uint64(counter), _p(out, _u8p))
    return out.tobytes()


# ---- batched transport AEAD ---------------------------------------------

def seal_batch(keys, peer, counters, inbuf, in_off, in_len, out, out_off,
               nthreads: int = 1) -> None:
    n = len(in_len)
    _lib.bnko_seal_batch(_p(keys, _u8p), _p(peer, _u32p), _p(counters, _u64p),
                         _p(inbuf, _u8p), _p(in_off, _u64p), _p(in_len, _u32p),
                         _p(out, _u8p), _p(out_off, _u64p), C.c_uint32(n),
                         C.c_int(nthreads))


def open_batch(keys, peer, counters, inbuf, in_off, in_len, out, out_off,
               nthreads: int = 1) -> np.ndarray:
    n = len(in_len)
    verdict = np.zeros(n, np.uint8)
    _lib.bnko_open_batch(_p(keys, _u8p), _p(peer, _u32p), _p(counters, _u64p),
                         _p(inbuf, _u8p), _p(in_off, _u64p), _p(in_len, _u32p),
                         _p(out, _u8p), _p(out_off, _u64p), _p(verdict, _u8p),
                         C.c_uint32(n), C.c_int(nthreads))
    return verdict


# ---- filter --------------------------------------------------------------

class _Prefix(C.Structure):
    _fields_ = [("addr", C.c_uint32), ("bits", C.c_int32), ("is4", C.c_int32)]


class _PortRange(C.Structure):
    _fields_ = [("first", C.c_uint16), ("last", C.c_uint16)]


class _Rule(C.Structure):
    _fields_ = [("srcs", C.POINTER(_Prefix)), ("n_srcs", C.c_uint32),
                ("proto", C.c_char_p), ("ports", C.POINTER(_PortRange)),
                ("n_ports", C.c_uint32)]


class _Parsed(C.Structure):
    _fields_ = [("proto", C.c_uint8), ("src", C.c_uint32), ("dst", C.c_uint32),
                ("src_port", C.c_uint16), ("dst_port", C.c_uint16),
                ("proto_name", C.c_char_p), ("icmp_type", C.c_uint8)]


def _mk_rules(rules):
    """rules: iterable of (srcs, proto, ports); srcs = [(addr_u32, bits)] or
    [(addr_u32, bits, is4)], ports = [(first, last)]."""
    keep = []
    arr = (_Rule * max(len(rules), 1))()
    for i, (srcs, proto, ports) in enumerate(rules):
        ps = (_Prefix * max(len(srcs), 1))()
        for j, s in enumerate(srcs):
            ps[j].addr, ps[j].bits = s[0], s[1]
            ps[j].is4 = s[2] if len(s) > 2 else 1
        pr = (_PortRange * max(len(ports), 1))()
        for j, (a, b) in enumerate(ports):
            pr[j].first, pr[j].last = a, b
        pb = proto.encode() if isinstance(proto, str) else proto
        keep += [ps, pr, pb]
        arr[i].srcs, arr[i].n_srcs = ps, len(srcs)
        arr[i].proto = pb
        arr[i].ports, arr[i].n_ports = pr, len(ports)
    return arr, keep


def rule_match(rule, src: int, proto: str, dst_port: int) -> bool:
    arr, keep = _mk_rules([rule])
    _lib.bnko_rule_match.restype = C.c_int
    return bool(_lib.bnko_rule_match(C.byref(arr[0]), C.c_uint32(src),
                                     proto.encode(), C.c_uint16(dst_port)))


def parse(pkt: bytes):
    """Returns None or (proto, src, dst, src_port, dst_port, icmp_type)."""
    out = _Parsed()
    buf = _b(pkt) if len(pkt) else np.zeros(1, np.uint8)
    _lib.bnko_parse.restype = C.c_int
    ok = _lib.bnko_parse(_p(buf, _u8p), C.c_size_t(len(pkt)), C.byref(out))
    if not ok:
        return None
    return (out.proto, out.src, out.dst, out.src_port, out.dst_port,
            out.icmp_type)


class Filter:
    """Mirror of the reference's filter.Filter over the C oracle."""

    def __init__(self):
        _lib.bnko_filter_new.restype = C.c_void_p
        self._f = C.c_void_p(_lib.bnko_filter_new())

    def __del__(self):
        # (at interpreter exit the module's globals may be gone before the object is)
        if getattr(self, "_f", None) and _lib is not None:
            _lib.bnko_filter_free(self._f)
            self._f = None

    def set_rules(self, rules) -> None:
        arr, keep = _mk_rules(list(rules))
        _lib.bnko_filter_set_rules(self._f, arr, C.c_uint32(len(rules)))

    def set_allow_all(self) -> None:
        _lib.bnko_filter_set_allow_all(self._f)

    def check_inbound(self, pkt: bytes | None, now_ns: int) -> bool:
        pkt = pkt or b""
        buf = _b(pkt) if len(pkt) else np.zeros(1, np.uint8)
        _lib.bnko_filter_check_inbound.restype = C.c_int
        return bool(_lib.bnko_filter_check_inbound(
            self._f, _p(buf, _u8p), C.c_size_t(len(pkt)), C.c_int64(now_ns)))

    def note_outbound(self, pkt: bytes | None, now_ns: int) -> None:
        pkt = pkt or b""
        buf = _b(pkt) if len(pkt) else np.zeros(1, np.uint8)
        _lib.bnko_filter_note_outbound(self._f, _p(buf, _u8p),
                                       C.c_size_t(len(pkt)), C.c_int64(now_ns))

    def check_inbound_batch(self, pkts, off, lens, now_ns: int) -> np.ndarray:
        v = np.zeros(len(lens), np.uint8)
        _lib.bnko_filter_check_inbound_batch(
            self._f, _p(pkts, _u8p), _p(off, _u64p), _p(lens, _u32p),
            C.c_uint32(len(lens)), C.c_int64(now_ns), _p(v, _u8p))
        return v

    def note_outbound_batch(self, pkts, off, lens, now_ns: int) -> None:
        _lib.bnko_filter_note_outbound_batch(
            self._f, _p(pkts, _u8p), _p(off, _u64p), _p(lens, _u32p),
            C.c_uint32(len(lens)), C.c_int64(now_ns))

    def flow_count(self) -> int:
        _lib.bnko_filter_flow_count.restype = C.c_uint32
        return int(_lib.bnko_filter_flow_count(self._f))

    def flows(self) -> dict:
        """{(remote, remote_port, local_port, proto): expiry_ns}"""
        n = self.flow_count()
        key = np.zeros(max(n, 1), np.uint64)
        proto = np.zeros(max(n, 1), np.uint8)
        exp = np.zeros(max(n, 1), np.int64)
        _lib.bnko_filter_flow_dump.restype = C.c_uint32
        k = _lib.bnko_filter_flow_dump(self._f, _p(key, _u64p),
                                       _p(proto, _u8p), _p(exp, _i64p))
        out = {}
        for i in range(k):
            kk = int(key[i])
            out[(kk >> 32, (kk >> 16) & 0xFFFF, kk & 0xFFFF,
                 int(proto[i]))] = int(exp[i])
        return out

    def relay_fused_batch(self, keys_in, peer_in, ctr_in, keys_out, peer_out,
                          ctr_base_out, inbuf, in_off, in_len, out, out_off,
                          now_ns: int):
        n = len(in_len)
        verdict = np.zeros(n, np.uint8)
        ctr_out = np.zeros(n, np.uint64)
        _lib.bnko_relay_fused_batch(
            self._f, _p(keys_in, _u8p), _p(peer_in, _u32p), _p(ctr_in, _u64p),
            _p(keys_out, _u8p), _p(peer_out, _u32p), _p(ctr_base_out, _u64p),
            C.c_uint32(len(ctr_base_out)), _p(inbuf, _u8p), _p(in_off, _u64p),
            _p(in_len, _u32p), _p(out, _u8p), _p(out_off, _u64p),
            C.c_int64(now_ns), _p(verdict, _u8p), _p(ctr_out, _u64p),
            C.c_uint32(n))
        return verdict, ctr_out


# ---- WireGuard transport framing (parity unpinned: see bnk_oracle.h) -----

WG_OK, WG_KEEPALIVE, WG_BAD_HEADER, WG_UNKNOWN_INDEX, WG_AUTH_FAIL, WG_BAD_IP, \
    WG_NOT_ALLOWED = range(7)

_lib.bnko_wg_padding.restype = C.c_uint32
_lib.bnko_wg_encap.restype = C.c_uint32
_lib.bnko_wg_decap.restype = C.c_int
_lib.bnko_replay_validate.restype = C.c_int


def wg_padding(length: int, mtu: int) -> int:
    return int(_lib.bnko_wg_padding(C.c_uint32(length), C.c_uint32(mtu)))


def wg_encap(plain: bytes, mtu: int, key: bytes, remote_index: int, counter: int) -> bytes:
    """One transport datagram for `plain`."""
    slot = np.zeros(16 + len(plain) + 16 + 16, np.uint8)
    slot[16:16 + len(plain)] = np.frombuffer(plain, np.uint8)
    n = _lib.bnko_wg_encap(_p(slot, _u8p), C.c_uint32(len(plain)), C.c_uint32(mtu),
                           _p(_b(key), _u8p), C.c_uint32(remote_index), C.c_uint64(counter))
    return slot[:n].tobytes()


def _mk_wg_peers(peers) -> np.ndarray:
    """[(local_index, remote_index, allowed_net, allowed_mask)] -> u32[n, 4]"""
    return np.ascontiguousarray(np.array(peers, dtype=np.uint32).reshape(-1, 4))


def wg_decap(wire: bytes, peers, keys_recv: np.ndarray):
    """-> (result, plaintext bytes, peer, counter)"""
    pe = _mk_wg_peers(peers)
    src = _b(wire) if len(wire) else np.zeros(1, np.uint8)
    out = np.zeros(max(len(wire), 1), np.uint8)
    out_len = C.c_uint32()
    peer = C.c_uint32()
    counter = C.c_uint64()
    rc = _lib.bnko_wg_decap(_p(src, _u8p), C.c_uint32(len(wire)), C.c_void_p(pe.ctypes.data),
                            _p(np.ascontiguousarray(keys_recv).reshape(-1), _u8p),
                            C.c_uint32(pe.shape[0]), _p(out, _u8p), C.byref(out_len),
                            C.byref(peer), C.byref(counter))
    return int(rc), out[:out_len.value].tobytes(), int(peer.value), int(counter.value)


class ReplayFilter:
    """RFC 6479 window (bnko_replay)."""

    def __init__(self):
        self._s = np.zeros(129, np.uint64)
        _lib.bnko_replay_reset(C.c_void_p(self._s.ctypes.data))

    def reset(self) -> None:
        _lib.bnko_replay_reset(C.c_void_p(self._s.ctypes.data))

    def validate(self, counter: int, limit: int = (1 << 64) - (1 << 13) - 1) -> bool:
        return bool(_lib.bnko_replay_validate(C.c_void_p(self._s.ctypes.data),
                                              C.c_uint64(counter), C.c_uint64(limit)))


# ---- OpenSSL as a second CPU baseline ------------------------------------

def ossl_available() -> bool:
    return bool(_lib.bnko_ossl_available())


def ossl_seal_open_batch(keys, peer, counters, inbuf, off, lens, sealed, opened, nthreads: int) -> int:
    """EVP_chacha20_poly1305 seal then open of every packet; returns how many
    round trips verified."""
    _lib.bnko_ossl_seal_open_batch.restype = C.c_uint32
    return int(_lib.bnko_ossl_seal_open_batch(
        _p(keys, _u8p), _p(peer, _u32p), _p(counters, _u64p), _p(inbuf, _u8p), _p(off, _u64p),
        _p(lens, _u32p), _p(sealed, _u8p), _p(opened, _u8p), C.c_uint32(len(lens)),
        C.c_int(nthreads)))
