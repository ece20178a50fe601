"""ctypes binding of libbnkhip.so (the C ABI in include/bnkhip.h).

There is no fallback: if the shared library is missing or no gfx950 device is
present, loading or ``Context()`` raises.  Buffers may be numpy arrays (host
memory), torch tensors (host or device, by ``.data_ptr()``) or plain integer
device addresses.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# BNK_HIP_SO: another build of the same library (an experiment beside the in-tree one)
SO_PATH = os.environ.get("BNK_HIP_SO") or os.path.join(_HERE, "libbnkhip.so")

MEM_HOST, MEM_DEVICE = 0, 1
KEYS_SEND, KEYS_RECV = 0, 1
RELAY_OK, RELAY_FORGED, RELAY_DENIED = 0, 1, 2
E_INVAL, E_NODEV, E_HIP, E_NOMEM, E_RANGE, E_STATE = -1, -2, -3, -4, -5, -6
NOALLOC_MAX_PACKETS = 1 << 20
WG_REJECT_AFTER_MESSAGES = (1 << 64) - (1 << 13) - 1


class BnkError(RuntimeError):
    def __init__(self, code: int, text: str):
        super().__init__(f"libbnkhip error {code}: {text}")
        self.code = code


class Batch(C.Structure):
    """struct bnk_batch"""
    _fields_ = [("base", C.c_void_p), ("bytes", C.c_uint64), ("n", C.c_uint32),
                ("mem", C.c_uint32), ("offsets", C.c_void_p), ("stride", C.c_uint32),
                ("len", C.c_uint32), ("lens", C.c_void_p), ("peer", C.c_void_p),
                ("counters", C.c_void_p), ("counter0", C.c_uint64)]


WG_OK, WG_KEEPALIVE, WG_BAD_HEADER, WG_UNKNOWN_INDEX, WG_AUTH_FAIL, WG_BAD_IP, \
    WG_NOT_ALLOWED = range(7)
WG_FILTERED = 7
WG_REPLAY = 8


class Rule(C.Structure):
    """struct bnk_rule"""
    _fields_ = [("src_net", C.c_uint32), ("src_mask", C.c_uint32),
                ("port_first", C.c_uint16), ("port_last", C.c_uint16),
                ("proto", C.c_uint8), ("pad", C.c_uint8 * 3)]


class CoalesceStats(C.Structure):
    """struct bnk_coalesce_stats"""
    _fields_ = [(k, C.c_uint64) for k in ("calls", "packets", "batches", "largest_batch", "largest_callers",
                                          "full_windows", "timed_out", "retried", "gather_ns", "enqueue_ns",
                                          "wait_ns")]

    def as_dict(self) -> dict:
        return {k: int(getattr(self, k)) for k, _ in self._fields_}


class Counters(C.Structure):
    """struct bnk_counters"""
    _fields_ = [(k, C.c_uint64) for k in ("sealed", "opened", "rejected", "allowed", "denied", "delivered",
                                          "keepalive", "replayed", "bad_header", "unknown_index", "bad_ip",
                                          "not_allowed", "relayed")]

    def as_dict(self) -> dict:
        return {k: int(getattr(self, k)) for k, _ in self._fields_}


_lib = None


def load() -> C.CDLL:
    """Loads the HIP library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            raise FileNotFoundError(
                f"{SO_PATH} is missing: build it with `make -C bnk_amd/csrc` "
                "(or __graft_entry__.build()); there is no CPU fallback")
        lib = C.CDLL(SO_PATH)
        lib.bnk_last_error.restype = C.c_char_p
        lib.bnk_last_error.argtypes = [C.c_void_p]
        lib.bnk_stream.restype = C.c_void_p
        lib.bnk_stream.argtypes = [C.c_void_p]
        lib.bnk_shutdown.restype = None
        lib.bnk_shutdown.argtypes = [C.c_void_p]
        _lib = lib
    return _lib


def _ptr(x) -> int | None:
    if x is None:
        return None
    if isinstance(x, (int, np.integer)):
        return int(x)
    if isinstance(x, np.ndarray):
        assert x.flags["C_CONTIGUOUS"], "numpy buffers must be contiguous"
        return x.ctypes.data
    if hasattr(x, "data_ptr"):
        return int(x.data_ptr())
    raise TypeError(f"cannot take the address of {type(x)!r}")


def make_batch(base, nbytes: int, n: int, mem: int, *, offsets=None, stride: int = 0,
               length: int = 0, lens=None, peer=None, counters=None,
               counter0: int = 0) -> Batch:
    b = Batch()
    b.base = _ptr(base)
    b.bytes = nbytes
    b.n = n
    b.mem = mem
    b.offsets = _ptr(offsets)
    b.stride = stride
    b.len = length
    b.lens = _ptr(lens)
    b.peer = _ptr(peer)
    b.counters = _ptr(counters)
    b.counter0 = counter0
    b._keep = (base, offsets, lens, peer, counters)
    return b


def flatten_rules(rules) -> np.ndarray:
    """[(srcs, proto, ports)] in the reference's CompiledRule shape
    (internal/acl/acl.go:33-42) -> array of bnk_rule tuples, one per (prefix,
    port range) pair.  srcs = [(addr_u32, bits[, is4])], proto is the
    reference's string, ports = [(first, last)]."""
    out = []
    for srcs, proto, ports in rules:
        p = {"tcp": 6, "udp": 17, "icmp": 1}.get(proto)
        if p is None:
            continue  # acl.go:150: no parsed packet carries another name
        pr = [(0, 0)] if p == 1 else list(ports)  # acl.go:163-165 icmp ignores ports
        for s in srcs:
            addr, bits = s[0], s[1]
            is4 = s[2] if len(s) > 2 else 1
            if bits < 0 or bits > 32 or not is4:
                continue  # netip.Prefix.Contains is false for these
            mask = 0 if bits == 0 else (0xFFFFFFFF << (32 - bits)) & 0xFFFFFFFF
            for lo, hi in pr:
                out.append((addr & mask, mask, lo, hi, p))
    arr = (Rule * max(len(out), 1))()
    for i, (net, mask, lo, hi, p) in enumerate(out):
        arr[i].src_net, arr[i].src_mask = net, mask
        arr[i].port_first, arr[i].port_last, arr[i].proto = lo, hi, p
    return arr, len(out)


def rules_from_netmap_json(doc: str | bytes):
    """(filter_enabled, [(src_net, src_mask, first, last, proto)]) from a netmap
    JSON document; raises BnkError(E_INVAL) on a document Go would reject.
    Needs no GPU."""
    lib = load()
    raw = doc.encode() if isinstance(doc, str) else bytes(doc)
    n = C.c_uint32()
    en = C.c_int()
    err = C.create_string_buffer(256)
    cap = 64
    while True:
        arr = (Rule * cap)()
        rc = lib.bnk_rules_from_netmap_json(raw, C.c_size_t(len(raw)), arr, C.c_uint32(cap),
                                            C.byref(n), C.byref(en), err, C.c_size_t(256))
        if rc != 0:
            raise BnkError(rc, err.value.decode())
        if n.value <= cap:
            break
        cap = n.value
    return bool(en.value), [(arr[i].src_net, arr[i].src_mask, arr[i].port_first,
                             arr[i].port_last, arr[i].proto) for i in range(n.value)]


class Context:
    """One bnk_ctx: a GPU, a stream, key tables, a filter."""

    def __init__(self, device: int = 0):
        self._lib = load()
        h = C.c_void_p()
        rc = self._lib.bnk_init(C.c_int(device), C.byref(h))
        if rc != 0:
            raise BnkError(rc, (self._lib.bnk_last_error(None) or b"").decode())
        self._h = h

    def close(self) -> None:
        if getattr(self, "_h", None):
            self._lib.bnk_shutdown(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _chk(self, rc: int) -> None:
        if rc != 0:
            raise BnkError(rc, (self._lib.bnk_last_error(self._h) or b"").decode())

    # ---- memory ----
    @property
    def stream(self) -> int:
        return int(self._lib.bnk_stream(self._h) or 0)

    def sync(self) -> None:
        self._chk(self._lib.bnk_sync(self._h))

    def dev_alloc(self, nbytes: int) -> int:
        p = C.c_void_p()
        self._chk(self._lib.bnk_dev_alloc(self._h, C.c_size_t(nbytes), C.byref(p)))
        return int(p.value)

    def dev_free(self, ptr: int) -> None:
        self._chk(self._lib.bnk_dev_free(self._h, C.c_void_p(ptr)))

    def ring_alloc(self, nbytes: int) -> np.ndarray:
        """Pinned host ring as a numpy u8 view (free with ring_free)."""
        p = C.c_void_p()
        self._chk(self._lib.bnk_ring_alloc(self._h, C.c_size_t(nbytes), C.byref(p)))
        buf = (C.c_uint8 * nbytes).from_address(p.value)
        arr = np.frombuffer(buf, dtype=np.uint8)
        self._rings = getattr(self, "_rings", {})
        self._rings[arr.ctypes.data] = p.value
        return arr

    def set_coalesce(self, max_packets: int, max_wait_us: int = 30, expect_callers: int = 0) -> None:
        """Merging of small host calls from several threads into one batch
        (max_packets 0: off).  Results per call are unchanged."""
        self._chk(self._lib.bnk_set_coalesce(self._h, C.c_uint32(max_packets), C.c_uint32(max_wait_us),
                                             C.c_uint32(expect_callers)))

    def coalesce_stats(self) -> dict:
        st = CoalesceStats()
        self._chk(self._lib.bnk_coalesce_stats_get(self._h, C.byref(st)))
        return st.as_dict()

    def counters(self) -> dict:
        """Packets by outcome since the context was made or the counters were reset."""
        c = Counters()
        self._chk(self._lib.bnk_counters_get(self._h, C.byref(c)))
        return c.as_dict()

    def counters_reset(self) -> None:
        self._chk(self._lib.bnk_counters_reset(self._h))

    def counters_enable(self, on: bool) -> None:
        self._chk(self._lib.bnk_counters_enable(self._h, C.c_int(1 if on else 0)))

    def set_spread_max_packets(self, max_packets: int) -> None:
        """Batches of at most this many packets run one wave per packet
        (0: always one lane per packet).  A tuning knob, results are the same."""
        self._chk(self._lib.bnk_set_spread_max_packets(self._h, C.c_uint32(max_packets)))

    def ring_free(self, arr: np.ndarray) -> None:
        p = self._rings.pop(arr.ctypes.data)
        self._chk(self._lib.bnk_ring_free(self._h, C.c_void_p(p)))

    def to_device(self, dev_ptr: int, host: np.ndarray) -> None:
        self._chk(self._lib.bnk_copy_to_device(self._h, C.c_void_p(dev_ptr),
                                               C.c_void_p(host.ctypes.data),
                                               C.c_size_t(host.nbytes)))

    def to_host(self, host: np.ndarray, dev_ptr: int) -> None:
        self._chk(self._lib.bnk_copy_to_host(self._h, C.c_void_p(host.ctypes.data),
                                             C.c_void_p(dev_ptr), C.c_size_t(host.nbytes)))

    def upload(self, host: np.ndarray) -> int:
        host = np.ascontiguousarray(host)
        p = self.dev_alloc(max(host.nbytes, 16))
        if host.nbytes:
            self.to_device(p, host)
        return p

    # ---- AEAD ----
    def keys_set(self, which: int, keys: np.ndarray) -> None:
        keys = np.ascontiguousarray(keys, dtype=np.uint8).reshape(-1, 32)
        self._chk(self._lib.bnk_keys_set(self._h, C.c_int(which), C.c_void_p(keys.ctypes.data),
                                         C.c_uint32(keys.shape[0])))

    def seal(self, inb: Batch, outb: Batch) -> None:
        self._chk(self._lib.bnk_aead_seal_batch(self._h, C.byref(inb), C.byref(outb)))

    def seal_noalloc(self, inb: Batch, outb: Batch) -> None:
        """bnk_aead_seal_batch_noalloc: device batches only, allocates nothing."""
        self._chk(self._lib.bnk_aead_seal_batch_noalloc(self._h, C.byref(inb), C.byref(outb)))

    def open(self, inb: Batch, outb: Batch, verdict) -> None:
        self._chk(self._lib.bnk_aead_open_batch(self._h, C.byref(inb), C.byref(outb),
                                                C.c_void_p(_ptr(verdict))))

    # ---- filter ----
    def filter_set_rules(self, rules) -> None:
        """rules: the reference's CompiledRule shape, see flatten_rules."""
        arr, n = flatten_rules(rules)
        self._chk(self._lib.bnk_filter_set_rules(self._h, arr, C.c_uint32(n)))

    def filter_set_rule_tuples(self, arr, n: int) -> None:
        self._chk(self._lib.bnk_filter_set_rules(self._h, arr, C.c_uint32(n)))

    def filter_apply_netmap_json(self, doc: str | bytes) -> None:
        raw = doc.encode() if isinstance(doc, str) else bytes(doc)
        self._chk(self._lib.bnk_filter_apply_netmap_json(self._h, raw, C.c_size_t(len(raw))))

    def filter_set_allow_all(self) -> None:
        self._chk(self._lib.bnk_filter_set_allow_all(self._h))

    def filter_note_outbound(self, pkts: Batch, now_ns: int) -> None:
        self._chk(self._lib.bnk_filter_note_outbound_batch(self._h, C.byref(pkts),
                                                           C.c_int64(now_ns)))

    def filter_check_inbound(self, pkts: Batch, now_ns: int, verdict) -> None:
        self._chk(self._lib.bnk_filter_check_inbound_batch(
            self._h, C.byref(pkts), C.c_int64(now_ns), C.c_void_p(_ptr(verdict))))

    def _ptr_list(self, pkts):
        n = len(pkts)
        bufs = [np.frombuffer(p, np.uint8) if len(p) else np.zeros(1, np.uint8) for p in pkts]
        ptrs = (C.c_void_p * max(n, 1))(*[b.ctypes.data for b in bufs])
        lens = np.array([len(p) for p in pkts], np.uint32)
        return bufs, ptrs, lens

    def filter_note_outbound_ptrs(self, pkts, now_ns: int) -> None:
        bufs, ptrs, lens = self._ptr_list(pkts)
        self._chk(self._lib.bnk_filter_note_outbound_ptrs(
            self._h, ptrs, C.c_void_p(lens.ctypes.data), C.c_uint32(len(pkts)),
            C.c_int64(now_ns)))

    def filter_check_inbound_ptrs(self, pkts, now_ns: int) -> np.ndarray:
        bufs, ptrs, lens = self._ptr_list(pkts)
        v = np.zeros(max(len(pkts), 1), np.uint8)
        self._chk(self._lib.bnk_filter_check_inbound_ptrs(
            self._h, ptrs, C.c_void_p(lens.ctypes.data), C.c_uint32(len(pkts)),
            C.c_int64(now_ns), C.c_void_p(v.ctypes.data)))
        return v[:len(pkts)]

    def filter_flow_count(self) -> int:
        c = C.c_uint32()
        self._chk(self._lib.bnk_filter_flow_count(self._h, C.byref(c)))
        return int(c.value)

    def filter_flows(self) -> dict:
        """{(remote, remote_port, local_port, proto): expiry_ns}"""
        cap = self.filter_flow_count() + 16
        key = np.zeros(cap, np.uint64)
        proto = np.zeros(cap, np.uint8)
        exp = np.zeros(cap, np.int64)
        c = C.c_uint32()
        self._chk(self._lib.bnk_filter_flow_dump(
            self._h, C.c_void_p(key.ctypes.data), C.c_void_p(proto.ctypes.data),
            C.c_void_p(exp.ctypes.data), C.c_uint32(cap), C.byref(c)))
        out = {}
        for i in range(c.value):
            k = int(key[i])
            out[(k >> 32, (k >> 16) & 0xFFFF, k & 0xFFFF, int(proto[i]))] = int(exp[i])
        return out

    # ---- fused relay ----
    def relay_fused(self, inb: Batch, peer_out, ctr_base_out, n_peers_out: int, now_ns: int,
                    outb: Batch, verdict, ctr_out) -> None:
        self._chk(self._lib.bnk_relay_fused_batch(
            self._h, C.byref(inb), C.c_void_p(_ptr(peer_out)), C.c_void_p(_ptr(ctr_base_out)),
            C.c_uint32(n_peers_out), C.c_int64(now_ns), C.byref(outb),
            C.c_void_p(_ptr(verdict)), C.c_void_p(_ptr(ctr_out))))

    # ---- WireGuard transport framing ----
    def wg_peers_set(self, peers) -> None:
        """peers: [(local_index, remote_index, allowed_net, allowed_mask)]"""
        arr = np.ascontiguousarray(np.array(peers, dtype=np.uint32).reshape(-1, 4))
        self._chk(self._lib.bnk_wg_peers_set(self._h, C.c_void_p(arr.ctypes.data),
                                             C.c_uint32(arr.shape[0])))

    def wg_peer_set(self, row: int, peer, key_send=None, key_recv=None) -> None:
        """One peer's new keypair: replaces row `row` (peer table and both key
        tables) and restarts only that row's send counter."""
        arr = np.ascontiguousarray(np.array(peer, dtype=np.uint32).reshape(4))
        ks = None if key_send is None else np.ascontiguousarray(key_send, dtype=np.uint8).reshape(32)
        kr = None if key_recv is None else np.ascontiguousarray(key_recv, dtype=np.uint8).reshape(32)
        self._chk(self._lib.bnk_wg_peer_set(self._h, C.c_uint32(row), C.c_void_p(arr.ctypes.data),
                                            C.c_void_p(_ptr(ks)), C.c_void_p(_ptr(kr))))

    def wg_send_counter_set(self, row: int, value: int) -> None:
        self._chk(self._lib.bnk_wg_send_counter_set(self._h, C.c_uint32(row), C.c_uint64(value)))

    def wg_set_replay(self, on: bool) -> None:
        """Anti-replay windows on (default) or off for the decapsulating calls."""
        self._chk(self._lib.bnk_wg_set_replay(self._h, C.c_int(1 if on else 0)))

    def wg_set_fused(self, on: bool) -> None:
        """Framing of large batches inside the AEAD launch (default) or in kernels of its own."""
        self._chk(self._lib.bnk_wg_set_fused(self._h, C.c_int(1 if on else 0)))

    def wg_send_counters(self, n: int) -> np.ndarray:
        out = np.zeros(max(n, 1), np.uint64)
        self._chk(self._lib.bnk_wg_send_counters(self._h, C.c_void_p(out.ctypes.data),
                                                 C.c_uint32(n)))
        return out[:n]

    def wg_encap(self, slots: Batch, mtu: int, wire_len) -> None:
        self._chk(self._lib.bnk_wg_encap_batch(self._h, C.byref(slots), C.c_uint32(mtu),
                                               C.c_void_p(_ptr(wire_len))))

    def wg_decap(self, wire: Batch, outb: Batch, result, out_len, peer, counter) -> None:
        self._chk(self._lib.bnk_wg_decap_batch(
            self._h, C.byref(wire), C.byref(outb), C.c_void_p(_ptr(result)),
            C.c_void_p(_ptr(out_len)), C.c_void_p(_ptr(peer)), C.c_void_p(_ptr(counter))))

    def wg_decap_filter(self, wire: Batch, outb: Batch, now_ns: int, result, out_len, peer,
                        counter) -> None:
        self._chk(self._lib.bnk_wg_decap_filter_batch(
            self._h, C.byref(wire), C.byref(outb), C.c_int64(now_ns), C.c_void_p(_ptr(result)),
            C.c_void_p(_ptr(out_len)), C.c_void_p(_ptr(peer)), C.c_void_p(_ptr(counter))))

    def wg_note_encap(self, slots: Batch, mtu: int, now_ns: int, wire_len) -> None:
        self._chk(self._lib.bnk_wg_note_encap_batch(self._h, C.byref(slots), C.c_uint32(mtu),
                                                    C.c_int64(now_ns), C.c_void_p(_ptr(wire_len))))


class HostFilter:
    """The reference's filter.Filter method set (internal/filter/filter.go:41-59,
    121, 189) over a Context, one packet per call."""

    def __init__(self, ctx: Context | None = None):
        self.ctx = ctx or Context()

    def set_rules(self, rules) -> None:
        self.ctx.filter_set_rules(rules)

    def set_allow_all(self) -> None:
        self.ctx.filter_set_allow_all()

    def check_inbound(self, pkt, now_ns: int) -> bool:
        return bool(self.ctx.filter_check_inbound_ptrs([pkt or b""], now_ns)[0])

    def note_outbound(self, pkt, now_ns: int) -> None:
        self.ctx.filter_note_outbound_ptrs([pkt or b""], now_ns)

    def flows(self) -> dict:
        return self.ctx.filter_flows()

    def flow_count(self) -> int:
        return self.ctx.filter_flow_count()
