"""Seeded synthetic inputs for the benchmark configurations.

Every generator is a pure function of (configuration number, size): the same
bytes come out on every machine, so the GPU path, the CPU checker and the
committed golden fixtures all see identical inputs.  The byte source is
SplitMix64 run in counter mode (output k is mix(seed + k * golden)), which
vectorises in numpy.

Packet construction follows the reference's own test helpers
(internal/filter/filter_test.go:13-54: 20-byte IPv4 header 0x45, total length,
TTL 64, protocol, addresses; TCP 20-byte header; UDP 8-byte header; ICMP
8-byte echo).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

MASTER_SEED = 0x626E6B2026  # "bnk " .. 0x2026
T0_NS = 1_700_000_000 * 1_000_000_000  # filter_test.go:60
TAG = 16

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def splitmix64(seed: int, n: int, start: int = 0) -> np.ndarray:
    """Outputs start+1 .. start+n of SplitMix64 seeded with ``seed``."""
    with np.errstate(over="ignore"):
        z = np.arange(start + 1, start + n + 1, dtype=np.uint64)
        z *= _GOLDEN
        z += np.uint64(seed & 0xFFFFFFFFFFFFFFFF)
        t = z >> np.uint64(30)
        z ^= t
        z *= _M1
        np.right_shift(z, np.uint64(27), out=t)
        z ^= t
        z *= _M2
        np.right_shift(z, np.uint64(31), out=t)
        z ^= t
        return z


def stream_seed(cfg: int, stream: int) -> int:
    """Independent sub-seed for stream ``stream`` of configuration ``cfg``."""
    return int(splitmix64(MASTER_SEED ^ cfg, 1, start=stream)[0])


def rand_bytes(seed: int, nbytes: int) -> np.ndarray:
    words = splitmix64(seed, (nbytes + 7) // 8)
    return words.view(np.uint8)[:nbytes]


def rand_bytes_torch(seed: int, nbytes: int, device):
    """Same bytes as rand_bytes, produced by torch on ``device`` (int64
    arithmetic wraps like uint64; right shifts are made logical by masking)."""
    import torch
    n = (nbytes + 7) // 8

    def lsr(z, s):
        return (z >> s) & ((1 << (64 - s)) - 1)

    def s64(v):  # Python int -> the int64 with the same 64-bit pattern
        v &= 0xFFFFFFFFFFFFFFFF
        return v - (1 << 64) if v >= (1 << 63) else v

    k = torch.arange(1, n + 1, dtype=torch.int64, device=device)
    z = k * s64(0x9E3779B97F4A7C15) + s64(seed)
    z = (z ^ lsr(z, 30)) * s64(0xBF58476D1CE4E5B9)
    z = (z ^ lsr(z, 27)) * s64(0x94D049BB133111EB)
    z = z ^ lsr(z, 31)
    return z.view(torch.uint8)[:nbytes]


def aead_uniform_torch(cfg: int, n: int, length: int, stride: int, device):
    """The plaintext arena of aead_uniform(cfg, n, length, stride) as a torch
    uint8 tensor [n, stride] on ``device``, byte for byte."""
    import torch
    plain = torch.zeros((n, stride), dtype=torch.uint8, device=device)
    plain[:, :length] = rand_bytes_torch(stream_seed(cfg, 1), n * length, device).view(n, length)
    return plain


def rand_u64(seed: int, n: int) -> np.ndarray:
    return splitmix64(seed, n)


def rand_below(seed: int, n: int, bound: int) -> np.ndarray:
    """Uniform integers in [0, bound) (multiply-shift on the top 32 bits)."""
    hi = splitmix64(seed, n) >> np.uint64(32)
    return ((hi * np.uint64(bound)) >> np.uint64(32)).astype(np.uint32)


def permutation(seed: int, n: int) -> np.ndarray:
    """Seeded shuffle: order of n distinct SplitMix64 draws (stable sort)."""
    return np.argsort(splitmix64(seed, n), kind="stable").astype(np.uint32)


def align_up(x: int, a: int) -> int:
    return (x + a - 1) // a * a


# --------------------------------------------------------------------------
# AEAD batches
# --------------------------------------------------------------------------

@dataclass
class AeadBatch:
    """A batch of transport payloads laid out in one arena.

    Packet i's plaintext is ``plain[off[i] : off[i] + lens[i]]``; the sealed
    form occupies ``lens[i] + 16`` bytes at the same offset of a second arena
    of the same size (every slot leaves room for the tag).
    """
    keys: np.ndarray       # [n_peers, 32] u8
    peer: np.ndarray       # [n] u32
    counters: np.ndarray   # [n] u64
    lens: np.ndarray       # [n] u32 plaintext lengths
    off: np.ndarray        # [n] u64 slot offsets
    plain: np.ndarray      # arena, u8
    stride: int = 0        # nonzero when slots are uniform
    meta: dict = field(default_factory=dict)

    @property
    def n(self) -> int:
        return int(self.lens.shape[0])

    @property
    def arena_bytes(self) -> int:
        return int(self.plain.shape[0]) if self.plain is not None else int(self.meta["total"])


def aead_uniform(cfg: int, n: int, length: int = 1420, stride: int | None = None,
                 counter0: int = 0) -> AeadBatch:
    """Configurations 1 and 2: one peer key, ``n`` payloads of ``length``
    uniform-random bytes, counters counter0 .. counter0+n-1, packet slots at a
    16-byte-aligned stride."""
    if stride is None:
        stride = align_up(length + TAG, 16)
    keys = rand_bytes(stream_seed(cfg, 0), 32).reshape(1, 32)
    plain = np.zeros(n * stride, np.uint8)
    body = rand_bytes(stream_seed(cfg, 1), n * length).reshape(n, length)
    plain.reshape(n, stride)[:, :length] = body
    return AeadBatch(
        keys=keys,
        peer=np.zeros(n, np.uint32),
        counters=np.arange(counter0, counter0 + n, dtype=np.uint64),
        lens=np.full(n, length, np.uint32),
        off=np.arange(n, dtype=np.uint64) * np.uint64(stride),
        plain=plain, stride=stride,
        meta={"cfg": cfg, "length": length})


IMIX_SIZES = (60, 576, 1420)
_IMIX_PATTERN = np.array([60] * 7 + [576] * 4 + [1420], np.uint32)


def imix_lengths(seed: int, n: int) -> np.ndarray:
    """Sizes 60/576/1420 in a 7:4:1 ratio (index mod 12), seeded shuffle."""
    base = _IMIX_PATTERN[np.arange(n) % 12]
    return base[permutation(seed, n)]


def per_peer_sequence(peer: np.ndarray, n_peers: int) -> np.ndarray:
    """seq[i] = number of earlier packets in the batch with the same peer."""
    order = np.argsort(peer, kind="stable")
    sorted_peer = peer[order]
    start = np.searchsorted(sorted_peer, np.arange(n_peers, dtype=peer.dtype))
    rank_sorted = np.arange(peer.shape[0], dtype=np.uint64) - start[sorted_peer].astype(np.uint64)
    seq = np.empty(peer.shape[0], np.uint64)
    seq[order] = rank_sorted
    return seq


def _imix_slots(lens: np.ndarray, align: int) -> np.ndarray:
    a = np.uint64(align)
    return ((lens.astype(np.uint64) + np.uint64(TAG) + a - np.uint64(1)) // a) * a


def aead_imix(cfg: int, n: int, n_peers: int = 256, payload: bool = True,
              lens: np.ndarray | None = None, align: int = 16) -> AeadBatch:
    """Configuration 3 (and the AEAD half of 5): IMIX sizes, ``n_peers`` keys,
    per-peer counter = random base below 2^48 plus the per-peer sequence
    number; slots back to back, each starting at a multiple of ``align`` bytes
    (16: as tight as the kernels' fast path allows, packets share 128-byte
    lines; 128: every packet in lines of its own, as in a ring of buffers)."""
    if lens is None:
        lens = imix_lengths(stream_seed(cfg, 2), n)
    lens = lens.astype(np.uint32)
    keys = rand_bytes(stream_seed(cfg, 0), 32 * n_peers).reshape(n_peers, 32)
    peer = rand_below(stream_seed(cfg, 3), n, n_peers)
    base = rand_u64(stream_seed(cfg, 4), n_peers) >> np.uint64(16)
    counters = base[peer] + per_peer_sequence(peer, n_peers)
    slot = _imix_slots(lens, align)
    off = np.zeros(n, np.uint64)
    np.cumsum(slot[:-1], out=off[1:])
    total = int(off[-1] + slot[-1]) if n else 0
    plain = None
    if payload:
        # random fill of the whole arena, then clear the tag/pad gaps so the
        # arena content is a function of the packets only
        plain = rand_bytes(stream_seed(cfg, 1), total)
        gap = (slot - lens.astype(np.uint64)).astype(np.int64)
        end = (off + lens.astype(np.uint64)).astype(np.int64)
        for k in range(int(gap.max()) if n else 0):
            sel = gap > k
            plain[end[sel] + k] = 0
    return AeadBatch(keys=keys, peer=peer, counters=counters, lens=lens, off=off,
                     plain=plain, stride=0,
                     meta={"cfg": cfg, "n_peers": n_peers, "total": total, "align": align})


def imix_plain_torch(b: AeadBatch, device):
    """The arena aead_imix(..., payload=True) would hold, built by torch on
    ``device`` (for sizes where the numpy path takes too long)."""
    import torch
    total = b.meta["total"]
    plain = rand_bytes_torch(stream_seed(b.meta["cfg"], 1), total, device).clone()
    slot = _imix_slots(b.lens, b.meta.get("align", 16))
    gap = (slot - b.lens.astype(np.uint64)).astype(np.int64)
    end = (b.off + b.lens.astype(np.uint64)).astype(np.int64)
    for k in range(int(gap.max()) if b.n else 0):
        sel = gap > k
        plain[torch.from_numpy(end[sel] + k).to(device)] = 0
    return plain


def forge_tags(cfg: int, sealed: np.ndarray, off: np.ndarray, lens: np.ndarray,
               fraction: float) -> np.ndarray:
    """Flip one seeded bit in the tag of floor(fraction * n) seeded packets of
    the sealed arena (in place).  Returns the boolean mask of forged packets."""
    n = lens.shape[0]
    k = int(fraction * n)
    forged = np.zeros(n, bool)
    if k == 0:
        return forged
    which = permutation(stream_seed(cfg, 5), n)[:k]
    bit = rand_below(stream_seed(cfg, 6), k, 128)
    pos = off[which] + lens[which].astype(np.uint64) + (bit >> 3).astype(np.uint64)
    sealed[pos.astype(np.int64)] ^= (np.uint8(1) << (bit & 7).astype(np.uint8))
    forged[which] = True
    return forged


# --------------------------------------------------------------------------
# IPv4 packet construction (filter_test.go:13-54)
# --------------------------------------------------------------------------

def ip(s: str) -> int:
    a, b, c, d = (int(x) for x in s.split("."))
    return a << 24 | b << 16 | c << 8 | d


def ipv4(proto: int, src: int, dst: int, payload: bytes) -> bytes:
    pkt = bytearray(20 + len(payload))
    pkt[0] = 0x45
    pkt[2:4] = (len(pkt) & 0xFFFF).to_bytes(2, "big")
    pkt[8] = 64
    pkt[9] = proto
    pkt[12:16] = src.to_bytes(4, "big")
    pkt[16:20] = dst.to_bytes(4, "big")
    pkt[20:] = payload
    return bytes(pkt)


def tcp(src: int, dst: int, sport: int, dport: int, syn: bool = True) -> bytes:
    hdr = bytearray(20)
    hdr[0:2] = sport.to_bytes(2, "big")
    hdr[2:4] = dport.to_bytes(2, "big")
    hdr[12] = 5 << 4
    hdr[13] = 0x02 if syn else 0x10
    return ipv4(6, src, dst, bytes(hdr))


def udp(src: int, dst: int, sport: int, dport: int) -> bytes:
    hdr = bytearray(8)
    hdr[0:2] = sport.to_bytes(2, "big")
    hdr[2:4] = dport.to_bytes(2, "big")
    hdr[4:6] = (8).to_bytes(2, "big")
    return ipv4(17, src, dst, bytes(hdr))


def icmp_echo(src: int, dst: int, reply: bool = False) -> bytes:
    hdr = bytearray(8)
    hdr[0] = 0 if reply else 8
    return ipv4(1, src, dst, bytes(hdr))


# --------------------------------------------------------------------------
# ACL / conntrack workload (configuration 4)
# --------------------------------------------------------------------------

CGNAT_BASE = 100 << 24 | 64 << 16  # 100.64.0.0/10
RECORD_STRIDE = 32                 # 20-byte IPv4 header + 8 L4 bytes, padded to 32
_WELL_KNOWN = (80, 443, 22, 53, 25, 123, 8080, 3389, 5432, 3306, 6379, 8443, 21, 23, 110, 143)


def zipf_ports(seed: int, n: int, s: float = 1.1) -> np.ndarray:
    """Ports drawn from Zipf(s) over ranks 1..65535; rank 1.. map to the
    well-known ports above, the remaining ranks to a seeded permutation of all
    other ports."""
    ranks = np.arange(1, 65536, dtype=np.float64)
    cdf = np.cumsum(ranks ** (-s))
    cdf /= cdf[-1]
    u = (splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    r = np.searchsorted(cdf, u, side="left")
    rest = np.setdiff1d(np.arange(1, 65536, dtype=np.uint32), np.array(_WELL_KNOWN, np.uint32))
    rest = rest[permutation(seed ^ 0x5A5A, rest.shape[0])]
    table = np.concatenate([np.array(_WELL_KNOWN, np.uint32), rest])
    return table[np.minimum(r, table.shape[0] - 1)].astype(np.uint32)


def proto_mix(seed: int, n: int) -> np.ndarray:
    """TCP:UDP:ICMP = 6:3:1 as IP protocol numbers."""
    r = rand_below(seed, n, 10)
    return np.where(r < 6, 6, np.where(r < 9, 17, 1)).astype(np.uint32)


def header_records(proto: np.ndarray, src: np.ndarray, dst: np.ndarray, sport: np.ndarray,
                   dport: np.ndarray) -> np.ndarray:
    """[n, 32] u8 records: IPv4 header as filter_test.go:13-24 builds it (0x45,
    total length 28, TTL 64) followed by 8 L4 bytes (ports first for TCP/UDP;
    echo request type 8 for ICMP)."""
    n = proto.shape[0]
    rec = np.zeros((n, RECORD_STRIDE), np.uint8)
    rec[:, 0] = 0x45
    rec[:, 3] = 28
    rec[:, 8] = 64
    rec[:, 9] = proto
    for k in range(4):
        rec[:, 12 + k] = (src >> (24 - 8 * k)) & 0xFF
        rec[:, 16 + k] = (dst >> (24 - 8 * k)) & 0xFF
    l4 = proto != 1
    rec[l4, 20] = (sport[l4] >> 8) & 0xFF
    rec[l4, 21] = sport[l4] & 0xFF
    rec[l4, 22] = (dport[l4] >> 8) & 0xFF
    rec[l4, 23] = dport[l4] & 0xFF
    rec[~l4, 20] = 8
    return rec


@dataclass
class AclWorkload:
    rules_ref: list            # [(srcs, proto_name, ports)] in the reference's shape
    rule_tuples: np.ndarray    # [n_rules, 5] u32: net, mask, first, last, proto
    note_batches: list         # [(now_ns, records [m, 32] u8)] ascending in time
    check: np.ndarray          # [n, 32] u8 records
    now_ns: int
    record_len: int = 28


def acl_workload(cfg: int = 4, n: int = 1 << 22, n_rules: int = 4096, n_flows: int = 65536,
                 note_rounds: int = 16, mirror_fraction: float = 0.125) -> AclWorkload:
    """Configuration 4: ``n`` inbound headers against ``n_rules`` single-prefix
    single-range rules and a flow table built by ``n_flows`` earlier outbound
    packets noted at t0 - U[0, 150 s) (so some are expired at check time t0)."""
    ss = lambda k: stream_seed(cfg, k)  # noqa: E731
    # rules: prefix length uniform /16../32 under 100.64/10, proto 6:3:1, one
    # port range (half single ports, else geometric width)
    bits = 16 + rand_below(ss(10), n_rules, 17)
    host = rand_below(ss(11), n_rules, 1 << 22)
    mask = ((0xFFFFFFFF << (32 - bits.astype(np.uint64))) & 0xFFFFFFFF).astype(np.uint32)
    net = ((CGNAT_BASE | host) & mask).astype(np.uint32)
    rproto = proto_mix(ss(12), n_rules)
    first = zipf_ports(ss(13), n_rules)
    single = rand_below(ss(14), n_rules, 2) == 0
    u = (splitmix64(ss(15), n_rules) >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    width = np.where(single, 0, np.floor(np.log(np.maximum(u, 1e-12)) / np.log(0.99)).astype(np.int64))
    last = np.minimum(first.astype(np.int64) + width, 65535).astype(np.uint32)
    tuples = np.stack([net, mask, first, last, rproto], axis=1).astype(np.uint32)
    name = {6: "tcp", 17: "udp", 1: "icmp"}
    rules_ref = [([(int(net[i]), int(bits[i]))], name[int(rproto[i])],
                  [] if rproto[i] == 1 else [(int(first[i]), int(last[i]))]) for i in range(n_rules)]

    # earlier outbound traffic from this host
    self_addr = CGNAT_BASE | 1
    fproto = proto_mix(ss(20), n_flows)
    fdst = (CGNAT_BASE | rand_below(ss(21), n_flows, 1 << 22)).astype(np.uint32)
    fsport = (32768 + rand_below(ss(22), n_flows, 28000)).astype(np.uint32)
    fdport = zipf_ports(ss(23), n_flows)
    age_ns = (splitmix64(ss(24), n_flows) % np.uint64(150 * 1_000_000_000)).astype(np.int64)
    order = np.argsort(-age_ns, kind="stable")  # oldest first
    rec = header_records(fproto, np.full(n_flows, self_addr, np.uint32), fdst, fsport, fdport)
    note_batches = []
    for chunk in np.array_split(order, note_rounds):
        if chunk.shape[0] == 0:
            continue
        # one `now` per batch, as one tun.Read delivers: the batch's newest packet
        now = T0_NS - int(age_ns[chunk].min())
        note_batches.append((now, np.ascontiguousarray(rec[chunk])))

    # inbound headers to check at t0
    cproto = proto_mix(ss(30), n)
    csrc = (CGNAT_BASE | rand_below(ss(31), n, 1 << 22)).astype(np.uint32)
    cdst = np.full(n, self_addr, np.uint32)
    csport = zipf_ports(ss(32), n)
    cdport = zipf_ports(ss(33), n)
    # a seeded share of them are replies to recorded flows
    m = int(mirror_fraction * n)
    if m and n_flows:
        which = permutation(ss(34), n)[:m]
        pick = rand_below(ss(35), m, n_flows)
        cproto[which] = fproto[pick]
        csrc[which] = fdst[pick]
        csport[which] = fdport[pick]
        cdport[which] = fsport[pick]
    check = header_records(cproto, csrc, cdst, csport, cdport)
    return AclWorkload(rules_ref=rules_ref, rule_tuples=tuples, note_batches=note_batches,
                       check=check, now_ns=T0_NS)


# --------------------------------------------------------------------------
# Fused relay workload (configuration 5)
# --------------------------------------------------------------------------

@dataclass
class RelayWorkload:
    batch: AeadBatch           # inbound plaintexts (before sealing), keys = inbound keys
    keys_out: np.ndarray       # [n_peers, 32]
    peer_out: np.ndarray       # [n] u32
    ctr_base_out: np.ndarray   # [n_peers] u64
    rules_ref: list
    note_batch: tuple          # (now_ns, records) noted before the relay step
    denied: np.ndarray         # [n] bool: constructed to fail the filter
    flow_allowed: np.ndarray   # [n] bool: pass only through the flow table
    forged_fraction: float
    now_ns: int


def relay_workload(cfg: int = 5, n: int = 1 << 22, n_peers: int = 4096, n_rules: int = 4096,
                   forged_fraction: float = 0.005, denied_fraction: float = 0.05,
                   flow_fraction: float = 0.01, payload: bool = True, align: int = 16) -> RelayWorkload:
    """Configuration 5: IMIX packets whose plaintext starts with an IPv4 + L4
    header.  denied_fraction of them come from 10.0.0.0/8, which no rule
    covers; flow_fraction come from 10.0.0.0/8 too but answer a noted outbound
    flow; every other packet is built to match one seeded rule."""
    ss = lambda k: stream_seed(cfg, k)  # noqa: E731
    acl = acl_workload(cfg, n=1, n_rules=n_rules, n_flows=0)
    t = acl.rule_tuples
    b = aead_imix(cfg, n, n_peers=n_peers, payload=payload, align=align)
    pick = rand_below(ss(40), n, n_rules)
    net, mask, first, last, rproto = (t[pick, k] for k in range(5))
    r1 = splitmix64(ss(41), n)
    src = (net | ((r1 & np.uint64(0xFFFFFFFF)).astype(np.uint32) & ~mask)).astype(np.uint32)
    span = (last - first + 1).astype(np.uint64)
    dport = (first + ((r1 >> np.uint64(32)) % span).astype(np.uint32)).astype(np.uint32)
    sport = (1024 + rand_below(ss(42), n, 60000)).astype(np.uint32)
    proto = rproto.copy()
    order = permutation(ss(43), n)
    n_denied = int(denied_fraction * n)
    n_flow = int(flow_fraction * n)
    denied = np.zeros(n, bool)
    flow_allowed = np.zeros(n, bool)
    denied[order[:n_denied]] = True
    flow_allowed[order[n_denied:n_denied + n_flow]] = True
    outside = denied | flow_allowed
    ten = (10 << 24 | rand_below(ss(44), n, 1 << 24)).astype(np.uint32)
    src[outside] = ten[outside]
    # flow-admitted packets must not be ICMP duplicates of each other's keys;
    # give them tcp/udp and distinct port pairs
    proto[flow_allowed] = np.where(rand_below(ss(45), n, 2)[flow_allowed] == 0, 6, 17)
    self_addr = CGNAT_BASE | 1
    rec = header_records(proto, src, np.full(n, self_addr, np.uint32), sport, dport)
    # total length field = plaintext length (not looked at by the filter)
    rec[:, 2] = (b.lens >> 8) & 0xFF
    rec[:, 3] = b.lens & 0xFF
    if payload:
        off64 = b.off.astype(np.int64)
        for k in range(28):
            b.plain[off64 + k] = rec[:, k]
    # the outbound packets this host sent earlier, which the flow_allowed ones answer
    fa = np.flatnonzero(flow_allowed)
    note_rec = header_records(proto[fa], np.full(fa.shape[0], self_addr, np.uint32), src[fa],
                              dport[fa], sport[fa])
    keys_out = rand_bytes(ss(46), 32 * n_peers).reshape(n_peers, 32)
    peer_out = rand_below(ss(47), n, n_peers)
    ctr_base_out = rand_u64(ss(48), n_peers) >> np.uint64(16)
    b.meta["headers"] = rec
    return RelayWorkload(batch=b, keys_out=keys_out, peer_out=peer_out, ctr_base_out=ctr_base_out,
                         rules_ref=acl.rules_ref, note_batch=(T0_NS - 1_000_000_000, note_rec),
                         denied=denied, flow_allowed=flow_allowed,
                         forged_fraction=forged_fraction, now_ns=T0_NS)


def relay_forged_bits(w: RelayWorkload, cfg: int = 5):
    """Which packets of the relay's inbound traffic carry a forged tag, and
    how: (packet indices, byte position of the flipped bit in the sealed arena,
    the bit as a mask).  forged_fraction of the packets, one seeded bit of the
    16-byte tag each."""
    b = w.batch
    n = b.n
    k = int(w.forged_fraction * n)
    which = permutation(stream_seed(cfg, 5), n)[:k].astype(np.int64)
    bit = rand_below(stream_seed(cfg, 6), k, 128)
    pos = b.off[which].astype(np.int64) + b.lens[which].astype(np.int64) + (bit >> 3).astype(np.int64)
    return which, pos, (1 << (bit & 7)).astype(np.uint8)


def relay_plain_torch(w: RelayWorkload, device):
    """Plaintext arena of a relay_workload(..., payload=False), built on
    ``device``: the IMIX payload with each packet's 28 header bytes written in."""
    import torch
    plain = imix_plain_torch(w.batch, device)
    rec = torch.from_numpy(np.ascontiguousarray(w.batch.meta["headers"][:, :28])).to(device)
    off = torch.from_numpy(w.batch.off.astype(np.int64)).to(device)
    for k in range(28):
        plain[off + k] = rec[:, k]
    return plain
