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
        k = np.arange(start + 1, start + n + 1, dtype=np.uint64)
        z = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + k * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def stream_seed(cfg: int, stream: int) -> int:
    """Independent sub-seed for stream ``stream`` of configuration ``cfg``."""
    return int(splitmix64(MASTER_SEED ^ cfg, 1, start=stream)[0])


def rand_bytes(seed: int, nbytes: int) -> np.ndarray:
    words = splitmix64(seed, (nbytes + 7) // 8)
    return words.view(np.uint8)[:nbytes].copy()


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
        return int(self.plain.shape[0])


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


def aead_imix(cfg: int, n: int, n_peers: int = 256, payload: np.ndarray | None = None,
              lens: np.ndarray | None = None) -> AeadBatch:
    """Configuration 3 (and the AEAD half of 5): IMIX sizes, ``n_peers`` keys,
    per-peer counter = random base below 2^48 plus the per-peer sequence
    number; slots packed back to back at 16-byte alignment."""
    if lens is None:
        lens = imix_lengths(stream_seed(cfg, 2), n)
    lens = lens.astype(np.uint32)
    keys = rand_bytes(stream_seed(cfg, 0), 32 * n_peers).reshape(n_peers, 32)
    peer = rand_below(stream_seed(cfg, 3), n, n_peers)
    base = rand_u64(stream_seed(cfg, 4), n_peers) >> np.uint64(16)
    counters = base[peer] + per_peer_sequence(peer, n_peers)
    slot = ((lens.astype(np.uint64) + np.uint64(TAG + 15)) // np.uint64(16)) * np.uint64(16)
    off = np.zeros(n, np.uint64)
    np.cumsum(slot[:-1], out=off[1:])
    total = int(off[-1] + slot[-1]) if n else 0
    plain = np.zeros(total, np.uint8)
    if payload is None:
        # random fill of the whole arena, then clear the tag/pad gaps so the
        # arena content is a function of the packets only
        plain[:] = rand_bytes(stream_seed(cfg, 1), total)
        mark = np.zeros(total + 1, np.int32)
        np.add.at(mark, off.astype(np.int64), 1)
        np.add.at(mark, (off + lens.astype(np.uint64)).astype(np.int64), -1)
        inside = np.cumsum(mark)[:total] > 0
        plain[~inside] = 0
    else:
        plain[:] = payload
    return AeadBatch(keys=keys, peer=peer, counters=counters, lens=lens, off=off,
                     plain=plain, stride=0, meta={"cfg": cfg, "n_peers": n_peers})


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
