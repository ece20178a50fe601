"""WireGuard transport framing on the GPU (bnk_wg_encap_batch /
bnk_wg_decap_batch) against the oracle's per-packet definition: identical
datagrams, results, lengths, peers, counters and plaintext bytes.  The oracle's
framing itself is spec-derived (wireguard-go is not in the reference tree), so
this is parity with the restated protocol, not with a reference artefact."""
import struct

import numpy as np
import pytest

from bnk_amd import workloads as W

pytestmark = pytest.mark.gpu

N_PEERS = 37
MTU = 1420


def _peers(rng):
    local = rng.permutation(1 << 20)[:N_PEERS].astype(np.uint32) * 4099 + 17
    remote = rng.integers(0, 1 << 32, N_PEERS, dtype=np.uint64).astype(np.uint32)
    net = (0x64400000 + np.arange(N_PEERS, dtype=np.uint32) * 256 + 1).astype(np.uint32)
    mask = np.full(N_PEERS, 0xFFFFFFFF, np.uint32)
    mask[::5] = 0xFFFFFF00  # a few peers own a /24
    return [(int(a), int(b), int(c), int(d)) for a, b, c, d in zip(local, remote, net, mask)]


def _inner(rng, peers, p, length):
    """An IPv4 packet of `length` bytes from peer p's allowed address."""
    if length < 20:
        return bytes(length)  # too short for IPv4; version nibble 0
    pkt = bytearray(rng.integers(0, 256, length, dtype=np.uint8).tobytes())
    pkt[0] = 0x45
    pkt[2:4] = struct.pack(">H", length)
    pkt[12:16] = struct.pack(">I", peers[p][2])
    return bytes(pkt)


def _layout(rng, sizes, misalign=False):
    """Slot offsets: 16-aligned with random gaps, or arbitrary."""
    gaps = rng.integers(0, 5, len(sizes)) * 16
    off = np.zeros(len(sizes), np.uint64)
    pos = 0
    for i, s in enumerate(sizes):
        pos += int(gaps[i])
        if misalign:
            pos += int(rng.integers(0, 16))
        else:
            pos = (pos + 15) & ~15
        off[i] = pos
        pos += int(s)
    return off, pos + 64


def _ctx(peers, keys_send=None, keys_recv=None):
    from bnk_amd import lib
    ctx = lib.Context(0)
    if keys_send is not None:
        ctx.keys_set(lib.KEYS_SEND, keys_send)
    if keys_recv is not None:
        ctx.keys_set(lib.KEYS_RECV, keys_recv)
    ctx.wg_peers_set(peers)
    # these tests look at the framing alone and hand the same datagrams in more
    # than once; the anti-replay windows have tests/test_gpu_wg_replay.py
    ctx.wg_set_replay(False)
    return ctx


def _launch_shape(ctx, fused):
    """"wave": small batches take a wave per packet with the framing inside the
    AEAD launch (the default); "lane": every batch takes a lane per packet,
    framing inside as well; "separate": a lane per packet between framing
    kernels of their own."""
    if fused != "wave":
        ctx.set_spread_max_packets(0)
    if fused == "separate":
        ctx.wg_set_fused(False)


@pytest.mark.parametrize("mem", ["host", "ring", "device"])
@pytest.mark.parametrize("misalign", [False, True])
@pytest.mark.parametrize("n", [3000, 700])
@pytest.mark.parametrize("fused", ["wave", "lane", "separate"])
def test_encap_matches_oracle(mem, misalign, n, fused):
    """"ring": the slots lie in a pinned ring of the context, which small
    batches seal in place without staging copies.  700 packets also take the
    one-launch counter assignment, 3000 the sorted one.  fused: host batches
    this small are framed by the wave-per-packet AEAD launch itself; with the
    threshold at zero the framing kernels run around a lane-per-packet launch,
    as they do for large batches."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(11 + misalign)
    peers = _peers(rng)
    keys = rng.integers(0, 256, (N_PEERS, 32), dtype=np.uint8)
    lens = rng.choice([0, 1, 15, 16, 17, 20, 40, 63, 64, 65, 127, 128, 129, 576, 1399, 1408, 1419, 1420],
                      n).astype(np.uint32)
    lens[:200] = rng.integers(0, MTU + 1, 200)
    peer = rng.integers(0, N_PEERS, n).astype(np.uint32)
    room = 16 + lens.astype(np.int64) + 15 + 16
    off, total = _layout(rng, room, misalign)
    arena = np.full(total, 0xEE, np.uint8)
    plains = []
    for i in range(n):
        pt = _inner(rng, peers, int(peer[i]), int(lens[i]))
        plains.append(pt)
        arena[int(off[i]) + 16:int(off[i]) + 16 + len(pt)] = np.frombuffer(pt, np.uint8)
    ctx = _ctx(peers, keys_send=keys)
    _launch_shape(ctx, fused)
    next_ctr = np.zeros(N_PEERS, np.uint64)
    for round_ in range(2):  # the second batch continues the peers' counters
        want = arena.copy()
        want_len = np.zeros(n, np.uint32)
        for i in range(n):
            p = int(peer[i])
            w = O.wg_encap(plains[i], MTU, keys[p].tobytes(), peers[p][1], int(next_ctr[p]))
            next_ctr[p] += 1
            want[int(off[i]):int(off[i]) + len(w)] = np.frombuffer(w, np.uint8)
            want_len[i] = len(w)
        if mem == "host":
            got = arena.copy()
            got_len = np.zeros(n, np.uint32)
            ctx.wg_encap(lib.make_batch(got, got.nbytes, n, lib.MEM_HOST, offsets=off, lens=lens, peer=peer),
                         MTU, got_len)
        elif mem == "ring":
            ring = ctx.ring_alloc(arena.nbytes + 48)
            view = ring[48:]  # an arena that starts inside the ring
            view[:] = arena
            got_len = np.zeros(n, np.uint32)
            ctx.wg_encap(lib.make_batch(view, arena.nbytes, n, lib.MEM_HOST, offsets=off, lens=lens, peer=peer),
                         MTU, got_len)
            got = np.array(view)
            ctx.ring_free(ring)
        else:
            dev = torch.device("cuda:0")
            d_arena = torch.from_numpy(arena).to(dev)
            d_off = torch.from_numpy(off.astype(np.int64)).to(dev)
            d_lens = torch.from_numpy(lens.astype(np.int32)).to(dev)
            d_peer = torch.from_numpy(peer.astype(np.int32)).to(dev)
            d_wl = torch.zeros(n, dtype=torch.int32, device=dev)
            torch.cuda.synchronize()
            ctx.wg_encap(lib.make_batch(d_arena, d_arena.numel(), n, lib.MEM_DEVICE, offsets=d_off,
                                        lens=d_lens, peer=d_peer), MTU, d_wl)
            ctx.sync()
            got = d_arena.cpu().numpy()
            got_len = d_wl.cpu().numpy().astype(np.uint32)
        assert np.array_equal(got_len, want_len)
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, f"first differing byte at {bad[:5]}"  # gaps keep their 0xEE fill
        assert np.array_equal(ctx.wg_send_counters(N_PEERS), next_ctr)
    ctx.close()


@pytest.mark.parametrize("fused", ["wave", "lane", "separate"])
@pytest.mark.parametrize("length,mtu", [(100, 1420), (1500, 1420), (1413, 1420), (37, 0), (0, 1420), (2839, 1420)])
def test_encap_uniform_slots_one_peer_and_padding_rules(fused, length, mtu):
    """Uniform slots without length or peer arrays (everything goes to peer 0),
    and the padding rule at its corners: a packet longer than the MTU pads its
    remainder, one just below the MTU pads up to it and no further, mtu 0 means
    no cap, an empty packet is a keepalive."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(length * 7 + mtu)
    peers = _peers(rng)
    keys = rng.integers(0, 256, (N_PEERS, 32), dtype=np.uint8)
    n = 300
    stride = (16 + length + 15 + 16 + 15) & ~15
    arena = rng.integers(0, 256, n * stride, dtype=np.uint8)
    want = arena.copy()
    want_len = np.zeros(n, np.uint32)
    for i in range(n):
        pt = arena[i * stride + 16:i * stride + 16 + length].tobytes()
        w = O.wg_encap(pt, mtu, keys[0].tobytes(), peers[0][1], i)
        want[i * stride:i * stride + len(w)] = np.frombuffer(w, np.uint8)
        want_len[i] = len(w)
    assert want_len[0] == 32 + length + O.wg_padding(length, mtu)
    ctx = _ctx(peers, keys_send=keys)
    _launch_shape(ctx, fused)
    for mem in ("pageable", "ring"):
        ring = ctx.ring_alloc(arena.nbytes) if mem == "ring" else None
        got = ring if ring is not None else arena.copy()
        got[:] = arena
        got_len = np.zeros(n, np.uint32)
        ctx.wg_send_counter_set(0, 0)  # the same keypair from the start again (test only: reuses nonces)
        ctx.wg_encap(lib.make_batch(got, arena.nbytes, n, lib.MEM_HOST, stride=stride, length=length), mtu, got_len)
        assert np.array_equal(got_len, want_len), mem
        bad = np.flatnonzero(np.array(got) != want)
        assert bad.size == 0, f"{mem}: first differing byte at {bad[:5]}"
        if ring is not None:
            ctx.ring_free(ring)
    ctx.close()


@pytest.mark.parametrize("n_peers", [700, 5000])
def test_many_peers_counters_and_index_lookup(n_peers):
    """A peer table of hundreds and of thousands of rows, batches large enough for
    the lane-per-packet launches: send counters follow each peer's order in the
    batch (700 rows: counted per tile; 5000: beyond what that holds in LDS, so
    sorted), every datagram finds its sender through the hash form of the
    receiver-index map (indices chosen to collide), and an index nobody owns is
    told apart."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(n_peers)
    # local indices in a few clusters of consecutive numbers: long probe chains
    local = (np.repeat(rng.integers(0, 1 << 32, 8, dtype=np.uint64), (n_peers + 7) // 8)[:n_peers]
             + np.arange(n_peers, dtype=np.uint64) * 0x10000).astype(np.uint32)
    assert np.unique(local).size == n_peers
    remote = rng.integers(0, 1 << 32, n_peers, dtype=np.uint64).astype(np.uint32)
    net = (0x64400000 + np.arange(n_peers, dtype=np.uint32)).astype(np.uint32)
    peers = np.stack([local, remote, net, np.full(n_peers, 0xFFFFFFFF, np.uint32)], 1)
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    n, length, mtu = 9000, 44, 1420
    stride = 112
    peer = rng.integers(0, n_peers, n).astype(np.uint32)
    peer[:50] = 3  # a run of one peer
    arena = rng.integers(0, 256, n * stride, dtype=np.uint8)
    v = arena.reshape(n, stride)
    v[:, 16] = 0x45
    v[:, 18], v[:, 19] = length >> 8, length & 255
    for k in range(4):
        v[:, 16 + 12 + k] = (net[peer] >> (24 - 8 * k)) & 255
    plain = v[:, 16:16 + length].copy()
    ctx = lib.Context(0)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    # both ends in one table: what a peer expects in the header is what we look up
    peers[:, 1] = peers[:, 0]
    ctx.wg_peers_set(peers)
    ctx.set_spread_max_packets(0)
    wire_len = np.zeros(n, np.uint32)
    ctx.wg_encap(lib.make_batch(arena, arena.nbytes, n, lib.MEM_HOST, stride=stride, length=length, peer=peer),
                 mtu, wire_len)
    padded = length + O.wg_padding(length, mtu)
    assert (wire_len == 32 + padded).all()
    hdr = v[:, :16].copy().view(np.uint32).reshape(n, 4)
    assert (hdr[:, 0] == 4).all() and np.array_equal(hdr[:, 1], local[peer])
    got_ctr = hdr[:, 2].astype(np.uint64) | hdr[:, 3].astype(np.uint64) << np.uint64(32)
    assert np.array_equal(got_ctr, W.per_peer_sequence(peer, n_peers))
    assert np.array_equal(ctx.wg_send_counters(n_peers), np.bincount(peer, minlength=n_peers).astype(np.uint64))
    i = 4321
    assert v[i, :32 + padded].tobytes() == O.wg_encap(plain[i].tobytes(), mtu, keys[peer[i]].tobytes(),
                                                     int(local[peer[i]]), int(got_ctr[i]))
    # back in: a few datagrams carry an index one off a real one
    strangers = rng.permutation(n)[:40]
    hdr_view = v[:, :16].view(np.uint32).reshape(n, 4)
    free = np.setdiff1d(local[peer[strangers]] + np.uint32(1), local)
    hdr_view[strangers[:free.size], 1] = free
    strangers = strangers[:free.size]
    out = np.zeros(n * stride, np.uint8)
    res = np.full(n, 99, np.uint8)
    out_len = np.zeros(n, np.uint32)
    got_peer = np.zeros(n, np.uint32)
    got_c = np.zeros(n, np.uint64)
    ctx.wg_decap(lib.make_batch(arena, arena.nbytes, n, lib.MEM_HOST, stride=stride, length=32 + padded),
                 lib.make_batch(out, out.nbytes, n, lib.MEM_HOST, stride=stride), res, out_len, got_peer, got_c)
    want_res = np.zeros(n, np.uint8)
    want_res[strangers] = lib.WG_UNKNOWN_INDEX
    assert np.array_equal(res, want_res)
    ok = want_res == 0
    assert np.array_equal(got_peer[ok], peer[ok]) and (got_peer[~ok] == 0xFFFFFFFF).all()
    assert np.array_equal(got_c[ok], got_ctr[ok]) and (out_len[ok] == length).all()
    assert np.array_equal(out.reshape(n, stride)[ok, :length], plain[ok])
    ctx.close()


@pytest.mark.parametrize("fused", ["wave", "lane", "separate"])
@pytest.mark.parametrize("inner", [0, 28, 1000, 1420])
def test_decap_uniform_datagrams(fused, inner):
    """Datagrams of one size at a uniform stride, no length array: keepalives
    (inner 0), the smallest UDP packet, ordinary and MTU-sized ones."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(inner + 3)
    peers = _peers(rng)
    keys = rng.integers(0, 256, (N_PEERS, 32), dtype=np.uint8)
    n = 257
    wires = []
    for i in range(n):
        p = int(rng.integers(0, N_PEERS))
        pt = _inner(rng, peers, p, inner) if inner else b""
        wires.append(O.wg_encap(pt, MTU, keys[p].tobytes(), peers[p][0], 5 + i))
    wlen = len(wires[0])
    assert all(len(w) == wlen for w in wires)
    stride = (wlen + 31) & ~15
    arena = np.full(n * stride, 0xEE, np.uint8)
    for i, w in enumerate(wires):
        arena[i * stride:i * stride + wlen] = np.frombuffer(w, np.uint8)
    want = np.array([(lambda r: (r[0], len(r[1]), r[2], r[3]))(O.wg_decap(w, peers, keys)) for w in wires], np.uint64)
    assert (want[:, 0] == (O.WG_OK if inner else O.WG_KEEPALIVE)).all()
    ctx = _ctx(peers, keys_recv=keys)
    _launch_shape(ctx, fused)
    for mem in ("pageable", "ring"):
        rings = [ctx.ring_alloc(arena.nbytes), ctx.ring_alloc(arena.nbytes)] if mem == "ring" else []
        src = rings[0] if rings else arena.copy()
        out = rings[1] if rings else np.zeros_like(arena)
        src[:] = arena
        out[:] = 0x77
        res, olen = np.full(n, 99, np.uint8), np.full(n, 99, np.uint32)
        gp, gc = np.full(n, 99, np.uint32), np.full(n, 99, np.uint64)
        ctx.wg_decap(lib.make_batch(src, arena.nbytes, n, lib.MEM_HOST, stride=stride, length=wlen),
                     lib.make_batch(out, arena.nbytes, n, lib.MEM_HOST, stride=stride), res, olen, gp, gc)
        assert np.array_equal(res, want[:, 0].astype(np.uint8)), mem
        assert np.array_equal(olen, want[:, 1].astype(np.uint32)) and np.array_equal(gp, want[:, 2].astype(np.uint32))
        assert np.array_equal(gc, want[:, 3])
        got = np.array(out).reshape(n, stride)
        for i in (0, n // 2, n - 1):
            rc, pt, _, _ = O.wg_decap(wires[i], peers, keys)
            assert got[i, :len(pt)].tobytes() == pt
            assert (got[i, wlen - 32:] == 0x77).all()  # nothing beyond the padded plaintext
        for r in rings:
            ctx.ring_free(r)
    ctx.close()


@pytest.mark.parametrize("mem", ["pageable", "ring"])
@pytest.mark.parametrize("n,spread_max", [(600, 4096), (600, 0), (6000, 4096), (9000, 4096)])
def test_decap_in_place(mem, n, spread_max):
    """wireguard-go opens a datagram in place: the plaintext lands 16 bytes into
    the datagram it came from.  Header and tag bytes stay as they were.  9000
    full-size datagrams (13 MB) go through in overlapped chunks."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(n + spread_max)
    peers = _peers(rng)
    keys = rng.integers(0, 256, (N_PEERS, 32), dtype=np.uint8)
    plains, wires = [], []
    for i in range(n):
        p = int(rng.integers(0, N_PEERS))
        pt = _inner(rng, peers, p, 1400 if n == 9000 else int(rng.choice([20, 64, 300, 1400])))
        plains.append(pt)
        wires.append(O.wg_encap(pt, MTU, keys[p].tobytes(), peers[p][0], i))
    lens = np.array([len(w) for w in wires], np.uint32)
    off, total = _layout(rng, lens)
    assert (n == 9000) == (total > 12 << 20)
    arena = np.full(total, 0xEE, np.uint8)
    for i, w in enumerate(wires):
        arena[int(off[i]):int(off[i]) + len(w)] = np.frombuffer(w, np.uint8)
    want = arena.copy()
    for i, w in enumerate(wires):
        padded = len(w) - 32
        rc, pt, p, c = O.wg_decap(w, peers, keys)
        assert rc == O.WG_OK
        full = O.aead_open(keys[p].tobytes(), O.wg_nonce(c), w[16:])[1]  # padding included
        assert len(full) == padded
        want[int(off[i]) + 16:int(off[i]) + 16 + padded] = np.frombuffer(full, np.uint8)
    ctx = _ctx(peers, keys_recv=keys)
    ctx.set_spread_max_packets(spread_max)
    ring = ctx.ring_alloc(total) if mem == "ring" else None
    buf = ring if ring is not None else arena.copy()
    buf[:] = arena
    res, olen = np.full(n, 99, np.uint8), np.zeros(n, np.uint32)
    gp, gc = np.zeros(n, np.uint32), np.zeros(n, np.uint64)
    ctx.wg_decap(lib.make_batch(buf, total, n, lib.MEM_HOST, offsets=off, lens=lens),
                 lib.make_batch(buf, total, n, lib.MEM_HOST, offsets=off + np.uint64(16)), res, olen, gp, gc)
    assert (res == 0).all() and np.array_equal(olen, np.array([len(p) for p in plains], np.uint32))
    bad = np.flatnonzero(np.array(buf) != want)
    assert bad.size == 0, f"first differing byte at {bad[:5]}"
    if ring is not None:
        ctx.ring_free(ring)
    ctx.close()


def _decap_cases(rng, peers, keys, n):
    """Datagrams as the remote peers would send them, most of them damaged in
    one of the ways the receive path must tell apart."""
    from oracle import binding as O
    wires, kinds = [], []
    for i in range(n):
        p = int(rng.integers(0, N_PEERS))
        kind = int(rng.integers(0, 14))
        length = int(rng.choice([20, 21, 28, 40, 64, 100, 576, 1300, 1420]))
        pt = bytearray(_inner(rng, peers, p, length))
        if kind == 1:
            pt = bytearray()                           # keepalive
        elif kind == 2:
            pt[2:4] = struct.pack(">H", max(20, length - int(rng.integers(0, 9))))  # trailing bytes
        elif kind == 3:
            pt[0] = int(rng.choice([0x05, 0x55, 0x75, 0xF5]))
        elif kind == 4:
            pt[2:4] = struct.pack(">H", length + 16)
        elif kind == 5:
            pt[2:4] = struct.pack(">H", int(rng.integers(0, 20)))
        elif kind == 6:
            pt[12:16] = struct.pack(">I", peers[p][2] ^ 0x00010000)  # outside the allowed prefix
        elif kind == 7:
            pt = bytearray(max(length, 40))
            pt[0] = 0x60
            pt[4:6] = struct.pack(">H", len(pt) - 40 + int(rng.integers(0, 2)) * 8)
        elif kind == 8:
            pt = pt[:int(rng.integers(1, 20))]
            pt[0] = 0x45
        ctr = int(rng.integers(0, 1 << 62))
        w = bytearray(O.wg_encap(bytes(pt), MTU, keys[p].tobytes(), peers[p][0], ctr))
        if kind == 9:
            w[int(rng.integers(8, len(w)))] ^= 1 << int(rng.integers(0, 8))   # counter, body or tag
        elif kind == 10:
            w[0:4] = struct.pack("<I", int(rng.choice([0, 1, 2, 3, 5, 0x0400, 0x04000000])))
        elif kind == 11:
            w = w[:int(rng.integers(0, 32))]
        elif kind == 12:
            w[4:8] = struct.pack("<I", peers[p][0] ^ 0x40000000)
        elif kind == 13:
            w[4:8] = struct.pack("<I", peers[(p + 1) % N_PEERS][0])           # someone else's index
        wires.append(bytes(w))
        kinds.append(kind)
    return wires, np.array(kinds)


@pytest.mark.parametrize("mem", ["host", "ring", "device"])
@pytest.mark.parametrize("aligned", [True, False])
@pytest.mark.parametrize("fused", ["wave", "lane", "separate"])
def test_decap_matches_oracle(mem, aligned, fused):
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(23 + aligned)
    peers = _peers(rng)
    keys = rng.integers(0, 256, (N_PEERS, 32), dtype=np.uint8)
    n = 4000
    wires, kinds = _decap_cases(rng, peers, keys, n)
    lens = np.array([len(w) for w in wires], np.uint32)
    off, total = _layout(rng, lens, misalign=not aligned)
    arena = np.full(total, 0xEE, np.uint8)
    for i, w in enumerate(wires):
        arena[int(off[i]):int(off[i]) + len(w)] = np.frombuffer(w, np.uint8)
    # plaintext slot i sits 16 bytes into a copy of the wire layout, so that
    # ciphertext and plaintext share their position within a 128-byte line
    out_off = off + np.uint64(16)
    want_out = np.full(total + 16, 0x77, np.uint8)
    want = np.zeros((n, 4), np.uint64)
    for i, w in enumerate(wires):
        rc, pt, p, c = O.wg_decap(w, peers, keys)
        want[i] = (rc, len(pt), p, c)
        plen = max(len(w) - 32, 0)
        if rc not in (O.WG_BAD_HEADER, O.WG_UNKNOWN_INDEX):
            # an opened packet leaves its whole plaintext (padding included), a
            # failed open leaves zeros
            if rc == O.WG_AUTH_FAIL:
                body = bytes(plen)
            else:
                ok, body = O.aead_open(keys[p].tobytes(), O.wg_nonce(c), w[16:])
                assert ok
            want_out[int(out_off[i]):int(out_off[i]) + plen] = np.frombuffer(body, np.uint8)
    assert len(set(want[:, 0].tolist())) == 7  # every result class occurs
    ctx = _ctx(peers, keys_recv=keys)
    _launch_shape(ctx, fused)
    if mem == "host":
        got_out = np.full(total + 16, 0x77, np.uint8)
        res = np.full(n, 99, np.uint8)
        olen = np.full(n, 99, np.uint32)
        gp = np.full(n, 99, np.uint32)
        gc = np.full(n, 99, np.uint64)
        ctx.wg_decap(lib.make_batch(arena, arena.nbytes, n, lib.MEM_HOST, offsets=off, lens=lens),
                     lib.make_batch(got_out, got_out.nbytes, n, lib.MEM_HOST, offsets=out_off),
                     res, olen, gp, gc)
    elif mem == "ring":
        r_in, r_out = ctx.ring_alloc(arena.nbytes + 80), ctx.ring_alloc(total + 16)
        r_in[80:] = arena
        r_out[:] = 0x77
        res = np.full(n, 99, np.uint8)
        olen = np.full(n, 99, np.uint32)
        gp = np.full(n, 99, np.uint32)
        gc = np.full(n, 99, np.uint64)
        ctx.wg_decap(lib.make_batch(r_in[80:], arena.nbytes, n, lib.MEM_HOST, offsets=off, lens=lens),
                     lib.make_batch(r_out, total + 16, n, lib.MEM_HOST, offsets=out_off),
                     res, olen, gp, gc)
        got_out = np.array(r_out)
        ctx.ring_free(r_in)
        ctx.ring_free(r_out)
    else:
        dev = torch.device("cuda:0")
        d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
        d_arena, d_off, d_lens = d(arena), d(off.astype(np.int64)), d(lens.astype(np.int32))
        d_ooff = d(out_off.astype(np.int64))
        d_out = torch.full((total + 16,), 0x77, dtype=torch.uint8, device=dev)
        d_res = torch.full((n,), 99, dtype=torch.uint8, device=dev)
        d_olen = torch.zeros(n, dtype=torch.int32, device=dev)
        d_gp = torch.zeros(n, dtype=torch.int32, device=dev)
        d_gc = torch.zeros(n, dtype=torch.int64, device=dev)
        torch.cuda.synchronize()
        ctx.wg_decap(lib.make_batch(d_arena, d_arena.numel(), n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens),
                     lib.make_batch(d_out, d_out.numel(), n, lib.MEM_DEVICE, offsets=d_ooff),
                     d_res, d_olen, d_gp, d_gc)
        ctx.sync()
        got_out = d_out.cpu().numpy()
        res = d_res.cpu().numpy()
        olen = d_olen.cpu().numpy().astype(np.uint32)
        gp = d_gp.cpu().numpy().astype(np.uint32)
        gc = d_gc.cpu().numpy().astype(np.uint64)
    assert np.array_equal(res, want[:, 0].astype(np.uint8))
    assert np.array_equal(olen, want[:, 1].astype(np.uint32))
    assert np.array_equal(gp, want[:, 2].astype(np.uint32))
    assert np.array_equal(gc, want[:, 3])
    bad = np.flatnonzero(got_out != want_out)
    assert bad.size == 0, f"first differing byte at {bad[:5]}"
    ctx.close()


@pytest.mark.parametrize("n_peers", [65, 4097, 70000])
@pytest.mark.parametrize("fused", ["wave", "lane", "separate"])
def test_receiver_index_lookup_in_large_peer_tables(n_peers, fused):
    """The sender is found by its receiver index in a sorted table: searched 64
    entries at a time by the lanes of a wave (small batches), or by binary
    search per packet (70000 peers do not fit the LDS copy and are searched in
    memory).  Indices at both ends of the table, unknown ones below, between
    and above: results, peers and counters against the oracle."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(n_peers)
    local = (rng.permutation(1 << 22)[:n_peers].astype(np.uint64) * 1021 + 5).astype(np.uint32)
    peers = [(int(local[i]), i, 0x64400001 + i, 0xFFFFFFFF) for i in range(n_peers)]
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    srt = np.sort(local)
    n = 600 if n_peers < 10000 else 200  # the oracle rebuilds its table per packet
    who = rng.integers(0, n_peers, n)
    who[:4] = [int(np.argmin(local)), int(np.argmax(local)), 0, n_peers - 1]
    wires = []
    for i in range(n):
        p = int(who[i])
        pt = bytearray(rng.integers(0, 256, 48, dtype=np.uint8).tobytes())
        pt[0] = 0x45
        pt[2:4] = struct.pack(">H", 48)
        pt[12:16] = struct.pack(">I", peers[p][2])
        w = bytearray(O.wg_encap(bytes(pt), MTU, keys[p].tobytes(), peers[p][0], 1000 + i))
        if i % 5 == 4:  # an index nobody owns
            bogus = [int(srt[0]) - 1, int(srt[-1]) + 1, int(srt[len(srt) // 2]) + 1, 0, 0xFFFFFFFF][(i // 5) % 5]
            w[4:8] = struct.pack("<I", bogus & 0xFFFFFFFF)
        wires.append(bytes(w))
    lens = np.array([len(w) for w in wires], np.uint32)
    off = np.arange(n, dtype=np.uint64) * 128
    arena = np.zeros(n * 128, np.uint8)
    for i, w in enumerate(wires):
        arena[i * 128:i * 128 + len(w)] = np.frombuffer(w, np.uint8)
    want = np.array([(lambda r: (r[0], len(r[1]), r[2], r[3]))(O.wg_decap(w, peers, keys)) for w in wires],
                    np.uint64)
    assert (want[:, 0] == O.WG_UNKNOWN_INDEX).sum() >= n // 5 - 1 and (want[:, 0] == 0).sum() >= n // 2
    ctx = _ctx(peers, keys_recv=keys)
    _launch_shape(ctx, fused)
    out = np.zeros(n * 128, np.uint8)
    res, olen = np.full(n, 99, np.uint8), np.full(n, 99, np.uint32)
    gp, gc = np.full(n, 99, np.uint32), np.full(n, 99, np.uint64)
    ctx.wg_decap(lib.make_batch(arena, arena.nbytes, n, lib.MEM_HOST, offsets=off, lens=lens),
                 lib.make_batch(out, out.nbytes, n, lib.MEM_HOST, offsets=off), res, olen, gp, gc)
    assert np.array_equal(res, want[:, 0].astype(np.uint8))
    assert np.array_equal(olen, want[:, 1].astype(np.uint32))
    assert np.array_equal(gp, want[:, 2].astype(np.uint32))
    assert np.array_equal(gc, want[:, 3])
    ctx.close()


def _filter_setup(rng, peers):
    """Rules that let some peers reach some ports, and a few recorded outbound
    flows whose replies must pass without a rule."""
    rules = [([(peers[p][2], 32)], "tcp", [(22, 22), (8000, 8100)]) for p in range(0, N_PEERS, 3)]
    rules += [([(0x64400000, 16)], "udp", [(53, 53)]), ([(peers[1][2], 32)], "icmp", [])]
    local = 0x64700001
    noted = [W.udp(local, peers[p][2], 4000 + p, 9000 + p) for p in range(2, N_PEERS, 4)]
    noted += [W.tcp(local, peers[p][2], 5000 + p, 443) for p in range(3, N_PEERS, 5)]
    return rules, local, noted


@pytest.mark.parametrize("mem", ["host", "ring", "device"])
@pytest.mark.parametrize("fused", ["wave", "lane", "separate"])
def test_decap_with_the_inbound_filter_in_one_call(mem, fused):
    """bnk_wg_decap_filter_batch = decapsulate, then CheckInbound with one `now`
    on what was delivered: results (FILTERED for the denied), plaintexts,
    peers, counters and the flow table afterwards against the oracle's two
    steps, and against the library's own two calls."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(77)
    peers = _peers(rng)
    keys = rng.integers(0, 256, (N_PEERS, 32), dtype=np.uint8)
    rules, local, noted = _filter_setup(rng, peers)
    t0 = 1_700_000_000 * 10**9
    n = 1500
    wires = []
    for i in range(n):
        p = int(rng.integers(0, N_PEERS))
        src = peers[p][2]
        kind = int(rng.integers(0, 8))
        if kind == 0:
            pt = W.tcp(src, local, 40000 + i, int(rng.choice([22, 23, 8000, 8100, 8101, 443])))
        elif kind == 1:
            pt = W.udp(src, local, int(rng.choice([53, 9000 + p])), int(rng.choice([53, 4000 + p, 4001])))
        elif kind == 2:
            pt = W.tcp(src, local, 443, 5000 + p, syn=False)      # reply to a recorded flow, or not
        elif kind == 3:
            pt = W.icmp_echo(src, local)
        elif kind == 4:
            pt = W.udp(src ^ 0x00010000, local, 53, 53)           # not the peer's address
        elif kind == 5:
            pt = b""                                              # keepalive
        elif kind == 6:
            pt = W.tcp(src, local, 1, 22) + bytes(int(rng.integers(0, 40)))  # trailing bytes beyond the IP length
        else:
            pt = W.ipv4(47, src, local, bytes(8))                 # a protocol the filter does not parse
        w = bytearray(O.wg_encap(pt, MTU, keys[p].tobytes(), peers[p][0], 100 + i))
        if i % 19 == 0:
            w[-1] ^= 1
        wires.append(bytes(w))
    lens = np.array([len(w) for w in wires], np.uint32)
    off, total = _layout(rng, lens)
    arena = np.full(total, 0xEE, np.uint8)
    for i, w in enumerate(wires):
        arena[int(off[i]):int(off[i]) + len(w)] = np.frombuffer(w, np.uint8)
    out_off = off + np.uint64(16)

    # the oracle's two steps
    ora = O.Filter()
    ora.set_rules(rules)
    for pkt in noted:
        ora.note_outbound(pkt, t0 - 10**9)
    want = np.zeros((n, 4), np.uint64)
    for i, w in enumerate(wires):
        rc, pt, p, c = O.wg_decap(w, peers, keys)
        if rc == O.WG_OK and not ora.check_inbound(pt, t0):
            rc = lib.WG_FILTERED
        want[i] = (rc, len(pt), p, c)
    assert {0, 1, 4, 6, 7} <= set(want[:, 0].tolist())
    assert 0.2 < (want[:, 0] == 7).mean() < 0.7 and (want[:, 0] == 0).mean() > 0.1

    def fresh_ctx():
        ctx = _ctx(peers, keys_recv=keys)
        _launch_shape(ctx, fused)
        ctx.filter_set_rules(rules)
        for pkt in noted:
            ctx.filter_note_outbound_ptrs([pkt], t0 - 10**9)
        return ctx

    ctx = fresh_ctx()
    res, olen = np.full(n, 99, np.uint8), np.full(n, 99, np.uint32)
    gp, gc = np.full(n, 99, np.uint32), np.full(n, 99, np.uint64)
    if mem == "device":
        dev = torch.device("cuda:0")
        d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
        d_arena, d_off, d_lens, d_ooff = d(arena), d(off.astype(np.int64)), d(lens.astype(np.int32)), d(out_off.astype(np.int64))
        d_out = torch.full((total + 16,), 0x77, dtype=torch.uint8, device=dev)
        d_res = torch.full((n,), 99, dtype=torch.uint8, device=dev)
        d_olen, d_gp = torch.zeros(n, dtype=torch.int32, device=dev), torch.zeros(n, dtype=torch.int32, device=dev)
        d_gc = torch.zeros(n, dtype=torch.int64, device=dev)
        torch.cuda.synchronize()
        ctx.wg_decap_filter(lib.make_batch(d_arena, d_arena.numel(), n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens),
                            lib.make_batch(d_out, d_out.numel(), n, lib.MEM_DEVICE, offsets=d_ooff),
                            t0, d_res, d_olen, d_gp, d_gc)
        ctx.sync()
        got_out = d_out.cpu().numpy()
        res, olen = d_res.cpu().numpy(), d_olen.cpu().numpy().astype(np.uint32)
        gp, gc = d_gp.cpu().numpy().astype(np.uint32), d_gc.cpu().numpy().astype(np.uint64)
    else:
        rings = []
        if mem == "ring":
            rings = [ctx.ring_alloc(arena.nbytes), ctx.ring_alloc(total + 16)]
            rings[0][:] = arena
            src, got_out = rings
        else:
            src, got_out = arena, np.zeros(total + 16, np.uint8)
        got_out[:] = 0x77
        ctx.wg_decap_filter(lib.make_batch(src, arena.nbytes, n, lib.MEM_HOST, offsets=off, lens=lens),
                            lib.make_batch(got_out, total + 16, n, lib.MEM_HOST, offsets=out_off),
                            t0, res, olen, gp, gc)
        got_out = np.array(got_out)
        for r in rings:
            ctx.ring_free(r)
    assert np.array_equal(res, want[:, 0].astype(np.uint8))
    assert np.array_equal(olen, want[:, 1].astype(np.uint32))
    assert np.array_equal(gp, want[:, 2].astype(np.uint32))
    assert np.array_equal(gc, want[:, 3])
    assert ctx.filter_flows() == ora.flows()

    # the library's own two calls leave the same plaintexts and the same table
    ctx2 = fresh_ctx()
    out2 = np.full(total + 16, 0x77, np.uint8)
    r2, l2 = np.zeros(n, np.uint8), np.zeros(n, np.uint32)
    p2, c2 = np.zeros(n, np.uint32), np.zeros(n, np.uint64)
    ctx2.wg_decap(lib.make_batch(arena, arena.nbytes, n, lib.MEM_HOST, offsets=off, lens=lens),
                  lib.make_batch(out2, out2.nbytes, n, lib.MEM_HOST, offsets=out_off), r2, l2, p2, c2)
    v2 = np.zeros(n, np.uint8)
    ctx2.filter_check_inbound(lib.make_batch(out2, out2.nbytes, n, lib.MEM_HOST, offsets=out_off, lens=l2), t0, v2)
    assert np.array_equal(got_out, out2)
    assert np.array_equal(np.where((r2 == 0) & (v2 == 0), 7, r2), res)
    assert ctx2.filter_flows() == ctx.filter_flows()
    # allow-all: nothing is filtered
    ctx2.filter_set_allow_all()
    ctx2.wg_decap_filter(lib.make_batch(arena, arena.nbytes, n, lib.MEM_HOST, offsets=off, lens=lens),
                         lib.make_batch(out2, out2.nbytes, n, lib.MEM_HOST, offsets=out_off), t0, r2, l2, p2, c2)
    assert not (r2 == 7).any() and np.array_equal(r2 == 0, np.isin(res, (0, 7)))
    ctx.close()
    ctx2.close()


@pytest.mark.parametrize("mem", ["host", "ring"])
@pytest.mark.parametrize("n", [900, 3000])
def test_note_outbound_and_encap_in_one_call(mem, n):
    """bnk_wg_note_encap_batch = NoteOutbound with one `now` on every
    plaintext, then encapsulate: the datagrams of bnk_wg_encap_batch and the
    flow table of bnk_filter_note_outbound_batch, both against the oracle."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(5 + n)
    peers = _peers(rng)
    keys = rng.integers(0, 256, (N_PEERS, 32), dtype=np.uint8)
    t0 = 1_700_000_000 * 10**9
    local = 0x64700001
    peer = rng.integers(0, N_PEERS, n).astype(np.uint32)
    plains = []
    for i in range(n):
        dst = peers[int(peer[i])][2]
        kind = i % 5
        if kind == 0:
            plains.append(W.tcp(local, dst, 30000 + (i % 2000), 443))
        elif kind == 1:
            plains.append(W.udp(local, dst, 30000 + (i % 500), 53))
        elif kind == 2:
            plains.append(W.icmp_echo(local, dst))
        elif kind == 3:
            plains.append(bytes(int(rng.integers(0, 19))))       # too short to be noted
        else:
            plains.append(W.tcp(local, dst, 1234, 80) + bytes(int(rng.integers(0, 600))))
    lens = np.array([len(p) for p in plains], np.uint32)
    room = 16 + lens.astype(np.int64) + 15 + 16
    off, total = _layout(rng, room)
    arena = np.full(total, 0xEE, np.uint8)
    for i, pt in enumerate(plains):
        arena[int(off[i]) + 16:int(off[i]) + 16 + len(pt)] = np.frombuffer(pt, np.uint8)
    ora = O.Filter()
    ora.set_rules([])
    want = arena.copy()
    want_len = np.zeros(n, np.uint32)
    next_ctr = np.zeros(N_PEERS, np.uint64)
    for i, pt in enumerate(plains):
        ora.note_outbound(pt, t0)
        p = int(peer[i])
        w = O.wg_encap(pt, MTU, keys[p].tobytes(), peers[p][1], int(next_ctr[p]))
        next_ctr[p] += 1
        want[int(off[i]):int(off[i]) + len(w)] = np.frombuffer(w, np.uint8)
        want_len[i] = len(w)
    ctx = _ctx(peers, keys_send=keys)
    ctx.filter_set_rules([])
    ring = ctx.ring_alloc(total) if mem == "ring" else None
    got = ring if mem == "ring" else arena.copy()
    got[:] = arena
    got_len = np.zeros(n, np.uint32)
    ctx.wg_note_encap(lib.make_batch(got, total, n, lib.MEM_HOST, offsets=off, lens=lens, peer=peer), MTU, t0, got_len)
    assert np.array_equal(got_len, want_len)
    assert np.array_equal(np.array(got), want)
    assert ctx.filter_flows() == ora.flows() and ora.flow_count() > n // 4
    if ring is not None:
        ctx.ring_free(ring)
    ctx.close()


def test_one_call_paths_through_the_chunked_route():
    """13 MB of full-size packets in pinned rings: NoteOutbound + encapsulate
    and decapsulate + CheckInbound each in one call (overlapped chunks) against
    the library's separate calls, which the tests above hold to the oracle:
    same datagrams, results and flow tables."""
    from bnk_amd import lib
    rng = np.random.default_rng(99)
    peers = _peers(rng)
    keys = rng.integers(0, 256, (N_PEERS, 32), dtype=np.uint8)
    rules, local, noted = _filter_setup(rng, peers)
    t0 = 1_700_000_000 * 10**9
    n, stride = 9000, 1504
    peer = rng.integers(0, N_PEERS, n).astype(np.uint32)
    lens = np.full(n, 1400, np.uint32)
    off = np.arange(n, dtype=np.uint64) * stride
    arena = np.zeros(n * stride, np.uint8)
    rows = arena.reshape(n, stride)
    for i in range(n):
        p = int(peer[i])
        # send side: packets from this node to the peer, recorded as outbound flows; the
        # receive side below sees the same bytes arriving from the peer's address
        pkt = W.udp(peers[p][2], local, 53 if i % 3 else 9999, 4000 + (i % 50)) if i % 2 else \
            W.tcp(peers[p][2], local, 40000 + (i % 999), 22 if i % 4 else 23)
        rows[i, 16:16 + len(pkt)] = np.frombuffer(pkt, np.uint8)
        rows[i, 18], rows[i, 19] = 1400 >> 8, 1400 & 255  # IP total length = the whole slot payload
    assert arena.nbytes > 12 << 20

    def make(send):
        c = _ctx(peers, keys_send=keys if send else None, keys_recv=None if send else keys)
        c.filter_set_rules(rules)
        return c

    # --- send side
    a, b = make(True), make(True)
    ra, rb = a.ring_alloc(arena.nbytes), b.ring_alloc(arena.nbytes)
    ra[:] = arena
    rb[:] = arena
    wl_a, wl_b = np.zeros(n, np.uint32), np.zeros(n, np.uint32)
    a.wg_note_encap(lib.make_batch(ra, arena.nbytes, n, lib.MEM_HOST, offsets=off, lens=lens, peer=peer), MTU, t0, wl_a)
    b.filter_note_outbound(lib.make_batch(rb[16:], arena.nbytes - 16, n, lib.MEM_HOST, offsets=off, lens=lens), t0)
    b.wg_encap(lib.make_batch(rb, arena.nbytes, n, lib.MEM_HOST, offsets=off, lens=lens, peer=peer), MTU, wl_b)
    assert np.array_equal(wl_a, wl_b) and np.array_equal(np.array(ra), np.array(rb))
    assert a.filter_flows() == b.filter_flows() and a.filter_flow_count() > 100
    wire = np.array(ra)
    for c, r in ((a, ra), (b, rb)):
        c.ring_free(r)
        c.close()

    # --- receive side: the same datagrams, addressed to the receiver's indices
    rx_peers = [(p[1], p[0], p[2], p[3]) for p in peers]
    def make_rx():
        c = lib.Context(0)
        c.keys_set(lib.KEYS_RECV, keys)
        c.wg_peers_set(rx_peers)
        c.filter_set_rules(rules)
        for pkt in noted:
            c.filter_note_outbound_ptrs([pkt], t0 - 10**9)
        return c
    a, b = make_rx(), make_rx()
    ra, oa = a.ring_alloc(wire.nbytes), a.ring_alloc(wire.nbytes)
    rb, ob = b.ring_alloc(wire.nbytes), b.ring_alloc(wire.nbytes)
    for r in (ra, rb):
        r[:] = wire
    for r in (oa, ob):
        r[:] = 0x77
    out_off = off + np.uint64(16)
    res_a, res_b = np.zeros(n, np.uint8), np.zeros(n, np.uint8)
    la, lb = np.zeros(n, np.uint32), np.zeros(n, np.uint32)
    pa, pb = np.zeros(n, np.uint32), np.zeros(n, np.uint32)
    ca, cb = np.zeros(n, np.uint64), np.zeros(n, np.uint64)
    a.wg_decap_filter(lib.make_batch(ra, wire.nbytes, n, lib.MEM_HOST, offsets=off, lens=wl_a),
                      lib.make_batch(oa, wire.nbytes, n, lib.MEM_HOST, offsets=out_off), t0, res_a, la, pa, ca)
    b.wg_decap(lib.make_batch(rb, wire.nbytes, n, lib.MEM_HOST, offsets=off, lens=wl_a),
               lib.make_batch(ob, wire.nbytes, n, lib.MEM_HOST, offsets=out_off), res_b, lb, pb, cb)
    v = np.zeros(n, np.uint8)
    b.filter_check_inbound(lib.make_batch(ob, wire.nbytes, n, lib.MEM_HOST, offsets=out_off, lens=lb), t0, v)
    assert (res_b == 0).all()
    assert np.array_equal(res_a, np.where(v == 0, 7, 0)) and 0.5 < (res_a == 7).mean() < 0.99
    assert np.array_equal(la, lb) and np.array_equal(pa, pb) and np.array_equal(ca, cb)
    assert np.array_equal(np.array(oa), np.array(ob))
    assert a.filter_flows() == b.filter_flows()
    for c, rs in ((a, (ra, oa)), (b, (rb, ob))):
        for r in rs:
            c.ring_free(r)
        c.close()


def test_random_framing_batches_round_trip_through_rings_and_pageable_memory():
    """Forty batches of random size, length mix, MTU, alignment, memory kind and
    kernel choice: encapsulated datagrams against the oracle byte for byte,
    then decapsulated again (results, lengths, peers, counters, plaintexts)."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(4242)
    n_peers = 23
    local = rng.permutation(1 << 20)[:n_peers].astype(np.uint32) * 4099 + 17
    remote = rng.integers(0, 1 << 32, n_peers, dtype=np.uint64).astype(np.uint32)
    peers_tx = [(int(local[i]), int(remote[i]), 0x64400001 + i, 0xFFFFFFFF) for i in range(n_peers)]
    peers_rx = [(int(remote[i]), int(local[i]), 0x64400001 + i, 0xFFFFFFFF) for i in range(n_peers)]
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    tx, rx = lib.Context(0), lib.Context(0)
    tx.keys_set(lib.KEYS_SEND, keys)
    rx.keys_set(lib.KEYS_RECV, keys)
    ring_t, ring_r, ring_o = tx.ring_alloc(3 << 20), rx.ring_alloc(3 << 20), rx.ring_alloc(3 << 20)
    tx.wg_peers_set(peers_tx)
    rx.wg_peers_set(peers_rx)
    nxt = np.zeros(n_peers, np.uint64)  # the peers' send counters run on from batch to batch
    for it in range(40):
        n = int(rng.choice([1, 3, 64, 65, 200, 1024, 1025]))
        mtu = int(rng.choice([0, 1280, 1420]))
        lens = rng.choice([0, 1, 20, 21, 28, 40, 100, 576, 1279, 1280, 1400, 1420], n).astype(np.uint32)
        peer = rng.integers(0, n_peers, n).astype(np.uint32)
        slot = ((16 + lens.astype(np.int64) + 15 + 16 + 15) & ~15) + 16
        gaps = rng.integers(0, 16, n) if rng.integers(0, 2) else np.zeros(n, np.int64)
        off = (np.concatenate([[0], np.cumsum(slot)[:-1]]) + gaps).astype(np.uint64)
        total = int(slot.sum()) + 32
        arena = rng.integers(0, 256, total, dtype=np.uint8)
        for i in range(n):
            length, o = int(lens[i]), int(off[i]) + 16
            if length >= 20:
                arena[o] = 0x45
                arena[o + 2:o + 4] = np.frombuffer(struct.pack(">H", length), np.uint8)
                arena[o + 12:o + 16] = np.frombuffer(struct.pack(">I", peers_tx[int(peer[i])][2]), np.uint8)
        if it % 8 == 7:
            tx.wg_peers_set(peers_tx)  # the same table again: counters must not move
        spread = int(rng.choice([0, 4096]))
        tx.set_spread_max_packets(spread)
        rx.set_spread_max_packets(spread)
        in_rings = bool(rng.integers(0, 2))
        case = f"batch {it}: n={n} mtu={mtu} spread_max={spread} rings={in_rings}"
        want, want_len = arena.copy(), np.zeros(n, np.uint32)
        for i in range(n):
            p, o = int(peer[i]), int(off[i])
            w = O.wg_encap(arena[o + 16:o + 16 + int(lens[i])].tobytes(), mtu, keys[p].tobytes(),
                           peers_tx[p][1], int(nxt[p]))
            nxt[p] += 1
            want[o:o + len(w)] = np.frombuffer(w, np.uint8)
            want_len[i] = len(w)
        buf = ring_t[:total] if in_rings else arena.copy()
        buf[:] = arena
        got_len = np.zeros(n, np.uint32)
        tx.wg_encap(lib.make_batch(buf, total, n, lib.MEM_HOST, offsets=off, lens=lens, peer=peer), mtu, got_len)
        assert np.array_equal(got_len, want_len) and np.array_equal(np.array(buf), want), case
        src = ring_r[:total] if in_rings else want.copy()
        src[:] = want
        out = ring_o[:total + 16] if in_rings else np.zeros(total + 16, np.uint8)
        out[:] = 0x77
        res, olen = np.zeros(n, np.uint8), np.zeros(n, np.uint32)
        gp, gc = np.zeros(n, np.uint32), np.zeros(n, np.uint64)
        rx.wg_decap(lib.make_batch(src, total, n, lib.MEM_HOST, offsets=off, lens=want_len),
                    lib.make_batch(out, total + 16, n, lib.MEM_HOST, offsets=off + np.uint64(16)),
                    res, olen, gp, gc)
        for i in range(n):
            o = int(off[i])
            rc, pt, p, c = O.wg_decap(want[o:o + int(want_len[i])].tobytes(), peers_rx, keys)
            assert (rc, len(pt), p, c) == (int(res[i]), int(olen[i]), int(gp[i]), int(gc[i])), f"{case}, packet {i}"
            assert rc != 0 or out[o + 16:o + 16 + len(pt)].tobytes() == pt, f"{case}, packet {i}"
    for c, rings in ((tx, (ring_t,)), (rx, (ring_r, ring_o))):
        for r in rings:
            c.ring_free(r)
        c.close()


def test_encap_then_decap_round_trip_full_size():
    """2^20 MTU-sized slots, device resident: every datagram decapsulates to
    its plaintext under the mirrored peer table, counters are each peer's
    0..k-1 in batch order, and a sample is bit-exact against the oracle."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    dev = torch.device("cuda:0")
    n, n_peers, plen = 1 << 20, 1024, 1400
    stride = 1536  # slot: 16 headroom + 1400 + 8 pad + 16 tag = 1440
    rng = np.random.default_rng(5)
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    idx_a = (np.arange(n_peers, dtype=np.uint32) * 7919 + 3).astype(np.uint32)
    idx_b = (np.arange(n_peers, dtype=np.uint32) * 104729 + 11).astype(np.uint32)
    addr = (0x64400000 + np.arange(n_peers, dtype=np.uint32)).astype(np.uint32)
    full = np.full(n_peers, 0xFFFFFFFF, np.uint32)
    # side A sends with remote index idx_b; side B receives with local index idx_b
    side_a = np.stack([idx_a, idx_b, addr, full], 1)
    side_b = np.stack([idx_b, idx_a, addr, full], 1)
    peer = rng.integers(0, n_peers, n).astype(np.uint32)
    arena = W.rand_bytes_torch(W.stream_seed(2, 77), n * stride, dev).view(n, stride)
    d_peer = torch.from_numpy(peer.astype(np.int32)).to(dev)
    # valid IPv4 header fields where decap looks: version/IHL, total length, source
    arena[:, 16] = 0x45
    arena[:, 18] = plen >> 8
    arena[:, 19] = plen & 0xFF
    src = torch.from_numpy(addr.astype(np.int64)).to(dev)[d_peer.long()]
    for k in range(4):
        arena[:, 16 + 12 + k] = ((src >> (24 - 8 * k)) & 0xFF).to(torch.uint8)
    plain = arena[:, 16:16 + plen].clone()
    d_wl = torch.zeros(n, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    tx = lib.Context(0)
    tx.keys_set(lib.KEYS_SEND, keys)
    tx.wg_peers_set(side_a)
    tx.wg_encap(lib.make_batch(arena, arena.numel(), n, lib.MEM_DEVICE, stride=stride, length=plen,
                               peer=d_peer), MTU, d_wl)
    tx.sync()
    assert bool((d_wl == 1440).all())
    sent = np.bincount(peer, minlength=n_peers).astype(np.uint64)
    assert np.array_equal(tx.wg_send_counters(n_peers), sent)
    # sample against the oracle
    sample = rng.choice(n, 64, replace=False)
    rank = np.zeros(n, np.uint64)
    seen = np.zeros(n_peers, np.uint64)
    for i in range(n):
        rank[i] = seen[peer[i]]
        seen[peer[i]] += 1
    h_plain = plain[torch.from_numpy(sample).to(dev)].cpu().numpy()
    h_wire = arena[torch.from_numpy(sample).to(dev)].cpu().numpy()
    for j, i in enumerate(sample):
        p = int(peer[i])
        w = O.wg_encap(h_plain[j].tobytes(), MTU, keys[p].tobytes(), int(idx_b[p]), int(rank[i]))
        assert h_wire[j, :1440].tobytes() == w
    # receive side
    rx = lib.Context(0)
    rx.keys_set(lib.KEYS_RECV, keys)
    rx.wg_peers_set(side_b)
    out = torch.zeros(n, stride, dtype=torch.uint8, device=dev)
    d_res = torch.full((n,), 99, dtype=torch.uint8, device=dev)
    d_olen = torch.zeros(n, dtype=torch.int32, device=dev)
    d_gp = torch.zeros(n, dtype=torch.int32, device=dev)
    d_gc = torch.zeros(n, dtype=torch.int64, device=dev)
    torch.cuda.synchronize()
    # plaintext lands 16 bytes into its slot, in line with the ciphertext
    rx.wg_decap(lib.make_batch(arena, arena.numel(), n, lib.MEM_DEVICE, stride=stride, length=1440),
                lib.make_batch(out.view(-1)[16:], out.numel() - 16, n, lib.MEM_DEVICE, stride=stride),
                d_res, d_olen, d_gp, d_gc)
    rx.sync()
    assert bool((d_res == 0).all())
    assert bool((d_olen == plen).all())
    assert bool((d_gp == d_peer).all())
    assert np.array_equal(d_gc.cpu().numpy().astype(np.uint64), rank)
    assert torch.equal(out[:, 16:16 + plen], plain)
    tx.close()
    rx.close()


@pytest.mark.parametrize("n", [24000, 96000])
def test_large_host_rings_take_the_chunked_route(n):
    """Host rings of several chunks' worth (pinned, as a tunnel would use them):
    encapsulate in place and decapsulate chunk by chunk with upload, kernels
    and download overlapped; results equal the device-resident path's and a
    sample equals the oracle.  24000 packets make chunks small enough for a
    wave per packet, 96000 chunks of 6000 that take a lane per packet (framing
    and window-pass keys from the AEAD launches, chunk by chunk)."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(31)
    n_peers, stride = 64, 1536
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    idx_a = (np.arange(n_peers, dtype=np.uint32) * 7919 + 3).astype(np.uint32)
    idx_b = (np.arange(n_peers, dtype=np.uint32) * 104729 + 11).astype(np.uint32)
    addr = (0x64400000 + np.arange(n_peers, dtype=np.uint32)).astype(np.uint32)
    full = np.full(n_peers, 0xFFFFFFFF, np.uint32)
    peer = rng.integers(0, n_peers, n).astype(np.uint32)
    lens = rng.choice([28, 60, 576, 1300, 1420], n).astype(np.uint32)
    tx, rx = lib.Context(0), lib.Context(0)
    tx.keys_set(lib.KEYS_SEND, keys)
    tx.wg_peers_set(np.stack([idx_a, idx_b, addr, full], 1))
    rx.keys_set(lib.KEYS_RECV, keys)
    rx.wg_peers_set(np.stack([idx_b, idx_a, addr, full], 1))
    ring = tx.ring_alloc(n * stride)
    assert ring.nbytes > 8 * (4 << 20)
    ring[:] = 0xEE
    slots = ring.reshape(n, stride)
    plain = rng.integers(0, 256, (n, 1420), dtype=np.uint8)
    plain[:, 0] = 0x45
    plain[:, 2] = (lens >> 8).astype(np.uint8)
    plain[:, 3] = (lens & 0xFF).astype(np.uint8)
    for k in range(4):
        plain[:, 12 + k] = ((addr[peer] >> (24 - 8 * k)) & 0xFF).astype(np.uint8)
    for L in np.unique(lens):
        rows = np.flatnonzero(lens == L)
        slots[rows, 16:16 + L] = plain[rows, :L]
    wl = np.zeros(n, np.uint32)
    tx.wg_encap(lib.make_batch(ring, ring.nbytes, n, lib.MEM_HOST, stride=stride, lens=lens, peer=peer),
                MTU, wl)
    pad = np.minimum((lens.astype(np.int64) + 15) // 16 * 16, MTU) - lens  # never beyond the MTU
    assert np.array_equal(wl, (16 + lens + pad + 16).astype(np.uint32))
    rank = np.zeros(n, np.uint64)
    seen = np.zeros(n_peers, np.uint64)
    for i in range(n):
        rank[i] = seen[peer[i]]
        seen[peer[i]] += 1
    assert np.array_equal(tx.wg_send_counters(n_peers), seen)
    for i in rng.choice(n, 48, replace=False):
        p = int(peer[i])
        w = O.wg_encap(plain[i, :lens[i]].tobytes(), MTU, keys[p].tobytes(), int(idx_b[p]), int(rank[i]))
        assert slots[i, :len(w)].tobytes() == w
        assert (slots[i, len(w):] == 0xEE).all()  # the rest of the slot came back untouched
    # receive side: same ring as the wire, plaintext into a second ring
    out = rx.ring_alloc(n * stride)
    out[:] = 0x77
    res = np.full(n, 99, np.uint8)
    olen = np.zeros(n, np.uint32)
    gp = np.zeros(n, np.uint32)
    gc = np.zeros(n, np.uint64)
    ring.reshape(n, stride)[5, 40] ^= 1  # one forged datagram
    rx.wg_decap(lib.make_batch(ring, ring.nbytes, n, lib.MEM_HOST, stride=stride, lens=wl),
                lib.make_batch(out[16:], out.nbytes - 16, n, lib.MEM_HOST, stride=stride),
                res, olen, gp, gc)
    want_res = np.zeros(n, np.uint8)
    want_res[5] = O.WG_AUTH_FAIL
    assert np.array_equal(res, want_res)
    ok = res == 0
    assert np.array_equal(olen[ok], lens[ok]) and olen[5] == 0
    assert np.array_equal(gp, peer) and np.array_equal(gc, rank)
    o2 = out.reshape(n, stride)
    for L in np.unique(lens):
        rows = np.flatnonzero((lens == L) & ok)
        assert np.array_equal(o2[rows, 16:16 + L], plain[rows, :L])
    assert (o2[:, :16] == 0x77).all()  # bytes between packets survive
    assert not o2[5, 16:16 + int(wl[5]) - 32].any()  # a failed open leaves zeros
    tx.ring_free(ring)
    rx.ring_free(out)
    tx.close()
    rx.close()


def _encap_host(ctx, arena, off, lens, peer, mtu=MTU):
    from bnk_amd import lib
    got = arena.copy()
    wl = np.zeros(len(lens), np.uint32)
    ctx.wg_encap(lib.make_batch(got, got.nbytes, len(lens), lib.MEM_HOST, offsets=off, lens=lens, peer=peer),
                 mtu, wl)
    return got, wl


@pytest.mark.parametrize("fused", ["wave", "lane", "separate"])
@pytest.mark.parametrize("n", [400, 3000])
def test_rekey_of_one_peer_leaves_the_other_counters_alone(fused, n):
    """WireGuard peers rekey independently: installing peer A's new keypair
    (bnk_wg_peer_set, or bnk_wg_peers_set with A's row changed) restarts A's
    counter only; every other peer's next packet continues its sequence, so no
    (key, nonce) pair is ever used twice."""
    from oracle import binding as O
    rng = np.random.default_rng(77)
    peers = _peers(rng)
    keys = rng.integers(0, 256, (N_PEERS, 32), dtype=np.uint8)
    lens = rng.integers(20, 600, n).astype(np.uint32)
    peer = rng.integers(0, N_PEERS, n).astype(np.uint32)
    off, total = _layout(rng, 16 + lens.astype(np.int64) + 31)
    arena = np.full(total, 0xEE, np.uint8)
    plains = []
    for i in range(n):
        pt = _inner(rng, peers, int(peer[i]), int(lens[i]))
        plains.append(pt)
        arena[int(off[i]) + 16:int(off[i]) + 16 + len(pt)] = np.frombuffer(pt, np.uint8)
    ctx = _ctx(peers, keys_send=keys, keys_recv=keys)
    _launch_shape(ctx, fused)
    next_ctr = np.zeros(N_PEERS, np.uint64)

    def check_batch():
        want = arena.copy()
        for i in range(n):
            p = int(peer[i])
            w = O.wg_encap(plains[i], MTU, keys[p].tobytes(), peers[p][1], int(next_ctr[p]))
            next_ctr[p] += 1
            want[int(off[i]):int(off[i]) + len(w)] = np.frombuffer(w, np.uint8)
        got, _ = _encap_host(ctx, arena, off, lens, peer)
        assert np.array_equal(got, want)
        assert np.array_equal(ctx.wg_send_counters(N_PEERS), next_ctr)

    check_batch()
    assert next_ctr.min() > 0
    # peer 5 completes a handshake: new indices, new keys, counter back to 0
    a = 5
    peers[a] = (peers[a][0] ^ 0x5A5A0000, peers[a][1] ^ 0x00A5A500, peers[a][2], peers[a][3])
    keys[a] = rng.integers(0, 256, 32, dtype=np.uint8)
    ctx.wg_peer_set(a, peers[a], key_send=keys[a], key_recv=keys[a])
    next_ctr[a] = 0
    assert np.array_equal(ctx.wg_send_counters(N_PEERS), next_ctr)
    check_batch()
    # a netmap push re-installs the whole table: rows with unchanged indices go
    # on counting, the row with fresh indices (peer 9 rekeyed) starts over, and
    # a row added at the end starts at 0
    b = 9
    peers[b] = (peers[b][0] + 1, peers[b][1] + 1, peers[b][2], peers[b][3])
    grown = peers + [(0x7F000001, 0x12345678, 0x64410001, 0xFFFFFFFF)]
    keys = np.concatenate([keys, rng.integers(0, 256, (1, 32), dtype=np.uint8)])
    from bnk_amd import lib
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.wg_peers_set(grown)
    next_ctr[b] = 0
    got = ctx.wg_send_counters(N_PEERS + 1)
    assert np.array_equal(got[:N_PEERS], next_ctr) and got[N_PEERS] == 0
    ctx.wg_peers_set(peers)  # and shrinking keeps the rest
    check_batch()
    # a duplicate local index is refused and changes nothing
    with pytest.raises(lib.BnkError) as ei:
        ctx.wg_peer_set(3, (peers[4][0], 1, 2, 0xFFFFFFFF))
    assert ei.value.code == lib.E_INVAL
    with pytest.raises(lib.BnkError) as ei:
        ctx.wg_peer_set(N_PEERS, peers[0])
    assert ei.value.code == lib.E_RANGE
    check_batch()
    ctx.close()


@pytest.mark.parametrize("fused", ["wave", "lane", "separate"])
@pytest.mark.parametrize("n", [64, 2500])
def test_keypair_stops_sending_at_reject_after_messages(fused, n):
    """wireguard-go sends nothing under a keypair whose nonce counter has
    reached RejectAfterMessages = 2^64 - 2^13 - 1 (device/send.go): such packets
    come back with wire_len 0, untouched, and the counter stays at the limit."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(78)
    peers = _peers(rng)
    keys = rng.integers(0, 256, (N_PEERS, 32), dtype=np.uint8)
    lens = np.full(n, 100, np.uint32)
    peer = (np.arange(n) % 2).astype(np.uint32)  # peers 0 and 1 alternate
    off, total = _layout(rng, 16 + lens.astype(np.int64) + 31)
    arena = np.full(total, 0xEE, np.uint8)
    plains = []
    for i in range(n):
        pt = _inner(rng, peers, int(peer[i]), 100)
        plains.append(pt)
        arena[int(off[i]) + 16:int(off[i]) + 116] = np.frombuffer(pt, np.uint8)
    ctx = _ctx(peers, keys_send=keys)
    _launch_shape(ctx, fused)
    limit = lib.WG_REJECT_AFTER_MESSAGES
    ctx.wg_send_counter_set(0, limit - 3)
    ctx.wg_send_counter_set(1, (1 << 40) + 7)
    nxt = {0: limit - 3, 1: (1 << 40) + 7}
    want = arena.copy()
    want_len = np.zeros(n, np.uint32)
    for i in range(n):
        p = int(peer[i])
        if nxt[p] >= limit:
            continue
        w = O.wg_encap(plains[i], MTU, keys[p].tobytes(), peers[p][1], nxt[p])
        nxt[p] += 1
        want[int(off[i]):int(off[i]) + len(w)] = np.frombuffer(w, np.uint8)
        want_len[i] = len(w)
    got, got_len = _encap_host(ctx, arena, off, lens, peer)
    assert np.array_equal(got_len, want_len) and int((want_len[::2] > 0).sum()) == 3
    assert np.array_equal(got, want)
    ctr = ctx.wg_send_counters(2)
    assert int(ctr[0]) == limit and int(ctr[1]) == (1 << 40) + 7 + n // 2
    # nothing more goes out for peer 0 until it has a new keypair
    got, got_len = _encap_host(ctx, arena, off, lens, peer)
    assert not got_len[::2].any() and got_len[1::2].all()
    ctx.wg_peer_set(0, (peers[0][0] + 2, peers[0][1], peers[0][2], peers[0][3]), key_send=keys[0])
    got, got_len = _encap_host(ctx, arena, off, lens, peer)
    assert got_len.all() and int(ctx.wg_send_counters(1)[0]) == n // 2
    ctx.close()


def test_wg_argument_errors():
    from bnk_amd import lib
    ctx = lib.Context(0)
    arena = np.zeros(4096, np.uint8)
    wl_ = np.zeros(4, np.uint32)
    b = lib.make_batch(arena, arena.nbytes, 4, lib.MEM_HOST, stride=256, length=100)
    with pytest.raises(lib.BnkError) as ei:
        ctx.wg_encap(b, MTU, wl_)
    assert ei.value.code == lib.E_STATE  # no peer table
    with pytest.raises(lib.BnkError) as ei:
        ctx.wg_peers_set([(1, 2, 3, 0xFFFFFFFF), (1, 5, 6, 0xFFFFFFFF)])
    assert ei.value.code == lib.E_INVAL  # duplicate local index
    with pytest.raises(lib.BnkError) as ei:
        ctx.wg_peers_set([(1, 2, 3, 0xFF00FF00)])
    assert ei.value.code == lib.E_INVAL
    ctx.wg_peers_set([(1, 2, 3, 0xFFFFFFFF), (4, 5, 6, 0xFFFFFFFF)])
    with pytest.raises(lib.BnkError) as ei:
        ctx.wg_encap(b, MTU, wl_)
    assert ei.value.code == lib.E_STATE  # no send keys
    ctx.keys_set(lib.KEYS_SEND, np.zeros((2, 32), np.uint8))
    peer = np.array([0, 1, 2, 0], np.uint32)
    with pytest.raises(lib.BnkError) as ei:
        ctx.wg_encap(lib.make_batch(arena, arena.nbytes, 4, lib.MEM_HOST, stride=256, length=100,
                                    peer=peer), MTU, wl_)
    assert ei.value.code == lib.E_RANGE
    with pytest.raises(lib.BnkError) as ei:
        ctx.wg_encap(lib.make_batch(arena, 900, 4, lib.MEM_HOST, stride=256, length=100), MTU, wl_)
    assert ei.value.code == lib.E_INVAL  # last slot has no room for pad + tag
    assert np.array_equal(ctx.wg_send_counters(2), [0, 0])  # refused calls hand out no counters
    ctx.wg_encap(b, MTU, wl_)
    assert np.array_equal(wl_, [16 + 112 + 16] * 4)
    assert np.array_equal(ctx.wg_send_counters(2), [4, 0])
    ctx.close()


def test_full_size_tunnel_round_trips_device_resident():
    """2^20 MTU-sized packets across 1024 peers, device resident, the shape
    bench.py --workload wg times (framing inside the lane-per-packet launches,
    counters from the per-tile counting kernels, anti-replay windows on): two
    encapsulate + decapsulate trips, the second carrying the first one's
    counters on.  Counters follow each peer's order in the batch, every packet
    comes back as it went in, a sample of datagrams is bit-exact against the
    oracle, a trip of the same datagrams once more is all replays, and a few
    tampered datagrams come back as exactly what was done to them."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    dev = torch.device("cuda:0")
    n, n_peers, plen, mtu, stride = 1 << 20, 1024, 1420, 1420, 1456
    wire_len = 16 + plen + 16
    keys = W.rand_bytes(W.stream_seed(2, 40), n_peers * 32).reshape(n_peers, 32)
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
    d_res = torch.full((n,), 99, dtype=torch.uint8, device=dev)
    d_olen = torch.zeros(n, dtype=torch.int32, device=dev)
    d_gp = torch.zeros(n, dtype=torch.int32, device=dev)
    d_gc = torch.zeros(n, dtype=torch.int64, device=dev)
    torch.cuda.synchronize()
    ctx = lib.Context(0)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    ctx.wg_peers_set(np.stack([idx, idx, addr, full], 1))
    nbytes = n * stride
    seq = W.per_peer_sequence(peer, n_peers)
    per_trip = np.bincount(peer, minlength=n_peers).astype(np.uint64)
    sample = [0, 1, 4097, n // 2 + 5, n - 1]
    arenas = (a, b)
    for trip in range(2):
        cur, nxt = arenas[trip & 1], arenas[1 - (trip & 1)]
        plain_before = {i: cur[i * stride + 16:i * stride + 16 + plen].cpu().numpy().tobytes() for i in sample}
        ctx.wg_encap(lib.make_batch(cur, nbytes, n, lib.MEM_DEVICE, stride=stride, length=plen, peer=d_peer),
                     mtu, d_wl)
        ctx.sync()
        assert bool((d_wl == wire_len).all())
        want_ctr = seq + per_trip[peer] * np.uint64(trip)
        for i in sample:
            want = O.wg_encap(plain_before[i], mtu, keys[peer[i]].tobytes(), int(idx[peer[i]]), int(want_ctr[i]))
            assert cur[i * stride:i * stride + wire_len].cpu().numpy().tobytes() == want, (trip, i)
        ctx.wg_decap(lib.make_batch(cur, nbytes, n, lib.MEM_DEVICE, stride=stride, length=wire_len),
                     lib.make_batch(nxt[16:], nbytes, n, lib.MEM_DEVICE, stride=stride), d_res, d_olen, d_gp, d_gc)
        ctx.sync()
        assert bool((d_res == 0).all()) and bool((d_olen == plen).all()) and bool((d_gp == d_peer).all())
        assert np.array_equal(d_gc.cpu().numpy().astype(np.uint64), want_ctr)
        got = nxt[:n * stride].view(n, stride)[:, 16:16 + plen]
        assert torch.equal(got, first_plain)
    assert np.array_equal(ctx.wg_send_counters(n_peers), per_trip * np.uint64(2))
    # the last trip's datagrams (still in `cur`) once more: every one is a replay; before
    # that, tamper with a few: a flipped tag bit, a foreign index, a wrong type
    bad_tag, bad_idx, bad_type = [7, 70000], [8, 900000], [9]
    cv = cur[:n * stride].view(n, stride)
    cv[bad_tag, wire_len - 1] ^= 0x10
    cv[bad_idx, 5] ^= 0xFF
    cv[bad_type, 0] = 1
    torch.cuda.synchronize()
    scratch_out = torch.zeros_like(a)
    ctx.wg_decap(lib.make_batch(cur, nbytes, n, lib.MEM_DEVICE, stride=stride, length=wire_len),
                 lib.make_batch(scratch_out[16:], nbytes, n, lib.MEM_DEVICE, stride=stride), d_res, d_olen, d_gp, d_gc)
    ctx.sync()
    want_res = np.full(n, lib.WG_REPLAY, np.uint8)
    want_res[bad_tag] = lib.WG_AUTH_FAIL
    want_res[bad_idx] = lib.WG_UNKNOWN_INDEX
    want_res[bad_type] = lib.WG_BAD_HEADER
    assert np.array_equal(d_res.cpu().numpy(), want_res)
    assert bool((d_olen == 0).all())
    ctx.close()


@pytest.mark.parametrize("plen", [20, 40, 60, 100, 113])
def test_short_uniform_tunnel_batches_device_resident(plen):
    """Device-resident batches of short packets of one common length: the
    launches in which every wave takes the short path (three waves per SIMD)
    also do the framing -- header, padding as implied zeros, wire lengths on the
    way out; header checks, index lookup and the checks on the inner header on
    the way in.  Every datagram against the oracle, then decapsulated in line
    with the ciphertext, a forged one and a repeat among them."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    dev = torch.device("cuda:0")
    n, n_peers, stride = 20000 + 13, 37, 256
    rng = np.random.default_rng(900 + plen)
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    idx_a = (np.arange(n_peers, dtype=np.uint32) * 7919 + 3).astype(np.uint32)
    idx_b = (np.arange(n_peers, dtype=np.uint32) * 104729 + 11).astype(np.uint32)
    addr = (0x64400000 + np.arange(n_peers, dtype=np.uint32)).astype(np.uint32)
    full = np.full(n_peers, 0xFFFFFFFF, np.uint32)
    side_a = np.stack([idx_a, idx_b, addr, full], 1)
    side_b = np.stack([idx_b, idx_a, addr, full], 1)
    peer = rng.integers(0, n_peers, n).astype(np.uint32)
    h_arena = rng.integers(0, 256, (n, stride), dtype=np.uint8)
    h_arena[:, 16] = 0x45
    h_arena[:, 18], h_arena[:, 19] = plen >> 8, plen & 0xFF
    h_arena[:, 28:32] = addr[peer].astype(">u4").view(np.uint8).reshape(n, 4)
    plain = h_arena[:, 16:16 + plen].copy()
    arena = torch.from_numpy(h_arena).to(dev)
    d_peer = torch.from_numpy(peer.astype(np.int32)).to(dev)
    d_wl = torch.zeros(n, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    padded = (plen + 15) & ~15
    with lib.Context(0) as tx, lib.Context(0) as rx:
        tx.keys_set(lib.KEYS_SEND, keys)
        tx.wg_peers_set(side_a)
        tx.wg_encap(lib.make_batch(arena, arena.numel(), n, lib.MEM_DEVICE, stride=stride, length=plen, peer=d_peer),
                    MTU, d_wl)
        tx.sync()
        assert bool((d_wl == 16 + padded + 16).all())
        rank, seen = np.zeros(n, np.uint64), np.zeros(n_peers, np.uint64)
        for i in range(n):
            rank[i] = seen[peer[i]]
            seen[peer[i]] += 1
        wire = arena.cpu().numpy()
        for i in range(n):
            p = int(peer[i])
            w = O.wg_encap(plain[i].tobytes(), MTU, keys[p].tobytes(), int(idx_b[p]), int(rank[i]))
            assert wire[i, :len(w)].tobytes() == w, i
            assert np.array_equal(wire[i, len(w):], h_arena[i, len(w):]), i  # nothing beyond the datagram written
        # receive: packet 5 forged, packet 9 a copy of packet 8's datagram (a repeat)
        wire[5, 16 + 3] ^= 0x80
        wire[9] = wire[8]
        d_wire = torch.from_numpy(wire).to(dev)
        rx.keys_set(lib.KEYS_RECV, keys)
        rx.wg_peers_set(side_b)
        d_res = torch.full((n,), 99, dtype=torch.uint8, device=dev)
        d_olen = torch.zeros(n, dtype=torch.int32, device=dev)
        d_gp = torch.zeros(n, dtype=torch.int32, device=dev)
        d_gc = torch.zeros(n, dtype=torch.int64, device=dev)
        torch.cuda.synchronize()
        flat = d_wire.view(-1)
        rx.wg_decap(lib.make_batch(flat, flat.numel(), n, lib.MEM_DEVICE, stride=stride, length=16 + padded + 16),
                    lib.make_batch(flat[16:], flat.numel() - 16, n, lib.MEM_DEVICE, stride=stride),
                    d_res, d_olen, d_gp, d_gc)
        rx.sync()
        res = d_res.cpu().numpy()
        want = np.zeros(n, np.uint8)
        want[5], want[9] = lib.WG_AUTH_FAIL, lib.WG_REPLAY
        assert np.array_equal(res, want)
        olen = d_olen.cpu().numpy()
        assert (olen[want == 0] == plen).all() and olen[5] == 0 and olen[9] == 0
        got = d_wire.cpu().numpy()
        ok = np.flatnonzero(want == 0)
        assert np.array_equal(got[ok, 16:16 + plen], plain[ok])
        assert not got[5, 16:16 + padded].any()  # a rejected packet's plaintext is cleared
