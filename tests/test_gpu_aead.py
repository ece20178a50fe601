"""Parity of the HIP seal/open path (through the C ABI) with the CPU oracle:
bit-exact ciphertexts, tags, verdicts and rejected-plaintext zeroing."""
import hashlib
import json
import os

import numpy as np
import pytest

from bnk_amd import workloads as W

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from bnk_amd import lib
    c = lib.Context(0)
    yield c
    c.close()


@pytest.fixture(params=["wave_per_packet", "lane_per_packet"])
def small_ctx(request, ctx):
    """Small batches run one wave per packet by default; with the threshold at
    zero they take the lane-per-packet kernel the large batches use.  Tests of
    small batches run both ways."""
    ctx.set_spread_max_packets(4096 if request.param == "wave_per_packet" else 0)
    yield ctx
    ctx.set_spread_max_packets(4096)


def _oracle_seal(b):
    from oracle import binding as O
    out = np.zeros_like(b.plain)
    O.seal_batch(np.ascontiguousarray(b.keys), b.peer, b.counters, b.plain, b.off, b.lens,
                 out, b.off, 4)
    return out


def _gpu_seal_host(ctx, b, uniform):
    from bnk_amd import lib
    ctx.keys_set(lib.KEYS_SEND, b.keys)
    ctx.keys_set(lib.KEYS_RECV, b.keys)
    out = np.zeros_like(b.plain)
    if uniform:
        inb = lib.make_batch(b.plain, b.plain.nbytes, b.n, lib.MEM_HOST, stride=b.stride,
                             length=int(b.lens[0]), counter0=int(b.counters[0]))
        outb = lib.make_batch(out, out.nbytes, b.n, lib.MEM_HOST, stride=b.stride)
    else:
        inb = lib.make_batch(b.plain, b.plain.nbytes, b.n, lib.MEM_HOST, offsets=b.off,
                             lens=b.lens, peer=b.peer, counters=b.counters)
        outb = lib.make_batch(out, out.nbytes, b.n, lib.MEM_HOST, offsets=b.off)
    ctx.seal(inb, outb)
    return out


def _gpu_open_host(ctx, b, sealed, uniform):
    from bnk_amd import lib
    out = np.full_like(b.plain, 0xEE)
    verdict = np.full(b.n, 7, np.uint8)
    ct_lens = (b.lens + 16).astype(np.uint32)
    if uniform:
        inb = lib.make_batch(sealed, sealed.nbytes, b.n, lib.MEM_HOST, stride=b.stride,
                             length=int(ct_lens[0]), counter0=int(b.counters[0]))
        outb = lib.make_batch(out, out.nbytes, b.n, lib.MEM_HOST, stride=b.stride)
    else:
        inb = lib.make_batch(sealed, sealed.nbytes, b.n, lib.MEM_HOST, offsets=b.off,
                             lens=ct_lens, peer=b.peer, counters=b.counters)
        outb = lib.make_batch(out, out.nbytes, b.n, lib.MEM_HOST, offsets=b.off)
    ctx.open(inb, outb, verdict)
    return out, verdict


def _packets_equal(a, b, off, lens, extra=0):
    """Compare only the packet bytes (the gaps of `a` keep their fill)."""
    for i in range(len(lens)):
        o, L = int(off[i]), int(lens[i]) + extra
        if not np.array_equal(a[o:o + L], b[o:o + L]):
            return i
    return -1


def test_cfg1_against_oracle_and_openssl_fixture(small_ctx):
    ctx = small_ctx
    b = W.aead_uniform(1, 128, 1420)
    got = _gpu_seal_host(ctx, b, uniform=True)
    want = _oracle_seal(b)
    assert np.array_equal(got.reshape(128, b.stride)[:, :1436],
                          want.reshape(128, b.stride)[:, :1436])
    # bytes of each slot beyond the tag stay as the caller left them
    assert not got.reshape(128, b.stride)[:, 1436:].any()
    g = json.load(open(os.path.join(os.path.dirname(__file__), "golden",
                                    "aead_cfg1_openssl.json")))
    sealed = got.reshape(128, b.stride)[:, :1436]
    assert hashlib.sha256(sealed.tobytes()).hexdigest() == g["sha256_all_sealed"]
    for idx, hx in g["packets"].items():
        assert sealed[int(idx)].tobytes().hex() == hx
    back, verdict = _gpu_open_host(ctx, b, got, uniform=True)
    assert verdict.tolist() == [1] * 128
    assert np.array_equal(back.reshape(128, b.stride)[:, :1420],
                          b.plain.reshape(128, b.stride)[:, :1420])
    assert (back.reshape(128, b.stride)[:, 1420:] == 0xEE).all()


EDGE_LENS = [0, 1, 3, 4, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 79, 80, 127, 128, 129,
             255, 256, 575, 576, 1419, 1420, 1421, 1424, 1500, 4096, 9000]


def test_edge_lengths_and_high_counters(small_ctx):
    ctx = small_ctx
    lens = np.array(EDGE_LENS * 3, np.uint32)
    b = W.aead_imix(11, len(lens), n_peers=5, lens=lens)
    # counters straddling 2^32 and the top of the 64-bit range
    b.counters[:8] = np.array([0, 1, 0xFFFFFFFF, 1 << 32, (1 << 32) + 1, (1 << 63),
                               (1 << 64) - 2, (1 << 64) - 1], np.uint64)
    got = _gpu_seal_host(ctx, b, uniform=False)
    want = _oracle_seal(b)
    assert _packets_equal(got, want, b.off, b.lens, 16) == -1
    assert np.array_equal(got, want)  # gaps untouched too (both started from zeros)
    back, verdict = _gpu_open_host(ctx, b, got, uniform=False)
    assert verdict.all()
    assert _packets_equal(back, b.plain, b.off, b.lens) == -1


@pytest.mark.parametrize("half", [0, 1])
@pytest.mark.parametrize("misalign", [False, True])
def test_every_length_through_one_wave_and_beyond(small_ctx, half, misalign):
    """Every plaintext length from 0 to 4200 bytes: all the shapes of a packet
    spread over a wave (cells, blocks, lanes partly filled, the 63-block limit
    at 4032 bytes and the single-lane fallback beyond it), at aligned and at
    arbitrary byte offsets, forged tags among them."""
    from bnk_amd import lib
    from oracle import binding as O
    ctx = small_ctx
    lens = np.arange(half, 4201, 2, dtype=np.uint32)
    n = len(lens)
    rng = np.random.default_rng(40 + half + 2 * misalign)
    rng.shuffle(lens)
    gaps = rng.integers(0, 16, n) if misalign else np.zeros(n, np.int64)
    room = ((lens.astype(np.int64) + 16 + 15) & ~15) + 16
    off = (np.concatenate([[0], np.cumsum(room)[:-1]]) + gaps).astype(np.uint64)
    total = int(room.sum()) + 16
    plain = rng.integers(0, 256, total, dtype=np.uint8)
    keys = rng.integers(0, 256, (3, 32), dtype=np.uint8)
    peer = rng.integers(0, 3, n).astype(np.uint32)
    counters = rng.integers(0, 1 << 63, n, dtype=np.uint64)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    want = np.full(total, 0x5A, np.uint8)
    O.seal_batch(keys, peer, counters, plain, off, lens, want, off, 4)
    got = np.full(total, 0x5A, np.uint8)
    ctx.seal(lib.make_batch(plain, total, n, lib.MEM_HOST, offsets=off, lens=lens, peer=peer, counters=counters),
             lib.make_batch(got, total, n, lib.MEM_HOST, offsets=off))
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, f"first differing byte at {bad[:3]}"
    forged = W.forge_tags(41, got, off, lens, 0.05)
    ct_lens = (lens + 16).astype(np.uint32)
    back = np.full(total, 0xEE, np.uint8)
    verdict = np.full(n, 7, np.uint8)
    ctx.open(lib.make_batch(got, total, n, lib.MEM_HOST, offsets=off, lens=ct_lens, peer=peer, counters=counters),
             lib.make_batch(back, total, n, lib.MEM_HOST, offsets=off), verdict)
    oback = np.full(total, 0xEE, np.uint8)
    overdict = O.open_batch(keys, peer, counters, got, off, ct_lens, oback, off, 4)
    assert np.array_equal(verdict, overdict) and np.array_equal(verdict == 0, forged)
    assert np.array_equal(back, oback)


@pytest.mark.parametrize("n", [64, 128, 100])
def test_unsorted_mixed_lengths_within_a_wave(small_ctx, n):
    ctx = small_ctx
    """Up to 64 packets are not grouped by length, so one wave holds long and
    short packets at once: the lines inside every packet of the wave take the
    unchecked route, the others the bounds-checked one, and a partly filled
    wave takes the checked one throughout.  Every alignment class of a
    128-byte line occurs as the first byte of some packet."""
    rng = np.random.default_rng(n)
    lens = rng.integers(130, 1500, n).astype(np.uint32)
    lens[::7] = rng.choice([128, 129, 255, 256, 257, 1408, 1420, 1499], len(lens[::7]))
    b = W.aead_imix(13, n, n_peers=3, lens=lens)
    assert len({int(o) & 127 for o in b.off}) >= 6
    got = _gpu_seal_host(ctx, b, uniform=False)
    want = _oracle_seal(b)
    assert np.array_equal(got, want)
    W.forge_tags(13, got, b.off, b.lens, 0.1)
    back, verdict = _gpu_open_host(ctx, b, got, uniform=False)
    from oracle import binding as O
    oback = np.full_like(b.plain, 0xEE)
    overdict = O.open_batch(np.ascontiguousarray(b.keys), b.peer, b.counters, got, b.off,
                            (b.lens + 16).astype(np.uint32), oback, b.off, 2)
    assert np.array_equal(verdict, overdict) and 0 < int((verdict == 0).sum()) < n
    assert np.array_equal(back, oback)


def test_imix_multi_peer_with_forged_tags(small_ctx):
    ctx = small_ctx
    from oracle import binding as O
    b = W.aead_imix(3, 6000, n_peers=256)
    got = _gpu_seal_host(ctx, b, uniform=False)
    want = _oracle_seal(b)
    assert np.array_equal(got, want)
    forged = W.forge_tags(3, got, b.off, b.lens, 0.01)
    assert forged.sum() == 60
    back, verdict = _gpu_open_host(ctx, b, got, uniform=False)
    oback = np.full_like(b.plain, 0xEE)
    overdict = O.open_batch(np.ascontiguousarray(b.keys), b.peer, b.counters, got, b.off,
                            (b.lens + 16).astype(np.uint32), oback, b.off, 4)
    assert np.array_equal(verdict, overdict)
    assert np.array_equal(verdict == 0, forged)
    assert np.array_equal(back, oback)  # rejected plaintexts are zero-filled
    i = int(np.flatnonzero(forged)[0])
    o, L = int(b.off[i]), int(b.lens[i])
    assert not back[o:o + L].any()


def test_maximum_packet_sizes(small_ctx):
    ctx = small_ctx
    """Jumbo frames and the largest length a 16-bit IP total-length field can
    name (65,535), next to minimum-size packets: more ChaCha20 blocks than the
    length grouping has bins, in both memory paths' batch sizes."""
    lens = np.array([65535, 65519, 65520, 9000, 8999, 9001, 4096, 60, 0, 1] * 7, np.uint32)
    b = W.aead_imix(15, len(lens), n_peers=4, lens=lens)
    got = _gpu_seal_host(ctx, b, uniform=False)
    want = _oracle_seal(b)
    assert np.array_equal(got, want)
    forged = W.forge_tags(15, got, b.off, b.lens, 0.1)
    back, verdict = _gpu_open_host(ctx, b, got, uniform=False)
    assert np.array_equal(verdict == 0, forged)
    for i in range(b.n):
        o, L = int(b.off[i]), int(b.lens[i])
        if forged[i]:
            assert not back[o:o + L].any()
        else:
            assert np.array_equal(back[o:o + L], b.plain[o:o + L])


@pytest.mark.parametrize("layout", ["offsets", "reversed", "in_place", "uniform"])
def test_large_host_batches_take_the_chunked_route(ctx, layout):
    """Host batches of several chunks' worth are uploaded, computed and
    downloaded chunk by chunk with the three overlapped; a layout whose packets
    do not ascend through the arena takes the single-shot route.  Either way:
    oracle-exact bytes, verdicts, zero-filled rejects and untouched gaps."""
    from bnk_amd import lib
    from oracle import binding as O
    if layout == "uniform":
        n, L, stride = 20000, 1420, 1472
        b = W.aead_uniform(14, n, L, stride=stride, counter0=1 << 33)
    else:
        n = 40000
        b = W.aead_imix(14, n, n_peers=64)
    assert b.plain.nbytes > 3 * (4 << 20)
    off = b.off
    peer, counters, lens = b.peer, b.counters, b.lens
    if layout == "reversed":
        perm = np.arange(n)[::-1].copy()
        off, peer, counters, lens = off[perm].copy(), peer[perm].copy(), counters[perm].copy(), lens[perm].copy()
    keys = np.ascontiguousarray(b.keys)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    want = np.full_like(b.plain, 0x5A)
    O.seal_batch(keys, peer, counters, b.plain, off, lens, want, off, 4)
    ct_lens = (lens + 16).astype(np.uint32)

    def batch(buf, ln, with_meta=True):
        if layout == "uniform":
            return lib.make_batch(buf, buf.nbytes, n, lib.MEM_HOST, stride=b.stride,
                                  length=int(ln[0]) if with_meta else 0, counter0=1 << 33)
        return lib.make_batch(buf, buf.nbytes, n, lib.MEM_HOST, offsets=off,
                              lens=ln if with_meta else None, peer=peer if with_meta else None,
                              counters=counters if with_meta else None)

    if layout == "in_place":
        got = b.plain.copy()
        ctx.seal(batch(got, lens), batch(got, lens, False))
        # only the packets and their tags changed
        assert _packets_equal(got, want, off, lens, 16) == -1
        mask = np.ones(got.size, bool)
        for o, l in zip(off.astype(np.int64), lens.astype(np.int64)):
            mask[o:o + l + 16] = False
        assert np.array_equal(got[mask], b.plain[mask])
    else:
        got = np.full_like(b.plain, 0x5A)
        ctx.seal(batch(b.plain, lens), batch(got, lens, False))
        assert np.array_equal(got, want)  # the 0x5A between packets survived
    forged = W.forge_tags(14, got, off, lens, 0.02)
    back = np.full_like(b.plain, 0xEE)
    verdict = np.full(n, 7, np.uint8)
    ctx.open(batch(got, ct_lens), batch(back, lens, False), verdict)
    oback = np.full_like(b.plain, 0xEE)
    overdict = O.open_batch(keys, peer, counters, got, off, ct_lens, oback, off, 4)
    assert np.array_equal(verdict, overdict)
    assert np.array_equal(verdict == 0, forged) and forged.sum() == int(0.02 * n)
    assert np.array_equal(back, oback)


@pytest.mark.parametrize("layout", ["offsets", "reversed", "in_place", "uniform"])
@pytest.mark.parametrize("n", [1, 70, 3000])
def test_small_batches_in_pinned_rings(small_ctx, layout, n):
    """Host batches of up to a few megabytes whose arenas are pinned rings of
    the context are read and written in place by the kernels (no staging
    copies).  Same bar as the staged routes: oracle-exact bytes, verdicts,
    zero-filled rejects and untouched gaps."""
    ctx = small_ctx
    from bnk_amd import lib
    from oracle import binding as O
    if layout == "uniform":
        b = W.aead_uniform(15, n, 333, stride=352, counter0=(1 << 40) + 5)
    else:
        b = W.aead_imix(15, n, n_peers=8)
    off, peer, counters, lens = b.off, b.peer, b.counters, b.lens
    if layout == "reversed":
        perm = np.arange(n)[::-1].copy()
        off, peer, counters, lens = off[perm].copy(), peer[perm].copy(), counters[perm].copy(), lens[perm].copy()
    keys = np.ascontiguousarray(b.keys)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    want = np.full_like(b.plain, 0x5A)
    O.seal_batch(keys, peer, counters, b.plain, off, lens, want, off, 4)
    ct_lens = (lens + 16).astype(np.uint32)
    nbytes = b.plain.nbytes
    rings = [ctx.ring_alloc(nbytes + 64) for _ in range(3)]
    # arenas that start inside a ring, not at its base
    src, got, back = (r[32:32 + nbytes] for r in rings)

    def batch(buf, ln, with_meta=True):
        if layout == "uniform":
            return lib.make_batch(buf, nbytes, n, lib.MEM_HOST, stride=b.stride,
                                  length=int(ln[0]) if with_meta else 0, counter0=(1 << 40) + 5)
        return lib.make_batch(buf, nbytes, n, lib.MEM_HOST, offsets=off,
                              lens=ln if with_meta else None, peer=peer if with_meta else None,
                              counters=counters if with_meta else None)

    try:
        if layout == "in_place":
            got[:] = b.plain
            ctx.seal(batch(got, lens), batch(got, lens, False))
            assert _packets_equal(got, want, off, lens, 16) == -1
            mask = np.ones(got.size, bool)
            for o, l in zip(off.astype(np.int64), lens.astype(np.int64)):
                mask[o:o + l + 16] = False
            assert np.array_equal(got[mask], b.plain[mask])
        else:
            src[:] = b.plain
            got[:] = 0x5A
            ctx.seal(batch(src, lens), batch(got, lens, False))
            assert np.array_equal(got, want)
        forged = W.forge_tags(15, got, off, lens, 0.1) if n > 1 else np.zeros(1, bool)
        back[:] = 0xEE
        verdict = np.full(n, 7, np.uint8)
        ctx.open(batch(got, ct_lens), batch(back, lens, False), verdict)
        oback = np.full_like(b.plain, 0xEE)
        overdict = O.open_batch(keys, peer, counters, np.array(got), off, ct_lens, oback, off, 4)
        assert np.array_equal(verdict, overdict)
        assert np.array_equal(verdict == 0, forged)
        assert np.array_equal(back, oback)
        # a ring that has been freed is staged like any other host memory
        spare = ctx.ring_alloc(nbytes)
        ctx.ring_free(spare)
    finally:
        for r in rings:
            ctx.ring_free(r)


def test_random_shapes_through_pinned_rings(ctx):
    """Three hundred batches of random size (1 to 5000 packets), length mix,
    alignment and kernel choice, one after the other through the same rings
    and the same context: every sealed byte and every gap against the oracle,
    every packet back."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(2026)
    n_keys = 9
    keys = rng.integers(0, 256, (n_keys, 32), dtype=np.uint8)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    rings = [ctx.ring_alloc(9 << 20) for _ in range(3)]
    try:
        for it in range(300):
            n = int(rng.choice([1, 2, 63, 64, 65, 128, 500, 1024, 3000, 5000]))
            lens = rng.integers(0, int(rng.choice([64, 200, 1500])) + 1, n).astype(np.uint32)
            room = ((lens.astype(np.int64) + 16 + 15) & ~15) + 16
            gaps = rng.integers(0, 16, n) if rng.integers(0, 2) else np.zeros(n, np.int64)
            off = (np.concatenate([[0], np.cumsum(room)[:-1]]) + gaps).astype(np.uint64)
            total = int(room.sum()) + 16
            ctx.set_spread_max_packets(int(rng.choice([0, 4096])))
            plain = rng.integers(0, 256, total, dtype=np.uint8)
            peer = rng.integers(0, n_keys, n).astype(np.uint32)
            counters = rng.integers(0, 1 << 63, n, dtype=np.uint64)
            want = np.full(total, 0x5A, np.uint8)
            O.seal_batch(keys, peer, counters, plain, off, lens, want, off, 4)
            a, b, c = (r[:total] for r in rings)
            a[:] = plain
            b[:] = 0x5A
            c[:] = 0xEE
            ctx.seal(lib.make_batch(a, total, n, lib.MEM_HOST, offsets=off, lens=lens, peer=peer, counters=counters),
                     lib.make_batch(b, total, n, lib.MEM_HOST, offsets=off))
            assert np.array_equal(b, want), f"batch {it}: {n} packets"
            verdict = np.zeros(n, np.uint8)
            ctx.open(lib.make_batch(b, total, n, lib.MEM_HOST, offsets=off, lens=(lens + 16).astype(np.uint32),
                                    peer=peer, counters=counters),
                     lib.make_batch(c, total, n, lib.MEM_HOST, offsets=off), verdict)
            assert verdict.all() and _packets_equal(c, plain, off, lens) == -1, f"batch {it}: {n} packets"
    finally:
        ctx.set_spread_max_packets(4096)
        for r in rings:
            ctx.ring_free(r)


def test_in_place_and_unaligned_slots(small_ctx):
    ctx = small_ctx
    """WireGuard seals in place at offset 16 of its buffers; slots need not be
    16-byte aligned."""
    from bnk_amd import lib
    from oracle import binding as O
    n, L, stride = 70, 1001, 1051  # odd stride: every alignment class occurs
    b = W.aead_uniform(12, n, L, stride=stride, counter0=5)
    ctx.keys_set(lib.KEYS_SEND, b.keys)
    ctx.keys_set(lib.KEYS_RECV, b.keys)
    arena = np.concatenate([np.full(13, 0x5A, np.uint8), b.plain])  # odd base offset
    view = arena[13:]
    work = arena.copy()
    wv = work[13:]
    inb = lib.make_batch(wv, wv.nbytes, n, lib.MEM_HOST, stride=stride, length=L, counter0=5)
    ctx.seal(inb, inb)
    want = np.zeros_like(b.plain)
    O.seal_batch(np.ascontiguousarray(b.keys), b.peer, b.counters, b.plain, b.off, b.lens,
                 want, b.off, 2)
    g2 = wv.reshape(n, stride)
    w2 = want.reshape(n, stride)
    assert np.array_equal(g2[:, :L + 16], w2[:, :L + 16])
    assert np.array_equal(g2[:, L + 16:], view.reshape(n, stride)[:, L + 16:])
    assert (work[:13] == 0x5A).all()
    verdict = np.zeros(n, np.uint8)
    opb = lib.make_batch(wv, wv.nbytes, n, lib.MEM_HOST, stride=stride, length=L + 16, counter0=5)
    ctx.open(opb, opb, verdict)
    assert verdict.all()
    assert np.array_equal(wv.reshape(n, stride)[:, :L], view.reshape(n, stride)[:, :L])


@pytest.mark.parametrize("mem", ["pageable", "ring"])
def test_short_and_error_paths(small_ctx, mem):
    ctx = small_ctx
    from bnk_amd import lib
    b = W.aead_uniform(13, 4, 32)
    ctx.keys_set(lib.KEYS_SEND, b.keys)
    ctx.keys_set(lib.KEYS_RECV, b.keys)
    # ciphertext shorter than a tag: verdict 0, nothing written
    rings = [ctx.ring_alloc(64) for _ in range(3)] if mem == "ring" else []
    buf, out, ka = rings if rings else (np.zeros(64, np.uint8), np.zeros(64, np.uint8), np.zeros(32, np.uint8))
    buf[:] = 0
    out[:] = 0xEE
    ka = ka[:32]
    ka[:] = 0
    v = np.full(2, 9, np.uint8)
    inb = lib.make_batch(buf, 64, 2, lib.MEM_HOST, stride=32, length=15)
    outb = lib.make_batch(out, 64, 2, lib.MEM_HOST, stride=32)
    ctx.open(inb, outb, v)
    assert v.tolist() == [0, 0] and (out == 0xEE).all()
    # empty batch is a no-op
    ctx.seal(lib.make_batch(buf, 64, 0, lib.MEM_HOST), lib.make_batch(out, 64, 0, lib.MEM_HOST))
    # packet outside the arena
    with pytest.raises(lib.BnkError) as ei:
        ctx.seal(lib.make_batch(buf, 64, 2, lib.MEM_HOST, stride=32, length=32),
                 lib.make_batch(out, 64, 2, lib.MEM_HOST, stride=32))
    assert ei.value.code == lib.E_INVAL
    # peer beyond the key table
    with pytest.raises(lib.BnkError) as ei:
        ctx.seal(lib.make_batch(buf, 64, 2, lib.MEM_HOST, stride=32, length=8,
                                peer=np.array([0, 3], np.uint32)),
                 lib.make_batch(out, 64, 2, lib.MEM_HOST, stride=32))
    assert ei.value.code == lib.E_RANGE
    # keepalive: empty plaintext seals to just a tag, and opens
    ctx.seal(lib.make_batch(ka, 32, 2, lib.MEM_HOST, stride=16, length=0, counter0=9),
             lib.make_batch(ka, 32, 2, lib.MEM_HOST, stride=16))
    from oracle import binding as O
    assert ka[:16].tobytes() == O.aead_seal(b.keys[0].tobytes(), O.wg_nonce(9), b"")
    v = np.zeros(2, np.uint8)
    ctx.open(lib.make_batch(ka, 32, 2, lib.MEM_HOST, stride=16, length=16, counter0=9),
             lib.make_batch(ka, 32, 2, lib.MEM_HOST, stride=16), v)
    assert v.tolist() == [1, 1]
    for r in rings:
        ctx.ring_free(r)


def test_device_resident_large_batch_properties(ctx):
    """At a size the oracle cannot finish quickly: seal -> open round trip is
    the identity, every verdict is 1, and a sample of packets is bit-exact
    against the oracle."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    n, L, stride = 1 << 18, 1420, 1440
    key = W.rand_bytes(W.stream_seed(2, 0), 32).reshape(1, 32)
    ctx.keys_set(lib.KEYS_SEND, key)
    ctx.keys_set(lib.KEYS_RECV, key)
    g = torch.Generator(device="cuda").manual_seed(2)
    pt = torch.randint(0, 256, (n, stride), dtype=torch.uint8, device="cuda", generator=g)
    ct = torch.zeros_like(pt)
    back = torch.zeros_like(pt)
    verdict = torch.zeros(n, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    nb = n * stride
    ctx.seal(lib.make_batch(pt, nb, n, lib.MEM_DEVICE, stride=stride, length=L, counter0=1000),
             lib.make_batch(ct, nb, n, lib.MEM_DEVICE, stride=stride))
    ctx.open(lib.make_batch(ct, nb, n, lib.MEM_DEVICE, stride=stride, length=L + 16,
                            counter0=1000),
             lib.make_batch(back, nb, n, lib.MEM_DEVICE, stride=stride), verdict)
    ctx.sync()
    assert bool(verdict.all())
    assert torch.equal(back[:, :L], pt[:, :L])
    assert not bool(back[:, L:].any())
    for i in (0, 1, 63, 64, 4097, n - 1):
        want = O.aead_seal(key.tobytes(), O.wg_nonce(1000 + i), pt[i, :L].cpu().numpy().tobytes())
        assert ct[i, :L + 16].cpu().numpy().tobytes() == want
    # linearity of the stream cipher: ct(a) ^ ct(b) == a ^ b under the same nonce
    pt2 = pt.clone(); pt2[:, :L] ^= 0x3C
    ct2 = torch.zeros_like(pt)
    torch.cuda.synchronize()  # torch's fills run on its own stream
    ctx.seal(lib.make_batch(pt2, nb, n, lib.MEM_DEVICE, stride=stride, length=L, counter0=1000),
             lib.make_batch(ct2, nb, n, lib.MEM_DEVICE, stride=stride))
    ctx.sync()
    assert bool(((ct[:, :L] ^ ct2[:, :L]) == 0x3C).all())
    assert not torch.equal(ct[:, L:L + 16], ct2[:, L:L + 16])


@pytest.mark.parametrize("align", [16, 128])
def test_cfg3_full_size_imix_with_forged_tags(ctx, align):
    """Configuration 3 at full size (2^20 IMIX packets, 256 peers, 1 % of the
    tags with one seeded bit flipped), device resident, slots back to back at
    16-byte alignment (packets share 128-byte lines) and at 128 (the layout
    bench.py times): rejects are exactly the forged packets and their plaintext
    is zero, every other packet opens to what was sealed, nothing between
    packets is written, and a sample of sealed packets is bit-exact against the
    oracle."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    n = 1 << 20
    b = W.aead_imix(3, n, n_peers=256, payload=False, align=align)
    dev = torch.device("cuda:0")
    total = b.meta["total"]
    plain = W.imix_plain_torch(b, dev)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    d_off, d_peer, d_ctr = d(b.off.astype(np.int64)), d(b.peer.astype(np.int32)), d(b.counters.astype(np.int64))
    d_lens, d_ctl = d(b.lens.astype(np.int32)), d((b.lens + 16).astype(np.int32))
    sealed = torch.full((total,), 0x5A, dtype=torch.uint8, device=dev)
    back = torch.full((total,), 0xA5, dtype=torch.uint8, device=dev)
    v = torch.full((n,), 7, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    keys = np.ascontiguousarray(b.keys)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    ctx.seal(lib.make_batch(plain, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens, peer=d_peer,
                            counters=d_ctr),
             lib.make_batch(sealed, total, n, lib.MEM_DEVICE, offsets=d_off))
    ctx.sync()
    # sample against the oracle, all three sizes
    for L in W.IMIX_SIZES:
        for i in np.flatnonzero(b.lens == L)[[0, 1, -1]]:
            o = int(b.off[i])
            pt = plain[o:o + L].cpu().numpy().tobytes()
            want = O.aead_seal(keys[b.peer[i]].tobytes(), O.wg_nonce(int(b.counters[i])), pt)
            assert sealed[o:o + L + 16].cpu().numpy().tobytes() == want
    # forge 1 % of the tags
    k = int(0.01 * n)
    which = W.permutation(W.stream_seed(3, 5), n)[:k].astype(np.int64)
    bit = W.rand_below(W.stream_seed(3, 6), k, 128)
    pos = b.off[which].astype(np.int64) + b.lens[which].astype(np.int64) + (bit >> 3).astype(np.int64)
    sealed[d(pos)] ^= d((1 << (bit & 7)).astype(np.uint8))
    torch.cuda.synchronize()
    ctx.open(lib.make_batch(sealed, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_ctl, peer=d_peer,
                            counters=d_ctr),
             lib.make_batch(back, total, n, lib.MEM_DEVICE, offsets=d_off), v)
    ctx.sync()
    forged = np.zeros(n, bool)
    forged[which] = True
    assert k == 10485 and np.array_equal(v.cpu().numpy() == 0, forged)
    # byte-level expectation: packet bytes = plaintext (zeros where forged), everything else untouched
    is_pkt = torch.zeros(total + 1, dtype=torch.int32, device=dev)
    is_pkt.index_add_(0, d_off, torch.ones(n, dtype=torch.int32, device=dev))
    is_pkt.index_add_(0, d_off + d_lens.long(), -torch.ones(n, dtype=torch.int32, device=dev))
    inside = torch.cumsum(is_pkt[:total], 0) > 0
    zero = torch.zeros(total + 1, dtype=torch.int32, device=dev)
    f_off, f_len = d_off[d(which)], d_lens.long()[d(which)]
    zero.index_add_(0, f_off, torch.ones(k, dtype=torch.int32, device=dev))
    zero.index_add_(0, f_off + f_len, -torch.ones(k, dtype=torch.int32, device=dev))
    zeroed = torch.cumsum(zero[:total], 0) > 0
    want = torch.where(inside, torch.where(zeroed, torch.zeros_like(plain), plain),
                       torch.full_like(plain, 0xA5))
    assert torch.equal(back, want)


def test_concurrent_callers_share_one_context(ctx):
    """wireguard-go calls Seal from one goroutine per peer: entry points on one
    context may be called from several threads at once and are serialised
    inside the library; every caller gets its own correct result."""
    import threading
    from bnk_amd import lib
    b0 = W.aead_imix(21, 3000, n_peers=8)
    keys = np.ascontiguousarray(b0.keys)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    want = _oracle_seal(b0)
    errors = []

    def worker(tid):
        rings = []
        try:
            # odd threads keep their packets in pinned rings of the shared context
            # (allocated, used in place and freed while the others are calling)
            if tid % 2:
                rings = [ctx.ring_alloc(b0.plain.nbytes) for _ in range(2)]
            for it in range(6):
                out = rings[0] if rings else np.zeros_like(b0.plain)
                out[:] = 0
                ctx.seal(lib.make_batch(b0.plain, b0.plain.nbytes, b0.n, lib.MEM_HOST, offsets=b0.off,
                                        lens=b0.lens, peer=b0.peer, counters=b0.counters),
                         lib.make_batch(out, out.nbytes, b0.n, lib.MEM_HOST, offsets=b0.off))
                if not np.array_equal(out, want):
                    errors.append((tid, it, "seal"))
                back = rings[1] if rings else np.zeros_like(b0.plain)
                back[:] = 0
                v = np.zeros(b0.n, np.uint8)
                ctx.open(lib.make_batch(out, out.nbytes, b0.n, lib.MEM_HOST, offsets=b0.off,
                                        lens=(b0.lens + 16).astype(np.uint32), peer=b0.peer,
                                        counters=b0.counters),
                         lib.make_batch(back, back.nbytes, b0.n, lib.MEM_HOST, offsets=b0.off), v)
                if not (v.all() and _packets_equal(back, b0.plain, b0.off, b0.lens) == -1):
                    errors.append((tid, it, "open"))
        except Exception as e:  # noqa: BLE001
            errors.append((tid, repr(e)))
        finally:
            for r in rings:
                ctx.ring_free(r)

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors[:3]


@pytest.mark.parametrize("length", [0, 1, 15, 16, 17, 60, 63, 64, 65, 100, 127, 128, 129])
@pytest.mark.parametrize("stride,shift", [(256, 0), (160, 16), (176, 48)])
def test_uniform_short_device_batches_against_the_oracle(ctx, length, stride, shift):
    """Device-resident batches of one common length up to 128 bytes with every
    packet 16-byte aligned at the same place of a line in both arenas run in a
    launch of their own (more waves per SIMD); 129 bytes and the strides that
    put packets across two lines take the other paths.  Every ciphertext and
    tag against the oracle, the round trip, and a forged tag's zero-fill."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    n = 40000 + 37  # beyond the wave-per-packet launches, and not a whole number of waves
    rng = np.random.default_rng(1000 + length)
    keys = rng.integers(0, 256, (3, 32), dtype=np.uint8)
    ctx.keys_set(lib.KEYS_SEND, keys)
    ctx.keys_set(lib.KEYS_RECV, keys)
    peer = rng.integers(0, 3, n).astype(np.uint32)
    ctr = rng.integers(0, 1 << 62, n).astype(np.uint64)
    nb = n * stride + shift + 64
    plain = rng.integers(0, 256, nb, dtype=np.uint8)
    off = (np.arange(n, dtype=np.uint64) * np.uint64(stride)) + np.uint64(shift)
    want = np.zeros(nb, np.uint8)
    O.seal_batch(keys, peer, ctr, plain, off, np.full(n, length, np.uint32), want, off, 4)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")  # noqa: E731
    d_plain, d_ct = d(plain), torch.zeros(nb, dtype=torch.uint8, device="cuda:0")
    d_back = torch.full((nb,), 0xEE, dtype=torch.uint8, device="cuda:0")
    d_peer, d_ctr = d(peer.astype(np.int32)), d(ctr.astype(np.int64))
    verdict = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
    torch.cuda.synchronize()
    view = lambda t: t[shift:]  # noqa: E731  (the batch starts `shift` bytes into the allocation)
    ctx.seal(lib.make_batch(view(d_plain), nb - shift, n, lib.MEM_DEVICE, stride=stride, length=length, peer=d_peer,
                            counters=d_ctr),
             lib.make_batch(view(d_ct), nb - shift, n, lib.MEM_DEVICE, stride=stride))
    ctx.sync()
    got = d_ct.cpu().numpy()
    assert np.array_equal(got, want)  # nothing between or beyond the packets was written either
    forged = rng.choice(n, 9, replace=False)
    got2 = got.copy()
    got2[(off[forged] + np.uint64(length + 5)).astype(np.int64)] ^= 0x40
    d_ct2 = d(got2)
    torch.cuda.synchronize()
    ctx.open(lib.make_batch(view(d_ct2), nb - shift, n, lib.MEM_DEVICE, stride=stride, length=length + 16,
                            peer=d_peer, counters=d_ctr),
             lib.make_batch(view(d_back), nb - shift, n, lib.MEM_DEVICE, stride=stride), verdict)
    ctx.sync()
    v = verdict.cpu().numpy()
    expect_v = np.ones(n, np.uint8)
    expect_v[forged] = 0
    assert np.array_equal(v, expect_v)
    back = d_back.cpu().numpy()
    expect = np.full(nb, 0xEE, np.uint8)
    for i in range(n):
        o = int(off[i])
        expect[o:o + length] = 0 if v[i] == 0 else plain[o:o + length]
    assert np.array_equal(back, expect)
