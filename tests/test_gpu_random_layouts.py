"""Large device-resident batches with seeded random lengths, alignments and
peers: sealed arenas equal the oracle's byte for byte (bytes between packets
included), forged tags are rejected and their plaintext left as zeros, every
other packet opens to what was sealed.  Each seed picks a length mix (uniform
random up to 1500, the IMIX sizes, short packets only, or block and line
boundaries with a 4100-byte packet among them) and a layout (slots at 1-, 4-,
16- or 128-byte alignment), so the aligned, short, unaligned and generic
paths of the lane-per-packet kernels all see ragged input."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(16))
def test_random_lengths_and_alignments_match_the_oracle(seed):
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(1000 + seed)
    dev = torch.device("cuda:0")
    n_peers = 33
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    n = int(rng.choice([30000, 70000]))
    kind = seed % 4
    if kind == 0:
        lens = rng.integers(0, 1501, n)
    elif kind == 1:
        lens = rng.choice([60, 576, 1420], n, p=[7 / 12, 4 / 12, 1 / 12])
    elif kind == 2:
        lens = rng.integers(0, 130, n)
    else:
        lens = rng.choice([0, 1, 15, 16, 17, 63, 64, 65, 127, 128, 129, 1419, 1420, 4100], n)
    lens = lens.astype(np.uint32)
    align = [1, 4, 16, 128][(seed // 4 + seed) % 4]
    if align == 1:
        gap = rng.integers(0, 16, n)
    elif align == 4:
        gap = rng.integers(0, 4, n) * 4
    else:
        gap = np.zeros(n, np.int64)
    unit = 128 if align == 128 else 16
    room = ((lens.astype(np.int64) + 16 + unit - 1) // unit) * unit + (16 if align < 16 else 0)
    off = (np.concatenate([[0], np.cumsum(room)[:-1]]) + gap).astype(np.uint64)
    total = int(room.sum()) + 32
    plain = rng.integers(0, 256, total, dtype=np.uint8)
    peer = rng.integers(0, n_peers, n).astype(np.uint32)
    ctrs = rng.integers(0, 1 << 63, n, dtype=np.uint64)
    want = np.full(total, 0x5A, np.uint8)
    O.seal_batch(keys, peer, ctrs, plain, off, lens, want, off, 8)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    d_plain = d(plain)
    d_sealed = torch.full((total,), 0x5A, dtype=torch.uint8, device=dev)
    d_off, d_len, d_ctl = d(off.astype(np.int64)), d(lens.astype(np.int32)), d((lens + 16).astype(np.int32))
    d_peer, d_ctr = d(peer.astype(np.int32)), d(ctrs.astype(np.int64))
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_SEND, keys)
        ctx.keys_set(lib.KEYS_RECV, keys)
        ctx.seal(lib.make_batch(d_plain, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_len, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(d_sealed, total, n, lib.MEM_DEVICE, offsets=d_off))
        ctx.sync()
        got = d_sealed.cpu().numpy()
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, f"kind {kind} align {align}: first differing byte at {bad[:4]}"
        forged = rng.permutation(n)[:40]
        pos = off[forged].astype(np.int64) + lens[forged].astype(np.int64) + 3
        d_sealed[d(pos)] ^= 0x40
        d_back = torch.full((total,), 0xA5, dtype=torch.uint8, device=dev)
        d_v = torch.full((n,), 9, dtype=torch.uint8, device=dev)
        ctx.open(lib.make_batch(d_sealed, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_ctl, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(d_back, total, n, lib.MEM_DEVICE, offsets=d_off), d_v)
        ctx.sync()
    exp_v = np.ones(n, np.uint8)
    exp_v[forged] = 0
    assert np.array_equal(d_v.cpu().numpy(), exp_v)
    expect = np.full(total, 0xA5, np.uint8)
    length, at = lens.astype(np.int64), off.astype(np.int64)
    for k in range(int(length.max())):
        sel = length > k
        expect[at[sel] + k] = np.where(exp_v[sel] == 1, plain[at[sel] + k], 0)
    assert np.array_equal(d_back.cpu().numpy(), expect)


def _layout(rng, lens, extra, align, fixed_gap=None):
    """Slots back to back, each holding lens[i] + extra bytes, starting at a multiple of 16
    plus a gap that is a multiple of `align` below 16 (or `fixed_gap` for every packet)."""
    room = ((lens.astype(np.int64) + extra + 15) // 16) * 16 + 16
    if fixed_gap is not None:
        gap = np.full(len(lens), fixed_gap, np.int64)
    elif align >= 16:
        gap = np.zeros(len(lens), np.int64)
    else:
        gap = rng.integers(0, 16 // align, len(lens)) * align
    off = (np.concatenate([[0], np.cumsum(room)[:-1]]) + gap).astype(np.uint64)
    return off, int(room.sum()) + 32


@pytest.mark.parametrize("src_align,dst_align,src_gap,dst_gap", [
    (1, 4, None, None),   # input anywhere, output on words: whole destination cells, word-shifted
    (4, 1, None, None),   # output anywhere: misaligned stores
    (4, 4, None, None),   # both on words, each packet with skews of its own
    (16, 4, None, None),
    (4, 16, None, None),
    (4, 4, 4, 12),        # one skew for every packet of the batch, different on the two sides
    (16, 16, None, None), # both on cells but in different places within their lines
])
def test_source_and_destination_laid_out_independently(src_align, dst_align, src_gap, dst_gap):
    """Seal and open between arenas whose packets sit at unrelated alignments: sealed
    bytes equal the oracle's, the bytes between packets stay as they were, forged tags
    are rejected and everything else opens to the plaintext."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(4242 + 16 * src_align + dst_align)
    dev = torch.device("cuda:0")
    n, n_peers = 40000, 17
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    lens = rng.choice([0, 1, 3, 16, 17, 60, 63, 64, 65, 127, 128, 129, 255, 576, 1419, 1420, 1500], n).astype(np.uint32)
    off_p, total_p = _layout(rng, lens, 0, src_align, src_gap)
    off_s, total_s = _layout(rng, lens, 16, dst_align, dst_gap)
    if src_align == 16 and dst_align == 16:
        off_s = off_s + np.uint64(48)  # cells on both sides, 48 bytes apart within their lines
        total_s += 48
    plain = rng.integers(0, 256, total_p, dtype=np.uint8)
    peer = rng.integers(0, n_peers, n).astype(np.uint32)
    ctrs = rng.integers(0, 1 << 63, n, dtype=np.uint64)
    want = np.full(total_s, 0x5A, np.uint8)
    O.seal_batch(keys, peer, ctrs, plain, off_p, lens, want, off_s, 8)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    d_plain = d(plain)
    d_sealed = torch.full((total_s,), 0x5A, dtype=torch.uint8, device=dev)
    d_offp, d_offs = d(off_p.astype(np.int64)), d(off_s.astype(np.int64))
    d_len, d_ctl = d(lens.astype(np.int32)), d((lens + 16).astype(np.int32))
    d_peer, d_ctr = d(peer.astype(np.int32)), d(ctrs.astype(np.int64))
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_SEND, keys)
        ctx.keys_set(lib.KEYS_RECV, keys)
        ctx.seal(lib.make_batch(d_plain, total_p, n, lib.MEM_DEVICE, offsets=d_offp, lens=d_len, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(d_sealed, total_s, n, lib.MEM_DEVICE, offsets=d_offs))
        ctx.sync()
        got = d_sealed.cpu().numpy()
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, f"first differing sealed byte at {bad[:4]}"
        forged = rng.permutation(n)[:30]
        pos = off_s[forged].astype(np.int64) + lens[forged].astype(np.int64) + 5
        d_sealed[d(pos)] ^= 0x01
        # open back into an arena laid out like the plaintext's
        d_back = torch.full((total_p,), 0xA5, dtype=torch.uint8, device=dev)
        d_v = torch.full((n,), 9, dtype=torch.uint8, device=dev)
        ctx.open(lib.make_batch(d_sealed, total_s, n, lib.MEM_DEVICE, offsets=d_offs, lens=d_ctl, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(d_back, total_p, n, lib.MEM_DEVICE, offsets=d_offp), d_v)
        ctx.sync()
    exp_v = np.ones(n, np.uint8)
    exp_v[forged] = 0
    assert np.array_equal(d_v.cpu().numpy(), exp_v)
    expect = np.full(total_p, 0xA5, np.uint8)
    length, at = lens.astype(np.int64), off_p.astype(np.int64)
    for k in range(int(length.max())):
        sel = length > k
        expect[at[sel] + k] = np.where(exp_v[sel] == 1, plain[at[sel] + k], 0)
    assert np.array_equal(d_back.cpu().numpy(), expect)


@pytest.mark.parametrize("align", [4, 16, 1])
def test_seal_and_open_in_place(align):
    """One arena for both sides: every packet is sealed where it lies (its slot has
    room for the tag) and opened there again."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(777 + align)
    dev = torch.device("cuda:0")
    n, n_peers = 50000, 5
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    lens = rng.choice([0, 2, 16, 31, 60, 64, 100, 128, 130, 576, 1420, 1421], n).astype(np.uint32)
    off, total = _layout(rng, lens, 16, align)
    arena = rng.integers(0, 256, total, dtype=np.uint8)
    peer = rng.integers(0, n_peers, n).astype(np.uint32)
    ctrs = rng.integers(0, 1 << 63, n, dtype=np.uint64)
    want = arena.copy()
    O.seal_batch(keys, peer, ctrs, arena, off, lens, want, off, 8)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    d_arena = d(arena)
    d_off, d_len, d_ctl = d(off.astype(np.int64)), d(lens.astype(np.int32)), d((lens + 16).astype(np.int32))
    d_peer, d_ctr = d(peer.astype(np.int32)), d(ctrs.astype(np.int64))
    d_v = torch.zeros(n, dtype=torch.uint8, device=dev)
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_SEND, keys)
        ctx.keys_set(lib.KEYS_RECV, keys)
        ctx.seal(lib.make_batch(d_arena, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_len, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(d_arena, total, n, lib.MEM_DEVICE, offsets=d_off))
        ctx.sync()
        got = d_arena.cpu().numpy()
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, f"first differing sealed byte at {bad[:4]}"
        ctx.open(lib.make_batch(d_arena, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_ctl, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(d_arena, total, n, lib.MEM_DEVICE, offsets=d_off), d_v)
        ctx.sync()
    assert bool(d_v.all())
    back = d_arena.cpu().numpy()
    # the plaintext is back; the 16 bytes after it still hold the tag
    at, length = off.astype(np.int64), lens.astype(np.int64)
    expect = want.copy()
    for k in range(int(length.max())):
        sel = length > k
        expect[at[sel] + k] = arena[at[sel] + k]
    assert np.array_equal(back, expect)


@pytest.mark.parametrize("n", [1 << 20, (1 << 20) + 1])
def test_length_grouping_on_either_side_of_its_launch_shapes(n):
    """2^20 packets are grouped by length in two launches (every scatter block scans the
    histogram itself), one packet more in three (a scan launch in between).  Two batches
    in a row through one context, the second with other lengths: both sealed arenas equal
    the oracle's, so each shape also left the histogram cleared for the next grouping."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(77 + (n & 1))
    dev = torch.device("cuda:0")
    n_peers = 5
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_SEND, keys)
        for top in (40, 150):
            lens = rng.integers(0, top + 1, n).astype(np.uint32)
            off, total = _layout(rng, lens, 16, 16)
            plain = rng.integers(0, 256, total, dtype=np.uint8)
            peer = rng.integers(0, n_peers, n).astype(np.uint32)
            ctrs = rng.integers(0, 1 << 63, n, dtype=np.uint64)
            want = np.full(total, 0x5A, np.uint8)
            O.seal_batch(keys, peer, ctrs, plain, off, lens, want, off, 8)
            d_sealed = torch.full((total,), 0x5A, dtype=torch.uint8, device=dev)
            d_off = d(off.astype(np.int64))
            ctx.seal(lib.make_batch(d(plain), total, n, lib.MEM_DEVICE, offsets=d_off, lens=d(lens.astype(np.int32)),
                                    peer=d(peer.astype(np.int32)), counters=d(ctrs.astype(np.int64))),
                     lib.make_batch(d_sealed, total, n, lib.MEM_DEVICE, offsets=d_off))
            ctx.sync()
            bad = np.flatnonzero(d_sealed.cpu().numpy() != want)
            assert bad.size == 0, f"lengths up to {top}: first differing byte at {bad[:4]}"
