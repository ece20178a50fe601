"""Device-resident batches whose offsets and lengths live in device memory
cannot be checked by the host: the lanes compare every packet with the arena
size the caller declared.  A packet reaching beyond it is left alone (verdict
0), the rest of the batch is processed as usual, nothing outside the arena is
read for a result or written, and bnk_sync reports BNK_E_INVAL.  The arenas
here sit between guard bands inside a larger allocation, so an escaped write
would be seen rather than fault."""
import numpy as np
import pytest

from bnk_amd import workloads as W

pytestmark = pytest.mark.gpu

GUARD = 4096


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


class Banded:
    """An arena of `nbytes` bytes between two guard bands of 0xC3."""

    def __init__(self, content: np.ndarray):
        import torch
        self.n = content.nbytes
        host = np.full(self.n + 2 * GUARD, 0xC3, np.uint8)
        host[GUARD:GUARD + self.n] = content
        self.t = torch.from_numpy(host).to("cuda:0")
        self.ptr = self.t.data_ptr() + GUARD

    def arena(self) -> np.ndarray:
        return self.t[GUARD:GUARD + self.n].cpu().numpy()

    def guards_intact(self) -> bool:
        h = self.t.cpu().numpy()
        return bool((h[:GUARD] == 0xC3).all() and (h[GUARD + self.n:] == 0xC3).all())


def _expect_inval(ctx):
    from bnk_amd import lib
    with pytest.raises(lib.BnkError) as ei:
        ctx.sync()
    assert ei.value.code == lib.E_INVAL
    ctx.sync()  # the condition is reported once


@pytest.mark.parametrize("n,spread_max", [(300, 4096), (300, 0), (9000, 4096)])
def test_seal_and_open_skip_packets_outside_the_arena(n, spread_max):
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    b = W.aead_imix(41, n, n_peers=8)
    keys = np.ascontiguousarray(b.keys)
    total = b.plain.nbytes
    want = np.zeros_like(b.plain)
    O.seal_batch(keys, b.peer, b.counters, b.plain, b.off, b.lens, want, b.off, 4)
    # three kinds of bad packet: offset far outside, offset inside but the tag
    # would stick out, and an absurd length
    bad = np.array([5, n // 2, n - 3])
    off = b.off.copy()
    lens = b.lens.copy()
    off[bad[0]] = total + (1 << 30)
    off[bad[1]] = total - int(lens[bad[1]]) - 8  # ciphertext fits, the tag does not
    lens[bad[2]] = 0x7FFFFF00
    good = np.ones(n, bool)
    good[bad] = False
    with lib.Context(0) as ctx:
        ctx.set_spread_max_packets(spread_max)
        ctx.keys_set(lib.KEYS_SEND, keys)
        ctx.keys_set(lib.KEYS_RECV, keys)
        src, dst = Banded(b.plain), Banded(np.full(total, 0x5A, np.uint8))
        d_off, d_lens = _dev(off.astype(np.int64)), _dev(lens.astype(np.int32))
        d_peer, d_ctr = _dev(b.peer.astype(np.int32)), _dev(b.counters.astype(np.int64))
        torch.cuda.synchronize()
        ctx.seal(lib.make_batch(src.ptr, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(dst.ptr, total, n, lib.MEM_DEVICE, offsets=d_off))
        _expect_inval(ctx)
        assert src.guards_intact() and dst.guards_intact()
        expect = np.full(total, 0x5A, np.uint8)
        for i in np.flatnonzero(good):
            o, L = int(b.off[i]), int(b.lens[i]) + 16
            expect[o:o + L] = want[o:o + L]
        assert np.array_equal(dst.arena(), expect)

        # open of the oracle's sealed packets with the same three offenders
        ct_lens = (b.lens + 16).astype(np.uint32)
        ct_lens[bad[2]] = 0x7FFFFF00
        sealed, back = Banded(want), Banded(np.full(total, 0xA5, np.uint8))
        off2 = off.copy()
        off2[bad[1]] = total - int(ct_lens[bad[1]]) + 4  # the ciphertext itself sticks out
        d_off2, d_ctl = _dev(off2.astype(np.int64)), _dev(ct_lens.astype(np.int32))
        v = torch.full((n,), 7, dtype=torch.uint8, device="cuda:0")
        torch.cuda.synchronize()
        ctx.open(lib.make_batch(sealed.ptr, total, n, lib.MEM_DEVICE, offsets=d_off2, lens=d_ctl, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(back.ptr, total, n, lib.MEM_DEVICE, offsets=d_off2), v)
        _expect_inval(ctx)
        assert sealed.guards_intact() and back.guards_intact()
        assert np.array_equal(v.cpu().numpy(), good.astype(np.uint8))
        expect = np.full(total, 0xA5, np.uint8)
        for i in np.flatnonzero(good):
            o, L = int(b.off[i]), int(b.lens[i])
            expect[o:o + L] = b.plain[o:o + L]
        assert np.array_equal(back.arena(), expect)


@pytest.mark.parametrize("n,spread_max", [(300, 4096), (300, 0), (9000, 4096)])
def test_uniform_input_with_device_output_offsets_is_checked(n, spread_max):
    """The input is a uniform stride and length (nothing of it lies in device
    arrays), only the output offsets do: the lanes still check where they write."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(5)
    L, stride = 200, 224
    key = rng.integers(0, 256, (1, 32), dtype=np.uint8)
    plain = rng.integers(0, 256, n * stride, dtype=np.uint8)
    off = (np.arange(n, dtype=np.uint64) * stride)
    lens = np.full(n, L, np.uint32)
    zeros = np.zeros(n, np.uint32)
    ctrs = np.arange(n, dtype=np.uint64) + 9
    want = np.full(n * stride, 0x5A, np.uint8)
    O.seal_batch(key, zeros, ctrs, plain, off, lens, want, off, 4)
    bad = np.array([2, n // 2, n - 1])
    out_off = off.copy()
    out_off[bad[0]] = n * stride + (1 << 33)
    out_off[bad[1]] = n * stride - L - 8      # ciphertext fits, the tag does not
    out_off[bad[2]] = n * stride              # starts at the arena's end
    good = np.ones(n, bool)
    good[bad] = False
    with lib.Context(0) as ctx:
        ctx.set_spread_max_packets(spread_max)
        ctx.keys_set(lib.KEYS_SEND, key)
        ctx.keys_set(lib.KEYS_RECV, key)
        src, dst = Banded(plain), Banded(np.full(n * stride, 0x5A, np.uint8))
        d_out_off = _dev(out_off.astype(np.int64))
        torch.cuda.synchronize()
        ctx.seal(lib.make_batch(src.ptr, plain.nbytes, n, lib.MEM_DEVICE, stride=stride, length=L, counter0=9),
                 lib.make_batch(dst.ptr, plain.nbytes, n, lib.MEM_DEVICE, offsets=d_out_off))
        _expect_inval(ctx)
        assert src.guards_intact() and dst.guards_intact()
        expect = np.full(n * stride, 0x5A, np.uint8)
        for i in np.flatnonzero(good):
            o = int(off[i])
            expect[o:o + L + 16] = want[o:o + L + 16]
        assert np.array_equal(dst.arena(), expect)

        # open of the oracle's sealed packets, plaintexts to checked offsets
        sealed, back = Banded(want), Banded(np.full(n * stride, 0xA5, np.uint8))
        out_off[bad[1]] = n * stride - L + 3  # the plaintext itself sticks out
        d_out_off = _dev(out_off.astype(np.int64))
        v = torch.full((n,), 7, dtype=torch.uint8, device="cuda:0")
        torch.cuda.synchronize()
        ctx.open(lib.make_batch(sealed.ptr, plain.nbytes, n, lib.MEM_DEVICE, stride=stride, length=L + 16,
                                counter0=9),
                 lib.make_batch(back.ptr, plain.nbytes, n, lib.MEM_DEVICE, offsets=d_out_off), v)
        _expect_inval(ctx)
        assert sealed.guards_intact() and back.guards_intact()
        assert np.array_equal(v.cpu().numpy(), good.astype(np.uint8))
        expect = np.full(n * stride, 0xA5, np.uint8)
        for i in np.flatnonzero(good):
            o = int(off[i])
            expect[o:o + L] = plain[o:o + L]
        assert np.array_equal(back.arena(), expect)


@pytest.mark.parametrize("n,spread_max", [(300, 4096), (9000, 4096)])
def test_length_words_near_2_to_32_do_not_wrap_past_the_check(n, spread_max):
    """len + 16 and len + padding are not 32-bit sums: a length word of
    0xFFFFFFF0 or more in an arena of any size is refused, not wrapped to a
    small number that passes."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    b = W.aead_imix(43, n, n_peers=4)
    keys = np.ascontiguousarray(b.keys)
    total = b.plain.nbytes
    want = np.zeros_like(b.plain)
    O.seal_batch(keys, b.peer, b.counters, b.plain, b.off, b.lens, want, b.off, 4)
    bad = np.array([1, n // 2, n - 2])
    lens = b.lens.copy()
    lens[bad] = [0xFFFFFFF0, 0xFFFFFFFF, 0xFFFFFFF5]
    good = np.ones(n, bool)
    good[bad] = False
    with lib.Context(0) as ctx:
        ctx.set_spread_max_packets(spread_max)
        ctx.keys_set(lib.KEYS_SEND, keys)
        src, dst = Banded(b.plain), Banded(np.full(total, 0x5A, np.uint8))
        d_off, d_lens = _dev(b.off.astype(np.int64)), _dev(lens.view(np.int32))
        d_peer, d_ctr = _dev(b.peer.astype(np.int32)), _dev(b.counters.astype(np.int64))
        torch.cuda.synchronize()
        # the declared arena size is beyond 4 GiB, so that only a wrapped sum could pass
        # for the offenders (the good packets all lie within the real allocation)
        ctx.seal(lib.make_batch(src.ptr, 1 << 33, n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(dst.ptr, 1 << 33, n, lib.MEM_DEVICE, offsets=d_off))
        _expect_inval(ctx)
        assert src.guards_intact() and dst.guards_intact()
        expect = np.full(total, 0x5A, np.uint8)
        for i in np.flatnonzero(good):
            o, L = int(b.off[i]), int(b.lens[i]) + 16
            expect[o:o + L] = want[o:o + L]
        assert np.array_equal(dst.arena(), expect)


def test_filter_skips_packets_outside_the_arena():
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    n = 5000
    w = W.acl_workload(n=n, n_rules=256, n_flows=512)
    rec = np.ascontiguousarray(w.check).reshape(-1)
    off = np.arange(n, dtype=np.uint64) * 32
    lens = np.full(n, 28, np.uint32)
    ora = O.Filter()
    ora.set_rules(w.rules_ref)
    with lib.Context(0) as ctx:
        ctx.filter_set_rules(w.rules_ref)
        for now, r in w.note_batches:
            buf = np.ascontiguousarray(r).reshape(-1)
            o2 = np.arange(r.shape[0], dtype=np.uint64) * 32
            l2 = np.full(r.shape[0], 28, np.uint32)
            ora.note_outbound_batch(buf, o2, l2, now)
            # one noted packet lies outside: it must not enter the table
            o3 = o2.copy()
            o3[1] = buf.nbytes + 77
            skipped = np.ones(r.shape[0], bool)
            arena = Banded(buf)
            d_o, d_l = _dev(o3.astype(np.int64)), _dev(l2.astype(np.int32))
            torch.cuda.synchronize()
            ctx.filter_note_outbound(lib.make_batch(arena.ptr, buf.nbytes, r.shape[0], lib.MEM_DEVICE,
                                                    offsets=d_o, lens=d_l), now)
            _expect_inval(ctx)
            # the skipped packet goes in by a second, well-formed call
            ctx.filter_note_outbound(lib.make_batch(arena.ptr, buf.nbytes, 1, lib.MEM_DEVICE,
                                                    offsets=_dev(o2[1:2].astype(np.int64)),
                                                    lens=_dev(l2[1:2].astype(np.int32))), now)
            ctx.sync()
        assert ctx.filter_flows() == ora.flows()
        want = ora.check_inbound_batch(rec, off, lens, w.now_ns)
        bad = np.array([0, 1234, n - 1])
        off_b, lens_b = off.copy(), lens.copy()
        off_b[bad[0]] = rec.nbytes - 20        # the header's end sticks out
        off_b[bad[1]] = 1 << 40
        lens_b[bad[2]] = 64                    # length says more than the arena holds
        want[bad] = 0
        arena = Banded(rec)
        v = torch.full((n,), 9, dtype=torch.uint8, device="cuda:0")
        d_o, d_l = _dev(off_b.astype(np.int64)), _dev(lens_b.astype(np.int32))
        torch.cuda.synchronize()
        ctx.filter_check_inbound(lib.make_batch(arena.ptr, rec.nbytes, n, lib.MEM_DEVICE, offsets=d_o,
                                                lens=d_l), w.now_ns, v)
        _expect_inval(ctx)
        assert np.array_equal(v.cpu().numpy(), want)
        assert arena.guards_intact()


@pytest.mark.parametrize("n", [500, 5000])
def test_framing_skips_slots_outside_the_arena(n):
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(99)
    n_peers = 9
    peers = [(1000 + 7 * i, 5000 + 11 * i, 0x64400001 + i, 0xFFFFFFFF) for i in range(n_peers)]
    rx_peers = [(p[1], p[0], p[2], p[3]) for p in peers]
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    lens = rng.choice([20, 40, 100, 576, 1400], n).astype(np.uint32)
    peer = rng.integers(0, n_peers, n).astype(np.uint32)
    slot = ((16 + lens.astype(np.int64) + 15 + 16 + 15) & ~15)
    off = np.concatenate([[0], np.cumsum(slot)[:-1]]).astype(np.uint64)
    total = int(slot.sum())
    arena = rng.integers(0, 256, total, dtype=np.uint8)
    for i in range(n):
        o = int(off[i]) + 16
        arena[o] = 0x45
        arena[o + 2:o + 4] = np.frombuffer(int(lens[i]).to_bytes(2, "big"), np.uint8)
        arena[o + 12:o + 16] = np.frombuffer(peers[int(peer[i])][2].to_bytes(4, "big"), np.uint8)
    bad = np.array([3, n // 3, n - 1])
    off_b = off.copy()
    off_b[bad[0]] = total + 5
    off_b[bad[1]] = total - 40              # header fits, the rest does not
    off_b[bad[2]] = total - int(lens[bad[2]]) - 20   # the tag sticks out
    good = np.ones(n, bool)
    good[bad] = False
    want = arena.copy()
    want_len = np.zeros(n, np.uint32)
    nxt = np.zeros(n_peers, np.uint64)
    for i in range(n):
        p, o = int(peer[i]), int(off[i])
        if good[i]:
            wdg = O.wg_encap(arena[o + 16:o + 16 + int(lens[i])].tobytes(), 1420, keys[p].tobytes(), peers[p][1],
                             int(nxt[p]))
            want[o:o + len(wdg)] = np.frombuffer(wdg, np.uint8)
            want_len[i] = len(wdg)
        nxt[p] += 1  # a counter was handed out before the slot was looked at
    with lib.Context(0) as tx, lib.Context(0) as rx:
        tx.keys_set(lib.KEYS_SEND, keys)
        tx.wg_peers_set(peers)
        slots = Banded(arena)
        d_off, d_lens, d_peer = _dev(off_b.astype(np.int64)), _dev(lens.astype(np.int32)), _dev(peer.astype(np.int32))
        d_wl = torch.full((n,), 77, dtype=torch.int32, device="cuda:0")
        torch.cuda.synchronize()
        tx.wg_encap(lib.make_batch(slots.ptr, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens, peer=d_peer),
                    1420, d_wl)
        _expect_inval(tx)
        assert slots.guards_intact()
        assert np.array_equal(d_wl.cpu().numpy().astype(np.uint32), want_len)
        assert np.array_equal(slots.arena(), want)

        # the datagrams back in, with the same three offsets broken
        rx.keys_set(lib.KEYS_RECV, keys)
        rx.wg_peers_set(rx_peers)
        wire, out = Banded(want), Banded(np.full(total, 0x77, np.uint8))
        wl_b = want_len.copy()
        wl_b[bad] = (16 + lens[bad] + 15) // 16 * 16 + 16
        d_wlen = _dev(wl_b.astype(np.int32))
        res = torch.full((n,), 99, dtype=torch.uint8, device="cuda:0")
        olen = torch.zeros(n, dtype=torch.int32, device="cuda:0")
        gp = torch.zeros(n, dtype=torch.int32, device="cuda:0")
        gc = torch.zeros(n, dtype=torch.int64, device="cuda:0")
        torch.cuda.synchronize()
        rx.wg_decap(lib.make_batch(wire.ptr, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_wlen),
                    lib.make_batch(out.ptr, total, n, lib.MEM_DEVICE, offsets=d_off), res, olen, gp, gc)
        _expect_inval(rx)
        assert wire.guards_intact() and out.guards_intact()
        r = res.cpu().numpy()
        assert (r[good] == lib.WG_OK).all() and (r[bad] == lib.WG_BAD_HEADER).all()
        got = out.arena()
        expect = np.full(total, 0x77, np.uint8)
        for i in np.flatnonzero(good):
            o, L = int(off[i]), int(want_len[i]) - 32
            expect[o:o + L] = arena[o + 16:o + 16 + L] if L <= int(lens[i]) else np.concatenate(
                [arena[o + 16:o + 16 + int(lens[i])], np.zeros(L - int(lens[i]), np.uint8)])
        assert np.array_equal(got, expect)


def test_relay_skips_packets_outside_the_arenas():
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    n = 6000
    w = W.relay_workload(n=n, n_peers=64, n_rules=128)
    b = w.batch
    keys_in, keys_out = np.ascontiguousarray(b.keys), np.ascontiguousarray(w.keys_out)
    sealed = np.zeros_like(b.plain)
    O.seal_batch(keys_in, b.peer, b.counters, b.plain, b.off, b.lens, sealed, b.off, 4)
    W.forge_tags(5, sealed, b.off, b.lens, w.forged_fraction)
    total = sealed.nbytes
    ct_lens = (b.lens + 16).astype(np.uint32)
    bad = np.array([7, n // 2])
    # the oracle sees the two offenders as truncated packets (FORGED, no nonce
    # used), the GPU sees them with offsets outside the arena
    ct_trunc = ct_lens.copy()
    ct_trunc[bad] = 9
    off_b = b.off.copy()
    off_b[bad[0]] = total + 100
    off_b[bad[1]] = total - 10
    ora = O.Filter()
    ora.set_rules(w.rules_ref)
    now, rec = w.note_batch
    m = rec.shape[0]
    buf = np.ascontiguousarray(rec).reshape(-1)
    ora.note_outbound_batch(buf, np.arange(m, dtype=np.uint64) * 32, np.full(m, 28, np.uint32), now)
    want_out = np.full_like(sealed, 0x3C)
    want_v, want_c = ora.relay_fused_batch(keys_in, b.peer, b.counters, keys_out, w.peer_out, w.ctr_base_out,
                                           sealed, b.off, ct_trunc, want_out, b.off, w.now_ns)
    assert (want_v[bad] == lib.RELAY_FORGED).all()
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_RECV, keys_in)
        ctx.keys_set(lib.KEYS_SEND, keys_out)
        ctx.filter_set_rules(w.rules_ref)
        ctx.filter_note_outbound(lib.make_batch(buf, buf.nbytes, m, lib.MEM_HOST, stride=32, length=28), now)
        src, dst = Banded(sealed), Banded(np.full(total, 0x3C, np.uint8))
        d = _dev
        d_off, d_lens = d(off_b.astype(np.int64)), d(ct_lens.astype(np.int32))
        d_peer, d_ctr = d(b.peer.astype(np.int32)), d(b.counters.astype(np.int64))
        d_po, d_cb = d(w.peer_out.astype(np.int32)), d(w.ctr_base_out.astype(np.int64))
        v = torch.full((n,), 9, dtype=torch.uint8, device="cuda:0")
        co = torch.zeros(n, dtype=torch.int64, device="cuda:0")
        torch.cuda.synchronize()
        ctx.relay_fused(lib.make_batch(src.ptr, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens, peer=d_peer,
                                       counters=d_ctr),
                        d_po, d_cb, len(w.ctr_base_out), w.now_ns,
                        lib.make_batch(dst.ptr, total, n, lib.MEM_DEVICE, offsets=d_off), v, co)
        _expect_inval(ctx)
        assert src.guards_intact() and dst.guards_intact()
        assert np.array_equal(v.cpu().numpy(), want_v)
        assert np.array_equal(co.cpu().numpy().astype(np.uint64), want_c)
        assert np.array_equal(dst.arena(), want_out)
