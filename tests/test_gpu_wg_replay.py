"""The anti-replay windows of bnk_wg_decap_batch (RFC 6479 as wireguard-go's
replay.Filter, one per peer, on the device, a whole batch at a time) against
the sequential filter of the oracle (bnko_replay_validate) fed packet by
packet in batch order, with wireguard-go's ordering: every authentic packet
goes through its peer's window before its inner header counts.  The window
itself is pinned on the CPU (tests/cpp/replay_test.cpp, tests/test_oracle_wg.py);
like the rest of the framing it is spec-derived, not a reference artefact."""
import struct

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

P = 6
LIMIT = (1 << 64) - (1 << 13) - 1
WINDOW = 8128


def _peers():
    tx = [(1000 + 13 * i, 7000 + 17 * i, 0x64400001 + i, 0xFFFFFFFF) for i in range(P)]
    rx = [(p[1], p[0], p[2], p[3]) for p in tx]
    return tx, rx


def _inner(rng, src, length, kind):
    if kind == "keepalive":
        return b""
    pkt = bytearray(rng.integers(0, 256, length, dtype=np.uint8).tobytes())
    pkt[0] = 0x45 if kind != "badip" else 0x15
    pkt[2:4] = struct.pack(">H", length)
    pkt[12:16] = struct.pack(">I", src if kind != "notallowed" else src ^ 0x00010000)
    return bytes(pkt)


def _counters(rng, n, last):
    """A walk around each peer's newest counter: forward steps, repeats,
    reordering, the window's edges on both sides, far jumps."""
    peer = rng.integers(0, P, n)
    ctr = np.zeros(n, np.uint64)
    last = list(last)
    recent = [[] for _ in range(P)]
    for i in range(n):
        p = int(peer[i])
        r = rng.random()
        if r < 0.55:
            c = last[p] + int(rng.integers(1, 4))
        elif r < 0.70 and recent[p]:
            c = recent[p][int(rng.integers(0, len(recent[p])))]          # an exact repeat
        elif r < 0.80:
            c = max(0, last[p] - int(rng.integers(0, 200)))              # a little late
        elif r < 0.86:
            c = max(0, last[p] - WINDOW + int(rng.integers(-2, 3)))      # the far edge of the window
        elif r < 0.90:
            c = last[p] + int(rng.integers(60, 70)) * int(rng.integers(1, 200))  # over one or many blocks
        elif r < 0.93:
            c = last[p] + WINDOW + int(rng.integers(-2, 3)) + 64         # just beyond a whole ring
        elif r < 0.95:
            c = 0
        else:
            c = last[p] + int(rng.integers(1, 3))
        c = min(c, LIMIT + 3)
        ctr[i] = c
        if c < LIMIT:
            last[p] = max(last[p], c)
        recent[p] = (recent[p] + [c])[-50:]
    return peer.astype(np.uint32), ctr, last


def _batch(rng, tx, keys, n, last, near_limit=False):
    from oracle import binding as O
    peer, ctr, last = _counters(rng, n, last)
    if near_limit:
        ctr[:6] = np.array([LIMIT - 2, LIMIT - 1, LIMIT, LIMIT + 1, LIMIT - 1, LIMIT - 2], np.uint64)
        peer[:6] = 0
    kinds = rng.choice(["ok", "ok", "ok", "ok", "keepalive", "notallowed", "badip", "forged"], n)
    wires, offs, pos = [], np.zeros(n, np.uint64), 0
    for i in range(n):
        p = int(peer[i])
        inner = _inner(rng, tx[p][2], int(rng.choice([20, 28, 60, 200, 576])), kinds[i])
        w = bytearray(O.wg_encap(inner, 1420, keys[p].tobytes(), tx[p][1], int(ctr[i])))
        if kinds[i] == "forged":
            w[-1] ^= 1
        offs[i] = pos
        wires.append(bytes(w))
        pos += (len(w) + 15) & ~15
    arena = np.zeros(pos + 16, np.uint8)
    for i, w in enumerate(wires):
        arena[int(offs[i]):int(offs[i]) + len(w)] = np.frombuffer(w, np.uint8)
    lens = np.array([len(w) for w in wires], np.uint32)
    return arena, offs, lens, wires, last


def _expect(wires, rx, keys, filters):
    """Oracle result per packet, then the sequential window per peer in batch order."""
    from bnk_amd import lib
    from oracle import binding as O
    n = len(wires)
    res, olen, peer, ctr = np.zeros(n, np.uint8), np.zeros(n, np.uint32), np.zeros(n, np.uint32), np.zeros(n, np.uint64)
    for i, w in enumerate(wires):
        rc, pt, p, c = O.wg_decap(w, rx, keys)
        res[i], olen[i], peer[i], ctr[i] = rc, len(pt), p, c
        if rc not in (lib.WG_BAD_HEADER, lib.WG_UNKNOWN_INDEX, lib.WG_AUTH_FAIL):
            if not filters[p].validate(c):
                res[i], olen[i] = lib.WG_REPLAY, 0
    return res, olen, peer, ctr


@pytest.mark.parametrize("mode", ["host_fused", "host_unfused", "device_large", "device_separate", "ring_fused"])
def test_replay_windows_match_the_sequential_filter(mode):
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(2024)
    tx, rx = _peers()
    keys = rng.integers(0, 256, (P, 32), dtype=np.uint8)
    filters = [O.ReplayFilter() for _ in range(P)]
    last = [0] * P
    sizes = {"host_fused": [1, 64, 300, 1024, 700], "host_unfused": [300, 1024, 2000, 150],
             "device_large": [5000, 1025, 9000, 3000], "device_separate": [3000, 1025, 6000],
             "ring_fused": [128, 900, 128]}[mode]
    seen = set()
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_RECV, keys)
        ctx.wg_peers_set(rx)
        if mode == "host_unfused":
            ctx.set_spread_max_packets(0)
        if mode == "device_separate":
            ctx.wg_set_fused(False)  # the framing, and the window pass's sort keys, from kernels of their own
        for b, n in enumerate(sizes):
            arena, offs, lens, wires, last = _batch(rng, tx, keys, n, last, near_limit=(b == 2))
            want = _expect(wires, rx, keys, filters)
            total = arena.nbytes
            if mode in ("device_large", "device_separate"):
                d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")  # noqa: E731
                d_arena, d_out = d(arena), torch.zeros(total, dtype=torch.uint8, device="cuda:0")
                res = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
                olen = torch.zeros(n, dtype=torch.int32, device="cuda:0")
                gp = torch.zeros(n, dtype=torch.int32, device="cuda:0")
                gc = torch.zeros(n, dtype=torch.int64, device="cuda:0")
                d_off, d_len = d(offs.astype(np.int64)), d(lens.astype(np.int32))
                torch.cuda.synchronize()
                ctx.wg_decap(lib.make_batch(d_arena, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_len),
                             lib.make_batch(d_out, total, n, lib.MEM_DEVICE, offsets=d_off), res, olen, gp, gc)
                ctx.sync()
                got = (res.cpu().numpy(), olen.cpu().numpy().astype(np.uint32), gp.cpu().numpy().astype(np.uint32),
                       gc.cpu().numpy().astype(np.uint64))
            else:
                rings = []
                if mode == "ring_fused":
                    rings = [ctx.ring_alloc(total), ctx.ring_alloc(total)]
                    rings[0][:] = arena
                src = rings[0] if rings else arena
                out = rings[1] if rings else np.zeros(total, np.uint8)
                res, olen = np.zeros(n, np.uint8), np.zeros(n, np.uint32)
                gp, gc = np.zeros(n, np.uint32), np.zeros(n, np.uint64)
                ctx.wg_decap(lib.make_batch(src, total, n, lib.MEM_HOST, offsets=offs, lens=lens),
                             lib.make_batch(out, total, n, lib.MEM_HOST, offsets=offs), res, olen, gp, gc)
                got = (res, olen, gp, gc)
                for r in rings:
                    ctx.ring_free(r)
            bad = np.flatnonzero(got[0] != want[0])
            assert bad.size == 0, f"batch {b}: result differs at {bad[:5]}: got {got[0][bad[:5]]} want {want[0][bad[:5]]}"
            assert np.array_equal(got[1], want[1]) and np.array_equal(got[2], want[2]) and np.array_equal(got[3], want[3])
            seen.update(np.unique(want[0]).tolist())
    # the walk exercised every outcome, replays among them
    assert {lib.WG_OK, lib.WG_KEEPALIVE, lib.WG_AUTH_FAIL, lib.WG_BAD_IP, lib.WG_NOT_ALLOWED, lib.WG_REPLAY} <= seen


def test_a_rekeyed_peer_starts_with_an_empty_window_and_the_switch_turns_windows_off():
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(7)
    tx, rx = _peers()
    keys = rng.integers(0, 256, (P, 32), dtype=np.uint8)

    def decap(ctx, wires):
        n = len(wires)
        offs = np.arange(n, dtype=np.uint64) * 128
        arena = np.zeros(n * 128, np.uint8)
        for i, w in enumerate(wires):
            arena[i * 128:i * 128 + len(w)] = np.frombuffer(w, np.uint8)
        lens = np.array([len(w) for w in wires], np.uint32)
        out = np.zeros_like(arena)
        res, olen, gp, gc = np.zeros(n, np.uint8), np.zeros(n, np.uint32), np.zeros(n, np.uint32), np.zeros(n, np.uint64)
        ctx.wg_decap(lib.make_batch(arena, arena.nbytes, n, lib.MEM_HOST, offsets=offs, lens=lens),
                     lib.make_batch(out, out.nbytes, n, lib.MEM_HOST, offsets=offs), res, olen, gp, gc)
        return res.tolist()

    def dg(p, c, key=None, remote=None):
        inner = _inner(rng, tx[p][2], 40, "ok")
        return O.wg_encap(inner, 1420, (keys[p] if key is None else key).tobytes(), tx[p][1] if remote is None else remote, c)

    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_RECV, keys)
        ctx.wg_peers_set(rx)
        assert decap(ctx, [dg(0, 5), dg(1, 5), dg(0, 5), dg(0, 4)]) == [lib.WG_OK, lib.WG_OK, lib.WG_REPLAY, lib.WG_OK]
        assert decap(ctx, [dg(0, 5), dg(0, 4), dg(1, 5), dg(0, 6)]) == [lib.WG_REPLAY] * 3 + [lib.WG_OK]
        # peer 0 rekeys: new indices, new key, and a window that has seen nothing;
        # peer 1's window stands
        new_key = rng.integers(0, 256, 32, dtype=np.uint8)
        ctx.wg_peer_set(0, (rx[0][0] + 1, rx[0][1], rx[0][2], rx[0][3]), key_recv=new_key)
        assert decap(ctx, [dg(0, 5, new_key, rx[0][0] + 1), dg(1, 5), dg(0, 5)]) == \
            [lib.WG_OK, lib.WG_REPLAY, lib.WG_UNKNOWN_INDEX]
        # the same table again keeps the windows; a changed row starts over
        rows = [(rx[0][0] + 1, rx[0][1], rx[0][2], rx[0][3])] + rx[1:]
        ctx.wg_peers_set(rows)
        assert decap(ctx, [dg(0, 5, new_key, rx[0][0] + 1), dg(1, 5)]) == [lib.WG_REPLAY, lib.WG_REPLAY]
        rows[1] = (rx[1][0] + 1, rx[1][1], rx[1][2], rx[1][3])
        ctx.wg_peers_set(rows)
        assert decap(ctx, [dg(1, 5, None, rx[1][0] + 1), dg(0, 5, new_key, rx[0][0] + 1)]) == [lib.WG_OK, lib.WG_REPLAY]
        # windows off: nothing is turned away and nothing is recorded
        ctx.wg_set_replay(False)
        assert decap(ctx, [dg(2, 9), dg(2, 9)]) == [lib.WG_OK, lib.WG_OK]
        ctx.wg_set_replay(True)
        assert decap(ctx, [dg(2, 9), dg(2, 9)]) == [lib.WG_OK, lib.WG_REPLAY]


def _traffic(tx_ctx, tx_peers, n_a, n_b, n_total, inner_len, jump_rows, rng):
    """Datagrams for a large decapsulating batch without a per-packet oracle:
    two encapsulated batches (between them some peers' send counters jump ahead
    by more than a window, so that the first batch's packets of those peers are
    too old once a second-batch packet has been seen), then a shuffled mix of
    both with repeats.  Returns the wire arena, offsets, lengths, and each
    datagram's sender and counter as the sending side knows them."""
    from bnk_amd import lib
    n_peers = len(tx_peers)
    slot = (16 + inner_len + 15 + 16 + 15) & ~15
    per = []
    for k, n in enumerate((n_a, n_b)):
        peer = rng.integers(0, n_peers, n).astype(np.uint32)
        # half of either batch belongs to the peers that jump, so that they have old
        # packets to be refused and new ones to refuse them
        peer[: n // 2] = rng.choice(jump_rows, n // 2).astype(np.uint32)
        arena = rng.integers(0, 256, n * slot, dtype=np.uint8)
        rows = arena.reshape(n, slot)
        rows[:, 16] = 0x45
        rows[:, 18], rows[:, 19] = inner_len >> 8, inner_len & 255
        allowed = np.array([t[2] for t in tx_peers], np.uint32)[peer]
        rows[:, 28:32] = allowed.astype(">u4").view(np.uint8).reshape(n, 4)
        wl = np.zeros(n, np.uint32)
        if k == 1:
            for r in jump_rows:
                tx_ctx.wg_send_counter_set(int(r), 9000 + int(r) % 7)
        tx_ctx.wg_encap(lib.make_batch(arena, arena.nbytes, n, lib.MEM_HOST, stride=slot, length=inner_len,
                                       peer=peer), 1420, wl)
        assert (wl == 16 + ((inner_len + 15) & ~15) + 16).all()
        per.append((arena.reshape(n, slot), peer, int(wl[0])))
    wire_len = per[0][2]
    src = np.concatenate([per[0][0], per[1][0]])[:, :wire_len]
    src_peer = np.concatenate([per[0][1], per[1][1]])
    pick = np.concatenate([np.arange(n_a + n_b), rng.integers(0, n_a + n_b, n_total - n_a - n_b)])
    rng.shuffle(pick)
    stride = (wire_len + 15) & ~15
    wire = np.zeros((n_total, stride), np.uint8)
    wire[:, :wire_len] = src[pick]
    ctr = wire[:, 8:16].copy().view("<u8").reshape(-1)
    return wire.reshape(-1), stride, wire_len, src_peer[pick], ctr


def _window_expectation(peer, ctr, n_peers_seen):
    from bnk_amd import lib
    from oracle import binding as O
    filters = {}
    want = np.zeros(len(peer), np.uint8)
    for i in range(len(peer)):
        f = filters.setdefault(int(peer[i]), O.ReplayFilter())
        want[i] = lib.WG_OK if f.validate(int(ctr[i])) else lib.WG_REPLAY
    return want


def test_window_pass_with_more_peers_than_a_packed_sort_key_holds():
    """70,000 peers and 40,000 packets: the sender's number and the packet's
    position no longer fit one 32-bit sort key, so the window pass sorts
    (sender, position) pairs.  Expected results come from the sequential
    filter fed, in batch order, the senders and counters the sending side
    assigned."""
    import torch
    from bnk_amd import lib
    rng = np.random.default_rng(77)
    n_peers, n_total = 70000, 40000
    tx = [(10 + 3 * i, 500000 + 5 * i, 0x64400000 + i, 0xFFFFFFFF) for i in range(n_peers)]
    rx = [(p[1], p[0], p[2], p[3]) for p in tx]
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    jump_rows = rng.choice(n_peers, 300, replace=False)
    with lib.Context(0) as txc, lib.Context(0) as rxc:
        txc.keys_set(lib.KEYS_SEND, keys)
        txc.wg_peers_set(tx)
        rxc.keys_set(lib.KEYS_RECV, keys)
        rxc.wg_peers_set(rx)
        wire, stride, wire_len, peer, ctr = _traffic(txc, tx, 12000, 8000, n_total, 40, jump_rows, rng)
        want = _window_expectation(peer, ctr, n_peers)
        d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")  # noqa: E731
        d_wire, d_out = d(wire), torch.zeros(wire.nbytes, dtype=torch.uint8, device="cuda:0")
        res = torch.zeros(n_total, dtype=torch.uint8, device="cuda:0")
        olen = torch.zeros(n_total, dtype=torch.int32, device="cuda:0")
        gp = torch.zeros(n_total, dtype=torch.int32, device="cuda:0")
        gc = torch.zeros(n_total, dtype=torch.int64, device="cuda:0")
        torch.cuda.synchronize()
        rxc.wg_decap(lib.make_batch(d_wire, wire.nbytes, n_total, lib.MEM_DEVICE, stride=stride, length=wire_len),
                     lib.make_batch(d_out, wire.nbytes, n_total, lib.MEM_DEVICE, stride=stride), res, olen, gp, gc)
        rxc.sync()
        assert np.array_equal(gp.cpu().numpy().astype(np.uint32), peer)
        assert np.array_equal(gc.cpu().numpy().astype(np.uint64), ctr)
        got = res.cpu().numpy()
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, f"result differs at {bad[:5]}: got {got[bad[:5]]} want {want[bad[:5]]}"
        assert (want == lib.WG_REPLAY).sum() > 1000 and (want == lib.WG_OK).sum() > 1000
        assert np.array_equal(olen.cpu().numpy() != 0, want == lib.WG_OK)


def test_window_pass_of_a_host_batch_that_goes_through_in_chunks():
    """A host batch beyond the size that runs in one piece is cut into chunks,
    each with a window pass of its own continuing the one before: results are
    those of the sequential filter over the whole batch in order."""
    from bnk_amd import lib
    rng = np.random.default_rng(78)
    n_peers, n_total = 40, 14000
    tx = [(100 + 3 * i, 9000 + 5 * i, 0x64400000 + i, 0xFFFFFFFF) for i in range(n_peers)]
    rx = [(p[1], p[0], p[2], p[3]) for p in tx]
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    with lib.Context(0) as txc, lib.Context(0) as rxc:
        txc.keys_set(lib.KEYS_SEND, keys)
        txc.wg_peers_set(tx)
        rxc.keys_set(lib.KEYS_RECV, keys)
        rxc.wg_peers_set(rx)
        wire, stride, wire_len, peer, ctr = _traffic(txc, tx, 6000, 5000, n_total, 1400, np.arange(0, n_peers, 3),
                                                     rng)
        assert wire.nbytes > (16 << 20)  # well beyond two chunks' worth
        want = _window_expectation(peer, ctr, n_peers)
        out = np.zeros(wire.nbytes, np.uint8)
        res, olen = np.zeros(n_total, np.uint8), np.zeros(n_total, np.uint32)
        gp, gc = np.zeros(n_total, np.uint32), np.zeros(n_total, np.uint64)
        rxc.wg_decap(lib.make_batch(wire, wire.nbytes, n_total, lib.MEM_HOST, stride=stride, length=wire_len),
                     lib.make_batch(out, out.nbytes, n_total, lib.MEM_HOST, stride=stride), res, olen, gp, gc)
        assert np.array_equal(gp, peer) and np.array_equal(gc, ctr)
        bad = np.flatnonzero(res != want)
        assert bad.size == 0, f"result differs at {bad[:5]}: got {res[bad[:5]]} want {want[bad[:5]]}"
        assert (want == lib.WG_REPLAY).sum() > 1000 and (want == lib.WG_OK).sum() > 1000


def test_window_pass_where_one_peer_fills_more_blocks_than_one_look_back_reads():
    """Two peers, one of them sending nearly everything: its run in sorted order
    spans well over a thousand blocks of 1024 positions, so the running maximum
    a block is handed comes from carries read in more than one step, and a late
    repeat of a counter that was ahead when it first came is found by a search
    that goes back across many blocks."""
    import torch
    from bnk_amd import lib
    rng = np.random.default_rng(79)
    n_total = 2_300_000
    tx = [(100, 9000, 0x64400000, 0xFFFFFFFF), (103, 9005, 0x64400001, 0xFFFFFFFF)]
    rx = [(p[1], p[0], p[2], p[3]) for p in tx]
    keys = rng.integers(0, 256, (2, 32), dtype=np.uint8)
    with lib.Context(0) as txc, lib.Context(0) as rxc:
        txc.keys_set(lib.KEYS_SEND, keys)
        txc.wg_peers_set(tx)
        rxc.keys_set(lib.KEYS_RECV, keys)
        rxc.wg_peers_set(rx)
        # (no jump: a window is far shorter than the batch, so most early packets are too old
        # by the time they come, the rest repeat or are fresh)
        wire, stride, wire_len, peer, ctr = _traffic(txc, tx, 700_000, 500_000, n_total, 40, np.array([0]), rng)
        # the first 1.2 million in sending order, so that long stretches are ahead of everything
        # before them, then the shuffled mix with its repeats
        order = np.argsort(ctr[:1_200_000], kind="stable")
        w2 = wire.reshape(n_total, stride)
        w2[:1_200_000] = w2[:1_200_000][order]
        peer[:1_200_000], ctr[:1_200_000] = peer[:1_200_000][order], ctr[:1_200_000][order]
        assert (peer == 0).sum() > 1_500_000
        want = _window_expectation(peer, ctr, 2)
        d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")  # noqa: E731
        d_wire, d_out = d(wire), torch.zeros(wire.nbytes, dtype=torch.uint8, device="cuda:0")
        res = torch.zeros(n_total, dtype=torch.uint8, device="cuda:0")
        olen = torch.zeros(n_total, dtype=torch.int32, device="cuda:0")
        gp = torch.zeros(n_total, dtype=torch.int32, device="cuda:0")
        gc = torch.zeros(n_total, dtype=torch.int64, device="cuda:0")
        torch.cuda.synchronize()
        rxc.wg_decap(lib.make_batch(d_wire, wire.nbytes, n_total, lib.MEM_DEVICE, stride=stride, length=wire_len),
                     lib.make_batch(d_out, wire.nbytes, n_total, lib.MEM_DEVICE, stride=stride), res, olen, gp, gc)
        rxc.sync()
        assert np.array_equal(gp.cpu().numpy().astype(np.uint32), peer)
        assert np.array_equal(gc.cpu().numpy().astype(np.uint64), ctr)
        got = res.cpu().numpy()
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, f"result differs at {bad[:5]}: got {got[bad[:5]]} want {want[bad[:5]]}"
        assert (want == lib.WG_REPLAY).sum() > 100_000 and (want == lib.WG_OK).sum() > 100_000
        # the same datagrams again: the windows have seen or passed every counter
        rxc.wg_decap(lib.make_batch(d_wire, wire.nbytes, n_total, lib.MEM_DEVICE, stride=stride, length=wire_len),
                     lib.make_batch(d_out, wire.nbytes, n_total, lib.MEM_DEVICE, stride=stride), res, olen, gp, gc)
        rxc.sync()
        assert (res.cpu().numpy() == lib.WG_REPLAY).all()


@pytest.mark.parametrize("peers", [1, 2, 40])
def test_window_pass_with_few_and_many_senders(peers, monkeypatch):
    """The same walk as above, device resident, with one sender (every run spans
    several blocks of the pass, so repeats are looked for across blocks and a
    block's running maximum comes from the blocks before it), two, and forty
    (short runs, several to a block), per packet against the sequential filter."""
    import torch
    import sys
    from bnk_amd import lib
    from oracle import binding as O
    monkeypatch.setattr(sys.modules[__name__], "P", peers)
    rng = np.random.default_rng(300 + peers)
    tx, rx = _peers()
    keys = rng.integers(0, 256, (peers, 32), dtype=np.uint8)
    filters = [O.ReplayFilter() for _ in range(peers)]
    last = [0] * peers
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_RECV, keys)
        ctx.wg_peers_set(rx)
        for b, n in enumerate([3000, 1100, 6000, 2500]):
            arena, offs, lens, wires, last = _batch(rng, tx, keys, n, last, near_limit=(b == 1))
            want = _expect(wires, rx, keys, filters)
            total = arena.nbytes
            d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")  # noqa: E731
            d_arena, d_out = d(arena), torch.zeros(total, dtype=torch.uint8, device="cuda:0")
            res = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
            olen = torch.zeros(n, dtype=torch.int32, device="cuda:0")
            gp = torch.zeros(n, dtype=torch.int32, device="cuda:0")
            gc = torch.zeros(n, dtype=torch.int64, device="cuda:0")
            d_off, d_len = d(offs.astype(np.int64)), d(lens.astype(np.int32))
            torch.cuda.synchronize()
            ctx.wg_decap(lib.make_batch(d_arena, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_len),
                         lib.make_batch(d_out, total, n, lib.MEM_DEVICE, offsets=d_off), res, olen, gp, gc)
            ctx.sync()
            got = res.cpu().numpy()
            bad = np.flatnonzero(got != want[0])
            assert bad.size == 0, f"batch {b}: result differs at {bad[:5]}: got {got[bad[:5]]} want {want[0][bad[:5]]}"
            assert np.array_equal(olen.cpu().numpy().astype(np.uint32), want[1])
            assert (want[0] == lib.WG_REPLAY).sum() > 50
