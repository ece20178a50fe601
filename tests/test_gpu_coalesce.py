"""Calls from several threads merged into one batch inside the library
(bnk_set_coalesce), the calling pattern of wireguard-go's per-peer goroutines
(internal/filter/filter.go:171-186, internal/magicsock/bind.go:326-328): every
caller must get exactly what its own call would have returned -- ciphertexts,
tags, verdicts, BNK_WG_* results, lengths, peers, counters -- and the state the
calls leave behind (send counters, anti-replay windows, flow table) must be
that of the calls run one after the other.  Checked against the CPU oracle per
call; the statistics show that the calls did share launches."""
import struct
import threading

import numpy as np
import pytest

from bnk_amd import workloads as W

pytestmark = pytest.mark.gpu

T = 8          # caller threads
PER = 96       # packets per call (wireguard-go hands over at most 128)
MTU = 1420
T0 = 1_700_000_000 * 10**9


def _run_threads(fns):
    """Runs fns[t]() on T threads released together; re-raises the first failure."""
    errs = [None] * len(fns)
    gate = threading.Barrier(len(fns))

    def body(t):
        try:
            gate.wait()
            fns[t]()
        except BaseException as e:  # noqa: BLE001
            errs[t] = e

    th = [threading.Thread(target=body, args=(t,)) for t in range(len(fns))]
    for x in th:
        x.start()
    for x in th:
        x.join()
    for e in errs:
        if e is not None:
            raise e


def test_seal_and_open_from_many_threads_share_launches_and_match_the_oracle():
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(11)
    n_peers = 2 * T
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    rounds = 6
    slot = 1536
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_SEND, keys)
        ctx.keys_set(lib.KEYS_RECV, keys)
        plain = ctx.ring_alloc(T * PER * slot)
        sealed = ctx.ring_alloc(T * PER * slot)
        back = ctx.ring_alloc(T * PER * slot)
        # an unreasonably long wait: the first window of each kind forms only
        # when all T callers have arrived, whatever the scheduler does
        ctx.set_coalesce(4096, 2_000_000, T)
        for r in range(rounds):
            plain[:] = rng.integers(0, 256, plain.size, dtype=np.uint8)
            sealed[:] = 0x5A
            back[:] = 0xA5
            calls = []
            for t in range(T):
                # four shapes of call: per-packet arrays, a uniform stride with
                # counter0, no peer array (peer 0), short ragged packets
                shape = (t + r) % 4
                n = PER - (t % 3)
                base = t * PER * slot
                if shape == 0:
                    lens = rng.choice([60, 576, 1420, 0, 1, 17], n).astype(np.uint32)
                    off = (np.arange(n, dtype=np.uint64) * slot + np.uint64(16 * (t % 2)))
                    peer = rng.integers(0, n_peers, n).astype(np.uint32)
                    ctr = rng.integers(0, 1 << 62, n).astype(np.uint64)
                    kw = dict(offsets=off, lens=lens, peer=peer, counters=ctr)
                elif shape == 1:
                    lens = np.full(n, 1420, np.uint32)
                    off = np.arange(n, dtype=np.uint64) * slot
                    peer = np.full(n, (2 * t) % n_peers, np.uint32)
                    ctr = np.arange(n, dtype=np.uint64) + np.uint64(1000 * r + 7)
                    kw = dict(stride=slot, length=1420, peer=peer, counter0=1000 * r + 7)
                elif shape == 2:
                    lens = np.full(n, 1420, np.uint32)
                    off = np.arange(n, dtype=np.uint64) * slot
                    peer = np.zeros(n, np.uint32)
                    ctr = rng.integers(0, 1 << 40, n).astype(np.uint64)
                    kw = dict(stride=slot, length=1420, counters=ctr)
                else:
                    lens = rng.integers(0, 130, n).astype(np.uint32)
                    off = np.arange(n, dtype=np.uint64) * slot + np.uint64(3)   # misaligned
                    peer = rng.integers(0, n_peers, n).astype(np.uint32)
                    ctr = rng.integers(0, 1 << 62, n).astype(np.uint64)
                    kw = dict(offsets=off, lens=lens, peer=peer, counters=ctr)
                calls.append(dict(n=n, base=base, lens=lens, off=off, peer=peer, ctr=ctr, kw=kw,
                                  verdict=np.full(n, 9, np.uint8)))
            nbytes = PER * slot

            def seal(t):
                c = calls[t]
                ctx.seal(lib.make_batch(plain[c["base"]:c["base"] + nbytes], nbytes, c["n"], lib.MEM_HOST, **c["kw"]),
                         lib.make_batch(sealed[c["base"]:c["base"] + nbytes], nbytes, c["n"], lib.MEM_HOST,
                                        offsets=c["kw"].get("offsets"), stride=c["kw"].get("stride", 0)))

            _run_threads([lambda t=t: seal(t) for t in range(T)])
            want = np.full(sealed.size, 0x5A, np.uint8)
            for t, c in enumerate(calls):
                O.seal_batch(keys, c["peer"], c["ctr"], np.array(plain), c["off"] + np.uint64(c["base"]), c["lens"],
                             want, c["off"] + np.uint64(c["base"]), 2)
            assert np.array_equal(np.array(sealed), want), "round %d: sealed bytes differ from the oracle" % r

            # forge some tags, then open from T threads
            forged = []
            for t, c in enumerate(calls):
                f = rng.random(c["n"]) < 0.1
                for i in np.flatnonzero(f):
                    sealed[c["base"] + int(c["off"][i]) + int(c["lens"][i]) + int(rng.integers(0, 16))] ^= 1 << int(rng.integers(0, 8))
                forged.append(f)

            def open_(t):
                c = calls[t]
                kw = dict(c["kw"])
                if "lens" in kw:
                    kw["lens"] = (c["lens"] + 16).astype(np.uint32)
                else:
                    kw["length"] = 1436
                ctx.open(lib.make_batch(sealed[c["base"]:c["base"] + nbytes], nbytes, c["n"], lib.MEM_HOST, **kw),
                         lib.make_batch(back[c["base"]:c["base"] + nbytes], nbytes, c["n"], lib.MEM_HOST,
                                        offsets=kw.get("offsets"), stride=kw.get("stride", 0)), c["verdict"])

            _run_threads([lambda t=t: open_(t) for t in range(T)])
            want_back = np.full(back.size, 0xA5, np.uint8)
            for t, c in enumerate(calls):
                v = O.open_batch(keys, c["peer"], c["ctr"], np.array(sealed), c["off"] + np.uint64(c["base"]),
                                 (c["lens"] + 16).astype(np.uint32), want_back, c["off"] + np.uint64(c["base"]), 2)
                assert np.array_equal(c["verdict"], v), "round %d caller %d: verdicts" % (r, t)
                assert np.array_equal(c["verdict"] == 0, forged[t])
            assert np.array_equal(np.array(back), want_back), "round %d: opened bytes differ from the oracle" % r
        st = ctx.coalesce_stats()
        assert st["calls"] == 2 * rounds * T and st["largest_callers"] == T, st
        assert st["batches"] < st["calls"] / 2 and st["retried"] == 0, st
        ctx.set_coalesce(0)
        for ring in (plain, sealed, back):
            ctx.ring_free(ring)


def _inner(rng, src, dst, kind, i):
    if kind == 0:
        return W.tcp(src, dst, 40000 + i % 20000, int(rng.choice([22, 23, 8000, 443])))
    if kind == 1:
        return W.udp(src, dst, int(rng.choice([53, 9000])), int(rng.choice([53, 4000, 4001])))
    if kind == 2:
        return W.icmp_echo(src, dst)
    if kind == 3:
        return b""  # keepalive
    body = rng.integers(0, 256, int(rng.integers(100, 1380)), dtype=np.uint8).tobytes()
    return _with_len(W.tcp(src, dst, 50000 + i % 1000, 8000), body)


def _with_len(pkt: bytes, body: bytes) -> bytes:
    """The packet with `body` appended and the IPv4 total length adjusted."""
    out = bytearray(pkt + body)
    out[2:4] = struct.pack(">H", len(out))
    return bytes(out)


def test_tunnel_calls_from_many_threads_match_the_oracle_call_by_call():
    """T sender threads (two peers each) and T receiver threads on two contexts,
    both merging: NoteOutbound + encapsulate, then decapsulate + CheckInbound of
    the same datagrams, then the same datagrams once more (all replays)."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(12)
    n_peers = 2 * T
    # sender's view: (local index, the receiver's index for us, the receiver's address)
    tx_peers = [(3000 + 7 * p, 9000 + 11 * p, 0x64500001 + p, 0xFFFFFFFF) for p in range(n_peers)]
    # receiver's view of the same keypairs: senders' inner source addresses are 100.64.0.x
    src_of = [0x64400001 + p for p in range(n_peers)]
    rx_peers = [(tx_peers[p][1], tx_peers[p][0], src_of[p], 0xFFFFFFFF) for p in range(n_peers)]
    keys = rng.integers(0, 256, (n_peers, 32), dtype=np.uint8)
    rules = [([(src_of[p], 32)], "tcp", [(22, 22), (8000, 8100)]) for p in range(0, n_peers, 2)]
    rules += [([(0x64400000, 16)], "udp", [(53, 53)])]
    local = 0x64700001
    slot = 1536
    rounds = 4
    with lib.Context(0) as txc, lib.Context(0) as rxc:
        txc.keys_set(lib.KEYS_SEND, keys)
        txc.wg_peers_set(tx_peers)
        txc.filter_set_rules(rules)
        rxc.keys_set(lib.KEYS_RECV, keys)
        rxc.wg_peers_set(rx_peers)
        rxc.filter_set_rules(rules)
        ring = txc.ring_alloc(T * PER * slot)
        wire = rxc.ring_alloc(T * PER * slot)
        out = rxc.ring_alloc(T * PER * slot)
        txc.set_coalesce(4096, 2_000_000, T)
        rxc.set_coalesce(4096, 2_000_000, T)
        ora_tx, ora_rx = O.Filter(), O.Filter()
        ora_tx.set_rules(rules)
        ora_rx.set_rules(rules)
        next_ctr = [0] * n_peers
        windows = [O.ReplayFilter() for _ in range(n_peers)]
        seen = set()
        for r in range(rounds):
            now = T0 + r * 10**9
            ring[:] = 0xEE
            calls = []
            for t in range(T):
                n = PER - 2 * (t % 4)
                peer = rng.choice([2 * t, 2 * t + 1], n).astype(np.uint32)
                inner = [_inner(rng, src_of[int(peer[i])] if rng.random() > 0.05 else src_of[int(peer[i])] ^ 0x100,
                                local, int(rng.integers(0, 5)), i) for i in range(n)]
                lens = np.array([len(x) for x in inner], np.uint32)
                off = np.arange(n, dtype=np.uint64) * slot
                base = t * PER * slot
                for i, x in enumerate(inner):
                    o = base + int(off[i]) + 16
                    ring[o:o + len(x)] = np.frombuffer(x, np.uint8)
                calls.append(dict(n=n, base=base, peer=peer, inner=inner, lens=lens, off=off,
                                  wire_len=np.zeros(n, np.uint32)))
            nbytes = PER * slot

            def send(t):
                c = calls[t]
                txc.wg_note_encap(lib.make_batch(ring[c["base"]:c["base"] + nbytes], nbytes, c["n"], lib.MEM_HOST,
                                                 offsets=c["off"], lens=c["lens"], peer=c["peer"]), MTU, now,
                                  c["wire_len"])

            _run_threads([lambda t=t: send(t) for t in range(T)])
            # oracle, call by call: one peer's packets all come from one caller, in order
            for t, c in enumerate(calls):
                for i in range(c["n"]):
                    p = int(c["peer"][i])
                    w = O.wg_encap(c["inner"][i], MTU, keys[p].tobytes(), tx_peers[p][1], next_ctr[p])
                    next_ctr[p] += 1
                    o = c["base"] + int(c["off"][i])
                    assert int(c["wire_len"][i]) == len(w)
                    assert bytes(ring[o:o + len(w)]) == w, "round %d caller %d packet %d: datagram" % (r, t, i)
                    ora_tx.note_outbound(c["inner"][i], now)
            assert np.array_equal(txc.wg_send_counters(n_peers), np.array(next_ctr, np.uint64))
            assert txc.filter_flows() == ora_tx.flows()

            # the receiving side: the same datagrams, a few tampered with
            wire[:] = ring
            for t, c in enumerate(calls):
                for i in np.flatnonzero(rng.random(c["n"]) < 0.04):
                    wire[c["base"] + int(c["off"][i]) + int(c["wire_len"][i]) - 1] ^= 0x80
            for again in (False, True):
                out[:] = 0x77
                for c in calls:
                    c["res"], c["olen"] = np.full(c["n"], 99, np.uint8), np.full(c["n"], 99, np.uint32)
                    c["gp"], c["gc"] = np.full(c["n"], 99, np.uint32), np.full(c["n"], 99, np.uint64)

                def recv(t):
                    c = calls[t]
                    rxc.wg_decap_filter(lib.make_batch(wire[c["base"]:c["base"] + nbytes], nbytes, c["n"], lib.MEM_HOST,
                                                       offsets=c["off"], lens=c["wire_len"]),
                                        lib.make_batch(out[c["base"]:c["base"] + nbytes], nbytes, c["n"], lib.MEM_HOST,
                                                       offsets=c["off"]), now, c["res"], c["olen"], c["gp"], c["gc"])

                _run_threads([lambda t=t: recv(t) for t in range(T)])
                for t, c in enumerate(calls):
                    for i in range(c["n"]):
                        o = c["base"] + int(c["off"][i])
                        dg = bytes(wire[o:o + int(c["wire_len"][i])])
                        rc, pt, p, ctr = O.wg_decap(dg, rx_peers, keys)
                        delivered = len(pt)
                        if rc not in (lib.WG_BAD_HEADER, lib.WG_UNKNOWN_INDEX, lib.WG_AUTH_FAIL):
                            # the window first, as wireguard-go's sequential receiver has it
                            if not windows[p].validate(ctr):
                                rc, delivered = lib.WG_REPLAY, 0
                            elif rc == lib.WG_OK and not ora_rx.check_inbound(pt, now):
                                rc = lib.WG_FILTERED
                        seen.add(rc)
                        assert (int(c["res"][i]), int(c["olen"][i])) == (rc, delivered), \
                            "round %d caller %d packet %d again=%s: got %d/%d want %d/%d" % (
                                r, t, i, again, c["res"][i], c["olen"][i], rc, delivered)
                        if rc not in (lib.WG_BAD_HEADER, lib.WG_UNKNOWN_INDEX):
                            assert (int(c["gp"][i]), int(c["gc"][i])) == (p, ctr)
                        if rc in (lib.WG_OK, lib.WG_FILTERED):
                            assert bytes(out[o:o + delivered]) == pt
                assert rxc.filter_flows() == ora_rx.flows()
        assert {lib.WG_OK, lib.WG_KEEPALIVE, lib.WG_AUTH_FAIL, lib.WG_NOT_ALLOWED, lib.WG_FILTERED,
                lib.WG_REPLAY} <= seen, seen
        for ctx in (txc, rxc):
            st = ctx.coalesce_stats()
            assert st["largest_callers"] == T and st["retried"] == 0 and st["batches"] < st["calls"] / 2, st
            ctx.set_coalesce(0)
        txc.ring_free(ring)
        rxc.ring_free(wire)
        rxc.ring_free(out)


def test_a_call_a_direct_call_would_refuse_is_refused_alone():
    """One caller of a window names a peer beyond the key table: it gets
    BNK_E_RANGE with its own message, every other caller of the window gets its
    results."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(13)
    keys = rng.integers(0, 256, (4, 32), dtype=np.uint8)
    slot, n = 256, 32
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_SEND, keys)
        ring = ctx.ring_alloc(T * n * slot)
        outr = ctx.ring_alloc(T * n * slot)
        ring[:] = rng.integers(0, 256, ring.size, dtype=np.uint8)
        outr[:] = 0x5A
        ctx.set_coalesce(4096, 2_000_000, T)
        peers = [rng.integers(0, 4, n).astype(np.uint32) for _ in range(T)]
        peers[3][5] = 4  # beyond the table
        ctrs = [rng.integers(0, 1 << 60, n).astype(np.uint64) for _ in range(T)]
        failed = [None] * T

        def seal(t):
            nb = n * slot
            try:
                ctx.seal(lib.make_batch(ring[t * nb:(t + 1) * nb], nb, n, lib.MEM_HOST, stride=slot, length=200,
                                        peer=peers[t], counters=ctrs[t]),
                         lib.make_batch(outr[t * nb:(t + 1) * nb], nb, n, lib.MEM_HOST, stride=slot))
            except lib.BnkError as e:
                failed[t] = e

        _run_threads([lambda t=t: seal(t) for t in range(T)])
        assert [f is not None for f in failed] == [t == 3 for t in range(T)]
        assert failed[3].code == lib.E_RANGE
        want = np.full(outr.size, 0x5A, np.uint8)
        off = np.arange(n, dtype=np.uint64) * slot
        for t in range(T):
            if t != 3:
                O.seal_batch(keys, peers[t], ctrs[t], np.array(ring), off + np.uint64(t * n * slot),
                             np.full(n, 200, np.uint32), want, off + np.uint64(t * n * slot), 1)
        assert np.array_equal(np.array(outr), want)
        assert ctx.coalesce_stats()["retried"] == 1
        # calls that do not qualify (pageable memory) run as before with merging on
        pt = rng.integers(0, 256, n * slot, dtype=np.uint8)
        ct = np.zeros(n * slot, np.uint8)
        ctx.seal(lib.make_batch(pt, pt.nbytes, n, lib.MEM_HOST, stride=slot, length=200, peer=peers[0], counters=ctrs[0]),
                 lib.make_batch(ct, ct.nbytes, n, lib.MEM_HOST, stride=slot))
        w2 = np.zeros_like(ct)
        O.seal_batch(keys, peers[0], ctrs[0], pt, off, np.full(n, 200, np.uint32), w2, off, 1)
        assert np.array_equal(ct, w2)
        ctx.set_coalesce(0)
        ctx.ring_free(ring)
        ctx.ring_free(outr)
