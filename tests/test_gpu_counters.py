"""The hot-path counters (bnk_counters_get): packets by outcome over every entry
point of a context.  They are an addition (the reference's filter drops
without counting, internal/filter/filter.go:100-145), so what is checked is
that they are the histogram of the result bytes the calls return -- which the
other tests pin against the oracle -- for host batches (counted on the host)
and device-resident ones (counted by a launch behind the batch) alike, that a
failed call counts nothing, and that merged calls count once."""
import threading

import numpy as np
import pytest

from bnk_amd import workloads as W

pytestmark = pytest.mark.gpu

ZERO = dict.fromkeys(("sealed", "opened", "rejected", "allowed", "denied", "delivered", "keepalive", "replayed",
                      "bad_header", "unknown_index", "bad_ip", "not_allowed", "relayed"), 0)


def test_seal_open_counts_host_and_device_and_reset():
    import torch
    from bnk_amd import lib
    rng = np.random.default_rng(5)
    n, length, stride = 3000, 60, 128
    keys = rng.integers(0, 256, (4, 32), dtype=np.uint8)
    peer = rng.integers(0, 4, n).astype(np.uint32)
    ctr = np.arange(n, dtype=np.uint64)
    plain = rng.integers(0, 256, n * stride, dtype=np.uint8)
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_SEND, keys)
        ctx.keys_set(lib.KEYS_RECV, keys)
        assert ctx.counters() == ZERO
        sealed = np.zeros_like(plain)
        ctx.seal(lib.make_batch(plain, plain.nbytes, n, lib.MEM_HOST, stride=stride, length=length, peer=peer,
                                counters=ctr),
                 lib.make_batch(sealed, sealed.nbytes, n, lib.MEM_HOST, stride=stride))
        forged = rng.choice(n, 7, replace=False)
        sealed.reshape(n, stride)[forged, length + 3] ^= 0x10
        back, verdict = np.zeros_like(plain), np.zeros(n, np.uint8)
        ctx.open(lib.make_batch(sealed, sealed.nbytes, n, lib.MEM_HOST, stride=stride, length=length + 16, peer=peer,
                                counters=ctr),
                 lib.make_batch(back, back.nbytes, n, lib.MEM_HOST, stride=stride), verdict)
        assert int(verdict.sum()) == n - 7
        assert ctx.counters() == {**ZERO, "sealed": n, "opened": n - 7, "rejected": 7}
        # the same open, device resident: one more of each
        d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")  # noqa: E731
        d_sealed, d_back, d_verdict = d(sealed), torch.zeros(plain.nbytes, dtype=torch.uint8, device="cuda:0"), \
            torch.zeros(n, dtype=torch.uint8, device="cuda:0")
        d_peer, d_ctr = d(peer.astype(np.int32)), d(ctr.astype(np.int64))
        torch.cuda.synchronize()
        for _ in range(2):
            ctx.open(lib.make_batch(d_sealed, sealed.nbytes, n, lib.MEM_DEVICE, stride=stride, length=length + 16,
                                    peer=d_peer, counters=d_ctr),
                     lib.make_batch(d_back, back.nbytes, n, lib.MEM_DEVICE, stride=stride), d_verdict)
        assert ctx.counters() == {**ZERO, "sealed": n, "opened": 3 * (n - 7), "rejected": 21}
        assert int(d_verdict.sum().item()) == n - 7
        # a call that fails counts nothing
        bad_peer = peer.copy()
        bad_peer[11] = 99
        with pytest.raises(lib.BnkError):
            ctx.seal(lib.make_batch(plain, plain.nbytes, n, lib.MEM_HOST, stride=stride, length=length,
                                    peer=bad_peer, counters=ctr),
                     lib.make_batch(sealed, sealed.nbytes, n, lib.MEM_HOST, stride=stride))
        assert ctx.counters()["sealed"] == n
        ctx.counters_reset()
        assert ctx.counters() == ZERO
        # switched off, calls are not counted (and a device-resident one launches nothing more)
        ctx.counters_enable(False)
        ctx.open(lib.make_batch(d_sealed, sealed.nbytes, n, lib.MEM_DEVICE, stride=stride, length=length + 16,
                                peer=d_peer, counters=d_ctr),
                 lib.make_batch(d_back, back.nbytes, n, lib.MEM_DEVICE, stride=stride), d_verdict)
        assert ctx.counters() == ZERO
        ctx.counters_enable(True)
        # a result array that does not start on a 16-byte boundary, and not a multiple of 16 long
        ctx.open(lib.make_batch(d_sealed, sealed.nbytes, n - 8, lib.MEM_DEVICE, stride=stride, length=length + 16,
                                peer=d_peer, counters=d_ctr),
                 lib.make_batch(d_back, back.nbytes, n - 8, lib.MEM_DEVICE, stride=stride), d_verdict[5:])
        late = int((forged >= n - 8).sum())
        assert ctx.counters() == {**ZERO, "opened": n - 8 - (7 - late), "rejected": 7 - late}


def test_merged_calls_count_once_each():
    from bnk_amd import lib
    rng = np.random.default_rng(6)
    threads, per, length, slot = 6, 100, 200, 256
    keys = rng.integers(0, 256, (threads, 32), dtype=np.uint8)
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_SEND, keys)
        ctx.keys_set(lib.KEYS_RECV, keys)
        a, b = ctx.ring_alloc(threads * per * slot), ctx.ring_alloc(threads * per * slot)
        a[:] = rng.integers(0, 256, a.size, dtype=np.uint8)
        ctx.set_coalesce(4096, 2_000_000, threads)
        verdicts = [np.zeros(per, np.uint8) for _ in range(threads)]
        gate = threading.Barrier(threads)
        errs = []

        def body(t):
            try:
                peer = np.full(per, t, np.uint32)
                lo = t * per * slot
                kw = dict(stride=slot, peer=peer)
                gate.wait()
                ctx.seal(lib.make_batch(a[lo:], per * slot, per, lib.MEM_HOST, length=length, counter0=t << 20, **kw),
                         lib.make_batch(b[lo:], per * slot, per, lib.MEM_HOST, stride=slot))
                if t == 2:
                    b[lo + 5 * slot + 1] ^= 1
                gate.wait()
                ctx.open(lib.make_batch(b[lo:], per * slot, per, lib.MEM_HOST, length=length + 16, counter0=t << 20,
                                        **kw),
                         lib.make_batch(a[lo:], per * slot, per, lib.MEM_HOST, stride=slot), verdicts[t])
            except BaseException as e:  # noqa: BLE001
                errs.append(e)
                gate.abort()

        th = [threading.Thread(target=body, args=(t,)) for t in range(threads)]
        for x in th:
            x.start()
        for x in th:
            x.join()
        assert not errs, errs
        assert ctx.coalesce_stats()["batches"] < 2 * threads  # they did share launches
        total = threads * per
        assert ctx.counters() == {**ZERO, "sealed": total, "opened": total - 1, "rejected": 1}
        ctx.ring_free(a)
        ctx.ring_free(b)


@pytest.mark.parametrize("where", ["host", "device"])
def test_tunnel_and_filter_counts_are_the_histogram_of_the_results(where):
    import torch
    from bnk_amd import lib
    from tests.test_gpu_wg_replay import P, _batch, _peers
    rng = np.random.default_rng(31)
    tx, rx = _peers()
    keys = rng.integers(0, 256, (P, 32), dtype=np.uint8)
    n = 4000
    arena, offs, lens, wires, _ = _batch(rng, tx, keys, n, [0] * P)
    # anything TCP, UDP or ICMP from anywhere may come in: the inner packets are random bytes
    # behind a valid IPv4 header, so most carry another protocol and are refused
    rules = [([(0, 0)], "tcp", [(0, 65535)]), ([(0, 0)], "udp", [(0, 65535)]), ([(0, 0)], "icmp", [])]
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_RECV, keys)
        ctx.wg_peers_set(rx)
        ctx.filter_set_rules(rules)
        res, olen = np.zeros(n, np.uint8), np.zeros(n, np.uint32)
        gp, gc = np.zeros(n, np.uint32), np.zeros(n, np.uint64)
        now = 1_700_000_000 * 10**9
        if where == "host":
            out = np.zeros(arena.nbytes, np.uint8)
            ctx.wg_decap_filter(lib.make_batch(arena, arena.nbytes, n, lib.MEM_HOST, offsets=offs, lens=lens),
                                lib.make_batch(out, out.nbytes, n, lib.MEM_HOST, offsets=offs), now, res, olen, gp, gc)
        else:
            d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")  # noqa: E731
            d_arena, d_out = d(arena), torch.zeros(arena.nbytes, dtype=torch.uint8, device="cuda:0")
            d_res = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
            d_olen = torch.zeros(n, dtype=torch.int32, device="cuda:0")
            d_gp = torch.zeros(n, dtype=torch.int32, device="cuda:0")
            d_gc = torch.zeros(n, dtype=torch.int64, device="cuda:0")
            d_off, d_len = d(offs.astype(np.int64)), d(lens.astype(np.int32))
            torch.cuda.synchronize()
            ctx.wg_decap_filter(lib.make_batch(d_arena, arena.nbytes, n, lib.MEM_DEVICE, offsets=d_off, lens=d_len),
                                lib.make_batch(d_out, arena.nbytes, n, lib.MEM_DEVICE, offsets=d_off), now, d_res,
                                d_olen, d_gp, d_gc)
            ctx.sync()
            res = d_res.cpu().numpy()
        hist = np.bincount(res, minlength=16)
        got = ctx.counters()
        assert got == {**ZERO, "delivered": hist[lib.WG_OK], "allowed": hist[lib.WG_OK],
                       "denied": hist[lib.WG_FILTERED], "keepalive": hist[lib.WG_KEEPALIVE],
                       "rejected": hist[lib.WG_AUTH_FAIL], "replayed": hist[lib.WG_REPLAY],
                       "bad_ip": hist[lib.WG_BAD_IP], "not_allowed": hist[lib.WG_NOT_ALLOWED],
                       "bad_header": hist[lib.WG_BAD_HEADER], "unknown_index": hist[lib.WG_UNKNOWN_INDEX]}
        # every kind of outcome the walk produces took part
        for k in ("delivered", "denied", "keepalive", "rejected", "replayed", "bad_ip", "not_allowed"):
            assert got[k] > 0, k
        assert sum(got[k] for k in got if k != "allowed") == n


def test_relay_and_standalone_filter_counts():
    from bnk_amd import lib
    w = W.relay_workload(n=12000, n_peers=64, n_rules=512)
    b = w.batch
    from oracle import binding as O
    sealed = np.zeros_like(b.plain)
    O.seal_batch(np.ascontiguousarray(b.keys), b.peer, b.counters, b.plain, b.off, b.lens, sealed, b.off, 4)
    W.forge_tags(5, sealed, b.off, b.lens, w.forged_fraction)
    ct_lens = (b.lens + 16).astype(np.uint32)
    with lib.Context(0) as ctx:
        ctx.filter_set_rules(w.rules_ref)
        ctx.keys_set(lib.KEYS_RECV, np.ascontiguousarray(b.keys))
        ctx.keys_set(lib.KEYS_SEND, np.ascontiguousarray(w.keys_out))
        out = np.zeros_like(b.plain)
        v, c = np.zeros(b.n, np.uint8), np.zeros(b.n, np.uint64)
        ctx.relay_fused(lib.make_batch(sealed, sealed.nbytes, b.n, lib.MEM_HOST, offsets=b.off, lens=ct_lens,
                                       peer=b.peer, counters=b.counters),
                        w.peer_out, w.ctr_base_out, len(w.ctr_base_out), w.now_ns,
                        lib.make_batch(out, out.nbytes, b.n, lib.MEM_HOST, offsets=b.off), v, c)
        hist = np.bincount(v, minlength=3)
        assert hist[1] > 0 and hist[2] > 0
        assert ctx.counters() == {**ZERO, "relayed": hist[0], "rejected": hist[1], "denied": hist[2]}
        ctx.counters_reset()
        # CheckInbound on its own, over the plaintexts
        verdict = np.zeros(b.n, np.uint8)
        ctx.filter_check_inbound(lib.make_batch(b.plain, b.plain.nbytes, b.n, lib.MEM_HOST, offsets=b.off,
                                                lens=b.lens), w.now_ns, verdict)
        assert 0 < int(verdict.sum()) < b.n
        assert ctx.counters() == {**ZERO, "allowed": int(verdict.sum()), "denied": b.n - int(verdict.sum())}
