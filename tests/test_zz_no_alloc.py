"""bnk_aead_seal_batch_noalloc (the entry point that allocates nothing: its
length-grouping scratch is a file-scope device array) against
bnk_aead_seal_batch, bit-exact, through the C ABI, on calls in a row that
share the array."""
import numpy as np
import pytest

from bnk_amd import workloads as W

pytestmark = pytest.mark.gpu


def _device_batch(b, dev):
    import torch
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    return dict(plain=d(b.plain), off=d(b.off.astype(np.int64)), lens=d(b.lens.astype(np.int32)),
                peer=d(b.peer.astype(np.int32)), ctr=d(b.counters.astype(np.int64)))


def _seal_both(ctx, b, dev):
    import torch
    from bnk_amd import lib
    t = _device_batch(b, dev)
    total = b.plain.nbytes
    outs = []
    for fn in (ctx.seal, ctx.seal_noalloc):
        out = torch.full((total,), 0x5A, dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        fn(lib.make_batch(t["plain"], total, b.n, lib.MEM_DEVICE, offsets=t["off"], lens=t["lens"],
                          peer=t["peer"], counters=t["ctr"]),
           lib.make_batch(out, total, b.n, lib.MEM_DEVICE, offsets=t["off"]))
        ctx.sync()
        outs.append(out.cpu().numpy())
    return outs


def test_noalloc_seal_matches_seal_on_calls_in_a_row():
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    dev = torch.device("cuda:0")
    with lib.Context(0) as ctx:
        # the second call is smaller than the first (stale order[] entries beyond
        # its packets must not matter), the third small enough for a wave per
        # packet (no grouping at all), the fourth large again
        for seed, n in ((31, 20000), (32, 6000), (33, 300), (34, 9000)):
            b = W.aead_imix(seed, n, n_peers=16)
            keys = np.ascontiguousarray(b.keys)
            ctx.keys_set(lib.KEYS_SEND, keys)
            ref, got = _seal_both(ctx, b, dev)
            assert np.array_equal(got, ref), "n=%d: differs from bnk_aead_seal_batch" % n
            want = np.full_like(b.plain, 0x5A)
            O.seal_batch(keys, b.peer, b.counters, b.plain, b.off, b.lens, want, b.off, 4)
            assert np.array_equal(got, want), "n=%d: differs from the oracle" % n
        # uniform layout, no per-packet arrays
        u = W.aead_uniform(35, 5000, 1420)
        ctx.keys_set(lib.KEYS_SEND, u.keys)
        pt = torch.from_numpy(u.plain).to(dev)
        outs = []
        for fn in (ctx.seal, ctx.seal_noalloc):
            out = torch.zeros_like(pt)
            torch.cuda.synchronize()
            fn(lib.make_batch(pt, pt.numel(), u.n, lib.MEM_DEVICE, stride=u.stride, length=1420,
                              counter0=int(u.counters[0])),
               lib.make_batch(out, pt.numel(), u.n, lib.MEM_DEVICE, stride=u.stride))
            ctx.sync()
            outs.append(out.cpu().numpy())
        assert np.array_equal(outs[0], outs[1])


def test_noalloc_seal_rejects_what_it_cannot_take():
    import torch
    from bnk_amd import lib
    dev = torch.device("cuda:0")
    with lib.Context(0) as ctx:
        key = np.zeros((1, 32), np.uint8)
        ctx.keys_set(lib.KEYS_SEND, key)
        buf = torch.zeros(4096, dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        # beyond the stated maximum
        with pytest.raises(lib.BnkError) as ei:
            n = lib.NOALLOC_MAX_PACKETS + 1
            ctx.seal_noalloc(lib.make_batch(buf, 4096, n, lib.MEM_DEVICE, stride=0, length=16),
                             lib.make_batch(buf, 4096, n, lib.MEM_DEVICE, stride=0))
        assert ei.value.code == lib.E_INVAL
        # host memory would need staging buffers
        h = np.zeros(4096, np.uint8)
        with pytest.raises(lib.BnkError) as ei:
            ctx.seal_noalloc(lib.make_batch(h, 4096, 4, lib.MEM_HOST, stride=64, length=16),
                             lib.make_batch(h, 4096, 4, lib.MEM_HOST, stride=64))
        assert ei.value.code == lib.E_INVAL
