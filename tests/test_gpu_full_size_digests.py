"""Configurations 2 and 3 at their full size (2^20 packets), device resident,
against SHA-256 digests of what OpenSSL seals for the same seeded inputs
(tests/golden/aead_cfg2_cfg3_digests.json, written by
tests/golden/make_aead_digests.py): every sealed byte of every packet, in the
slotted and in the packed layout, then the way back."""
import hashlib
import json
import os

import numpy as np
import pytest

from bnk_amd import workloads as W

pytestmark = pytest.mark.gpu

N = 1 << 20
GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "aead_cfg2_cfg3_digests.json")))


def _sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).data).hexdigest()


def test_cfg2_full_size_sealed_bytes_match_the_openssl_digest():
    import torch
    from bnk_amd import lib
    L, S = 1420, 1440
    g = GOLDEN["cfg2"]
    dev = torch.device("cuda:0")
    key = np.frombuffer(bytes.fromhex(g["key"]), np.uint8).reshape(1, 32)
    assert np.array_equal(key, W.rand_bytes(W.stream_seed(2, 0), 32).reshape(1, 32))
    plain = W.aead_uniform_torch(2, N, L, S, dev)
    assert _sha(plain[:, :L].cpu().numpy()) == g["sha256_plain"], "the generators disagree"
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_SEND, key)
        ctx.keys_set(lib.KEYS_RECV, key)
        # ---- 1440-byte slots ----
        sealed = torch.full_like(plain, 0x5A)
        torch.cuda.synchronize()
        ctx.seal(lib.make_batch(plain, N * S, N, lib.MEM_DEVICE, stride=S, length=L),
                 lib.make_batch(sealed, N * S, N, lib.MEM_DEVICE, stride=S))
        ctx.sync()
        h = sealed.cpu().numpy()
        assert _sha(h[:, :L + 16]) == g["sha256_sealed"]
        for i, want in g["sha256_of_packet"].items():
            assert _sha(h[int(i), :L + 16]) == want
        assert (h[:, L + 16:] == 0x5A).all()  # the four bytes behind every tag are not touched
        del h
        back = torch.full_like(plain, 0xA5)
        v = torch.zeros(N, dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        ctx.open(lib.make_batch(sealed, N * S, N, lib.MEM_DEVICE, stride=S, length=L + 16),
                 lib.make_batch(back, N * S, N, lib.MEM_DEVICE, stride=S), v)
        ctx.sync()
        assert bool(v.all()) and torch.equal(back[:, :L], plain[:, :L]) and bool((back[:, L:] == 0xA5).all())
        del back, sealed
        # ---- packed: plaintexts back to back at a 1420-byte stride, sealed at 1436 ----
        pk_plain = plain[:, :L].contiguous().view(-1)
        pk_sealed = torch.zeros(N * (L + 16), dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        ctx.seal(lib.make_batch(pk_plain, N * L, N, lib.MEM_DEVICE, stride=L, length=L),
                 lib.make_batch(pk_sealed, N * (L + 16), N, lib.MEM_DEVICE, stride=L + 16))
        ctx.sync()
        assert _sha(pk_sealed.cpu().numpy()) == g["sha256_sealed"]  # the arena is the concatenation
        pk_back = torch.zeros(N * L, dtype=torch.uint8, device=dev)
        v.zero_()
        torch.cuda.synchronize()
        ctx.open(lib.make_batch(pk_sealed, N * (L + 16), N, lib.MEM_DEVICE, stride=L + 16, length=L + 16),
                 lib.make_batch(pk_back, N * L, N, lib.MEM_DEVICE, stride=L), v)
        ctx.sync()
        assert bool(v.all()) and torch.equal(pk_back, pk_plain)


def _concat_sha(arena: np.ndarray, off, lens, extra: int) -> str:
    h = hashlib.sha256()
    mv = memoryview(arena)
    for o, n in zip(off.tolist(), lens.tolist()):
        h.update(mv[o:o + n + extra])
    return h.hexdigest()


def test_cfg3_full_size_sealed_bytes_match_the_openssl_digest():
    import torch
    from bnk_amd import lib
    g = GOLDEN["cfg3"]
    dev = torch.device("cuda:0")
    b = W.aead_imix(3, N, n_peers=256, payload=False)
    total = b.meta["total"]
    assert total == g["arena_bytes"] and int(b.lens.sum()) == g["payload_bytes"]
    plain = W.imix_plain_torch(b, dev)
    hp = plain.cpu().numpy()
    assert _concat_sha(hp, b.off, b.lens, 0) == g["sha256_plain"], "the generators disagree"
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    d_off, d_peer, d_ctr = d(b.off.astype(np.int64)), d(b.peer.astype(np.int32)), d(b.counters.astype(np.int64))
    d_lens, d_ctl = d(b.lens.astype(np.int32)), d((b.lens + 16).astype(np.int32))
    sealed = torch.full((total,), 0x5A, dtype=torch.uint8, device=dev)
    back = torch.full((total,), 0xA5, dtype=torch.uint8, device=dev)
    v = torch.zeros(N, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    keys = np.ascontiguousarray(b.keys)
    with lib.Context(0) as ctx:
        ctx.keys_set(lib.KEYS_SEND, keys)
        ctx.keys_set(lib.KEYS_RECV, keys)
        ctx.seal(lib.make_batch(plain, total, N, lib.MEM_DEVICE, offsets=d_off, lens=d_lens, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(sealed, total, N, lib.MEM_DEVICE, offsets=d_off))
        ctx.sync()
        hs = sealed.cpu().numpy()
        assert _concat_sha(hs, b.off, b.lens, 16) == g["sha256_sealed"]
        for i, want in g["sha256_of_packet"].items():
            o, n = int(b.off[int(i)]), int(b.lens[int(i)])
            assert _sha(hs[o:o + n + 16]) == want
        ctx.open(lib.make_batch(sealed, total, N, lib.MEM_DEVICE, offsets=d_off, lens=d_ctl, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(back, total, N, lib.MEM_DEVICE, offsets=d_off), v)
        ctx.sync()
        assert bool(v.all())
        assert _concat_sha(back.cpu().numpy(), b.off, b.lens, 0) == g["sha256_plain"]
