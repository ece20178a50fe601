"""The configurations at their full size, device resident, against committed
SHA-256 digests.  Configurations 2 and 3 (2^20 packets): what OpenSSL seals for
the same seeded inputs (tests/golden/aead_cfg2_cfg3_digests.json, written by
tests/golden/make_aead_digests.py), every sealed byte of every packet, in the
slotted and in the packed layout, then the way back.  Configurations 4 and 5
(2^22 packets): what the sequential CPU oracle computes
(tests/golden/filter_relay_digests.json, written by
tests/golden/make_filter_relay_digests.py), every verdict, counter, re-sealed
byte and flow-table entry."""
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


# ---- configurations 4 and 5 against the CPU oracle's digests ----------------

def _fr_golden():
    return json.load(open(os.path.join(os.path.dirname(__file__), "golden", "filter_relay_digests.json")))


def _flows_digest(flows: dict) -> str:
    import struct
    h = hashlib.sha256()
    for key in sorted(flows):
        h.update(struct.pack("<IHHBq", key[0], key[1], key[2], key[3], flows[key]))
    return h.hexdigest()


def test_cfg4_full_size_verdicts_and_flow_table_match_the_oracle_digest():
    """All 2^22 verdicts of configuration 4 and the flow table the batch leaves
    behind, byte for byte against what the sequential CPU oracle computed
    (tests/golden/filter_relay_digests.json, written by
    tests/golden/make_filter_relay_digests.py)."""
    import torch
    from bnk_amd import lib
    g = _fr_golden()["cfg4"]
    n = g["packets"]
    w = W.acl_workload(n=n)
    buf = np.ascontiguousarray(w.check).reshape(-1)
    assert hashlib.sha256(buf.data).hexdigest() == g["sha256_headers"], "the generators disagree"
    with lib.Context(0) as ctx:
        ctx.filter_set_rules(w.rules_ref)
        for now, rec in w.note_batches:
            r = np.ascontiguousarray(rec).reshape(-1)
            ctx.filter_note_outbound(lib.make_batch(r, r.nbytes, rec.shape[0], lib.MEM_HOST, stride=32, length=28),
                                     now)
        before = ctx.filter_flows()
        assert len(before) == g["flows_before"] and _flows_digest(before) == g["sha256_flows_before"]
        dev = torch.device("cuda:0")
        d_rec = torch.from_numpy(w.check).to(dev)
        d_v = torch.full((n,), 7, dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()
        ctx.filter_check_inbound(lib.make_batch(d_rec, n * 32, n, lib.MEM_DEVICE, stride=32, length=28), w.now_ns, d_v)
        ctx.sync()
        v = d_v.cpu().numpy()
        assert int(v.sum()) == g["allowed"]
        assert _sha(v) == g["sha256_verdicts"]
        after = ctx.filter_flows()
        assert len(after) == g["flows_after"] and _flows_digest(after) == g["sha256_flows_after"]


def test_cfg5_full_size_verdicts_counters_and_resealed_bytes_match_the_oracle_digest():
    """Configuration 5 at full size: every verdict, every outbound counter and
    every byte of every re-sealed packet against the sequential CPU oracle's
    digests; the slots of dropped packets keep what they held."""
    import torch
    from bnk_amd import lib
    g = _fr_golden()["cfg5"]
    n = g["packets"]
    w = W.relay_workload(n=n, payload=False, align=128)
    b = w.batch
    dev = torch.device("cuda:0")
    keys_in, keys_out = np.ascontiguousarray(b.keys), np.ascontiguousarray(w.keys_out)
    plain = W.relay_plain_torch(w, dev)
    total = plain.numel()
    assert total == g["arena_bytes"]
    assert _concat_sha(plain.cpu().numpy(), b.off, b.lens, 0) == g["sha256_plain"], "the generators disagree"
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    d_off, d_peer, d_ctr = d(b.off.astype(np.int64)), d(b.peer.astype(np.int32)), d(b.counters.astype(np.int64))
    d_lens, d_ctlens = d(b.lens.astype(np.int32)), d((b.lens + 16).astype(np.int32))
    d_peer_out, d_base = d(w.peer_out.astype(np.int32)), d(w.ctr_base_out.astype(np.int64))
    sealed = torch.zeros(total, dtype=torch.uint8, device=dev)
    out = torch.full((total,), 0x77, dtype=torch.uint8, device=dev)
    verdict = torch.full((n,), 9, dtype=torch.uint8, device=dev)
    ctr_out = torch.zeros(n, dtype=torch.int64, device=dev)
    torch.cuda.synchronize()
    with lib.Context(0) as ctx:
        ctx.filter_set_rules(w.rules_ref)
        now, rec = w.note_batch
        r = np.ascontiguousarray(rec).reshape(-1)
        ctx.filter_note_outbound(lib.make_batch(r, r.nbytes, rec.shape[0], lib.MEM_HOST, stride=32, length=28), now)
        # the inbound traffic: sealed under the inbound keys, 0.5 % of the tags forged
        ctx.keys_set(lib.KEYS_SEND, keys_in)
        ctx.seal(lib.make_batch(plain, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens, peer=d_peer,
                                counters=d_ctr),
                 lib.make_batch(sealed, total, n, lib.MEM_DEVICE, offsets=d_off))
        ctx.sync()
        which, pos, mask = W.relay_forged_bits(w)
        sealed[d(pos)] ^= d(mask)
        torch.cuda.synchronize()
        assert _concat_sha(sealed.cpu().numpy(), b.off, b.lens, 16) == g["sha256_sealed_in"]
        ctx.keys_set(lib.KEYS_RECV, keys_in)
        ctx.keys_set(lib.KEYS_SEND, keys_out)
        ctx.relay_fused(lib.make_batch(sealed, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_ctlens,
                                       peer=d_peer, counters=d_ctr),
                        d_peer_out, d_base, len(w.ctr_base_out), w.now_ns,
                        lib.make_batch(out, total, n, lib.MEM_DEVICE, offsets=d_off), verdict, ctr_out)
        ctx.sync()
        v = verdict.cpu().numpy()
        c = ctr_out.cpu().numpy().astype("<u8")
        assert [int(x) for x in np.bincount(v, minlength=3)] == g["verdict_counts"]
        h = hashlib.sha256()
        h.update(np.ascontiguousarray(v).data)
        h.update(np.ascontiguousarray(c).data)
        assert h.hexdigest() == g["sha256_verdicts_and_counters"]
        o_host = out.cpu().numpy()
        ok = v == 0
        hr = hashlib.sha256()
        mv = memoryview(o_host)
        untouched = True
        for i, (o, L) in enumerate(zip(b.off.tolist(), b.lens.tolist())):
            if ok[i]:
                hr.update(mv[o:o + L + 16])
            elif untouched and i % 7 == 0:
                untouched = bool((o_host[o:o + L + 16] == 0x77).all())
        assert hr.hexdigest() == g["sha256_resealed"]
        assert untouched, "a dropped packet's slot in the output arena was written"
        for i, want in g["sha256_of_resealed_packet"].items():
            o, L = int(b.off[int(i)]), int(b.lens[int(i)])
            assert _sha(o_host[o:o + L + 16]) == want
        after = ctx.filter_flows()
        assert len(after) == g["flows_after"] and _flows_digest(after) == g["sha256_flows_after"]
