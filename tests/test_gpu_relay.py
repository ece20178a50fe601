"""Fused relay open -> filter -> re-seal on the GPU against the CPU
definition (oracle/relay.c): identical verdicts, outbound counters and output
ciphertexts."""
import numpy as np
import pytest

from bnk_amd import workloads as W

pytestmark = pytest.mark.gpu


def _note(ctx, ora, w):
    from bnk_amd import lib
    now, rec = w.note_batch
    m = rec.shape[0]
    buf = np.ascontiguousarray(rec).reshape(-1)
    if ora is not None:
        ora.note_outbound_batch(buf, np.arange(m, dtype=np.uint64) * 32, np.full(m, 28, np.uint32), now)
    ctx.filter_note_outbound(lib.make_batch(buf, buf.nbytes, m, lib.MEM_HOST, stride=32, length=28), now)


@pytest.mark.parametrize("mem", ["host", "ring"])
@pytest.mark.parametrize("n,n_peers", [(12000, 64), (900, 64), (40000, 64), (12000, 5000), (40000, 5000),
                                       (150000, 700)])
def test_relay_matches_oracle_host_path(mem, n, n_peers):
    """"ring": both arenas lie in pinned rings of the context, which batches of
    a few megabytes relay in place without staging copies.  900 packets also
    take the wave-per-packet kernels and the one-launch counter assignment;
    40000 (14 MB) go through in overlapped chunks, each continuing the
    counters of the one before; 150000 (52 MB) in chunks large enough for the
    lane-per-packet launches, the header records and the counting kernels,
    chunk by chunk.  With 64 or 700 peers the outbound counters come from the
    per-tile counting kernels, with 5000 (beyond what those hold in LDS) from
    the sort."""
    from bnk_amd import lib
    from oracle import binding as O
    w = W.relay_workload(n=n, n_peers=n_peers, n_rules=512)
    b = w.batch
    keys_in = np.ascontiguousarray(b.keys)
    keys_out = np.ascontiguousarray(w.keys_out)
    sealed = np.zeros_like(b.plain)
    O.seal_batch(keys_in, b.peer, b.counters, b.plain, b.off, b.lens, sealed, b.off, 4)
    forged = W.forge_tags(5, sealed, b.off, b.lens, w.forged_fraction)
    # a truncated packet is FORGED too
    ct_lens = (b.lens + 16).astype(np.uint32)
    ct_lens[7] = 9
    ora = O.Filter()
    ora.set_rules(w.rules_ref)
    ctx = lib.Context(0)
    ctx.filter_set_rules(w.rules_ref)
    ctx.keys_set(lib.KEYS_RECV, keys_in)
    ctx.keys_set(lib.KEYS_SEND, keys_out)
    _note(ctx, ora, w)
    want_out = np.full_like(b.plain, 0x77)
    want_v, want_c = ora.relay_fused_batch(keys_in, b.peer, b.counters, keys_out, w.peer_out,
                                           w.ctr_base_out, sealed, b.off, ct_lens, want_out, b.off,
                                           w.now_ns)
    rings = []
    if mem == "ring":
        rings = [ctx.ring_alloc(sealed.nbytes + 32), ctx.ring_alloc(sealed.nbytes)]
        rings[0][32:] = sealed
        sealed = rings[0][32:]
        got_out = rings[1]
        got_out[:] = 0x77
    else:
        got_out = np.full_like(b.plain, 0x77)
    got_v = np.full(b.n, 9, np.uint8)
    got_c = np.full(b.n, 123, np.uint64)
    ctx.relay_fused(
        lib.make_batch(sealed, sealed.nbytes, b.n, lib.MEM_HOST, offsets=b.off, lens=ct_lens,
                       peer=b.peer, counters=b.counters),
        w.peer_out, w.ctr_base_out, len(w.ctr_base_out), w.now_ns,
        lib.make_batch(got_out, got_out.nbytes, b.n, lib.MEM_HOST, offsets=b.off), got_v, got_c)
    assert np.array_equal(got_v, want_v)
    assert np.array_equal(got_c, want_c)
    assert np.array_equal(got_out, want_out)  # dropped packets' slots keep their 0x77 fill
    expect = np.where(forged, 1, np.where(w.denied, 2, 0))
    expect[7] = 1
    assert np.array_equal(got_v, expect)
    assert ctx.filter_flows() == ora.flows()
    # in allow-all mode nothing is DENIED
    ctx.filter_set_allow_all()
    ctx.relay_fused(
        lib.make_batch(sealed, sealed.nbytes, b.n, lib.MEM_HOST, offsets=b.off, lens=ct_lens,
                       peer=b.peer, counters=b.counters),
        w.peer_out, w.ctr_base_out, len(w.ctr_base_out), w.now_ns,
        lib.make_batch(got_out, got_out.nbytes, b.n, lib.MEM_HOST, offsets=b.off), got_v, got_c)
    assert np.array_equal(got_v == 1, expect == 1) and not (got_v == 2).any()
    for r in rings:
        ctx.ring_free(r)
    ctx.close()


@pytest.mark.parametrize("n", [12000, 900])
def test_relay_ip_options_and_ragged_headers(n):
    """The filter inside the relay reads each plaintext's first bytes from a
    compact record the open leaves behind (lane-per-packet launches), and goes
    back to the packet itself only for an IP header with options.  Packets
    with options (ports 4 to 40 bytes further in), packets cut short anywhere
    inside their headers, and non-IP payloads: verdicts, counters and output
    equal the oracle's."""
    from bnk_amd import lib
    from oracle import binding as O
    w = W.relay_workload(n=n, n_peers=16, n_rules=128, forged_fraction=0.01)
    b = w.batch
    rng = np.random.default_rng(n)
    plain = b.plain.copy()
    lens = b.lens.copy()
    off = b.off.astype(np.int64)
    kind = rng.integers(0, 10, n)
    for i in np.flatnonzero(kind == 0):                # options: ihl 6..15, ports moved
        if lens[i] < 576:
            continue
        words = int(rng.integers(6, 16))
        o = off[i]
        l4 = plain[o + 20:o + 28].copy()
        plain[o] = 0x40 | words
        plain[o + 20:o + 4 * words] = rng.integers(0, 256, 4 * words - 20, dtype=np.uint8)
        plain[o + 4 * words:o + 4 * words + 8] = l4
    short = np.flatnonzero(kind == 1)                  # cut inside the headers (or to nothing)
    lens[short] = rng.integers(0, 40, short.shape[0]).astype(lens.dtype)
    for i in np.flatnonzero(kind == 2):                # not IPv4
        plain[off[i]] = rng.integers(0, 256, dtype=np.uint8) | 0x20 if rng.integers(0, 2) else 0x60
    keys_in = np.ascontiguousarray(b.keys)
    keys_out = np.ascontiguousarray(w.keys_out)
    sealed = np.zeros_like(plain)
    O.seal_batch(keys_in, b.peer, b.counters, plain, b.off, lens, sealed, b.off, 4)
    W.forge_tags(5, sealed, b.off, lens, w.forged_fraction)
    ct_lens = (lens + 16).astype(np.uint32)
    ora = O.Filter()
    ora.set_rules(w.rules_ref)
    ctx = lib.Context(0)
    ctx.filter_set_rules(w.rules_ref)
    ctx.keys_set(lib.KEYS_RECV, keys_in)
    ctx.keys_set(lib.KEYS_SEND, keys_out)
    _note(ctx, ora, w)
    want_out = np.full_like(plain, 0x77)
    want_v, want_c = ora.relay_fused_batch(keys_in, b.peer, b.counters, keys_out, w.peer_out,
                                           w.ctr_base_out, sealed, b.off, ct_lens, want_out, b.off,
                                           w.now_ns)
    got_out = np.full_like(plain, 0x77)
    got_v = np.full(b.n, 9, np.uint8)
    got_c = np.full(b.n, 123, np.uint64)
    ctx.relay_fused(
        lib.make_batch(sealed, sealed.nbytes, b.n, lib.MEM_HOST, offsets=b.off, lens=ct_lens,
                       peer=b.peer, counters=b.counters),
        w.peer_out, w.ctr_base_out, len(w.ctr_base_out), w.now_ns,
        lib.make_batch(got_out, got_out.nbytes, b.n, lib.MEM_HOST, offsets=b.off), got_v, got_c)
    assert np.array_equal(got_v, want_v)
    assert np.array_equal(got_c, want_c)
    assert np.array_equal(got_out, want_out)
    # the options case is really in there, on both sides of the verdict
    opt = (kind == 0) & (lens >= 576)
    assert (want_v[opt] == 0).any() and opt.sum() > n // 50
    ctx.close()


def test_relay_full_size_device_resident_properties():
    """Configuration 5 at full size (2^22 IMIX packets, 4096 peers, 4096
    rules): verdicts equal the construction, counters equal base + per-peer
    rank among survivors in batch order, every re-sealed packet opens under the
    outbound key to the original plaintext, and a sample is bit-exact against
    the oracle."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    n = 1 << 22
    # slots at 128-byte alignment, the layout bench.py times (the smaller cases above
    # pack them at 16, where packets share lines)
    w = W.relay_workload(n=n, payload=False, align=128)
    b = w.batch
    dev = torch.device("cuda:0")
    keys_in = np.ascontiguousarray(b.keys)
    keys_out = np.ascontiguousarray(w.keys_out)
    plain = W.relay_plain_torch(w, dev)
    total = plain.numel()
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)  # noqa: E731
    d_off, d_peer, d_ctr = d(b.off.astype(np.int64)), d(b.peer.astype(np.int32)), d(b.counters.astype(np.int64))
    d_lens, d_ctlens = d(b.lens.astype(np.int32)), d((b.lens + 16).astype(np.int32))
    d_peer_out, d_base = d(w.peer_out.astype(np.int32)), d(w.ctr_base_out.astype(np.int64))
    sealed = torch.zeros(total, dtype=torch.uint8, device=dev)
    out = torch.full((total,), 0x77, dtype=torch.uint8, device=dev)
    verdict = torch.zeros(n, dtype=torch.uint8, device=dev)
    ctr_out = torch.zeros(n, dtype=torch.int64, device=dev)
    torch.cuda.synchronize()
    ctx = lib.Context(0)
    ctx.filter_set_rules(w.rules_ref)
    _note(ctx, None, w)
    # inbound traffic: sealed under the inbound keys, then 0.5 % of tags forged
    ctx.keys_set(lib.KEYS_SEND, keys_in)
    ctx.seal(lib.make_batch(plain, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_lens, peer=d_peer,
                            counters=d_ctr),
             lib.make_batch(sealed, total, n, lib.MEM_DEVICE, offsets=d_off))
    ctx.sync()
    which, pos, mask = W.relay_forged_bits(w)
    k = which.shape[0]
    sealed[d(pos)] ^= d(mask)
    forged = np.zeros(n, bool)
    forged[which] = True
    torch.cuda.synchronize()
    ctx.keys_set(lib.KEYS_RECV, keys_in)
    ctx.keys_set(lib.KEYS_SEND, keys_out)
    ctx.relay_fused(lib.make_batch(sealed, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_ctlens,
                                   peer=d_peer, counters=d_ctr),
                    d_peer_out, d_base, len(w.ctr_base_out), w.now_ns,
                    lib.make_batch(out, total, n, lib.MEM_DEVICE, offsets=d_off), verdict, ctr_out)
    ctx.sync()
    v = verdict.cpu().numpy()
    c = ctr_out.cpu().numpy().astype(np.uint64)
    expect = np.where(forged, 1, np.where(w.denied, 2, 0))
    assert np.array_equal(v, expect)
    assert abs((v == 2).mean() - 0.05) < 0.002 and (v == 1).sum() == k
    # the verdicts are counted for bnk_counters_get by a launch behind the relay's own
    got = ctx.counters()
    assert (got["relayed"], got["rejected"], got["denied"]) == (int((v == 0).sum()), k, int((v == 2).sum()))
    # counters: base + rank among the same peer's survivors, batch order
    ok = v == 0
    surv = np.flatnonzero(ok)
    want_c = np.zeros(n, np.uint64)
    want_c[surv] = w.ctr_base_out[w.peer_out[surv]] + W.per_peer_sequence(w.peer_out[surv],
                                                                        len(w.ctr_base_out))
    assert np.array_equal(c, want_c)
    # every survivor opens under the outbound key/counter to the original plaintext
    ctx.keys_set(lib.KEYS_RECV, keys_out)
    back = torch.zeros(total, dtype=torch.uint8, device=dev)
    v2 = torch.zeros(n, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()  # torch's fills run on its own stream
    ctx.open(lib.make_batch(out, total, n, lib.MEM_DEVICE, offsets=d_off, lens=d_ctlens,
                            peer=d_peer_out, counters=ctr_out),
             lib.make_batch(back, total, n, lib.MEM_DEVICE, offsets=d_off), v2)
    ctx.sync()
    assert np.array_equal(v2.cpu().numpy().astype(bool), ok)
    # compare plaintext bytes of survivors; dropped slots of `out` kept the fill
    o_host, p_host, b_host = out.cpu().numpy(), plain.cpu().numpy(), back.cpu().numpy()
    for i in np.concatenate([surv[:300], surv[-300:]]):
        o, L = int(b.off[i]), int(b.lens[i])
        assert np.array_equal(b_host[o:o + L], p_host[o:o + L])
        want = O.aead_seal(keys_out[w.peer_out[i]].tobytes(), O.wg_nonce(int(c[i])),
                           p_host[o:o + L].tobytes())
        assert o_host[o:o + L + 16].tobytes() == want
    for i in np.flatnonzero(~ok)[:300]:
        o, L = int(b.off[i]), int(b.lens[i])
        assert (o_host[o:o + L + 16] == 0x77).all()
    ctx.close()
