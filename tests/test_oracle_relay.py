"""Pins oracle/relay.c (the CPU definition of open -> filter -> re-seal, which
has no counterpart in the reference) on the CPU, without any part of it in the
expectation: verdicts from how the workload was constructed, outbound counters
from the workload's own per-peer sequence, output packets from single-packet
seals.  The GPU relay tests compare with this oracle afterwards."""
import numpy as np

from bnk_amd import workloads as W
from oracle import binding as O

RELAY_OK, RELAY_FORGED, RELAY_DENIED = 0, 1, 2


def _relay(n, n_peers, forged_fraction):
    w = W.relay_workload(n=n, n_peers=n_peers, n_rules=256, forged_fraction=forged_fraction)
    b = w.batch
    keys_in, keys_out = np.ascontiguousarray(b.keys), np.ascontiguousarray(w.keys_out)
    sealed = np.zeros_like(b.plain)
    O.seal_batch(keys_in, b.peer, b.counters, b.plain, b.off, b.lens, sealed, b.off, 4)
    forged = W.forge_tags(5, sealed, b.off, b.lens, forged_fraction)
    ct_lens = (b.lens + 16).astype(np.uint32)
    f = O.Filter()
    f.set_rules(w.rules_ref)
    now, rec = w.note_batch
    m = rec.shape[0]
    f.note_outbound_batch(np.ascontiguousarray(rec).reshape(-1), np.arange(m, dtype=np.uint64) * 32,
                          np.full(m, 28, np.uint32), now)
    out = np.full_like(sealed, 0x77)
    v, c = f.relay_fused_batch(keys_in, b.peer, b.counters, keys_out, w.peer_out, w.ctr_base_out,
                               sealed, b.off, ct_lens, out, b.off, w.now_ns)
    return w, forged, v, c, out


def test_relay_oracle_against_the_workload_construction():
    n, n_peers = 6000, 48
    w, forged, v, c, out = _relay(n, n_peers, 0.01)
    b = w.batch
    # verdicts: forged tags first, then the packets built to be denied; the
    # packets admitted only by a noted flow pass like the rule-matched ones
    want_v = np.where(forged, RELAY_FORGED, np.where(w.denied, RELAY_DENIED, RELAY_OK)).astype(np.uint8)
    assert int(forged.sum()) == int(0.01 * n) and 0 < int(w.denied.sum()) and 0 < int(w.flow_allowed.sum())
    assert np.array_equal(v, want_v)
    # counters: base of the outbound peer + how many earlier survivors share it
    ok = want_v == RELAY_OK
    seq = np.zeros(n, np.uint64)
    seq[ok] = W.per_peer_sequence(w.peer_out[ok], n_peers)
    want_c = np.where(ok, w.ctr_base_out[w.peer_out] + seq, 0).astype(np.uint64)
    assert np.array_equal(c, want_c)
    # a dropped packet uses no counter: every peer's counters are consecutive
    for p in range(n_peers):
        mine = np.sort(c[ok & (w.peer_out == p)])
        assert np.array_equal(mine, w.ctr_base_out[p] + np.arange(mine.shape[0], dtype=np.uint64))
    # output: survivors re-sealed under the outbound key, everything else untouched
    want_out = np.full_like(out, 0x77)
    for i in np.flatnonzero(ok):
        o, L = int(b.off[i]), int(b.lens[i])
        ct = O.aead_seal(w.keys_out[w.peer_out[i]].tobytes(), O.wg_nonce(int(want_c[i])),
                         b.plain[o:o + L].tobytes())
        want_out[o:o + L + 16] = np.frombuffer(ct, np.uint8)
    assert np.array_equal(out, want_out)


def test_relay_oracle_short_and_empty_inputs():
    f = O.Filter()  # allow-all: every authentic packet is relayed
    key = np.arange(32, dtype=np.uint8).reshape(1, 32)
    sealed = np.zeros(64, np.uint8)
    ka = O.aead_seal(key.tobytes(), O.wg_nonce(5), b"")          # a keepalive: 16 bytes, empty plaintext
    sealed[:16] = np.frombuffer(ka, np.uint8)
    off = np.array([0, 32], np.uint64)
    lens = np.array([16, 9], np.uint32)                           # the second is shorter than a tag
    out = np.full(64, 0x77, np.uint8)
    v, c = f.relay_fused_batch(key, np.zeros(2, np.uint32), np.array([5, 6], np.uint64), key,
                               np.zeros(2, np.uint32), np.array([100], np.uint64), sealed, off, lens,
                               out, off, 0)
    assert v.tolist() == [RELAY_OK, RELAY_FORGED] and c.tolist() == [100, 0]
    assert out[:16].tobytes() == O.aead_seal(key.tobytes(), O.wg_nonce(100), b"")
    assert (out[16:] == 0x77).all()
