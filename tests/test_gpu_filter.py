"""Parity of the HIP packet filter (through the C ABI) with the CPU oracle and
with the reference's own test cases: identical allow/deny verdicts and
identical flow-table contents."""
import numpy as np
import pytest

import filter_cases as FC
from bnk_amd import workloads as W

pytestmark = pytest.mark.gpu


def _new_filter():
    from bnk_amd import lib
    return lib.HostFilter(lib.Context(0))


@pytest.mark.parametrize("case", FC.FILTER_CASES, ids=lambda c: c.__name__)
def test_reference_filter_cases(case):
    case(_new_filter)


def _match(rule, src, proto, port):
    """acl.Match seen through the filter: one rule, empty flow table."""
    f = _new_filter()
    f.set_rules([rule])
    me = W.ip("100.64.0.1")
    pkt = {"tcp": W.tcp(src, me, 999, port), "udp": W.udp(src, me, 999, port),
           "icmp": W.icmp_echo(src, me)}[proto]
    return f.check_inbound(pkt, FC.T0)


@pytest.mark.parametrize("case", FC.MATCH_CASES, ids=lambda c: c.__name__)
def test_reference_match_cases(case):
    case(_match)


def _flat(rec):
    n = rec.shape[0]
    return (np.ascontiguousarray(rec).reshape(-1), np.arange(n, dtype=np.uint64) * 32,
            np.full(n, 28, np.uint32))


@pytest.mark.parametrize("n", [1 << 15, 70000])
def test_cfg4_small_verdicts_and_flow_table_match_oracle(n):
    """Host batches: up to 65,536 packets the kernel reads the gathered headers
    from pinned staging in place, above that they are uploaded first."""
    from bnk_amd import lib
    from oracle import binding as O
    w = W.acl_workload(n=n)
    ctx = lib.Context(0)
    ora = O.Filter()
    ctx.filter_set_rules(w.rules_ref)
    ora.set_rules(w.rules_ref)
    for now, rec in w.note_batches:
        buf, off, lens = _flat(rec)
        ora.note_outbound_batch(buf, off, lens, now)
        ctx.filter_note_outbound(
            lib.make_batch(buf, buf.nbytes, rec.shape[0], lib.MEM_HOST, stride=32, length=28), now)
        assert ctx.filter_flow_count() == ora.flow_count()
    assert ctx.filter_flows() == ora.flows()
    buf, off, lens = _flat(w.check)
    want = ora.check_inbound_batch(buf, off, lens, w.now_ns)
    got = np.full(w.check.shape[0], 9, np.uint8)
    ctx.filter_check_inbound(
        lib.make_batch(buf, buf.nbytes, w.check.shape[0], lib.MEM_HOST, stride=32, length=28),
        w.now_ns, got)
    assert np.array_equal(got, want)
    assert 0.05 < want.mean() < 0.95
    assert ctx.filter_flows() == ora.flows()
    # a second pass later in time: refreshed flows pass, the rest have expired
    later = w.now_ns + 31 * FC.SEC
    want2 = ora.check_inbound_batch(buf, off, lens, later)
    got2 = np.zeros_like(got)
    ctx.filter_check_inbound(
        lib.make_batch(buf, buf.nbytes, w.check.shape[0], lib.MEM_HOST, stride=32, length=28),
        later, got2)
    assert np.array_equal(got2, want2)
    assert ctx.filter_flows() == ora.flows()
    ctx.close()


def test_duplicates_in_one_batch_and_sweep_threshold():
    from bnk_amd import lib
    from oracle import binding as O
    ctx = lib.Context(0)
    ora = O.Filter()
    ctx.filter_set_rules([])
    ora.set_rules([])
    # 4096 distinct flows plus duplicates of the first hundred
    pk = [W.udp(FC.SELF, FC.PEER, 1000 + (i % 60000), 1 + i // 60000) for i in range(4096)]
    pk += pk[:100]
    for f in (ctx.filter_note_outbound_ptrs, lambda p, t: [ora.note_outbound(x, t) for x in p]):
        f(pk, FC.T0)
    assert ctx.filter_flow_count() == ora.flow_count() == 4096
    # no sweep at exactly 4096 even far in the future
    ctx.filter_note_outbound_ptrs(pk[:1], FC.T0 + 3600 * FC.SEC)
    ora.note_outbound(pk[0], FC.T0 + 3600 * FC.SEC)
    assert ctx.filter_flow_count() == ora.flow_count() == 4096
    # entry 4097 with now == exp of the old ones: After() is strict
    extra = W.udp(FC.SELF, FC.PEER, 9, 9)
    ctx.filter_note_outbound_ptrs([extra], FC.T0 + 30 * FC.SEC)
    ora.note_outbound(extra, FC.T0 + 30 * FC.SEC)
    assert ctx.filter_flow_count() == ora.flow_count() == 4097
    ctx.filter_note_outbound_ptrs([extra], FC.T0 + 30 * FC.SEC + 1)
    ora.note_outbound(extra, FC.T0 + 30 * FC.SEC + 1)
    assert ctx.filter_flow_count() == ora.flow_count() == 2
    assert ctx.filter_flows() == ora.flows()
    # replies: one batch holding the same reply many times plus misses
    replies = [W.udp(FC.PEER, FC.SELF, 9, 9)] * 70 + [W.udp(FC.PEER, FC.SELF, 9, 10)] * 5
    now = FC.T0 + 40 * FC.SEC
    got = ctx.filter_check_inbound_ptrs(replies, now)
    want = [ora.check_inbound(p, now) for p in replies]
    assert got.tolist() == [int(x) for x in want]
    # the same batch after expiry: all denied, entry deleted once
    now = FC.T0 + 3 * 3600 * FC.SEC
    got = ctx.filter_check_inbound_ptrs(replies, now)
    want = [ora.check_inbound(p, now) for p in replies]
    assert got.tolist() == [int(x) for x in want] == [0] * 75
    assert ctx.filter_flows() == ora.flows()
    assert ctx.filter_flow_count() == ora.flow_count() == 1
    ctx.close()


def test_rules_too_wide_to_expand_and_rule_edges():
    """Thousands of /0 rules over thousands of /32 cut points exceed the
    expansion budget: those rules are scanned linearly instead; verdicts must
    not change.  Also unmasked prefixes, /0, empty port lists, odd protocols."""
    from bnk_amd import lib
    from oracle import binding as O
    rng = np.random.default_rng(5)
    base = W.CGNAT_BASE
    rules = []
    for i in range(1500):
        rules.append(([(int(rng.integers(0, 1 << 32)), 0)], "tcp", [(2 * i, 2 * i)]))
    for i in range(3000):
        rules.append(([(base | int(rng.integers(0, 1 << 16)), 32)], "udp", [(53, 53)]))
    rules.append(([(base | 0x1234, 20), (W.ip("10.1.2.3"), 8)], "tcp", [(7000, 7010), (9000, 9000)]))
    rules.append(([(base, 10)], "icmp", [(1, 2)]))
    rules.append(([(base, 10)], "sctp", [(0, 65535)]))
    rules.append(([(base, 10)], "udp", []))
    rules.append(([(base, -1)], "tcp", [(0, 65535)]))
    rules.append(([(base, 32, 0)], "tcp", [(0, 65535)]))
    ctx = lib.Context(0)
    ora = O.Filter()
    ctx.filter_set_rules(rules)
    ora.set_rules(rules)
    n = 20000
    proto = W.proto_mix(1, n)
    src = (base | rng.integers(0, 1 << 16, n)).astype(np.uint32)
    src[:200] = rng.integers(0, 1 << 32, 200)
    dport = rng.integers(0, 3200, n).astype(np.uint32)
    dport[::7] = 53
    dport[::11] = 7005
    rec = W.header_records(proto, src, np.full(n, base | 1, np.uint32),
                           rng.integers(0, 65536, n).astype(np.uint32), dport)
    buf, off, lens = _flat(rec)
    want = ora.check_inbound_batch(buf, off, lens, FC.T0)
    got = np.zeros(n, np.uint8)
    ctx.filter_check_inbound(lib.make_batch(buf, buf.nbytes, n, lib.MEM_HOST, stride=32, length=28),
                             FC.T0, got)
    assert np.array_equal(got, want)
    assert 0.2 < want.mean() < 0.9
    ctx.close()


def test_ragged_and_malformed_batch():
    from bnk_amd import lib
    from oracle import binding as O
    rules = [([(0, 0)], "tcp", [(0, 65535)]), ([(0, 0)], "icmp", [])]
    good = W.tcp(FC.PEER, FC.SELF, 1, 2)
    opt = bytearray(good[:20]) + b"\x01" * 40 + good[20:]
    opt[0] = 0x4F
    pk = [good, good[:24], good[:23], good[:19], b"", bytes([0x60, 0, 0]), bytes(opt), bytes(opt[:63]),
          W.icmp_echo(FC.PEER, FC.SELF)[:21], W.icmp_echo(FC.PEER, FC.SELF)[:20],
          W.udp(FC.PEER, FC.SELF, 1, 2), good + bytes(1400)]
    ctx = lib.Context(0)
    ora = O.Filter()
    ctx.filter_set_rules(rules)
    ora.set_rules(rules)
    want = [int(ora.check_inbound(p, FC.T0)) for p in pk]
    assert want == [1, 1, 0, 0, 0, 0, 1, 0, 1, 0, 0, 1]
    assert ctx.filter_check_inbound_ptrs(pk, FC.T0).tolist() == want
    # the same packets as a ragged arena batch
    lens = np.array([len(p) for p in pk], np.uint32)
    off = np.zeros(len(pk), np.uint64)
    off[1:] = np.cumsum(lens[:-1] + 3)
    arena = np.zeros(int(off[-1] + lens[-1]), np.uint8)
    for o, p in zip(off, pk):
        arena[int(o):int(o) + len(p)] = np.frombuffer(p, np.uint8)
    got = np.zeros(len(pk), np.uint8)
    ctx.filter_check_inbound(lib.make_batch(arena, arena.nbytes, len(pk), lib.MEM_HOST, offsets=off,
                                            lens=lens), FC.T0, got)
    assert got.tolist() == want
    # allow-all mode passes even the malformed ones (filter.go:124-126)
    ctx.filter_set_allow_all()
    assert ctx.filter_check_inbound_ptrs(pk, FC.T0).tolist() == [1] * len(pk)
    ctx.close()


def test_cfg4_full_size_device_resident_properties():
    """2^22 headers, 4096 rules, 65,536 noted flows, device resident.  The
    oracle cannot scan this in seconds, so: (a) a seeded sample of packets is
    checked against the oracle -- valid because a packet's verdict within one
    batch equals its verdict against the table as it stood before the batch;
    (b) the verdicts of a permuted batch are the permuted verdicts; (c) the
    flow table matches the oracle's after the sample has been replayed."""
    import torch
    from bnk_amd import lib
    from oracle import binding as O
    w = W.acl_workload(n=1 << 22)
    n = w.check.shape[0]
    ctxs = [lib.Context(0), lib.Context(0)]
    ora = O.Filter()
    ora.set_rules(w.rules_ref)
    for c in ctxs:
        c.filter_set_rules(w.rules_ref)
    for now, rec in w.note_batches:
        buf, off, lens = _flat(rec)
        ora.note_outbound_batch(buf, off, lens, now)
        for c in ctxs:
            c.filter_note_outbound(
                lib.make_batch(buf, buf.nbytes, rec.shape[0], lib.MEM_HOST, stride=32, length=28), now)
    assert ctxs[0].filter_flows() == ora.flows()
    dev = torch.device("cuda:0")
    d_rec = torch.from_numpy(w.check).to(dev)
    d_v = torch.zeros(n, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    ctxs[0].filter_check_inbound(
        lib.make_batch(d_rec, n * 32, n, lib.MEM_DEVICE, stride=32, length=28), w.now_ns, d_v)
    ctxs[0].sync()
    v = d_v.cpu().numpy()
    # (a) sample parity
    pick = np.sort(W.permutation(99, n)[:1 << 14].astype(np.int64))
    buf, off, lens = _flat(w.check[pick])
    want = ora.check_inbound_batch(buf, off, lens, w.now_ns)
    assert np.array_equal(v[pick], want)
    # (b) permutation invariance on an identical second filter
    perm = W.permutation(98, n).astype(np.int64)
    d_rec2 = torch.from_numpy(np.ascontiguousarray(w.check[perm])).to(dev)
    d_v2 = torch.zeros(n, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    ctxs[1].filter_check_inbound(
        lib.make_batch(d_rec2, n * 32, n, lib.MEM_DEVICE, stride=32, length=28), w.now_ns, d_v2)
    ctxs[1].sync()
    assert np.array_equal(d_v2.cpu().numpy(), v[perm])
    assert ctxs[0].filter_flows() == ctxs[1].filter_flows()
    for c in ctxs:
        c.close()


def test_apply_netmap_json_end_to_end():
    """Engine.ApplyNetmap's filter half fed with the control server's wire
    format: the reference's integration test allows one port and blocks another
    (internal/dataplane/acl_integration_test.go:20-80)."""
    import json
    from bnk_amd import lib
    ctx = lib.Context(0)
    a, b = W.ip("100.64.0.1"), W.ip("100.64.0.2")
    doc = {"self_id": 2, "self_ip": "100.64.0.2/32", "peers": [], "filter_enabled": True,
           "filter": [{"srcs": ["100.64.0.1/32"], "proto": "tcp", "ports": [{"first": 7777, "last": 7777}]}]}
    ctx.filter_apply_netmap_json(json.dumps(doc))
    got = ctx.filter_check_inbound_ptrs([W.tcp(a, b, 40000, 7777), W.tcp(a, b, 40000, 8888),
                                         W.udp(a, b, 40000, 7777)], FC.T0)
    assert got.tolist() == [1, 0, 0]
    # a malformed push leaves the filter as it was
    with pytest.raises(lib.BnkError):
        ctx.filter_apply_netmap_json('{"filter_enabled":true,"filter":[{"srcs":["bogus"]}]}')
    assert ctx.filter_check_inbound_ptrs([W.tcp(a, b, 1, 7777)], FC.T0).tolist() == [1]
    # policy removed: allow-all again
    ctx.filter_apply_netmap_json(json.dumps({"self_id": 2, "peers": []}))
    assert ctx.filter_check_inbound_ptrs([W.tcp(a, b, 1, 8888)], FC.T0).tolist() == [1]
    ctx.close()
