"""Pins oracle/filter.c with the reference's own filter/acl test cases
(tests/filter_cases.py) and with a brute-force Python model on random input."""
import numpy as np
import pytest

import filter_cases as FC
from bnk_amd import workloads as W
from oracle import binding as O


@pytest.mark.parametrize("case", FC.FILTER_CASES, ids=lambda c: c.__name__)
def test_reference_filter_cases(case):
    case(O.Filter)


@pytest.mark.parametrize("case", FC.MATCH_CASES, ids=lambda c: c.__name__)
def test_reference_match_cases(case):
    case(O.rule_match)


def test_wrap_tun_write_semantics():
    # tun_test.go:43-66: batch of (allowed, denied) -> verdicts (1, 0) with one
    # `now`; the wrapper reports both written and forwards only the first.
    f = FC.ssh_only(O.Filter)
    a, d = W.tcp(FC.PEER, FC.SELF, 5555, 22), W.tcp(FC.PEER, FC.SELF, 5555, 23)
    buf = np.frombuffer(a + d, np.uint8).copy()
    off = np.array([0, len(a)], np.uint64)
    lens = np.array([len(a), len(d)], np.uint32)
    assert f.check_inbound_batch(buf, off, lens, FC.T0).tolist() == [1, 0]


def test_sweep_threshold_is_4096_and_strict():
    # filter.go:202-208: only when len(flows) > 4096, only entries with
    # now.After(exp)
    f = O.Filter()
    f.set_rules([])
    for i in range(4096):
        f.note_outbound(W.udp(FC.SELF, FC.PEER, 1000 + (i % 60000), 1 + i // 60000), FC.T0)
    assert f.flow_count() == 4096
    # far in the future but still only 4096 entries after the overwrite: no sweep
    f.note_outbound(W.udp(FC.SELF, FC.PEER, 1000, 1), FC.T0 + 3600 * FC.SEC)
    assert f.flow_count() == 4096
    # entry 4097 at exactly exp of the old ones: After is strict, nothing goes
    f.note_outbound(W.udp(FC.SELF, FC.PEER, 9, 9), FC.T0 + 30 * FC.SEC)
    assert f.flow_count() == 4097
    f.note_outbound(W.udp(FC.SELF, FC.PEER, 9, 9), FC.T0 + 30 * FC.SEC + 1)
    assert f.flow_count() == 2  # the refreshed first entry and (9, 9)


def _py_model(rules, flows, pkt, now):
    """Brute-force restatement in Python over dict/tuples."""
    if len(pkt) < 20 or pkt[0] >> 4 != 4:
        return False
    ihl = (pkt[0] & 15) * 4
    if ihl < 20 or len(pkt) < ihl:
        return False
    proto = pkt[9]
    src = int.from_bytes(pkt[12:16], "big")
    body = pkt[ihl:]
    sp = dp = 0
    if proto in (6, 17):
        if len(body) < 4:
            return False
        sp, dp = int.from_bytes(body[0:2], "big"), int.from_bytes(body[2:4], "big")
    elif proto == 1:
        if len(body) < 1:
            return False
    else:
        return False
    name = {6: "tcp", 17: "udp", 1: "icmp"}[proto]
    for srcs, rp, ports in rules:
        if rp != name:
            continue
        if not any(b == 0 or (src ^ a) >> (32 - b) == 0 for a, b in srcs):
            continue
        if name == "icmp" or any(lo <= dp <= hi for lo, hi in ports):
            return True
    k = (src, sp, dp, proto)
    if k in flows:
        if now < flows[k]:
            flows[k] = now + {6: 120, 17: 30, 1: 30}[proto] * FC.SEC
            return True
        del flows[k]
    return False


def test_random_rules_and_packets_vs_python_model():
    rng = np.random.default_rng(7)
    base = W.ip("100.64.0.0")
    for trial in range(20):
        rules = []
        for _ in range(int(rng.integers(0, 12))):
            srcs = [(base | int(rng.integers(0, 1 << 12)), int(rng.integers(20, 33)))
                    for _ in range(int(rng.integers(1, 3)))]
            proto = ["tcp", "udp", "icmp"][int(rng.integers(0, 3))]
            ports = []
            if proto != "icmp":
                for _ in range(int(rng.integers(0, 3))):
                    lo = int(rng.integers(0, 64)); ports.append((lo, lo + int(rng.integers(0, 8))))
            rules.append((srcs, proto, ports))
        f = O.Filter()
        f.set_rules(rules)
        flows = {}
        now = FC.T0
        for step in range(300):
            now += int(rng.integers(0, 20)) * FC.SEC
            a = base | int(rng.integers(0, 1 << 12))
            b = base | int(rng.integers(0, 1 << 12))
            sp, dp = int(rng.integers(0, 70)), int(rng.integers(0, 70))
            kind = int(rng.integers(0, 3))
            pkt = [W.tcp(a, b, sp, dp), W.udp(a, b, sp, dp), W.icmp_echo(a, b)][kind]
            if rng.random() < 0.3:
                f.note_outbound(pkt, now)
                proto = pkt[9]
                key = (b, dp, sp, proto) if proto != 1 else (b, 0, 0, 1)
                flows[key] = now + {6: 120, 17: 30, 1: 30}[proto] * FC.SEC
            else:
                assert f.check_inbound(pkt, now) == _py_model(rules, flows, pkt, now)
        assert f.flows() == flows
