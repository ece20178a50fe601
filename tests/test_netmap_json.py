"""The netmap JSON rule loader (host code of libbnkhip.so, no GPU needed).
Shapes come from the reference: field names from internal/netmap/netmap.go:44-53
and internal/acl/acl.go:33-42, rule shapes from internal/coord/server/policy_test.go:10-41
and internal/acl/acl_test.go:16-74."""
import json

import pytest

from bnk_amd import lib
from bnk_amd import workloads as W


def _rule(srcs, proto, ports=None):
    r = {"srcs": srcs, "proto": proto}
    if ports is not None:
        r["ports"] = [{"first": a, "last": b} for a, b in ports]
    return r


def test_policy_push_shape_tcp22_to_nas():
    # policy_test.go:10-41: nas receives one rule, tcp/22 from laptop
    doc = json.dumps({"self_id": 2, "self_ip": "100.64.0.2/32", "peers": [],
                      "filter_enabled": True,
                      "filter": [_rule(["100.64.0.1/32"], "tcp", [(22, 22)])]})
    en, t = lib.rules_from_netmap_json(doc)
    assert en and t == [(W.ip("100.64.0.1"), 0xFFFFFFFF, 22, 22, 6)]
    # the laptop: enforcement on, no allowances (omitempty drops "filter")
    en, t = lib.rules_from_netmap_json(json.dumps({"self_id": 1, "filter_enabled": True}))
    assert en and t == []
    # no policy at all: allow-all
    en, t = lib.rules_from_netmap_json(json.dumps({"self_id": 1, "peers": [{"id": 3, "name": "x",
                                                  "endpoints": ["203.0.113.9:41641"]}]}))
    assert not en and t == []


def test_group_rule_expands_to_prefix_times_range_tuples():
    # acl_test.go:16-44: three allowances, two sources each; icmp has no ports
    srcs = ["100.64.0.1/32", "100.64.0.2/32"]
    doc = json.dumps([_rule(srcs, "tcp", [(22, 22)]), _rule(srcs, "tcp", [(443, 443)]),
                      _rule(srcs, "icmp"), _rule(["100.64.0.0/10"], "udp", [(6000, 6100), (53, 53)])])
    en, t = lib.rules_from_netmap_json(doc)
    assert en
    a, b = W.ip("100.64.0.1"), W.ip("100.64.0.2")
    assert t == [(a, 0xFFFFFFFF, 22, 22, 6), (b, 0xFFFFFFFF, 22, 22, 6),
                 (a, 0xFFFFFFFF, 443, 443, 6), (b, 0xFFFFFFFF, 443, 443, 6),
                 (a, 0xFFFFFFFF, 0, 0, 1), (b, 0xFFFFFFFF, 0, 0, 1),
                 (W.ip("100.64.0.0"), 0xFFC00000, 6000, 6100, 17),
                 (W.ip("100.64.0.0"), 0xFFC00000, 53, 53, 17)]


def test_semantics_of_odd_rules_match_acl_match():
    doc = json.dumps([
        _rule(["100.64.3.99/24"], "udp", [(53, 53)]),        # host bits ignored by Contains
        _rule(["fd7a:115c::/48", "::ffff:1.2.3.4/128"], "tcp", [(1, 1)]),  # IPv6 never contains IPv4
        _rule([""], "tcp", [(1, 1)]),                         # the zero prefix
        _rule(["1.2.3.4/32"], "tcp"),                         # tcp without ports never matches
        _rule(["1.2.3.4/32"], "sctp", [(1, 1)]),              # unknown protocol string
        _rule(["0.0.0.0/0"], "icmp", [(5, 5)]),               # icmp ignores ports
        {"Srcs": ["9.9.9.9/32"], "PROTO": "tcp", "Ports": [{"First": 7, "LAST": 8}]},  # Go matches case-insensitively
        {"srcs": None, "proto": "tcp", "ports": None},
    ])
    en, t = lib.rules_from_netmap_json(doc)
    assert t == [(W.ip("100.64.3.0"), 0xFFFFFF00, 53, 53, 17), (0, 0, 0, 0, 1),
                 (W.ip("9.9.9.9"), 0xFFFFFFFF, 7, 8, 6)]


@pytest.mark.parametrize("doc", [
    '{"filter_enabled":true,"filter":[{"srcs":["100.64.0.1"],"proto":"tcp"}]}',        # no /bits
    '{"filter_enabled":true,"filter":[{"srcs":["100.64.0.1/33"],"proto":"tcp"}]}',
    '{"filter_enabled":true,"filter":[{"srcs":["100.064.0.1/32"],"proto":"tcp"}]}',    # leading zero
    '{"filter_enabled":true,"filter":[{"srcs":["100.64.0/24"],"proto":"tcp"}]}',
    '{"filter_enabled":true,"filter":[{"srcs":["1.2.3.4/032"],"proto":"tcp"}]}',
    '{"filter":[{"proto":"tcp","ports":[{"first":70000,"last":1}]}]}',
    '{"filter":[{"proto":"tcp","ports":[{"first":-1,"last":1}]}]}',
    '{"filter":[{"proto":"tcp","ports":[{"first":1.5,"last":2}]}]}',
    '{"filter_enabled":"yes"}',
    '{"filter":[{"proto":"tcp"}',
    '{"filter":[]} trailing',
    '',
])
def test_documents_go_would_reject(doc):
    with pytest.raises(lib.BnkError) as ei:
        lib.rules_from_netmap_json(doc)
    assert ei.value.code == lib.E_INVAL


def test_large_rule_set_and_escapes():
    rules = [_rule(["100.%d.%d.0/24" % (64 + i // 256, i % 256)], "tcp", [(i, i + 1)]) for i in range(3000)]
    doc = json.dumps({"filter_enabled": True, "filter": rules, "note": 'a "quoted" \u00e9 string',
                      "nested": {"x": [1, 2.5e3, {"y": None}], "z": True}})
    en, t = lib.rules_from_netmap_json(doc)
    assert en and len(t) == 3000 and t[2999] == (W.ip("100.75.183.0"), 0xFFFFFF00, 2999, 3000, 6)
