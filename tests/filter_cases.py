"""The reference's own filter and ACL test cases, restated once so the CPU
oracle and the HIP library are held to the same expectations.

Sources: internal/filter/filter_test.go:56-170, internal/filter/tun_test.go:43-94,
internal/acl/acl_test.go:83-114.  ``new_filter`` is a zero-argument factory
returning an object with the reference's method set: set_rules, set_allow_all,
check_inbound(pkt, now_ns), note_outbound(pkt, now_ns).
Rules are (srcs, proto, ports) with srcs = [(addr_u32, bits)], ports =
[(first, last)].
"""
from bnk_amd import workloads as W

SEC = 1_000_000_000
MIN = 60 * SEC
PEER = W.ip("100.64.0.9")
OTHER = W.ip("100.64.0.7")
SELF = W.ip("100.64.0.1")
T0 = W.T0_NS

SSH_ONLY = [([(PEER, 32)], "tcp", [(22, 22)])]


def ssh_only(new_filter):
    f = new_filter()
    f.set_rules(SSH_ONLY)
    return f


def case_allow_all_mode_passes_everything(new_filter):      # filter_test.go:73-78
    f = new_filter()
    assert f.check_inbound(W.tcp(PEER, SELF, 5555, 23), T0)


def case_rule_allows_matching_inbound(new_filter):          # :80-85
    f = ssh_only(new_filter)
    assert f.check_inbound(W.tcp(PEER, SELF, 5555, 22), T0)


def case_default_deny_drops_non_matching(new_filter):       # :87-98
    f = ssh_only(new_filter)
    assert not f.check_inbound(W.tcp(PEER, SELF, 5555, 23), T0)
    assert not f.check_inbound(W.tcp(OTHER, SELF, 5555, 22), T0)
    assert not f.check_inbound(W.udp(PEER, SELF, 53, 22), T0)


def case_return_traffic_allowed_via_flow_table(new_filter):  # :100-116
    f = ssh_only(new_filter)
    f.note_outbound(W.udp(SELF, PEER, 40000, 9999), T0)
    assert f.check_inbound(W.udp(PEER, SELF, 9999, 40000), T0 + 2 * SEC)
    assert not f.check_inbound(W.udp(PEER, SELF, 9999, 40000), T0 + 5 * MIN)
    assert not f.check_inbound(W.udp(PEER, SELF, 9998, 40000), T0 + SEC)


def case_tcp_return_flow_allowed(new_filter):               # :118-127
    f = ssh_only(new_filter)
    f.note_outbound(W.tcp(SELF, PEER, 40000, 8080, True), T0)
    assert f.check_inbound(W.tcp(PEER, SELF, 8080, 40000, False), T0 + SEC)
    assert not f.check_inbound(W.tcp(PEER, SELF, 8081, 40000, False), T0 + SEC)


def case_icmp_echo_reply_via_flow(new_filter):              # :129-138
    f = ssh_only(new_filter)
    f.note_outbound(W.icmp_echo(SELF, PEER, False), T0)
    assert f.check_inbound(W.icmp_echo(PEER, SELF, True), T0 + SEC)
    assert not f.check_inbound(W.icmp_echo(OTHER, SELF, True), T0 + SEC)


def case_icmp_rule_allows_inbound_ping(new_filter):         # :140-149
    f = new_filter()
    f.set_rules([([(PEER, 32)], "icmp", [])])
    assert f.check_inbound(W.icmp_echo(PEER, SELF, False), T0)


def case_malformed_and_non_ipv4_dropped(new_filter):        # :151-162
    f = ssh_only(new_filter)
    assert not f.check_inbound(bytes([0x60, 0x00, 0x00]), T0)
    assert not f.check_inbound(None, T0)
    assert not f.check_inbound(W.tcp(PEER, SELF, 1, 22)[:22], T0)


def case_set_allow_all_disables_enforcement(new_filter):    # :164-170
    f = ssh_only(new_filter)
    f.set_allow_all()
    assert f.check_inbound(W.tcp(OTHER, SELF, 5555, 23), T0)


def case_empty_rules_is_deny_all_but_flows(new_filter):     # tun_test.go:68-94
    f = new_filter()
    f.set_rules([])
    f.note_outbound(W.udp(SELF, PEER, 40000, 9999), T0)
    assert f.check_inbound(W.udp(PEER, SELF, 9999, 40000), T0)
    assert not f.check_inbound(W.udp(PEER, SELF, 9999, 40001), T0)


# ---- cases beyond the reference's tests: boundaries the source fixes ----

def case_expiry_boundary_is_strict(new_filter):
    # filter.go:140 now.Before(exp): now == exp denies and deletes
    f = ssh_only(new_filter)
    f.note_outbound(W.udp(SELF, PEER, 40000, 9999), T0)
    assert f.check_inbound(W.udp(PEER, SELF, 9999, 40000), T0 + 30 * SEC - 1)
    # that hit refreshed the flow to (T0+30s-1)+30s
    assert not f.check_inbound(W.udp(PEER, SELF, 9999, 40000), T0 + 60 * SEC - 1)
    # deleted now: even an earlier clock cannot revive it
    assert not f.check_inbound(W.udp(PEER, SELF, 9999, 40000), T0 + SEC)


def case_tcp_ttl_is_two_minutes(new_filter):                # filter.go:18-22
    f = ssh_only(new_filter)
    f.note_outbound(W.tcp(SELF, PEER, 40000, 8080), T0)
    assert f.check_inbound(W.tcp(PEER, SELF, 8080, 40000, False), T0 + 119 * SEC)
    f2 = ssh_only(new_filter)
    f2.note_outbound(W.tcp(SELF, PEER, 40000, 8080), T0)
    assert not f2.check_inbound(W.tcp(PEER, SELF, 8080, 40000, False), T0 + 120 * SEC)


def case_flows_survive_set_allow_all(new_filter):           # filter.go:54-59
    f = ssh_only(new_filter)
    f.note_outbound(W.udp(SELF, PEER, 40000, 9999), T0)
    f.set_allow_all()
    # not enforcing: NoteOutbound records nothing (filter.go:192-194)
    f.note_outbound(W.udp(SELF, PEER, 40001, 9999), T0)
    f.set_rules(SSH_ONLY)
    assert f.check_inbound(W.udp(PEER, SELF, 9999, 40000), T0 + SEC)
    assert not f.check_inbound(W.udp(PEER, SELF, 9999, 40001), T0 + SEC)


def case_parse_edges(new_filter):                           # filter.go:71-106
    f = new_filter()
    f.set_rules([([(0, 0)], "tcp", [(0, 65535)]), ([(0, 0)], "udp", [(0, 65535)]),
                 ([(0, 0)], "icmp", [])])
    good = bytearray(W.tcp(PEER, SELF, 1, 2))
    assert f.check_inbound(bytes(good), T0)
    assert f.check_inbound(bytes(good[:24]), T0)      # 4 body bytes suffice
    assert not f.check_inbound(bytes(good[:23]), T0)  # 3 do not
    assert not f.check_inbound(bytes(good[:19]), T0)  # shorter than a header
    v = bytearray(good); v[0] = 0x55
    assert not f.check_inbound(bytes(v), T0)          # version 5
    v = bytearray(good); v[0] = 0x44
    assert not f.check_inbound(bytes(v), T0)          # ihl 16 < 20
    # ihl 24 with options: ports are read after the options
    opt = bytearray(good[:20]) + b"\x01\x01\x01\x01" + good[20:]
    opt[0] = 0x46
    assert f.check_inbound(bytes(opt), T0)
    assert not f.check_inbound(bytes(opt[:27]), T0)
    v = bytearray(good); v[0] = 0x4F                  # ihl 60 > len 40
    assert not f.check_inbound(bytes(v), T0)
    v = bytearray(good); v[9] = 2                     # IGMP
    assert not f.check_inbound(bytes(v), T0)
    ic = W.icmp_echo(PEER, SELF)
    assert f.check_inbound(ic[:21], T0)               # one ICMP byte suffices
    assert not f.check_inbound(ic[:20], T0)
    # fragments, bad checksums, wrong total length are not looked at
    v = bytearray(good); v[6] = 0x20; v[7] = 0x10; v[2] = 0xFF; v[10] = 0xAB
    assert f.check_inbound(bytes(v), T0)


# ---- acl.Match (acl_test.go:83-114) ----

def case_compiled_rule_match(match):
    r = ([(W.ip("100.64.0.1"), 32)], "tcp", [(22, 22), (8000, 9000)])
    table = [("100.64.0.1", "tcp", 22, True), ("100.64.0.1", "tcp", 8500, True),
             ("100.64.0.1", "tcp", 23, False), ("100.64.0.1", "udp", 22, False),
             ("100.64.0.9", "tcp", 22, False)]
    for src, proto, port, want in table:
        assert match(r, W.ip(src), proto, port) is want, (src, proto, port)


def case_icmp_rule_ignores_ports(match):
    r = ([(W.ip("100.64.0.0"), 10)], "icmp", [])
    assert match(r, W.ip("100.64.0.1"), "icmp", 0)


def case_match_edges(match):
    ipx = W.ip("100.64.3.77")
    # tcp/udp rule with no ports never matches (acl.go:166-171)
    assert not match(([(ipx, 32)], "tcp", []), ipx, "tcp", 22)
    # unknown proto string never matches a parsed packet's name
    assert not match(([(ipx, 32)], "sctp", [(0, 65535)]), ipx, "tcp", 22)
    # host bits in an unmasked prefix are ignored by Contains
    assert match(([(W.ip("100.64.3.99"), 24)], "udp", [(53, 53)]), ipx, "udp", 53)
    assert not match(([(W.ip("100.64.4.99"), 24)], "udp", [(53, 53)]), ipx, "udp", 53)
    # /0 contains everything; the invalid prefix and IPv6 prefixes nothing
    assert match(([(0x01020304, 0)], "tcp", [(1, 1)]), ipx, "tcp", 1)
    assert not match(([(ipx, -1)], "tcp", [(1, 1)]), ipx, "tcp", 1)
    assert not match(([(ipx, 32, 0)], "tcp", [(1, 1)]), ipx, "tcp", 1)
    # port range ends are inclusive; second prefix / second range reachable
    r = ([(W.ip("10.0.0.0"), 8), (W.ip("100.64.0.0"), 10)], "tcp", [(10, 20), (30, 40)])
    for port, want in [(9, False), (10, True), (20, True), (21, False), (30, True),
                       (40, True), (41, False)]:
        assert match(r, ipx, "tcp", port) is want
    # icmp ignores ports even when the rule lists some
    assert match(([(ipx, 32)], "icmp", [(5, 5)]), ipx, "icmp", 0)


FILTER_CASES = [v for k, v in sorted(globals().items())
                if k.startswith("case_") and v.__code__.co_varnames[:1] == ("new_filter",)]
MATCH_CASES = [v for k, v in sorted(globals().items())
               if k.startswith("case_") and v.__code__.co_varnames[:1] == ("match",)]
