// Reads the filter part of a netmap document, the wire format in which the
// control server pushes compiled rules to a client:
//
//   {"self_id":7, ..., "filter_enabled":true,
//    "filter":[{"srcs":["100.64.0.1/32"],"proto":"tcp","ports":[{"first":22,"last":22}]}]}
//
// Field names are the reference's JSON tags (internal/netmap/netmap.go:44-53,
// internal/acl/acl.go:33-42).  Everything else in the document is skipped.  A
// bare array of rules is accepted too.  Prefixes follow netip.Prefix's text
// form: "a.b.c.d/n" (no leading zeros), "" for the zero prefix, IPv6 prefixes
// are recognised and yield no tuples because they never contain an IPv4
// address.  Go's decoder matches field names case-insensitively; so does this.
#pragma once

#include <stdint.h>
#include <string.h>

#include <string>
#include <vector>

#include "../../include/bnkhip.h"

namespace bnk {

struct NetmapFilter {
    bool filter_enabled = false;
    std::vector<bnk_rule> tuples; // one per (prefix, port range) pair
    uint32_t n_rules = 0;         // CompiledRule objects seen
};

class NetmapJson {
public:
    NetmapJson(const char *p, size_t n) : p_(p), end_(p + n) {}

    bool parse(NetmapFilter &out, std::string &err)
    {
        out = NetmapFilter{};
        ws();
        bool ok;
        if (peek() == '[') {
            out.filter_enabled = true;
            ok = rules(out);
        } else {
            ok = document(out);
        }
        if (ok) {
            ws();
            if (p_ != end_) ok = fail("trailing data after the document");
        }
        if (!ok) err = err_;
        return ok;
    }

private:
    const char *p_, *end_;
    std::string err_;

    bool fail(const std::string &m)
    {
        if (err_.empty()) err_ = "netmap JSON: " + m;
        return false;
    }
    char peek() const { return p_ < end_ ? *p_ : '\0'; }
    void ws()
    {
        while (p_ < end_ && (*p_ == ' ' || *p_ == '\t' || *p_ == '\n' || *p_ == '\r')) p_++;
    }
    bool expect(char c)
    {
        ws();
        if (peek() != c) return fail(std::string("expected '") + c + "'");
        p_++;
        return true;
    }
    static bool ieq(const std::string &a, const char *b)
    {
        if (a.size() != strlen(b)) return false;
        for (size_t i = 0; i < a.size(); i++) {
            char x = a[i], y = b[i];
            if (x >= 'A' && x <= 'Z') x = (char)(x - 'A' + 'a');
            if (x != y) return false;
        }
        return true;
    }

    bool string(std::string &s)
    {
        ws();
        if (peek() != '"') return fail("expected a string");
        p_++;
        s.clear();
        while (p_ < end_ && *p_ != '"') {
            unsigned char c = (unsigned char)*p_++;
            if (c < 0x20) return fail("control character in string");
            if (c != '\\') {
                s.push_back((char)c);
                continue;
            }
            if (p_ >= end_) return fail("unterminated escape");
            const char e = *p_++;
            switch (e) {
            case '"': s.push_back('"'); break;
            case '\\': s.push_back('\\'); break;
            case '/': s.push_back('/'); break;
            case 'b': s.push_back('\b'); break;
            case 'f': s.push_back('\f'); break;
            case 'n': s.push_back('\n'); break;
            case 'r': s.push_back('\r'); break;
            case 't': s.push_back('\t'); break;
            case 'u': {
                if (end_ - p_ < 4) return fail("short \\u escape");
                unsigned v = 0;
                for (int i = 0; i < 4; i++) {
                    const char h = *p_++;
                    v <<= 4;
                    if (h >= '0' && h <= '9') v |= (unsigned)(h - '0');
                    else if (h >= 'a' && h <= 'f') v |= (unsigned)(h - 'a' + 10);
                    else if (h >= 'A' && h <= 'F') v |= (unsigned)(h - 'A' + 10);
                    else return fail("bad \\u escape");
                }
                // the fields read here are ASCII; anything else only needs to differ
                s.push_back(v < 0x80 ? (char)v : '?');
                break;
            }
            default: return fail("bad escape");
            }
        }
        if (p_ >= end_) return fail("unterminated string");
        p_++;
        return true;
    }

    // Integer in [0, max]; JSON numbers with fractions or exponents do not
    // decode into Go's uint16 either.
    bool uint_value(uint32_t max, uint32_t &v)
    {
        ws();
        if (peek() < '0' || peek() > '9') return fail("expected a non-negative integer");
        if (peek() == '0' && p_ + 1 < end_ && p_[1] >= '0' && p_[1] <= '9') return fail("leading zero in number");
        uint64_t x = 0;
        while (p_ < end_ && *p_ >= '0' && *p_ <= '9') {
            x = x * 10 + (uint64_t)(*p_++ - '0');
            if (x > max) return fail("number out of range");
        }
        if (peek() == '.' || peek() == 'e' || peek() == 'E') return fail("expected an integer");
        v = (uint32_t)x;
        return true;
    }

    bool literal(const char *w)
    {
        const size_t n = strlen(w);
        if ((size_t)(end_ - p_) < n || memcmp(p_, w, n) != 0) return fail("bad literal");
        p_ += n;
        return true;
    }

    bool skip_value(int depth = 0)
    {
        if (depth > 64) return fail("nesting too deep");
        ws();
        const char c = peek();
        if (c == '"') {
            std::string s;
            return string(s);
        }
        if (c == '{' || c == '[') {
            const char close = c == '{' ? '}' : ']';
            p_++;
            ws();
            if (peek() == close) { p_++; return true; }
            for (;;) {
                if (c == '{') {
                    std::string k;
                    if (!string(k) || !expect(':')) return false;
                }
                if (!skip_value(depth + 1)) return false;
                ws();
                if (peek() == ',') { p_++; continue; }
                if (peek() == close) { p_++; return true; }
                return fail("expected ',' or a closing bracket");
            }
        }
        if (c == 't') return literal("true");
        if (c == 'f') return literal("false");
        if (c == 'n') return literal("null");
        if (c == '-' || (c >= '0' && c <= '9')) {
            p_++;
            while (p_ < end_ && ((*p_ >= '0' && *p_ <= '9') || *p_ == '.' || *p_ == 'e' || *p_ == 'E' ||
                                 *p_ == '+' || *p_ == '-'))
                p_++;
            return true;
        }
        return fail("unexpected character");
    }

    bool null_value()
    {
        ws();
        if (peek() == 'n') return literal("null");
        return false;
    }

    // netip.ParsePrefix restricted to what matters here.  kind: 0 invalid/zero
    // prefix, 4 IPv4 (addr, bits filled), 6 IPv6.
    bool prefix(const std::string &s, int &kind, uint32_t &addr, int &bits)
    {
        kind = 0;
        if (s.empty()) return true; // the zero Prefix marshals as ""
        const size_t slash = s.rfind('/');
        if (slash == std::string::npos) return fail("prefix \"" + s + "\": no '/'");
        const std::string ip = s.substr(0, slash), bs = s.substr(slash + 1);
        if (bs.empty() || bs.size() > 3) return fail("prefix \"" + s + "\": bad bits");
        if (bs.size() > 1 && bs[0] == '0') return fail("prefix \"" + s + "\": bad bits");
        int b = 0;
        for (char c : bs) {
            if (c < '0' || c > '9') return fail("prefix \"" + s + "\": bad bits");
            b = b * 10 + (c - '0');
        }
        if (ip.find(':') != std::string::npos) {
            if (b > 128 || ip.find('%') != std::string::npos) return fail("prefix \"" + s + "\": bad IPv6 prefix");
            for (char c : ip)
                if (!((c >= '0' && c <= '9') || (c >= 'a' && c <= 'f') || (c >= 'A' && c <= 'F') || c == ':' ||
                      c == '.'))
                    return fail("prefix \"" + s + "\": bad IPv6 address");
            kind = 6;
            return true;
        }
        if (b > 32) return fail("prefix \"" + s + "\": bits out of range");
        uint32_t a = 0;
        int fields = 0;
        size_t i = 0;
        while (i <= ip.size()) {
            size_t j = i;
            uint32_t v = 0;
            while (j < ip.size() && ip[j] >= '0' && ip[j] <= '9') {
                v = v * 10 + (uint32_t)(ip[j] - '0');
                if (v > 255) return fail("prefix \"" + s + "\": IPv4 field out of range");
                j++;
            }
            if (j == i) return fail("prefix \"" + s + "\": bad IPv4 address");
            if (j - i > 1 && ip[i] == '0') return fail("prefix \"" + s + "\": IPv4 field has a leading zero");
            a = a << 8 | v;
            fields++;
            if (j == ip.size()) break;
            if (ip[j] != '.') return fail("prefix \"" + s + "\": bad IPv4 address");
            i = j + 1;
        }
        if (fields != 4) return fail("prefix \"" + s + "\": bad IPv4 address");
        kind = 4;
        addr = a;
        bits = b;
        return true;
    }

    struct Rule {
        std::vector<std::pair<uint32_t, int>> srcs4; // (addr, bits) of the IPv4 prefixes
        std::string proto;
        std::vector<std::pair<uint32_t, uint32_t>> ports;
    };

    bool port_range(std::pair<uint32_t, uint32_t> &pr)
    {
        pr = {0, 0};
        if (!expect('{')) return false;
        ws();
        if (peek() == '}') { p_++; return true; }
        for (;;) {
            std::string k;
            if (!string(k) || !expect(':')) return false;
            if (ieq(k, "first")) {
                if (!null_value() && !uint_value(65535, pr.first)) return false;
            } else if (ieq(k, "last")) {
                if (!null_value() && !uint_value(65535, pr.second)) return false;
            } else if (!skip_value()) {
                return false;
            }
            ws();
            if (peek() == ',') { p_++; continue; }
            return expect('}');
        }
    }

    bool rule(Rule &r)
    {
        if (!expect('{')) return false;
        ws();
        if (peek() == '}') { p_++; return true; }
        for (;;) {
            std::string k;
            if (!string(k) || !expect(':')) return false;
            if (ieq(k, "srcs")) {
                r.srcs4.clear();
                if (!null_value()) {
                    if (!expect('[')) return false;
                    ws();
                    if (peek() == ']') p_++;
                    else
                        for (;;) {
                            std::string s;
                            if (!string(s)) return false;
                            int kind, bits = 0;
                            uint32_t addr = 0;
                            if (!prefix(s, kind, addr, bits)) return false;
                            if (kind == 4) r.srcs4.push_back({addr, bits});
                            ws();
                            if (peek() == ',') { p_++; continue; }
                            if (!expect(']')) return false;
                            break;
                        }
                }
            } else if (ieq(k, "proto")) {
                if (!null_value() && !string(r.proto)) return false;
            } else if (ieq(k, "ports")) {
                r.ports.clear();
                if (!null_value()) {
                    if (!expect('[')) return false;
                    ws();
                    if (peek() == ']') p_++;
                    else
                        for (;;) {
                            std::pair<uint32_t, uint32_t> pr;
                            if (!port_range(pr)) return false;
                            r.ports.push_back(pr);
                            ws();
                            if (peek() == ',') { p_++; continue; }
                            if (!expect(']')) return false;
                            break;
                        }
                }
            } else if (!skip_value()) {
                return false;
            }
            ws();
            if (peek() == ',') { p_++; continue; }
            return expect('}');
        }
    }

    // acl.CompiledRule -> (prefix, port range) tuples, as acl.Match reads them
    // (acl.go:149-172).
    static void flatten(const Rule &r, std::vector<bnk_rule> &out)
    {
        uint8_t proto;
        if (r.proto == "tcp") proto = 6;
        else if (r.proto == "udp") proto = 17;
        else if (r.proto == "icmp") proto = 1;
        else return;
        std::vector<std::pair<uint32_t, uint32_t>> ports = r.ports;
        if (proto == 1) ports = {{0, 0}};
        for (const auto &s : r.srcs4) {
            const uint32_t mask = s.second == 0 ? 0u : 0xFFFFFFFFu << (32 - s.second);
            for (const auto &pr : ports) {
                bnk_rule t{};
                t.src_net = s.first & mask;
                t.src_mask = mask;
                t.port_first = (uint16_t)pr.first;
                t.port_last = (uint16_t)pr.second;
                t.proto = proto;
                out.push_back(t);
            }
        }
    }

    bool rules(NetmapFilter &out)
    {
        out.tuples.clear();
        out.n_rules = 0;
        if (null_value()) return true;
        if (!expect('[')) return false;
        ws();
        if (peek() == ']') { p_++; return true; }
        for (;;) {
            Rule r;
            if (!rule(r)) return false;
            out.n_rules++;
            flatten(r, out.tuples);
            ws();
            if (peek() == ',') { p_++; continue; }
            return expect(']');
        }
    }

    bool document(NetmapFilter &out)
    {
        if (!expect('{')) return false;
        ws();
        if (peek() == '}') { p_++; return true; }
        for (;;) {
            std::string k;
            if (!string(k) || !expect(':')) return false;
            if (ieq(k, "filter_enabled")) {
                ws();
                if (peek() == 't') {
                    if (!literal("true")) return false;
                    out.filter_enabled = true;
                } else if (peek() == 'f') {
                    if (!literal("false")) return false;
                    out.filter_enabled = false;
                } else if (!null_value()) {
                    return fail("filter_enabled is not a boolean");
                }
            } else if (ieq(k, "filter")) {
                if (!rules(out)) return false;
            } else if (!skip_value()) {
                return false;
            }
            ws();
            if (peek() == ',') { p_++; continue; }
            return expect('}');
        }
    }
};

} // namespace bnk
