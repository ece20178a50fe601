// Mutation fuzzing of the hostile-input parsers on the CPU, meant for a build
// with AddressSanitizer and UndefinedBehaviorSanitizer (make san): the netmap
// JSON rule loader (bnk_amd/csrc/netmap_json.hpp), which reads what the control
// server pushes, and the datagram classifiers of the Bind mirror (IsDisco,
// IsSTUN in bnk_amd/host/bnk_bind.hpp), which see raw datagrams from the
// network.  The reference fuzzes its own hostile-input parser the same way
// (internal/disco/fuzz_test.go:6-15: the parser must never panic).  Every input
// lives in a heap block of exactly its size with no terminator, so a read one
// byte past the end is a report.  Seeded and bounded: usage
//     netmap_fuzz [inputs] [seed]
// Stops at the first fault (the sanitizers abort the process).
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <memory>
#include <random>
#include <string>
#include <vector>

#include "../../bnk_amd/csrc/netmap_json.hpp"
#include "../../bnk_amd/host/bnk_bind.hpp"

namespace {

// Valid documents to start from: the shapes the reference's policy tests push
// (internal/coord/server/policy_test.go:10-41, internal/acl/acl_test.go:16-74).
const char *kCorpus[] = {
    R"({"self_id":2,"self_ip":"100.64.0.2/32","peers":[],"filter_enabled":true,"filter":[{"srcs":["100.64.0.1/32"],"proto":"tcp","ports":[{"first":22,"last":22}]}]})",
    R"({"self_id":1,"filter_enabled":true})",
    R"({"self_id":1,"peers":[{"id":3,"name":"x","endpoints":["203.0.113.9:41641"],"key":"AAAA"}]})",
    R"([{"srcs":["100.64.0.1/32","100.64.0.2/32"],"proto":"tcp","ports":[{"first":22,"last":22}]},{"srcs":["100.64.0.0/10"],"proto":"udp","ports":[{"first":6000,"last":6100},{"first":53,"last":53}]},{"srcs":["100.64.0.1/32"],"proto":"icmp"}])",
    R"([{"Srcs":["9.9.9.9/32"],"PROTO":"tcp","Ports":[{"First":7,"LAST":8}]},{"srcs":null,"proto":"tcp","ports":null},{"srcs":["fd7a:115c::/48",""],"proto":"sctp","ports":[{"first":1,"last":65535}]}])",
    R"({"filter_enabled":false,"filter":[],"derp":{"a":[1,2.5e3,-0.1,true,false,null,"é\n\"\\"],"b":{"c":{}}}})",
    R"(  [ { "srcs" : [ "0.0.0.0/0" ] , "proto" : "icmp" , "ports" : [ { "first" : 5 , "last" : 5 } ] } ]  )",
};

const char *kTokens[] = {"{", "}", "[", "]", ",", ":", "\"", "\\", "\\u", "\\ud800", "null", "true", "false", "-", "1e999",
                         "0.", "65536", "4294967296", "99999999999999999999", "/33", "/-1", "/032", "256.1.1.1", "01.2.3.4",
                         "::ffff:1.2.3.4/128", "\"srcs\"", "\"proto\"", "\"ports\"", "\"first\"", "\"last\"", "\"filter\"",
                         "\"filter_enabled\"", "[[[[[[[[[[[[[[[[", "{\"a\":{\"a\":{\"a\":{\"a\":", "\x00", "\xff\xfe", " "};

std::string mutate(std::mt19937_64 &rng, std::string s)
{
    const int rounds = 1 + (int)(rng() % 6);
    for (int r = 0; r < rounds; r++) {
        const size_t n = s.size();
        switch (rng() % 9) {
        case 0: // flip a bit
            if (n) s[rng() % n] ^= (char)(1u << (rng() % 8));
            break;
        case 1: // overwrite a byte
            if (n) s[rng() % n] = (char)rng();
            break;
        case 2: // delete a run
            if (n) {
                const size_t a = rng() % n, len = 1 + rng() % std::min<size_t>(16, n - a);
                s.erase(a, len);
            }
            break;
        case 3: { // insert a token
            const char *t = kTokens[rng() % (sizeof kTokens / sizeof *kTokens)];
            s.insert(n ? rng() % (n + 1) : 0, t);
            break;
        }
        case 4: // truncate
            if (n) s.resize(rng() % n);
            break;
        case 5: // duplicate a run
            if (n) {
                const size_t a = rng() % n, len = 1 + rng() % std::min<size_t>(64, n - a);
                s.insert(rng() % (n + 1), s.substr(a, len));
            }
            break;
        case 6: { // splice in another document's tail
            const std::string o = kCorpus[rng() % (sizeof kCorpus / sizeof *kCorpus)];
            s = s.substr(0, n ? rng() % n : 0) + o.substr(rng() % o.size());
            break;
        }
        case 7: // a digit run becomes another number
            for (size_t i = 0; i < n; i++)
                if (s[i] >= '0' && s[i] <= '9' && rng() % 4 == 0) s[i] = (char)('0' + rng() % 10);
            break;
        default: // deep nesting in front
            s.insert(0, std::string(rng() % 300, rng() % 2 ? '[' : '{'));
            break;
        }
        if (s.size() > 1 << 16) s.resize(1 << 16);
    }
    return s;
}

} // namespace

int main(int argc, char **argv)
{
    const uint64_t inputs = argc > 1 ? strtoull(argv[1], nullptr, 0) : 1000000ull;
    const uint64_t seed = argc > 2 ? strtoull(argv[2], nullptr, 0) : 0x626E6B2026ull;
    std::mt19937_64 rng(seed);
    uint64_t accepted = 0, tuples = 0, disco = 0, stun = 0;
    // the unmutated corpus must parse
    for (const char *doc : kCorpus) {
        bnk::NetmapFilter nf;
        std::string err;
        if (!bnk::NetmapJson(doc, strlen(doc)).parse(nf, err)) {
            fprintf(stderr, "FAIL corpus document rejected: %s\n  %s\n", err.c_str(), doc);
            return 1;
        }
    }
    for (uint64_t i = 0; i < inputs; i++) {
        const std::string s = mutate(rng, kCorpus[rng() % (sizeof kCorpus / sizeof *kCorpus)]);
        // an exact-size heap block: nothing readable behind the last byte
        std::unique_ptr<char[]> buf(new char[s.size() ? s.size() : 1]);
        memcpy(buf.get(), s.data(), s.size());
        bnk::NetmapFilter nf;
        std::string err;
        const bool ok = bnk::NetmapJson(buf.get(), s.size()).parse(nf, err);
        if (ok) {
            accepted++;
            tuples += nf.tuples.size();
            for (const bnk_rule &t : nf.tuples)
                if (t.proto != 1 && t.proto != 6 && t.proto != 17) {
                    fprintf(stderr, "FAIL input %llu: tuple with protocol %u\n", (unsigned long long)i, t.proto);
                    return 1;
                }
        } else if (err.empty()) {
            fprintf(stderr, "FAIL input %llu: rejected without a message\n", (unsigned long long)i);
            return 1;
        }
        // the same bytes as a datagram from the network
        const uint8_t *p = reinterpret_cast<const uint8_t *>(buf.get());
        disco += bnk_host::IsDisco(p, s.size()) ? 1 : 0;
        stun += bnk_host::IsSTUN(p, s.size()) ? 1 : 0;
        if (i % 4 == 0) {
            // and datagrams that begin like the ones the classifiers look for
            const size_t len = rng() % 48;
            std::unique_ptr<uint8_t[]> d(new uint8_t[len ? len : 1]);
            for (size_t k = 0; k < len; k++) d[k] = (uint8_t)rng();
            if (rng() % 2) memcpy(d.get(), bnk_host::kDiscoMagic, std::min(len, bnk_host::kDiscoMagicLen));
            else if (len >= 8) { d[0] &= 0x3F; d[4] = 0x21; d[5] = 0x12; d[6] = 0xA4; d[7] = 0x42; }
            disco += bnk_host::IsDisco(d.get(), len) ? 1 : 0;
            stun += bnk_host::IsSTUN(d.get(), len) ? 1 : 0;
        }
    }
    printf("PASS fuzz: %llu inputs, %llu accepted (%llu tuples), %llu disco, %llu stun, seed %#llx\n",
           (unsigned long long)inputs, (unsigned long long)accepted, (unsigned long long)tuples,
           (unsigned long long)disco, (unsigned long long)stun, (unsigned long long)seed);
    return 0;
}
