/*
 * filter.c -- CPU restatement of the reference's userspace packet filter
 * (internal/filter/filter.go) and rule matcher (internal/acl/acl.go:149-172).
 *
 * Test infrastructure only: see bnk_oracle.h.  Each function names the
 * reference lines it follows.  Go's map[flowKey]time.Time is restated as a
 * chained hash map; time.Time values are Unix nanoseconds.
 */
#include "bnk_oracle.h"

#include <stdlib.h>
#include <string.h>

/* filter.go:18-22 */
#define UDP_FLOW_TTL_NS (30LL * 1000000000LL)
#define TCP_FLOW_TTL_NS (120LL * 1000000000LL)
#define ICMP_FLOW_TTL_NS (30LL * 1000000000LL)

/* ---- acl.go:149-172 ---- */

/* netip.Prefix.Contains for an IPv4 address: false for the invalid prefix
 * and for IPv6 prefixes; otherwise only the top `bits` bits are compared,
 * so host bits set in an unmasked prefix are ignored and /0 contains all. */
static int prefix_contains(const bnko_prefix *p, uint32_t ip)
{
    if (p->bits < 0 || p->bits > 32 || !p->is4) return 0;
    if (p->bits == 0) return 1;
    return ((ip ^ p->addr) >> (32 - p->bits)) == 0;
}

int bnko_rule_match(const bnko_rule *r, uint32_t src, const char *proto,
                    uint16_t dst_port)
{
    if (strcmp(proto, r->proto) != 0) return 0; /* acl.go:150-152 */
    int in_src = 0;                             /* acl.go:153-159 */
    for (uint32_t i = 0; i < r->n_srcs; i++) {
        if (prefix_contains(&r->srcs[i], src)) {
            in_src = 1;
            break;
        }
    }
    if (!in_src) return 0;                        /* acl.go:160-162 */
    if (strcmp(r->proto, "icmp") == 0) return 1;  /* acl.go:163-165 */
    for (uint32_t i = 0; i < r->n_ports; i++) {   /* acl.go:166-170 */
        if (dst_port >= r->ports[i].first && dst_port <= r->ports[i].last)
            return 1;
    }
    return 0; /* acl.go:171 */
}

/* ---- filter.go:62-106 ---- */

static uint32_t be32(const uint8_t *p)
{
    return (uint32_t)p[0] << 24 | (uint32_t)p[1] << 16 | (uint32_t)p[2] << 8 |
           (uint32_t)p[3];
}
static uint16_t be16(const uint8_t *p)
{
    return (uint16_t)((uint16_t)p[0] << 8 | p[1]);
}

int bnko_parse(const uint8_t *pkt, size_t len, bnko_parsed *out)
{
    memset(out, 0, sizeof *out);
    if (len < 20 || (pkt[0] >> 4) != 4) return 0; /* filter.go:72-74 */
    size_t ihl = (size_t)(pkt[0] & 0x0F) * 4;     /* filter.go:75 */
    if (ihl < 20 || len < ihl) return 0;          /* filter.go:76-78 */
    out->proto = pkt[9];                          /* filter.go:79 */
    out->src = be32(pkt + 12);                    /* filter.go:80 */
    out->dst = be32(pkt + 16);                    /* filter.go:81 */
    const uint8_t *body = pkt + ihl;              /* filter.go:83 */
    size_t body_len = len - ihl;
    switch (out->proto) {
    case 6:
    case 17: /* filter.go:85-95 */
        if (body_len < 4) return 0;
        out->src_port = be16(body);
        out->dst_port = be16(body + 2);
        out->proto_name = out->proto == 6 ? "tcp" : "udp";
        break;
    case 1: /* filter.go:96-101 */
        if (body_len < 1) return 0;
        out->icmp_type = body[0];
        out->proto_name = "icmp";
        break;
    default: /* filter.go:102-104 */
        return 0;
    }
    return 1;
}

/* filter.go:108-117 */
int64_t bnko_flow_ttl_ns(uint8_t proto)
{
    switch (proto) {
    case 6:
        return TCP_FLOW_TTL_NS;
    case 1:
        return ICMP_FLOW_TTL_NS;
    default:
        return UDP_FLOW_TTL_NS;
    }
}

/* ---- flows map[flowKey]time.Time (filter.go:26-31, 37) ---- */

typedef struct flow_ent {
    uint32_t remote;
    uint16_t remote_port, local_port;
    uint8_t proto;
    int64_t expiry;
    struct flow_ent *next;
} flow_ent;

typedef struct {
    bnko_prefix *srcs;
    uint32_t n_srcs;
    char *proto;
    bnko_port_range *ports;
    uint32_t n_ports;
} own_rule;

struct bnko_filter {
    int enforce;
    own_rule *rules;
    uint32_t n_rules;
    flow_ent **buckets;
    uint32_t n_buckets; /* power of two */
    uint32_t n_flows;
    /* lower bound on every stored expiry; lets the :202-208 sweep skip the
     * scan when it provably deletes nothing (the result is unchanged) */
    int64_t min_expiry_lb;
};

static uint32_t flow_hash(uint32_t remote, uint16_t rp, uint16_t lp,
                          uint8_t proto)
{
    uint64_t x = (uint64_t)remote << 32 | (uint64_t)rp << 16 | lp;
    x ^= (uint64_t)proto * 0x9E3779B97F4A7C15ULL;
    x ^= x >> 33;
    x *= 0xff51afd7ed558ccdULL;
    x ^= x >> 33;
    x *= 0xc4ceb9fe1a85ec53ULL;
    x ^= x >> 33;
    return (uint32_t)x;
}

static void flows_rehash(bnko_filter *f, uint32_t nb)
{
    flow_ent **nbk = (flow_ent **)calloc(nb, sizeof *nbk);
    for (uint32_t b = 0; b < f->n_buckets; b++) {
        flow_ent *e = f->buckets[b];
        while (e) {
            flow_ent *nx = e->next;
            uint32_t h =
                flow_hash(e->remote, e->remote_port, e->local_port, e->proto) &
                (nb - 1);
            e->next = nbk[h];
            nbk[h] = e;
            e = nx;
        }
    }
    free(f->buckets);
    f->buckets = nbk;
    f->n_buckets = nb;
}

static flow_ent **flow_find(bnko_filter *f, uint32_t remote, uint16_t rp,
                            uint16_t lp, uint8_t proto)
{
    uint32_t h = flow_hash(remote, rp, lp, proto) & (f->n_buckets - 1);
    flow_ent **pp = &f->buckets[h];
    while (*pp) {
        flow_ent *e = *pp;
        if (e->remote == remote && e->remote_port == rp &&
            e->local_port == lp && e->proto == proto)
            return pp;
        pp = &e->next;
    }
    return pp; /* points at the NULL tail link of the bucket */
}

/* filter.go:41-43 */
bnko_filter *bnko_filter_new(void)
{
    bnko_filter *f = (bnko_filter *)calloc(1, sizeof *f);
    f->n_buckets = 1024;
    f->buckets = (flow_ent **)calloc(f->n_buckets, sizeof *f->buckets);
    f->min_expiry_lb = INT64_MAX;
    return f;
}

static void rules_free(bnko_filter *f)
{
    for (uint32_t i = 0; i < f->n_rules; i++) {
        free(f->rules[i].srcs);
        free(f->rules[i].proto);
        free(f->rules[i].ports);
    }
    free(f->rules);
    f->rules = NULL;
    f->n_rules = 0;
}

void bnko_filter_free(bnko_filter *f)
{
    if (!f) return;
    rules_free(f);
    for (uint32_t b = 0; b < f->n_buckets; b++) {
        flow_ent *e = f->buckets[b];
        while (e) {
            flow_ent *nx = e->next;
            free(e);
            e = nx;
        }
    }
    free(f->buckets);
    free(f);
}

/* filter.go:46-51 */
void bnko_filter_set_rules(bnko_filter *f, const bnko_rule *rules, uint32_t n)
{
    rules_free(f);
    f->enforce = 1;
    f->rules = (own_rule *)calloc(n ? n : 1, sizeof *f->rules);
    f->n_rules = n;
    for (uint32_t i = 0; i < n; i++) {
        own_rule *o = &f->rules[i];
        o->n_srcs = rules[i].n_srcs;
        o->srcs = (bnko_prefix *)malloc(sizeof(bnko_prefix) *
                                        (o->n_srcs ? o->n_srcs : 1));
        if (o->n_srcs)
            memcpy(o->srcs, rules[i].srcs, sizeof(bnko_prefix) * o->n_srcs);
        o->proto = strdup(rules[i].proto ? rules[i].proto : "");
        o->n_ports = rules[i].n_ports;
        o->ports = (bnko_port_range *)malloc(sizeof(bnko_port_range) *
                                             (o->n_ports ? o->n_ports : 1));
        if (o->n_ports)
            memcpy(o->ports, rules[i].ports,
                   sizeof(bnko_port_range) * o->n_ports);
    }
}

/* filter.go:54-59: enforcement off, rules dropped, flows kept */
void bnko_filter_set_allow_all(bnko_filter *f)
{
    rules_free(f);
    f->enforce = 0;
}

/* filter.go:121-147 */
int bnko_filter_check_inbound(bnko_filter *f, const uint8_t *pkt, size_t len,
                              int64_t now_ns)
{
    if (!f->enforce) return 1; /* :124-126 */
    bnko_parsed p;
    if (!bnko_parse(pkt, len, &p)) return 0; /* :127-130 */
    for (uint32_t i = 0; i < f->n_rules; i++) { /* :131-135 */
        const own_rule *o = &f->rules[i];
        bnko_rule r = {o->srcs, o->n_srcs, o->proto, o->ports, o->n_ports};
        if (bnko_rule_match(&r, p.src, p.proto_name, p.dst_port)) return 1;
    }
    /* :138 key = {remote: src, remotePort: srcPort, localPort: dstPort} */
    flow_ent **pp = flow_find(f, p.src, p.src_port, p.dst_port, p.proto);
    flow_ent *e = *pp;
    if (e) {                      /* :139 */
        if (now_ns < e->expiry) { /* :140 now.Before(exp) */
            e->expiry = now_ns + bnko_flow_ttl_ns(p.proto); /* :141 */
            if (e->expiry < f->min_expiry_lb) f->min_expiry_lb = e->expiry;
            return 1;
        }
        *pp = e->next; /* :144 delete */
        free(e);
        f->n_flows--;
    }
    return 0; /* :146 */
}

/* filter.go:189-209 */
void bnko_filter_note_outbound(bnko_filter *f, const uint8_t *pkt, size_t len,
                               int64_t now_ns)
{
    if (!f->enforce) return; /* :192-194 */
    bnko_parsed p;
    if (!bnko_parse(pkt, len, &p)) return; /* :195-198 */
    /* :199 key = {remote: dst, remotePort: dstPort, localPort: srcPort} */
    flow_ent **pp = flow_find(f, p.dst, p.dst_port, p.src_port, p.proto);
    int64_t exp = now_ns + bnko_flow_ttl_ns(p.proto);
    if (exp < f->min_expiry_lb) f->min_expiry_lb = exp;
    if (*pp) {
        (*pp)->expiry = exp; /* :200 */
    } else {
        flow_ent *e = (flow_ent *)calloc(1, sizeof *e);
        e->remote = p.dst;
        e->remote_port = p.dst_port;
        e->local_port = p.src_port;
        e->proto = p.proto;
        e->expiry = exp;
        *pp = e;
        f->n_flows++;
        if (f->n_flows > f->n_buckets) flows_rehash(f, f->n_buckets * 2);
    }
    if (f->n_flows > 4096 && now_ns > f->min_expiry_lb) { /* :202-208 */
        int64_t lb = INT64_MAX;
        for (uint32_t b = 0; b < f->n_buckets; b++) {
            flow_ent **q = &f->buckets[b];
            while (*q) {
                flow_ent *e = *q;
                if (now_ns > e->expiry) { /* now.After(exp) */
                    *q = e->next;
                    free(e);
                    f->n_flows--;
                } else {
                    if (e->expiry < lb) lb = e->expiry;
                    q = &e->next;
                }
            }
        }
        f->min_expiry_lb = lb;
    }
}

uint32_t bnko_filter_flow_count(const bnko_filter *f) { return f->n_flows; }

uint32_t bnko_filter_flow_dump(const bnko_filter *f, uint64_t *key,
                               uint8_t *proto, int64_t *expiry_ns)
{
    uint32_t k = 0;
    for (uint32_t b = 0; b < f->n_buckets; b++) {
        for (const flow_ent *e = f->buckets[b]; e; e = e->next) {
            key[k] = (uint64_t)e->remote << 32 | (uint64_t)e->remote_port << 16 |
                     e->local_port;
            proto[k] = e->proto;
            expiry_ns[k] = e->expiry;
            k++;
        }
    }
    return k;
}

/* filter.go:171-178: one `now`, one verdict per packet in order */
void bnko_filter_check_inbound_batch(bnko_filter *f, const uint8_t *pkts,
                                     const uint64_t *off, const uint32_t *len,
                                     uint32_t n, int64_t now_ns,
                                     uint8_t *verdict)
{
    for (uint32_t i = 0; i < n; i++)
        verdict[i] = (uint8_t)bnko_filter_check_inbound(f, pkts + off[i],
                                                        len[i], now_ns);
}

/* filter.go:160-167 */
void bnko_filter_note_outbound_batch(bnko_filter *f, const uint8_t *pkts,
                                     const uint64_t *off, const uint32_t *len,
                                     uint32_t n, int64_t now_ns)
{
    for (uint32_t i = 0; i < n; i++)
        bnko_filter_note_outbound(f, pkts + off[i], len[i], now_ns);
}
