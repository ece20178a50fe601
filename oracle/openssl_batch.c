/* TEST / BENCHMARK INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A second CPU baseline beside the scalar restatement: the same seal + open
 * batch run through OpenSSL's EVP_chacha20_poly1305 (hand-tuned assembly, the
 * closest thing on this machine to the assembly x/crypto uses in the Go
 * reference).  libcrypto is looked up at run time, so nothing links against
 * it; bnko_ossl_available() is 0 where it is missing. */
#include <dlfcn.h>
#include <pthread.h>
#include <stdint.h>
#include <string.h>

#include "bnk_oracle.h"

typedef void *(*fn_ctx_new)(void);
typedef void (*fn_ctx_free)(void *);
typedef const void *(*fn_cipher)(void);
typedef int (*fn_init)(void *, const void *, void *, const unsigned char *, const unsigned char *);
typedef int (*fn_update)(void *, unsigned char *, int *, const unsigned char *, int);
typedef int (*fn_final)(void *, unsigned char *, int *);
typedef int (*fn_ctrl)(void *, int, int, void *);

static struct {
    int tried, ok;
    fn_ctx_new ctx_new;
    fn_ctx_free ctx_free;
    fn_cipher cipher;
    fn_init enc_init, dec_init;
    fn_update enc_update, dec_update;
    fn_final enc_final, dec_final;
    fn_ctrl ctrl;
} L;

static pthread_once_t once = PTHREAD_ONCE_INIT;

static void load(void)
{
    const char *names[] = {"libcrypto.so.3", "libcrypto.so", "libcrypto.so.1.1"};
    void *h = NULL;
    for (unsigned i = 0; i < 3 && !h; i++) h = dlopen(names[i], RTLD_NOW | RTLD_LOCAL);
    L.tried = 1;
    if (!h) return;
    L.ctx_new = (fn_ctx_new)dlsym(h, "EVP_CIPHER_CTX_new");
    L.ctx_free = (fn_ctx_free)dlsym(h, "EVP_CIPHER_CTX_free");
    L.cipher = (fn_cipher)dlsym(h, "EVP_chacha20_poly1305");
    L.enc_init = (fn_init)dlsym(h, "EVP_EncryptInit_ex");
    L.dec_init = (fn_init)dlsym(h, "EVP_DecryptInit_ex");
    L.enc_update = (fn_update)dlsym(h, "EVP_EncryptUpdate");
    L.dec_update = (fn_update)dlsym(h, "EVP_DecryptUpdate");
    L.enc_final = (fn_final)dlsym(h, "EVP_EncryptFinal_ex");
    L.dec_final = (fn_final)dlsym(h, "EVP_DecryptFinal_ex");
    L.ctrl = (fn_ctrl)dlsym(h, "EVP_CIPHER_CTX_ctrl");
    L.ok = L.ctx_new && L.ctx_free && L.cipher && L.enc_init && L.dec_init && L.enc_update &&
           L.dec_update && L.enc_final && L.dec_final && L.ctrl;
}

int bnko_ossl_available(void)
{
    pthread_once(&once, load);
    return L.ok;
}

#define AEAD_GET_TAG 0x10
#define AEAD_SET_TAG 0x11

struct job {
    const uint8_t *keys;
    const uint32_t *peer;
    const uint64_t *counters;
    const uint8_t *in;
    const uint64_t *off;
    const uint32_t *len;
    uint8_t *sealed, *opened;
    uint32_t lo, hi;
    uint32_t ok;
};

static void *worker(void *arg)
{
    struct job *j = (struct job *)arg;
    /* one context per direction, bound to the cipher once: naming the cipher
     * again per packet makes OpenSSL 3 look it up under a global lock */
    void *ce = L.ctx_new(), *cd = L.ctx_new();
    L.enc_init(ce, L.cipher(), NULL, NULL, NULL);
    L.dec_init(cd, L.cipher(), NULL, NULL, NULL);
    for (uint32_t i = j->lo; i < j->hi; i++) {
        uint8_t nonce[12];
        bnko_wg_nonce(j->counters[i], nonce);
        const uint8_t *key = j->keys + 32 * (size_t)(j->peer ? j->peer[i] : 0);
        const uint8_t *pt = j->in + j->off[i];
        uint8_t *ct = j->sealed + j->off[i], *back = j->opened + j->off[i];
        const int n = (int)j->len[i];
        int m = 0, good = 1;
        good &= L.enc_init(ce, NULL, NULL, key, nonce);
        good &= L.enc_update(ce, ct, &m, pt, n);
        good &= L.enc_final(ce, ct + m, &m);
        good &= L.ctrl(ce, AEAD_GET_TAG, 16, ct + n);
        good &= L.dec_init(cd, NULL, NULL, key, nonce);
        good &= L.ctrl(cd, AEAD_SET_TAG, 16, ct + n);
        good &= L.dec_update(cd, back, &m, ct, n);
        good &= L.dec_final(cd, back + m, &m) > 0;
        j->ok += good ? 1u : 0u;
    }
    L.ctx_free(ce);
    L.ctx_free(cd);
    return NULL;
}

/* seal into `sealed` (len + 16 bytes per packet) and open again into `opened`,
 * packets split evenly over nthreads; returns how many round trips verified. */
uint32_t bnko_ossl_seal_open_batch(const uint8_t *keys, const uint32_t *peer, const uint64_t *counters,
                                   const uint8_t *in, const uint64_t *off, const uint32_t *len,
                                   uint8_t *sealed, uint8_t *opened, uint32_t n, int nthreads)
{
    if (!bnko_ossl_available()) return 0;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 64) nthreads = 64;
    pthread_t th[64];
    struct job jobs[64];
    for (int t = 0; t < nthreads; t++) {
        jobs[t] = (struct job){keys, peer, counters, in, off, len, sealed, opened,
                               (uint32_t)((uint64_t)n * t / nthreads),
                               (uint32_t)((uint64_t)n * (t + 1) / nthreads), 0};
        pthread_create(&th[t], NULL, worker, &jobs[t]);
    }
    uint32_t ok = 0;
    for (int t = 0; t < nthreads; t++) {
        pthread_join(th[t], NULL);
        ok += jobs[t].ok;
    }
    return ok;
}
