"""OpenSSL EVP_chacha20_poly1305 through ctypes: an independent library (not
the reference, not the oracle) used to pin the oracle on benchmark shapes and
to write tests/golden fixtures.  ``available()`` is False when libcrypto is
not on the machine; callers skip then."""
import ctypes as C
import ctypes.util

_lib = None


def _load():
    global _lib
    if _lib is None:
        name = ctypes.util.find_library("crypto")
        for cand in ([name] if name else []) + ["libcrypto.so.3", "libcrypto.so"]:
            try:
                _lib = C.CDLL(cand)
                break
            except OSError:
                continue
        if _lib is None:
            _lib = False
        else:
            _lib.EVP_CIPHER_CTX_new.restype = C.c_void_p
            _lib.EVP_chacha20_poly1305.restype = C.c_void_p
            _lib.EVP_chacha20.restype = C.c_void_p
    return _lib


def available() -> bool:
    return bool(_load())


_GET_TAG, _SET_TAG = 0x10, 0x11


def seal(key: bytes, nonce: bytes, pt: bytes, aad: bytes = b"") -> bytes:
    L = _load()
    ctx = C.c_void_p(L.EVP_CIPHER_CTX_new())
    try:
        assert L.EVP_EncryptInit_ex(ctx, C.c_void_p(L.EVP_chacha20_poly1305()),
                                    None, key, nonce) == 1
        n = C.c_int(0)
        if aad:
            assert L.EVP_EncryptUpdate(ctx, None, C.byref(n), aad, len(aad)) == 1
        out = C.create_string_buffer(len(pt) + 16)
        assert L.EVP_EncryptUpdate(ctx, out, C.byref(n), pt, len(pt)) == 1
        m = C.c_int(0)
        assert L.EVP_EncryptFinal_ex(ctx, C.byref(out, n.value), C.byref(m)) == 1
        tag = C.create_string_buffer(16)
        assert L.EVP_CIPHER_CTX_ctrl(ctx, _GET_TAG, 16, tag) == 1
        return out.raw[:len(pt)] + tag.raw
    finally:
        L.EVP_CIPHER_CTX_free(ctx)


def open_(key: bytes, nonce: bytes, ct: bytes, aad: bytes = b""):
    """Returns plaintext bytes or None when the tag does not verify."""
    L = _load()
    if len(ct) < 16:
        return None
    body, tag = ct[:-16], ct[-16:]
    ctx = C.c_void_p(L.EVP_CIPHER_CTX_new())
    try:
        assert L.EVP_DecryptInit_ex(ctx, C.c_void_p(L.EVP_chacha20_poly1305()),
                                    None, key, nonce) == 1
        assert L.EVP_CIPHER_CTX_ctrl(ctx, _SET_TAG, 16,
                                     C.create_string_buffer(tag, 16)) == 1
        n = C.c_int(0)
        if aad:
            assert L.EVP_DecryptUpdate(ctx, None, C.byref(n), aad, len(aad)) == 1
        out = C.create_string_buffer(max(len(body), 1))
        assert L.EVP_DecryptUpdate(ctx, out, C.byref(n), body, len(body)) == 1
        m = C.c_int(0)
        ok = L.EVP_DecryptFinal_ex(ctx, C.byref(out, n.value), C.byref(m))
        return out.raw[:len(body)] if ok > 0 else None
    finally:
        L.EVP_CIPHER_CTX_free(ctx)


def chacha20_stream(key: bytes, counter: int, nonce: bytes, data: bytes) -> bytes:
    """Raw ChaCha20: OpenSSL's 16-byte IV is LE32(counter) || nonce."""
    L = _load()
    ctx = C.c_void_p(L.EVP_CIPHER_CTX_new())
    try:
        iv = counter.to_bytes(4, "little") + nonce
        assert L.EVP_EncryptInit_ex(ctx, C.c_void_p(L.EVP_chacha20()), None,
                                    key, iv) == 1
        out = C.create_string_buffer(max(len(data), 1))
        n = C.c_int(0)
        assert L.EVP_EncryptUpdate(ctx, out, C.byref(n), data, len(data)) == 1
        return out.raw[:len(data)]
    finally:
        L.EVP_CIPHER_CTX_free(ctx)
