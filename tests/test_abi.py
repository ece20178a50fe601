"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and refuses to work without a GPU instead of falling back."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bnkhip.h")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(bnk_[a-z0-9_]+)\s*\(", src)))


def test_header_declares_the_expected_surface():
    names = _declared()
    for must in ("bnk_init", "bnk_shutdown", "bnk_keys_set", "bnk_aead_seal_batch",
                 "bnk_aead_open_batch", "bnk_filter_set_rules", "bnk_filter_set_allow_all",
                 "bnk_filter_note_outbound_batch", "bnk_filter_check_inbound_batch",
                 "bnk_relay_fused_batch", "bnk_ring_alloc", "bnk_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from bnk_amd import lib
    so = lib.load()
    for name in _declared():
        assert hasattr(so, name), f"{name} is declared in bnkhip.h but not exported"


def test_struct_layouts_match_the_header():
    from bnk_amd import lib
    # bnk_batch: void*, u64, u32, u32, ptr, u32, u32, ptr, ptr, ptr, u64
    assert C.sizeof(lib.Batch) == 72
    assert lib.Batch.offsets.offset == 24 and lib.Batch.lens.offset == 40
    assert lib.Batch.counter0.offset == 64
    # bnk_rule: u32, u32, u16, u16, u8, pad[3]
    assert C.sizeof(lib.Rule) == 16 and lib.Rule.proto.offset == 12


def test_no_gpu_means_an_error_not_a_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from bnk_amd import lib
    with pytest.raises(lib.BnkError) as ei:
        lib.Context(0)
    assert ei.value.code == lib.E_NODEV
    so = lib.load()
    # every entry point rejects a null context instead of crashing
    assert so.bnk_sync(None) == lib.E_INVAL
    assert so.bnk_aead_seal_batch(None, None, None) == lib.E_INVAL
    assert so.bnk_filter_set_allow_all(None) == lib.E_INVAL


def test_product_package_never_touches_the_oracle():
    # the CPU oracle is test infrastructure: nothing shipped may import, link
    # or even name it
    for top in ("bnk_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, top)):
            for f in files:
                if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp", ".inc")) or f == "Makefile":
                    text = open(os.path.join(dirpath, f), errors="ignore").read().lower()
                    assert "oracle" not in text, f"{os.path.join(dirpath, f)} names the oracle"


def test_rule_flattening_matches_reference_semantics():
    from bnk_amd import lib
    from bnk_amd import workloads as W
    arr, n = lib.flatten_rules([
        ([(W.ip("100.64.3.99"), 24), (W.ip("10.0.0.0"), 8)], "tcp", [(1, 2), (5, 5)]),
        ([(W.ip("1.2.3.4"), 32)], "icmp", [(9, 9)]),
        ([(W.ip("1.2.3.4"), 32)], "udp", []),          # never matches: no tuples
        ([(W.ip("1.2.3.4"), 32)], "sctp", [(1, 1)]),   # unknown proto: no tuples
        ([(W.ip("1.2.3.4"), -1)], "tcp", [(1, 1)]),    # invalid prefix: no tuples
        ([(0x01020304, 0)], "udp", [(7, 8)]),
    ])
    got = [(arr[i].src_net, arr[i].src_mask, arr[i].port_first, arr[i].port_last, arr[i].proto)
           for i in range(n)]
    assert got == [
        (W.ip("100.64.3.0"), 0xFFFFFF00, 1, 2, 6), (W.ip("100.64.3.0"), 0xFFFFFF00, 5, 5, 6),
        (W.ip("10.0.0.0"), 0xFF000000, 1, 2, 6), (W.ip("10.0.0.0"), 0xFF000000, 5, 5, 6),
        (W.ip("1.2.3.4"), 0xFFFFFFFF, 0, 0, 1),
        (0, 0, 7, 8, 17),
    ]


def test_allocation_failure_inside_the_library_is_an_error_code_not_an_unwind():
    """Nothing may throw across the C boundary: with the address space capped,
    parsing a netmap document that needs more memory than is left must come
    back as BNK_E_NOMEM (the std::bad_alloc is caught at the boundary), not
    abort the process.  Runs in a child process because of the cap."""
    import subprocess
    import sys
    code = r'''
import ctypes as C, resource, sys
sys.path.insert(0, %r)
from bnk_amd import lib
so = lib.load()
rule = b'{"srcs":["100.64.0.7/32","100.64.9.0/24"],"proto":"tcp","ports":[{"first":22,"last":22},{"first":80,"last":90}]},'
doc = b'{"filter_enabled":true,"filter":[' + rule * 1000000
doc = doc[:-1] + b']}'
vm = [int(l.split()[1]) * 1024 for l in open("/proc/self/status") if l.startswith("VmSize")][0]
resource.setrlimit(resource.RLIMIT_AS, (vm + (48 << 20), vm + (48 << 20)))
n = C.c_uint32(); en = C.c_int(); err = C.create_string_buffer(256)
arr = (lib.Rule * 16)()
rc = so.bnk_rules_from_netmap_json(doc, C.c_size_t(len(doc)), arr, C.c_uint32(16), C.byref(n),
                                   C.byref(en), err, C.c_size_t(256))
print("rc", rc, err.value.decode())
''' % ROOT
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-400:]
    assert r.stdout.strip() == "rc -4 out of host memory"
