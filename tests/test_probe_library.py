"""The benchmark's probe library (libbnkprobe.so): it loads and exports what its
header declares (no GPU needed), and on a GPU its issue probes show the two
rules the AEAD roofline is read against: plain instructions of two waves issue
together, rotates one wave at a time with the older wave first."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "bnk_amd", "probe", "bnkprobe.h")


def _declared():
    src = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(bnkp_[a-z0-9_]+)\s*\(", src)))


def test_probe_library_exports_every_declared_symbol():
    from bnk_amd import probe
    so = probe.load()
    names = _declared()
    assert {"bnkp_valu", "bnkp_copy", "bnkp_pair", "bnkp_mix", "bnkp_aead_compute", "bnkp_line_copy"} <= set(names)
    for name in names:
        assert hasattr(so, name), f"{name} is declared in bnkprobe.h but not exported"


def test_probe_rejects_bad_arguments_without_a_gpu_call():
    import ctypes as C
    from bnk_amd import probe
    so = probe.load()
    r = C.c_double()
    assert so.bnkp_valu(0, 999, 10, C.byref(r)) == -1
    assert so.bnkp_pair(0, 99, 0, 10, C.byref(r), C.byref(r)) == -1
    assert so.bnkp_mix(0, 0, 0, 10, C.byref(r)) == -1
    assert so.bnkp_copy(0, 100, 1, C.byref(r)) == -1
    assert so.bnkp_aead_compute(0, 1, 5, 48, C.byref(r)) == -1   # at most four waves per SIMD
    assert so.bnkp_aead_compute(0, 1, 2, 47, C.byref(r)) == -1   # blocks come in pairs
    assert so.bnkp_line_copy(0, 1024, 1441, 1420, 2, 1, 0, 1, C.byref(r)) == -1  # stride not a multiple of 16
    assert so.bnkp_line_copy(0, 1024, 1440, 1420, 2, 3, 0, 1, C.byref(r)) == -1  # a line is held one or two steps


@pytest.mark.gpu
def test_issue_probes_show_the_pairing_rules():
    from bnk_amd import probe
    alone, _ = probe.pair("v_add_u32", None, 4000)
    a, b = probe.pair("v_add_u32", "v_add_u32", 4000)
    # two waves of adds on one SIMD: each as fast as one alone (within a third)
    assert a < 1.35 * alone and b < 1.35 * alone
    a, b = probe.pair("v_add_u32", "v_alignbit_b32", 4000)
    # rotates beside an older wave's adds wait; the adds do not
    assert a < 1.35 * alone and b > 1.3 * alone
    plain = probe.mix(False, 2, 200)
    raised = probe.mix(True, 2, 200)
    assert plain > 20e12 and raised > 1.05 * plain


@pytest.mark.gpu
def test_arithmetic_alone_gains_from_a_second_wave_and_copy_streams():
    from bnk_amd import probe
    one = probe.aead_compute(True, 1, 24)
    two = probe.aead_compute(True, 2, 24)
    # a wave issues at most one instruction per 4.8 cycles: a second wave per SIMD nearly doubles the rate
    assert one > 10e9 and two > 1.5 * one
    single = probe.aead_compute(False, 2, 24)
    assert 0.7 * two < single < 1.1 * two
    assert probe.copy(1 << 28, 4) > 2e12
