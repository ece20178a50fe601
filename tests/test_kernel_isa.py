"""What the compiler made of the lane-per-packet AEAD kernels, read from its assembly
listing (no GPU needed: hipcc cross-compiles).

The kernels prefetch a packet's next line while they work on the current one.  That only
overlaps if no wait for *everything* in flight sits inside or right behind the group of
loads that fetches the line.  The compiler has put one there before (to protect a register
the last load of the group fills: the sealing launch then sat out a whole trip to memory in
every step, 5 % of its time), and nothing but its listing shows it.  The same listing says
whether a kernel spills registers, which at two waves per SIMD it must not."""
import os
import re
import subprocess
import tempfile

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "..", "bnk_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
WAVE_KERNELS = ("_ZN3bnk16aead_wave_kernelILb0EEEvNS_8AeadArgsE", "_ZN3bnk16aead_wave_kernelILb1EEEvNS_8AeadArgsE")
# seal, open, seal + framing, open + framing of a small batch: a wave per packet
SPREAD_KERNELS = tuple("_ZN3bnk18aead_spread_kernelILb%dELb%dEEEvNS_8AeadArgsE" % (o, w) for w in (0, 1) for o in (0, 1))


@pytest.fixture(scope="module")
def listing():
    if not os.path.exists(HIPCC):
        pytest.skip("no hipcc")
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "aead_kernels.s")
        # the library's own flags (bnk_amd/csrc/Makefile), to a device-side listing instead of an object
        cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "-S", "--cuda-device-only", os.path.join(CSRC, "aead_kernels.hip"), "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        return open(out).read()


def _body(listing, name):
    i = listing.index(name + ":")
    return listing[i:listing.index("s_endpgm", i)].split("\n")


@pytest.mark.parametrize("name", WAVE_KERNELS)
def test_no_wait_for_everything_among_the_loads_of_a_line(listing, name):
    lines = _body(listing, name)
    assert sum("global_load_dwordx4" in x for x in lines) >= 24, "not the kernel this test was written for"
    bad = []
    for k, text in enumerate(lines):
        if "s_waitcnt vmcnt(0)" in text:
            before = any("global_load_dwordx4" in x for x in lines[max(0, k - 6):k])
            after = any("global_load_dwordx4" in x for x in lines[k + 1:k + 3])
            if before and after:
                bad.append(k)
    assert not bad, "s_waitcnt vmcnt(0) between the loads of a line at listing lines %r of %s" % (bad, name)


@pytest.mark.parametrize("name", WAVE_KERNELS)
def test_the_wave_kernels_spill_nothing(listing, name):
    meta = listing[listing.index(".name:           " + name):]
    meta = meta[:meta.index(".wavefront_size")]
    get = lambda key: int(re.search(r"\.%s:\s+(\d+)" % key, meta).group(1))  # noqa: E731
    assert get("vgpr_spill_count") == 0 and get("private_segment_fixed_size") == 0
    assert get("vgpr_count") <= 256  # two waves per SIMD


@pytest.mark.parametrize("name", SPREAD_KERNELS)
def test_a_small_batch_packet_is_fetched_in_one_go(listing, name):
    """The wave-per-packet kernel reads a host batch over the link: every wait between two
    of its loads is a trip there and back.  A packet's four pieces, its last 1-15 bytes
    (three words, a halfword, a byte) and what goes with them must go out with no wait for
    memory among them (they did not while each sat under a branch of its own: the launch for
    128 packets took 17.8 us instead of 13.3)."""
    lines = _body(listing, name)
    best = run = 0
    for text in lines:
        t = text.strip()
        if t.startswith("global_load"):
            run += 1
            best = max(best, run)
        elif t.startswith("s_waitcnt") and "vmcnt" in t:
            run = 0
    assert best >= 9, "longest run of loads without a wait for memory is %d in %s" % (best, name)
