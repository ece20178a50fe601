"""The ring-based Bind mirror (bnk_amd/host/bnk_bind.hpp) over loopback UDP:
the reference's bind_batch_test.go / bind_transport_test.go / disco_demux_test.go
cases restated in tests/cpp/bind_test.cpp.  No GPU involved."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def test_ring_bind_over_loopback():
    subprocess.run(["make", "-s", "-C", os.path.join(HERE, "cpp"), "bind_test"], check=True)
    r = subprocess.run([os.path.join(HERE, "cpp", "bind_test")], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr


def test_batch_coalescer_with_a_stand_in_executor():
    """bnk_amd/host/bnk_coalesce.hpp: callers get their own verdicts, windows
    fill and flush, a lone caller waits at most the window, failures reach
    every caller (tests/cpp/coalesce_test.cpp)."""
    subprocess.run(["make", "-s", "-C", os.path.join(HERE, "cpp"), "coalesce_test"], check=True)
    r = subprocess.run([os.path.join(HERE, "cpp", "coalesce_test")], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
