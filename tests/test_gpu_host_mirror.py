"""Runs the C++ restatement of the reference's filter_test.go / tun_test.go
(tests/cpp/host_test.cpp) against the GPU through the C++ host mirror
(bnk_amd/host/bnk_host.hpp) and the C ABI."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def test_cpp_host_mirror_suite():
    exe = os.path.join(HERE, "cpp", "host_test")
    assert os.path.exists(exe), "build it first: make -C tests/cpp (or __graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "PASS all host-mirror tests" in r.stdout


def test_cpp_tunnel_over_loopback():
    """encapsulate -> sendmmsg from the pinned ring -> recvmmsg into a pinned
    ring -> decapsulate -> replay window (tests/cpp/tunnel_test.cpp)."""
    exe = os.path.join(HERE, "cpp", "tunnel_test")
    assert os.path.exists(exe), "build it first: make -C tests/cpp (or __graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "PASS tunnel over loopback" in r.stdout


def test_cpp_many_callers_merged_and_direct():
    """Sixteen threads calling with at most 128 packets each, as wireguard-go's
    per-peer goroutines do, with and without the library merging their calls
    (tests/cpp/callers_test.cpp over bnk_amd/host/bnk_callers.cpp)."""
    exe = os.path.join(HERE, "cpp", "callers_test")
    assert os.path.exists(exe), "build it first: make -C tests/cpp (or __graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "callers_test ok" in r.stdout
