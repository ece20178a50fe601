"""The kernels' per-lane ChaCha20 / Poly1305 arithmetic (bnk_amd/csrc/aead_lane.hpp)
compiled for the host and run against the RFC 8439 vectors -- including the
appendix A.3 Poly1305 carry cases that need a chosen r and s and so cannot be
reached through packets on the GPU -- and against the C oracle."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def test_lane_arithmetic_on_cpu():
    subprocess.run(["make", "-s", "-C", os.path.join(HERE, "..", "oracle")], check=True)
    subprocess.run(["make", "-s", "-C", os.path.join(HERE, "cpp"), "lane_test"], check=True)
    r = subprocess.run([os.path.join(HERE, "cpp", "lane_test")], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "PASS lane arithmetic" in r.stdout
