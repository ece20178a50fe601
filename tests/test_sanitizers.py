"""CPU builds of the host-side code under sanitizers, and the hostile-input
parsers under a seeded fuzzer.  The reference runs its tests under Go's race
detector (README.md:79) and fuzzes the parser that reads datagrams from the
network (internal/disco/fuzz_test.go:6-15); here:

  AddressSanitizer + UndefinedBehaviorSanitizer (any report ends the program)
      the kernels' lane arithmetic compiled for the host, the replay window,
      the Bind mirror over loopback, the filter-call coalescer, each with the C
      oracle's sources built the same way where they link it;
      the oracle's own Python tests against oracle/san/libbnkoracle.so;
      10^6 mutated netmap documents and datagrams through netmap_json.hpp,
      IsDisco and IsSTUN (tests/cpp/netmap_fuzz.cpp);
  ThreadSanitizer
      the coalescer and the Bind mirror, whose point is threads.

Nothing here touches the GPU; the GPU code is compiled without sanitizers."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CPP = os.path.join(HERE, "cpp")
ROOT = os.path.dirname(HERE)


def _run(path, *args, timeout=300):
    env = dict(os.environ, ASAN_OPTIONS="abort_on_error=0:detect_leaks=1", UBSAN_OPTIONS="halt_on_error=1",
               TSAN_OPTIONS="halt_on_error=1:second_deadlock_stack=1")
    r = subprocess.run([path, *args], capture_output=True, text=True, timeout=timeout, env=env)
    assert r.returncode == 0, "%s failed (%d):\n%s\n%s" % (path, r.returncode, r.stdout[-3000:], r.stderr[-6000:])
    assert "Sanitizer" not in r.stderr, r.stderr[-6000:]
    return r.stdout


def test_host_code_under_address_and_undefined_behaviour_sanitizers():
    subprocess.run(["make", "-s", "-C", CPP, "san"], check=True)
    assert "PASS lane arithmetic" in _run(os.path.join(CPP, "san", "lane_test"))
    assert "ok" in _run(os.path.join(CPP, "san", "replay_test"))
    assert "ok" in _run(os.path.join(CPP, "san", "coalesce_test"))
    assert "ok" in _run(os.path.join(CPP, "san", "bind_test"))


def test_netmap_documents_and_datagrams_under_the_fuzzer():
    subprocess.run(["make", "-s", "-C", CPP, "san/netmap_fuzz"], check=True)
    out = _run(os.path.join(CPP, "san", "netmap_fuzz"), "1000000", timeout=600)
    assert "PASS fuzz: 1000000 inputs" in out
    # a second seed, shorter: the run above is not the only path through the mutator
    assert "PASS fuzz: 100000 inputs" in _run(os.path.join(CPP, "san", "netmap_fuzz"), "100000", "12345")


def test_threaded_host_code_under_thread_sanitizer():
    subprocess.run(["make", "-s", "-C", CPP, "tsan"], check=True)
    assert "ok" in _run(os.path.join(CPP, "tsan", "coalesce_test"))
    assert "ok" in _run(os.path.join(CPP, "tsan", "bind_test"))


def test_oracle_tests_against_the_sanitizer_build_of_the_oracle():
    subprocess.run(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "san"], check=True)
    libasan = subprocess.run(["gcc", "-print-file-name=libasan.so"], capture_output=True, text=True,
                             check=True).stdout.strip()
    assert os.path.isabs(libasan), "gcc has no libasan.so"
    # Python itself is not built with the sanitizer, so its runtime is preloaded (ahead of
    # whatever is preloaded already); Python's own leaks at exit are not the oracle's
    preload = libasan + (":" + os.environ["LD_PRELOAD"] if os.environ.get("LD_PRELOAD") else "")
    env = dict(os.environ, LD_PRELOAD=preload, ASAN_OPTIONS="detect_leaks=0", UBSAN_OPTIONS="halt_on_error=1",
               BNK_ORACLE_SO=os.path.join(ROOT, "oracle", "san", "libbnkoracle.so"))
    tests = [os.path.join(HERE, "test_oracle_%s.py" % t) for t in ("aead", "filter", "relay", "wg")]
    r = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider", *tests],
                       capture_output=True, text=True, timeout=1500, env=env, cwd=ROOT)
    assert r.returncode == 0, r.stdout[-4000:] + r.stderr[-4000:]
    assert "Sanitizer" not in r.stderr and " passed" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
