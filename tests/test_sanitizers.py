"""The CPU-side C++ of this build under AddressSanitizer and UndefinedBehaviorSanitizer: the oracle (`make -C oracle asan`)
and the host mirror of ratchet's Tensor API (`ratchet_amd.build.build_host(sanitize=True)`) are rebuilt with
-fsanitize=address,undefined and the oracle, golden-vector and host-graph tests run once more against those builds, in a
child interpreter that has the sanitizer runtime loaded first.  GPU code is not involved (the sanitizers are host only).
"""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SUITES = ["tests/test_oracle_scalar.py", "tests/test_oracle_ops.py", "tests/test_oracle_16bit_stepwise.py", "tests/test_golden_vectors.py",
          "tests/test_host_graph.py"]


def _runtime(name):
    r = subprocess.run([os.environ.get("CXX", "g++"), "-print-file-name=" + name], capture_output=True, text=True)
    path = r.stdout.strip()
    return path if r.returncode == 0 and os.path.isabs(path) and os.path.exists(path) else None


def test_oracle_and_host_mirror_under_asan_and_ubsan():
    asan, ubsan = _runtime("libasan.so"), _runtime("libubsan.so")
    if not asan or not ubsan:
        pytest.skip("this compiler ships no shared sanitizer runtimes")
    sys.path.insert(0, ROOT)
    from ratchet_amd import build as hip_build

    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "asan"], check=True, capture_output=True)
    host_lib = hip_build.build_host(sanitize=True)
    env = dict(os.environ)
    env["RATCHET_ORACLE_LIB"] = os.path.join(ROOT, "oracle", "_asan", "libratchet_cpu_oracle.so")
    env["RATCHET_HOST_LIB"] = host_lib
    # the runtimes go in front of whatever is preloaded already; leaks are Python's own, the link-order check would
    # refuse a preloaded runtime, and torch / numpy pair allocators in ways ASan's new-delete check does not follow
    env["LD_PRELOAD"] = ":".join([asan, ubsan] + ([env["LD_PRELOAD"]] if env.get("LD_PRELOAD") else []))
    env["ASAN_OPTIONS"] = "detect_leaks=0:verify_asan_link_order=0:alloc_dealloc_mismatch=0:detect_odr_violation=0"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    probe = subprocess.run([sys.executable, "-c", "from oracle import cpu_oracle as o; import numpy as np; o.unary('neg', np.ones(4, np.float32))"],
                           cwd=ROOT, env=env, capture_output=True, text=True, timeout=300)
    if probe.returncode != 0 and "Sanitizer" not in probe.stderr and "runtime error" not in probe.stderr:
        pytest.skip("an interpreter with the sanitizer runtime preloaded does not start here: " + probe.stderr[-300:])
    r = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider"] + SUITES, cwd=ROOT, env=env,
                       capture_output=True, text=True, timeout=1500)
    report = r.stdout[-3000:] + r.stderr[-3000:]
    assert "ERROR: AddressSanitizer" not in report and "runtime error:" not in report, report
    assert r.returncode == 0, report
    assert " passed" in r.stdout
