"""The kernels' libm-level routines (ratchet_amd/csrc/rt_libm.h: tanhf, expm1f, expf, the bf16 rounding), compiled for
the host from the same text the GPU build uses and compared bit for bit with the C library, which is what the
reference's CPU executor calls (crates/ratchet-core/src/cpu/unary.rs:46-65).  No GPU needed."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_device_math_matches_the_c_library(tmp_path):
    exe = tmp_path / "device_math_check"
    subprocess.run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-fno-fast-math", "-I", os.path.join(ROOT, "ratchet_amd", "csrc"),
                    os.path.join(ROOT, "tests", "device_math_check.cpp"), "-o", str(exe), "-lm"], check=True)
    # every 101st float bit pattern (42 M inputs), every widened 16-bit value and the algorithms' breakpoints
    run = subprocess.run([str(exe), "101"], capture_output=True, text=True)
    assert run.returncode == 0, run.stdout + run.stderr
    fields = run.stdout.split()
    counts = dict(zip(fields[0::2], (int(v) for v in fields[1::2])))
    assert set(counts) == {"tanhf", "expm1f", "expf", "logf", "sinf", "cosf", "f2bf", "checked"}, run.stdout
    assert all(counts[k] == 0 for k in ("tanhf", "expm1f", "expf", "logf", "sinf", "cosf", "f2bf")), run.stdout
    assert counts["checked"] > 40_000_000
