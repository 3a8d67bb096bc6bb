"""AddressSanitizer + UndefinedBehaviorSanitizer runs of the code that executes on the host (CPU only, no GPU call):

* the CPU oracle (oracle/l2c.c): every operator and small models of every tensor-type mix in every arithmetic mode;
* the library's host-only arithmetic: the plan, stream offsets and typed-piece tables of the streaming decode kernel
  (csrc/k_flow.hip, host functions only; every table entry checked against the stream's bounds) and the synthetic-weight
  quantizers (csrc/synth.cpp).

The drivers under tests/sanitize/ are compiled here with the sanitizers (on the host side only for the HIP file) and
must exit 0 without a sanitizer report.  Device code is never run under a sanitizer."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "sanitize")


def _run(cmd, exe, tmp_path):
    r = subprocess.run(cmd, capture_output=True, text=True, cwd=ROOT)
    err = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l)
    assert r.returncode == 0, err
    r = subprocess.run([exe], capture_output=True, text=True, cwd=str(tmp_path),
                       env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1"))
    assert r.returncode == 0 and "silent" in r.stdout, r.stdout + r.stderr
    assert "ERROR: AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr


def test_oracle_under_sanitizers(tmp_path):
    gcc = shutil.which("gcc")
    if not gcc:
        pytest.skip("gcc not found")
    exe = str(tmp_path / "oracle_san")
    _run([gcc, "-std=c11", "-O1", "-g", "-fopenmp", "-ffp-contract=off", "-fsanitize=address,undefined",
          "-fno-sanitize-recover=all", "-static-libasan", os.path.join(SRC, "oracle_main.c"), "-o", exe, "-lm"], exe, tmp_path)


def test_host_arithmetic_under_sanitizers(tmp_path):
    hipcc = "/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else shutil.which("hipcc")
    if not hipcc:
        pytest.skip("hipcc not found")
    exe = str(tmp_path / "host_san")
    _run([hipcc, os.path.join(SRC, "host_main.hip"), "-o", exe, "-O1", "-g", "-std=c++17", "-ffp-contract=off",
          "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "llama2.jl_amd", "csrc"),
          "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
          "-Xarch_host", "-fno-sanitize-recover=all"], exe, tmp_path)
