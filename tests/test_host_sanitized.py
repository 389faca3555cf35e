"""The runtime's two byte-level parsers (custom-call attribute blobs, the constant-store
file) under AddressSanitizer and UndefinedBehaviorSanitizer on the host: a valid input, every
truncation of it and a few thousand seeded mutations must each be parsed or rejected, never
read out of bounds.  Driver: tests/native/host_parsers_fuzz.cc (host code only, built with
g++; no GPU, no HIP)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "bladedisc_amd", "csrc")


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_parsers_under_asan_ubsan(tmp_path):
    exe = str(tmp_path / "host_parsers_fuzz")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=all", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
           os.path.join(ROOT, "tests", "native", "host_parsers_fuzz.cc"),
           os.path.join(CSRC, "mlir", "ral", "context", "pdll_util.cc"),
           os.path.join(CSRC, "mlir", "ral", "ral_metadata.cc"), "-o", exe]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    scratch = tmp_path / "scratch"
    scratch.mkdir()
    run = subprocess.run([exe, str(scratch)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    assert run.stdout.strip().endswith("ok"), run.stdout + run.stderr


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_division_by_a_kernel_constant_matches_true_division(tmp_path):
    """The quotient the one-launch quantized linear forms from the scale's reciprocal and two
    fused multiply-adds (tests/native/div_by_constant_check.c restates it) against x / s: a
    strided sample of all x, every x around the rounding ties of the int8 result, 40 divisors."""
    exe = str(tmp_path / "div_by_constant_check")
    build = subprocess.run(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", "-o", exe,
                            os.path.join(ROOT, "tests", "native", "div_by_constant_check.c"), "-lm"],
                           capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([exe, "2053"], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0 and run.stdout.strip() == "ok", run.stdout + run.stderr
