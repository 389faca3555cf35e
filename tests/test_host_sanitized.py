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
