"""The kernels that are written to keep their working set in registers must not spill: the
compiler's resource remarks, recorded per object by the build, say how much scratch memory a
lane of each kernel uses."""
import glob
import json
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
OBJ = os.path.join(ROOT, "bladedisc_amd", "build")

# mangled-name fragments of the kernels in question
NO_SPILL = ("qconv_stream_kernel", "qgemm_persist_kernel", "qgemm_skinny_kernel", "qlinear",
            "quantize", "dequantize", "lut_u8", "minmax")
# the 256 x 256 tile on four waves keeps 256 accumulators per lane and spills part of their
# indexing; it is a cross-check variant that the library never picks by itself
ALLOWED = ("qgemm_pipe_kernelILi256ELi256ELi2ELi2E", "qgemm_mfma_kernelILi256ELi256E")


def _demangle(names):
    out = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True).stdout
    return dict(zip(names, out.splitlines()))


def test_register_resident_kernels_do_not_spill():
    files = sorted(glob.glob(os.path.join(OBJ, "*.o.resources.json")))
    if not files:
        pytest.skip("no resource records: the library was not built here")
    seen, spilled = 0, []
    for f in files:
        for name, res in json.load(open(f)).items():
            if "scratch_bytes_per_lane" not in res:
                continue
            watched = any(k in name for k in NO_SPILL) or "qgemm_pipe_kernel" in name
            if not watched or any(a in name for a in ALLOWED):
                continue
            seen += 1
            if res["scratch_bytes_per_lane"] > 0:
                spilled.append((name, res))
    assert seen > 50, "too few kernels recorded (%d): are the records stale?" % seen
    if spilled:
        pretty = _demangle([n for n, _ in spilled])
        raise AssertionError("kernels with scratch memory:\n" + "\n".join(
            "  %s: %s" % (pretty.get(n, n), r) for n, r in spilled))
