"""Builds libdisc_q8_ral.so: the gfx950 kernels, their C ABI and the RAL runtime.

Everything is compiled in-tree with hipcc for gfx950 only (hipcc cross-compiles
without a GPU).  Usage: ``python -m bladedisc_amd.build [--force]``.
"""
import concurrent.futures
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(PKG, "build")
LIB = os.path.join(PKG, "libdisc_q8_ral.so")
# The same library plus the entry points of tests/dq8_test_hooks.h (kernel variant selection,
# the MFMA layout probe): what the tests and tuning scripts load when they force a variant.
# The product library carries none of them.
HOOKS_LIB = os.path.join(PKG, "libdisc_q8_testhooks.so")
HOOKS_SRC = os.path.join(CSRC, "kernels", "qgemm.hip")     # compiled a second time with the hooks
EXPORTS = os.path.join(CSRC, "exports.map")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: the requantisation epilogue and quantize are defined as
#   separately rounded binary32 operations.
# packed-fp32-ops disabled: never let the compiler form v_pk_*_f32.
COMMON = [
    "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-Wall", "-Wno-unused-function",
    # the LDS-load helper names m0 as clobbered, which is what it does; clang remarks that m0
    # is a reserved register
    "-Wno-inline-asm",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    "-I" + os.path.join(CSRC, "kernels"),
]
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
          "-packed-fp32-ops"]


def sources():
    """Sources of the library: everything under csrc."""
    out = []
    for d, _, files in os.walk(CSRC):
        for f in sorted(files):
            if f.endswith((".hip", ".cc")):
                out.append(os.path.join(d, f))
    return sorted(out)


def _headers_mtime():
    m = 0.0
    for base in (CSRC, os.path.join(ROOT, "include")):
        for d, _, files in os.walk(base):
            for f in files:
                if f.endswith(".h"):
                    m = max(m, os.path.getmtime(os.path.join(d, f)))
    return m


def _compile(src, force, hdr_m, hooks=False):
    rel = os.path.relpath(src, CSRC).replace(os.sep, "_")
    obj = os.path.join(OBJ, rel + (".hooks.o" if hooks else ".o"))
    if (not force and os.path.exists(obj)
            and os.path.getmtime(obj) > max(os.path.getmtime(src), hdr_m)):
        return obj, ""
    cmd = [HIPCC] + COMMON + DEVICE + (["-DDQ8_TEST_HOOKS"] if hooks else []) + \
        ["-Rpass-analysis=kernel-resource-usage", "-x", "hip", "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    lines = (r.stdout + r.stderr).splitlines()
    log = "\n".join(l for l in lines if "packed-fp32-ops" not in l and "remark:" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    _record_resources(obj, lines)
    return obj, log


def _record_resources(obj, lines):
    """Registers and scratch of every kernel in the object, from the compiler's resource remarks,
    as <obj>.resources.json (read by tests/test_build_resources.py: the kernels that are meant
    to keep everything in registers must not spill)."""
    import json
    import re
    kernels, name = {}, None
    for l in lines:
        m = re.search(r"remark: .*Function Name: (\S+)", l)
        if m:
            name = m.group(1)
            kernels[name] = {}
            continue
        if name is None:
            continue
        for key, pat in (("vgprs", r"VGPRs: (\d+)"), ("agprs", r"AGPRs: (\d+)"),
                         ("scratch_bytes_per_lane", r"ScratchSize \[bytes/lane\]: (\d+)"),
                         ("lds_bytes", r"LDS Size \[bytes/block\]: (\d+)")):
            m = re.search("remark: .* " + pat, l)
            if m:
                kernels[name][key] = int(m.group(1))
    with open(obj + ".resources.json", "w") as f:
        json.dump(kernels, f, indent=0, sort_keys=True)


def build_test_code_objects():
    """Device code objects the GPU tests hand to ral_kernel_launch (tests/programs/*.hip ->
    *.hsaco next to the source), as a compiled program would carry them."""
    progs = os.path.join(ROOT, "tests", "programs")
    built = []
    for f in sorted(os.listdir(progs)):
        if not f.endswith(".hip"):
            continue
        out = os.path.join(progs, f[:-4] + ".hsaco")
        cmd = [HIPCC, "-O3", "-std=c++17", "--genco"] + DEVICE + ["-o", out, os.path.join(progs, f)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (f, r.stdout + r.stderr))
        built.append(out)
    return built


def build(force=False, verbose=False, jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    hdr_m = _headers_mtime()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        hooks_job = ex.submit(_compile, HOOKS_SRC, force, hdr_m, True)
        results = list(ex.map(lambda s: _compile(s, force, hdr_m), srcs))
        hooks_obj, hooks_log = hooks_job.result()
    results.append((None, hooks_log))
    objs = [o for o, _ in results if o]
    if verbose:
        for _, log in results:
            if log.strip():
                print(log)
    newest = max(os.path.getmtime(o) for o in objs)
    newest = max(newest, os.path.getmtime(EXPORTS))
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < newest:
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950",
               "-Wl,--version-script=" + EXPORTS, "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    newest = max(newest, os.path.getmtime(hooks_obj))
    if force or not os.path.exists(HOOKS_LIB) or os.path.getmtime(HOOKS_LIB) < newest:
        plain = os.path.join(OBJ, os.path.relpath(HOOKS_SRC, CSRC).replace(os.sep, "_") + ".o")
        cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", HOOKS_LIB] + \
            [o for o in objs if o != plain] + [hooks_obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link of the test-hooks library failed:\n" + r.stdout + r.stderr)
    return LIB


if __name__ == "__main__":
    path = build(force="--force" in sys.argv, verbose=True)
    build_test_code_objects()
    print("built", path)
