#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

Headline workload (BASELINE.json `metric`): int8 qgemm with M = N = K = 4096,
int8 values uniform in [-127,127], per-channel weight scales uniform in
[0.001,0.05], int32 accumulation, fused f32 bias + requantisation to int8
(round-half-to-even, saturate).  One "step" is one such GEMM; inputs are resident
in HBM before the timed region.  Prints ONE JSON line.

Extra (same line, under "extra"): quantize / dequantize GB/s on a 1 GiB f32 tensor
and the other BASELINE configs at a glance.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA peak, 5.0 POP/s
PEAK_HBM_GBPS = 8000.0    # MI355X HBM3E, 8 TB/s

# Bytes the L2s exchange with the memory side per launch of the headline kernel, from
# two rocprofv3 --pmc passes over this script (FETCH_SIZE, WRITE_SIZE; summary and
# commands in profiles/qgemm_4096_requant_hbm_traffic.md).  Counters cannot be read
# from inside the run, so the figure is recorded here for the size it was measured on.
MEASURED_TRAFFIC_BYTES = {4096: (98924 + 16384) * 1024}


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--size", type=int, default=4096, help="M = N = K of the headline GEMM")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    p.add_argument("--no-extra", action="store_true", help="skip the q/dq and sweep extras")
    p.add_argument("--pattern", choices=("uniform", "ones"), default="uniform",
                   help="operand values: 'uniform' is the benchmark's definition (integers uniform "
                        "in [-127,127]); 'ones' is a diagnosis aid that shows how much of the time "
                        "is the power drawn by toggling operands (same instructions, same traffic)")
    p.add_argument("--copy-probe", action="store_true",
                   help="also launch one plain streaming kernel of known size before the timed "
                        "loop (dst = src + 1 over 1 GiB of int8: reads 1 GiB, writes 1 GiB), the "
                        "yardstick for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE")
    return p.parse_args()


def make_problem(torch, size, seed=1236):
    """BASELINE config 3 inputs (seed = 1234 + config index)."""
    import numpy as np
    rng = np.random.default_rng(seed)
    m = n = k = size
    a = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    sw = rng.uniform(0.001, 0.05, n).astype(np.float32)
    sx = np.float32(0.02)
    # std of an accumulator of K products of two uniform[-127,127] integers
    std_acc = np.sqrt(k) * (127.0 * 128.0 / 3.0)
    so = np.float32(float(sx) * float(sw.mean()) * std_acc / 40.0)
    bias_q = (rng.standard_normal(n) * 10.0).astype(np.float32)  # bias / s_o
    return a, w, sx, sw, so, bias_q


class GemmCall:
    """dq8_qgemm bound once with all arguments, so the timed loop is one ctypes call
    per step."""

    def __init__(self, torch, a, w, sx, sw, so, bias, epilogue, bias_kind, out):
        from bladedisc_amd import _lib
        self.L = _lib.lib()
        self._keep = (a, w, sx, sw, so, bias, out)
        m, k = a.shape
        n = w.shape[0]
        vp = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None  # noqa: E731
        cnt = lambda t: t.numel() if t is not None else 0  # noqa: E731
        self.args = (vp(a), k, vp(w), k, vp(out), n, m, n, k, 0, 1, epilogue, vp(bias),
                     bias_kind, vp(sx), cnt(sx), vp(sw), cnt(sw), vp(so), cnt(so),
                     0, 0, 0, None, 0, C.c_void_p(torch.cuda.current_stream().cuda_stream))

    def __call__(self):
        st = self.L.dq8_qgemm(*self.args)
        if st != 0:
            raise RuntimeError(self.L.dq8_last_error().decode())


def time_steps(torch, fn, steps, warmup):
    """Wall time of exactly `steps` calls between two device syncs, plus the HIP
    event time over the same region on the launch stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0), e0.elapsed_time(e1) * 1e-3


def cpu_baseline(a, w, sx, sw, so, bias_q, budget_s=12.0):
    """The oracle (the restatement of the reference's x86 path: int32 GEMM, then the
    fused requantisation) on the host cores.  The same problem is repeated until
    about budget_s seconds of CPU work have been timed; for problems that would take
    longer than that, the first rows only."""
    import oracle as O
    n, k = w.shape
    probe_rows = min(a.shape[0], 256)

    def run(rows):
        acc, threads = O.gemm_s32_fast(a[:rows], w)
        O.requant_gpu(acc, sx, sw, so, bias_f32=bias_q)
        return threads

    run(probe_rows)                       # warm the thread pool and the caches
    t0 = time.perf_counter()
    run(probe_rows)
    t_probe = max(time.perf_counter() - t0, 1e-6)
    rows = int(min(a.shape[0], max(probe_rows, probe_rows * budget_s / t_probe)))
    rows -= rows % 4
    reps, dt, threads = 0, 0.0, 1
    t0 = time.perf_counter()
    while reps == 0 or dt < budget_s:
        threads = run(rows)
        reps += 1
        dt = time.perf_counter() - t0
    tops = 2.0 * rows * n * k * reps / dt / 1e12
    return {"value": round(tops, 4), "unit": "TOPS", "cores": int(threads), "kind": "port",
            "sample": "%d repetitions of the first %d of %d rows of the same %dx%dx%d problem "
                      "(int32 GEMM + fused requant), %.1f s of CPU time on the wall clock"
                      % (reps, rows, a.shape[0], a.shape[0], n, k, dt)}


def extras(torch, steps, warmup):
    """q/dq bandwidth on a tensor larger than the 256 MB last-level cache, and a few
    BERT-shaped GEMMs (dynamic M)."""
    from bladedisc_amd import kernels as K
    out = {}
    rows, cols = 65536, 4096
    x = torch.randn((rows, cols), device="cuda")
    q = torch.empty((rows, cols), dtype=torch.int8, device="cuda")
    f = torch.empty((rows, cols), device="cuda")
    s1 = torch.full((1,), 0.05, device="cuda")
    z1 = torch.zeros(1, dtype=torch.int32, device="cuda")
    sc = torch.full((cols,), 0.05, device="cuda")
    zc = torch.zeros(cols, dtype=torch.int32, device="cuda")
    sr = torch.full((rows,), 0.05, device="cuda")
    zr = torch.zeros(rows, dtype=torch.int32, device="cuda")
    nbytes = 5.0 * rows * cols
    reps = max(5, min(steps, 20))
    cases = (
            ("quantize_per_tensor", lambda: K.quantize(x, s1, z1, out=q)),
            ("dequantize_per_tensor", lambda: K.dequantize(q, s1, z1, out=f)),
            ("quantize_per_channel_last_axis", lambda: K.quantize(x, sc, zc, axis=1, out=q)),
            ("dequantize_per_channel_last_axis", lambda: K.dequantize(q, sc, zc, axis=1, out=f)),
            ("quantize_per_channel_axis0", lambda: K.quantize(x, sr, zr, axis=0, out=q)),
            ("dequantize_per_channel_axis0", lambda: K.dequantize(q, sr, zr, axis=0, out=f)))
    for _ in range(10):
        for _, fn in cases:
            fn()
    for name, fn in cases:
        # (freshly allocated device memory is slow for its first passes, hence the
        # warm-up rounds over all cases above)
        _, ev = time_steps(torch, fn, reps, 3)
        gbps = nbytes * reps / ev / 1e9
        out[name] = {"GB/s": round(gbps, 1), "frac_of_hbm_peak": round(gbps / PEAK_HBM_GBPS, 4),
                     "shape": [rows, cols], "bytes_per_elem": 5}
    del x, q, f
    sweep = {}
    for (m, n, k) in ((16, 768, 768), (128, 768, 768), (1000, 3072, 768), (4096, 768, 3072),
                      (16384, 768, 768)):
        a = torch.randint(-127, 128, (m, k), dtype=torch.int8, device="cuda")
        w = torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda")
        sx = torch.tensor([0.02], device="cuda")
        sw = torch.rand(n, device="cuda") * 0.049 + 0.001
        so = torch.tensor([20.0], device="cuda")
        o = torch.empty((m, n), dtype=torch.int8, device="cuda")
        call = GemmCall(torch, a, w, sx, sw, so, None, 1, 0, o)
        _, ev = time_steps(torch, call, 50, 5)
        us = ev / 50 * 1e6
        ops, byts = 2.0 * m * n * k, m * k + n * k + m * n + 4 * n
        sweep["%dx%dx%d" % (m, n, k)] = {
            "us": round(us, 2), "TOPS": round(ops / us / 1e6, 2),
            "GB/s": round(byts / us / 1e3, 1),
            "roofline_frac": round(max(ops / us / 1e6 / PEAK_INT8_TOPS,
                                       byts / us / 1e3 / PEAK_HBM_GBPS), 4)}
    out["qgemm_bert_shapes_requant_cpu"] = sweep
    # yardstick: the ROCm library int8 GEMM behind torch._int_mm (int32 output, no
    # epilogue) on the headline shape and data distribution -- a library, not the reference
    try:
        a = torch.randint(-127, 128, (4096, 4096), dtype=torch.int8, device="cuda")
        w = torch.randint(-127, 128, (4096, 4096), dtype=torch.int8, device="cuda")
        wt = w.t()
        _, ev = time_steps(torch, lambda: torch._int_mm(a, wt), 50, 5)
        o32 = torch.empty((4096, 4096), dtype=torch.int32, device="cuda")
        call = GemmCall(torch, a, w, None, None, None, None, 0, 0, o32)
        _, ev2 = time_steps(torch, call, 50, 5)
        out["rocm_library_int_mm_4096_s32"] = {
            "library_us": round(ev / 50 * 1e6, 2), "library_TOPS": round(2.0 * 4096 ** 3 / (ev / 50) / 1e12, 1),
            "dq8_qgemm_acc_s32_us": round(ev2 / 50 * 1e6, 2),
            "dq8_qgemm_acc_s32_TOPS": round(2.0 * 4096 ** 3 / (ev2 / 50) / 1e12, 1)}
    except Exception as exc:  # the yardstick is optional
        out["rocm_library_int_mm_4096_s32"] = {"error": str(exc)[:200]}
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); the hot path has no "
              "cross-GPU exchange to measure", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)

    size = args.size
    a, w, sx, sw, so, bias_q = make_problem(torch, size)
    if args.pattern == "ones":
        a[:] = 1
        w[:] = 1
    d = lambda v: torch.from_numpy(v).cuda()  # noqa: E731
    import numpy as np
    da, dw = d(a), d(w)
    dsx, dsw, dso = d(np.array([sx])), d(sw), d(np.array([so]))
    dbias = d(bias_q)
    out = torch.empty((size, size), dtype=torch.int8, device="cuda")
    # REQUANT_GPU epilogue (2) with an f32 bias (kind 2): out = sat8(rne(os[n]*acc + b[n]))
    call = GemmCall(torch, da, dw, dsx, dsw, dso, dbias, 2, 2, out)

    if args.copy_probe:
        src = torch.ones(1 << 30, dtype=torch.int8, device="cuda")
        dst = torch.empty_like(src)
        torch.add(src, 1, out=dst)
        torch.cuda.synchronize()
        del src, dst

    wall, ev = time_steps(torch, call, args.steps, args.warmup)
    ops = 2.0 * size * size * size
    ms_per_step = wall / args.steps * 1e3
    tops = ops * args.steps / wall / 1e12
    kernel_s = ev / args.steps
    achieved = ops / kernel_s / 1e12

    # saturated fraction of the output, reported with the number (degenerate scales
    # would make every parity check meaningless)
    o = out.cpu().numpy()
    sat_frac = float(((o == 127) | (o == -128)).mean())

    result = {
        "metric": "int8 qgemm TOPS (M=%d,K=N=%d)" % (size, size),
        "value": round(tops, 2),
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {
            "workload": "int8 qgemm M=N=K=%d: s8 x s8 -> s32, per-channel weight scales, fused "
                        "f32 bias + requant to s8 (round-half-even, saturate)" % size,
            "entry": "dq8_qgemm (C ABI), epilogue REQUANT_GPU",
            "saturated_fraction": round(sat_frac, 4),
            "operand_values": "uniform integers in [-127,127]" if args.pattern == "uniform"
                              else "all ones (diagnosis run, not the benchmark's data)",
        },
        "roofline": {
            "bound": "mfma",
            "achieved": round(achieved, 2),
            "peak": PEAK_INT8_TOPS,
            "unit": "TOP/s",
            "frac": round(achieved / PEAK_INT8_TOPS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(size) if args.pattern == "uniform" else None,
            "algorithmic_bytes": 3 * size * size + 8 * size,
            "kernel_us": round(kernel_s * 1e6, 2),
            "ops_per_launch": ops,
        },
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(a, w, sx, sw, so, bias_q)
    else:
        result["cpu_baseline"] = None
    if not args.no_extra:
        result["extra"] = extras(torch, args.steps, args.warmup)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
