#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

Headline workload (BASELINE.json `metric`): int8 qgemm with M = N = K = 4096,
int8 values uniform in [-127,127], per-channel weight scales uniform in
[0.001,0.05], int32 accumulation, fused f32 bias + requantisation to int8
(round-half-to-even, saturate).  One "step" is one such GEMM; inputs are resident
in HBM before the timed region.  Prints ONE JSON line.

Extra (same line, under "extra"): quantize / dequantize GB/s on a 1 GiB f32 tensor,
all five benchmark configurations next to the CPU oracle, and the ROCm library int8
GEMM as a yardstick.
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

def measured_traffic(size, kernel_name):
    """(bytes, note): what the L2s exchange with the memory side per launch of the headline
    kernel, from the record written next to the rocprofv3 --pmc summary of this command
    (profiles/qgemm_4096_requant_hbm_traffic.{md,json}: FETCH_SIZE and WRITE_SIZE in KiB per
    dispatch, each with the factor a kernel of known size reads under the same counter).
    Counters cannot be read from inside the run, so the figure is only reported when the record
    is for this size and for the kernel configuration the library picks now."""
    path = os.path.join(ROOT, "profiles", "qgemm_%d_requant_hbm_traffic.json" % size)
    if not os.path.exists(path):
        return None, "no counter record for this size under profiles/"
    with open(path) as f:
        rec = json.load(f)
    if rec.get("size") != size or rec.get("kernel") != kernel_name:
        return None, ("the counter record %s is for kernel %r, the library now picks %r: "
                      "re-measure" % (os.path.basename(path), rec.get("kernel"), kernel_name))
    byts = int((rec["fetch_size_kib_per_dispatch"] * rec["fetch_size_factor"]
                + rec["write_size_kib_per_dispatch"] * rec["write_size_factor"]) * 1024)
    return byts, ("recorded: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE passes over this command "
                  "(%s, kernel %s); counters cannot be read from inside the run"
                  % (rec.get("summary", path), rec.get("kernel_symbol", kernel_name)))


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    # After idling the GPU needs some tens of milliseconds of load before its clocks settle
    # (the first 300 launches of this 60 us kernel run 5-15 % slow): --prewarm-ms of the
    # same kernel run before the warm-up steps, untimed and reported separately.
    p.add_argument("--steps", type=int, default=400)
    p.add_argument("--warmup", type=int, default=50)
    p.add_argument("--prewarm-ms", type=float, default=50.0,
                   help="milliseconds of GPU time of the headline kernel before the warm-up "
                        "steps (0: none)")
    p.add_argument("--size", type=int, default=4096, help="M = N = K of the headline GEMM")
    p.add_argument("--workload", default="headline",
                   help="'headline' (default), or one parity-test configuration on its own, "
                        "e.g. for a profiler: 'gemm:MxKxN' (dynamic-M sweep shape, requant to "
                        "int8), 'conv:NAME' (NAME from baseline_configs.RESNET_CONVS), 'layer:NAME' (a layer of "
                        "the ResNet-50 sweep, HxHxCI_KxKxCO_sS), "
                        "'wo:MxKxN' (weight-only linear, f16 x uint8) or 'qlinear:MxKxN' "
                        "(quantize -> qgemm -> dequantize of f32 activations in one launch)")
    p.add_argument("--operands", choices=("config", "uniform", "ones", "zeros"), default="config",
                   help="with --workload gemm:MxKxN: the operand bytes -- the benchmark "
                        "configuration's quantized normals (default), uniform integers in "
                        "[-127,127], all ones or all zeros (the same instructions and traffic; "
                        "what differs is the switching power the data causes)")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    p.add_argument("--no-extra", action="store_true", help="skip the extras")
    p.add_argument("--no-two-stream", action="store_true",
                   help="skip the two-stream throughput leg (profiling runs: its overlapping "
                        "launches would blur per-kernel durations and counters)")
    p.add_argument("--extras", choices=("all", "qdq"), default="all",
                   help="'qdq': only the quantize / dequantize bandwidth cases (for profiling)")
    return p.parse_args()


def make_problem(torch, size):
    """BASELINE config 3 inputs."""
    from bladedisc_amd import baseline_configs as cfg
    c = cfg.config3(size)
    return c["a_q"], c["w_q"], c["sx"], c["sw"], c["so"], c["bias_q"]


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
                     0, 0, 0, None, 0)
        self.stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def __call__(self):
        st = self.L.dq8_qgemm(*self.args, self.stream)
        if st != 0:
            raise RuntimeError(self.L.dq8_last_error().decode())


class Timing(float):
    """Seconds per pass: the median over the timed graph replays (the float itself), with
    the fastest replay kept beside it."""

    def __new__(cls, median, fastest):
        t = super().__new__(cls, median)
        t.fastest = fastest
        return t


def time_graph(torch, calls, launches=20, replays=7, warm_replays=3, warm_seconds=0.03):
    """GPU time per pass over `calls` (objects with a .stream attribute and __call__)
    with the launches captured into a HIP graph, so that short kernels are timed back to
    back instead of at the rate Python can launch them.  The graph is first replayed untimed,
    at least warm_replays times and for at least warm_seconds (the first replays after capture
    upload the graph and, after idle, run at a lower clock: a single timed batch that includes
    them has read up to ten times too long for the shortest kernels, and 10-15 % too long for
    the long ones), then `replays` times with an event pair around each;
    returns the median as a Timing, the fastest replay in .fastest."""
    side = torch.cuda.Stream()
    saved = [c.stream for c in calls]
    graph = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.graph(graph, stream=side):
            handle = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            for c in calls:
                c.stream = handle
            for _ in range(launches):
                for c in calls:
                    c()
    finally:
        for c, st in zip(calls, saved):
            c.stream = st
    # warm: at least warm_replays replays and at least warm_seconds of GPU time (the CPU legs
    # between two measurements leave the GPU idle long enough for its clocks to drop)
    warm_t, warm_n = 0.0, 0
    while warm_n < max(3, warm_replays) or warm_t < warm_seconds:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(3):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        warm_t += e0.elapsed_time(e1) * 1e-3
        warm_n += 3
    times = []
    for _ in range(max(5, replays)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) * 1e-3 / launches)
    times.sort()
    return Timing(times[len(times) // 2], times[0])


def prewarm(torch, fn, min_seconds=0.05):
    """Runs fn back to back until at least min_seconds of GPU time have gone by: after
    idling, the clocks need some tens of milliseconds of load to settle.  Untimed work,
    reported separately from the warm-up steps.  Returns (launches, seconds)."""
    launches, total = 0, 0.0
    while total < min_seconds:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(100):
            fn()
        e1.record()
        torch.cuda.synchronize()
        launches += 100
        total += e0.elapsed_time(e1) * 1e-3
    return launches, total


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


class FnCall:
    """Adapter so that time_graph can drive any launcher that uses torch's current
    stream."""
    stream = None

    def __init__(self, fn):
        self.fn = fn

    def __call__(self):
        self.fn()


def cpu_time(fn, min_time=0.3, max_reps=10, min_reps=5):
    """Best wall time of fn over a few repetitions (at least min_reps, and at least
    min_time in total unless max_reps comes first); the minimum filters the scheduler
    stalls of a shared host."""
    fn()
    best, total, reps = float("inf"), 0.0, 0
    while reps < max_reps and (total < min_time or reps < min_reps):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best, total, reps = min(best, dt), total + dt, reps + 1
    return best


def roof(ops, byts, seconds):
    """TOP/s, GB/s and the larger of the two roofline fractions."""
    tops, gbps = ops / seconds / 1e12, byts / seconds / 1e9
    r = {"us": round(seconds * 1e6, 2), "TOPS": round(tops, 2), "GB/s": round(gbps, 1),
         "roofline_frac": round(max(tops / PEAK_INT8_TOPS, gbps / PEAK_HBM_GBPS), 4)}
    if isinstance(seconds, Timing):
        r["us_fastest_replay"] = round(seconds.fastest * 1e6, 2)
    return r


def config_reports(torch, K):
    """All five benchmark configurations: GPU time of the quantized operators (launches
    captured in a HIP graph, inputs resident) next to the CPU oracle on the host cores.
    Parity of exactly these inputs is what tests/test_gpu_configs.py checks."""
    import numpy as np
    import oracle as O
    from bladedisc_amd import baseline_configs as cfg
    dev = lambda v: torch.from_numpy(np.ascontiguousarray(v)).cuda()  # noqa: E731
    f1 = lambda v: dev(np.array([v], np.float32))                     # noqa: E731
    z1 = torch.zeros(1, dtype=torch.int32, device="cuda")
    rep = {}

    # ---- 1: single quantized linear, f32 in -> f32 out
    c = cfg.config1()
    x, wq, bias = dev(c["x"]), dev(c["w_q"]), dev(c["bias"])
    sx, sw, so = f1(c["sx"]), dev(c["sw"]), f1(c["so"])
    xq = torch.empty((64, 768), dtype=torch.int8, device="cuda")
    yq = torch.empty((64, 768), dtype=torch.int8, device="cuda")
    y = torch.empty((64, 768), device="cuda")
    chain = [FnCall(lambda: K.quantize(x, sx, z1, out=xq)),
             FnCall(lambda: K.qgemm(xq, wq, K.EPI_REQUANT_CPU, sx=sx, sw=sw, so=so, bias=bias, out=yq)),
             FnCall(lambda: K.dequantize(yq, so, z1, out=y))]
    gpu_s = time_graph(torch, chain)
    # the same with the trailing dequantize done in the GEMM's epilogue (bit-identical f32)
    fused = [chain[0],
             FnCall(lambda: K.qgemm(xq, wq, K.EPI_REQUANT_CPU_DEQUANT_F32, sx=sx, sw=sw, so=so,
                                    bias=bias, out=y))]
    gpu_fused_s = time_graph(torch, fused)
    # the whole chain as one launch: the activations are quantized on their way into the
    # matrix cores (dq8_qlinear_f32), the dequantize runs in the epilogue (bit-identical f32)
    one = [FnCall(lambda: K.qlinear_f32(x, wq, K.EPI_REQUANT_CPU_DEQUANT_F32, sx, sw, so,
                                        bias=bias, out=y))]
    gpu_one_s = time_graph(torch, one)

    def cpu1():
        q = O.quantize(c["x"], c["sx"], 0)
        acc, _ = O.gemm_s32_fast(q, c["w_q"])
        b32 = O.bias_f32_to_s32(c["bias"], float(c["sx"]), c["sw"])
        O.dequantize(O.requant_cpu(acc, float(c["sx"]), c["sw"], float(c["so"]), b32=b32), c["so"], 0)
    cpu_s = cpu_time(cpu1)
    rep["1_single_linear_64x768x768_q_gemm_dq"] = {
        "gpu_us": round(gpu_s * 1e6, 2), "cpu_us": round(cpu_s * 1e6, 1),
        "gpu_over_cpu": round(cpu_s / gpu_s, 1),
        "gpu_us_dequantize_in_epilogue": round(gpu_fused_s * 1e6, 2),
        "gpu_us_one_launch": round(gpu_one_s * 1e6, 2),
        "gpu_one_launch_over_cpu": round(cpu_s / gpu_one_s, 1)}

    # ---- 2: dynamic-M sweep, E1 requant, int8 out
    sweep = {}
    for (k, n) in cfg.BERT_LINEARS:
        for m in cfg.SWEEP_M:
            c = cfg.config2(m, k, n)
            a, w = dev(c["a_q"]), dev(c["w_q"])
            sx, sw, so = f1(c["sx"]), dev(c["sw"]), f1(c["so"])
            o = torch.empty((m, n), dtype=torch.int8, device="cuda")
            call = GemmCall(torch, a, w, sx, sw, so, None, 1, 0, o)
            gpu_s = time_graph(torch, [call])

            def cpu2():
                acc, _ = O.gemm_s32_fast(c["a_q"], c["w_q"])
                O.requant_cpu(acc, float(c["sx"]), c["sw"], float(c["so"]))
            cpu_s = cpu_time(cpu2, min_time=0.05, max_reps=8)
            r = roof(2.0 * m * n * k, m * k + n * k + m * n + 4 * n, gpu_s)
            r["cpu_us"] = round(cpu_s * 1e6, 1)
            sweep["M%d_K%d_N%d" % (m, k, n)] = r
    rep["2_dynamic_m_sweep_requant"] = sweep

    # ---- 3: 8192^3 next to the headline 4096^3
    c = cfg.config3(8192)
    a, w = dev(c["a_q"]), dev(c["w_q"])
    o = torch.empty((8192, 8192), dtype=torch.int8, device="cuda")
    call = GemmCall(torch, a, w, f1(c["sx"]), dev(c["sw"]), f1(c["so"]), dev(c["bias_q"]), 2, 2, o)
    # (as for the headline, the clocks settle over the first few dozen launches after idle:
    # 460 us for the first ones, 425-435 us from then on)
    _, ev = time_steps(torch, call, 40, 40)
    r = roof(2.0 * 8192 ** 3, 3 * 8192 ** 2 + 8 * 8192, ev / 40)

    def cpu3():
        acc, _ = O.gemm_s32_fast(c["a_q"], c["w_q"])
        O.requant_gpu(acc, c["sx"], c["sw"], c["so"], bias_f32=c["bias_q"])
    r["cpu_us"] = round(cpu_time(cpu3, min_time=0.0, max_reps=2, min_reps=2) * 1e6, 1)
    rep["3_large_square_8192_fused_bias_requant"] = r
    del a, w, o, call

    # ---- 4: int8 NHWC convolutions
    convs = {}
    for conv in cfg.RESNET_CONVS:
        c = cfg.config4(conv)
        nb, h, w_, ci, co, k = (conv[t] for t in ("nb", "h", "w", "ci", "co", "k"))
        pad4, md, osh = O.conv_attrs((nb, h, w_, ci), (co, k, k, ci), "NHWC", [1, 1, 1, 1],
                                     [1, 1, 1, 1], "EXPLICIT",
                                     explicit_paddings=[0, 0, conv["pad"], conv["pad"],
                                                        conv["pad"], conv["pad"], 0, 0])
        md[:12] = O.NHWC_OHWI_METADATA
        xq, wq = dev(c["x_q"]), dev(c["w_q"])
        sx, sw, so = f1(c["sx"]), dev(c["sw"]), f1(c["so"])
        o = torch.empty(tuple(osh), dtype=torch.int8, device="cuda")
        gpu_s = time_graph(torch, [FnCall(lambda: K.qconv2d(xq, wq, pad4, md, osh, K.EPI_REQUANT_CPU,
                                                            sx=sx, sw=sw, so=so, out=o))])
        mg, kg = nb * osh[1] * osh[2], k * k * ci
        r = roof(2.0 * mg * co * kg, nb * h * w_ * ci + co * kg + mg * co + 4 * co, gpu_s)
        # CPU: the GEMM the convolution reduces to (im2col done beforehand, not timed)
        cols = np.ascontiguousarray(np.lib.stride_tricks.sliding_window_view(
            np.pad(c["x_q"], ((0, 0), (conv["pad"],) * 2, (conv["pad"],) * 2, (0, 0))),
            (k, k), axis=(1, 2)).transpose(0, 1, 2, 4, 5, 3).reshape(mg, kg))
        wmat = c["w_q"].reshape(co, kg)

        def cpu4():
            acc, _ = O.gemm_s32_fast(cols, wmat)
            O.requant_cpu(acc, float(c["sx"]), c["sw"], float(c["so"]))
        r["cpu_us"] = round(cpu_time(cpu4, min_time=0.05, max_reps=8) * 1e6, 1)
        r["cpu_note"] = "int8 GEMM of the pre-built im2col matrix + requant"
        convs[conv["name"]] = r
        del cols
    rep["4_resnet_convs_requant"] = convs

    # ---- 4b: every distinct convolution of ResNet-50 at batch 32 (GPU only; operands drawn as
    # in config 4: activations max(N(0, 1), 0), weights N(0, 1) per output channel, both
    # quantized symmetrically to their maximum.  Uniform random bytes, which toggle far more
    # bits, run up to a third slower under sustained load: the clocks drop)
    sweep = {}
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4)
    for h, ci, co, k, stride, pad in cfg.RESNET50_LAYERS:
        ho = (h + 2 * pad - k) // stride + 1
        xf = torch.randn((32, h, h, ci), device="cuda", generator=gen).clamp_min_(0)
        xq = torch.round(xf * (127.0 / xf.max())).to(torch.int8)
        wf = torch.randn((co, k, k, ci), device="cuda", generator=gen)
        wq = torch.round(wf * (127.0 / wf.abs().amax(dim=(1, 2, 3), keepdim=True))).to(torch.int8)
        del xf, wf
        md = list(O.NHWC_OHWI_METADATA) + [stride, stride, 1, 1, 1]
        osh = [32, ho, ho, co]
        sx, so = f1(0.02), f1(20.0)
        sw = torch.rand(co, device="cuda", generator=gen) * 0.049 + 0.001
        o = torch.empty(tuple(osh), dtype=torch.int8, device="cuda")
        gpu_s = time_graph(torch, [FnCall(lambda: K.qconv2d(xq, wq, [pad] * 4, md, osh, K.EPI_REQUANT_CPU,
                                                            sx=sx, sw=sw, so=so, out=o))])
        sweep["%dx%dx%d_%dx%dx%d_s%d" % (h, h, ci, k, k, co, stride)] = roof(
            2.0 * 32 * ho * ho * co * k * k * ci, xq.numel() + wq.numel() + o.numel() + 4 * co, gpu_s)
        del xq, wq, o
    rep["4b_resnet50_layers_batch32_requant"] = sweep

    # ---- 5: quantized BERT-base encoder layer, batch 8
    from bladedisc_amd import bert_layer as B
    weights = cfg.config5_weights()
    layer = B.QuantBertLayer(weights, B.RawBackend())
    bert = {}
    for seq in cfg.BERT_SEQ_LENS:
        h = layer.embed(cfg.config5_tokens(8, seq))
        layer.calibrate(h)
        rec = {}
        layer.forward(h, rec)
        torch.cuda.synchronize()
        per, gpu_sum, cpu_sum = {}, 0.0, 0.0
        for name in B.LINEARS:
            r = rec[name]
            xin, xq, yq, yf = r["x"].contiguous(), r["x_q"], r["y_q"], r["y"]
            sx, sw, so = layer.s_in[name], layer.sw[name], layer.s_out[name]
            wq, bias = layer.w_q[name], layer.bias[name]
            chain = [FnCall(lambda: K.quantize(xin, sx, z1, out=xq)),
                     FnCall(lambda: K.qgemm(xq, wq, K.EPI_REQUANT_CPU, sx=sx, sw=sw, so=so,
                                            bias=bias, out=yq)),
                     FnCall(lambda: K.dequantize(yq, so, z1, out=yf))]
            gpu_s = time_graph(torch, chain)
            hx, hw, hb = xin.cpu().numpy(), wq.cpu().numpy(), layer.fb[name]
            fsx, fso, hsw = float(sx.cpu()[0]), float(so.cpu()[0]), sw.cpu().numpy()

            def cpu5():
                q = O.quantize(hx, fsx, 0)
                acc, _ = O.gemm_s32_fast(q, hw)
                b32 = O.bias_f32_to_s32(hb, fsx, hsw)
                O.dequantize(O.requant_cpu(acc, fsx, hsw, fso, b32=b32), fso, 0)
            cpu_s = cpu_time(cpu5, min_time=0.05, max_reps=8)
            m, kk = xin.shape
            n = wq.shape[0]
            per[name] = {"shape_MxKxN": [m, kk, n], "gpu_us": round(gpu_s * 1e6, 2),
                         "cpu_us": round(cpu_s * 1e6, 1)}
            gpu_sum += gpu_s
            cpu_sum += cpu_s
        # the whole layer (quantized operators + fp32 attention / LayerNorm / GELU in
        # PyTorch), eager launches from Python
        for _ in range(3):
            layer.forward(h)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            layer.forward(h)
        torch.cuda.synchronize()
        eager_us = (time.perf_counter() - t0) / 10 * 1e6
        # the same layer replayed from a HIP graph: as separate operators; with dequantize ->
        # GELU -> quantize between the FFN linears as one 256-entry table lookup on the int8
        # tensor; with each trailing dequantize done in its GEMM's epilogue as well; and with
        # the table and both residual additions in the epilogues too (all bit-identical)
        def replay_us(layer=layer, stream=None, **flags):
            saved = {k: getattr(layer, k) for k in flags}
            try:
                for k, v in flags.items():
                    setattr(layer, k, v)
                replay, _, _ = layer.capture(h, stream=stream)
                for _ in range(3):
                    replay()
                torch.cuda.synchronize()
                ts = []
                for _ in range(9):                   # median of batches of 4 replays
                    e0 = torch.cuda.Event(enable_timing=True)
                    e1 = torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(4):
                        replay()
                    e1.record()
                    torch.cuda.synchronize()
                    ts.append(e0.elapsed_time(e1) / 4)
                return round(sorted(ts)[len(ts) // 2] * 1e3, 1)
            except Exception as exc:  # capture is an optimisation, not the path under test
                return "capture failed: %s" % str(exc)[:100]
            finally:
                for k, v in saved.items():
                    setattr(layer, k, v)
        graph_us = replay_us()
        fused_us = replay_us(fuse_gelu=True)
        fused2_us = replay_us(fuse_gelu=True, fuse_dequant=True)
        fused3_us = replay_us(fuse_gelu=True, fuse_dequant=True, fuse_epilogue=True)
        # the same through the RAL entries (the plugin path): results from the context's pool,
        # the fused forms as ral_pdll_qgemm_fused
        from bladedisc_amd import ral
        rstream = torch.cuda.Stream()
        rctx = ral.RalContext(stream=rstream.cuda_stream)
        rex = rctx.execution()
        try:
            rlayer = B.QuantBertLayer(weights, B.RalBackend(rex))
            rlayer.calibrate(h)
            ral_graph_us = replay_us(layer=rlayer, stream=rstream)
            ral_fused3_us = replay_us(layer=rlayer, stream=rstream, fuse_gelu=True,
                                      fuse_dequant=True, fuse_epilogue=True)
        finally:
            torch.cuda.synchronize()
            rex.close()
            rctx.close()
        bert["seq%d" % seq] = {"linears_q_gemm_dq": per,
                               "quantized_ops_gpu_us": round(gpu_sum * 1e6, 2),
                               "quantized_ops_cpu_us": round(cpu_sum * 1e6, 1),
                               "layer_eager_wall_us": round(eager_us, 1),
                               "layer_graph_replay_us": graph_us,
                               "layer_graph_replay_fused_gelu_table_us": fused_us,
                               "layer_graph_replay_fused_gelu_table_and_dequantize_us": fused2_us,
                               "layer_graph_replay_fused_epilogues_us": fused3_us,
                               "layer_graph_replay_ral_entries_us": ral_graph_us,
                               "layer_graph_replay_ral_entries_fused_epilogues_us": ral_fused3_us}
    rep["5_bert_base_layer_batch8"] = bert
    return rep


def extras(torch, steps, warmup, which="all"):
    """q/dq bandwidth on a tensor larger than the 256 MB last-level cache, the five
    benchmark configurations against the CPU oracle, and a library yardstick."""
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
    # calibration statistic (running min / max): 4 bytes read per element
    lo1, hi1 = torch.full((1,), float("inf"), device="cuda"), torch.full((1,), float("-inf"), device="cuda")
    loc, hic = torch.full((cols,), float("inf"), device="cuda"), torch.full((cols,), float("-inf"), device="cuda")
    lor, hir = torch.full((rows,), float("inf"), device="cuda"), torch.full((rows,), float("-inf"), device="cuda")
    ws = torch.empty(1 << 24, dtype=torch.uint8, device="cuda")
    for name, fn in (("minmax_per_tensor", lambda: K.minmax(x, lo1, hi1, workspace=ws)),
                     ("minmax_per_channel_last_axis", lambda: K.minmax(x, loc, hic, axis=1, workspace=ws)),
                     ("minmax_per_channel_axis0", lambda: K.minmax(x, lor, hir, axis=0, workspace=ws))):
        _, ev = time_steps(torch, fn, reps, 3)
        gbps = 4.0 * rows * cols * reps / ev / 1e9
        out[name] = {"GB/s": round(gbps, 1), "frac_of_hbm_peak": round(gbps / PEAK_HBM_GBPS, 4),
                     "shape": [rows, cols], "bytes_per_elem": 4}
    # tf.QuantizeV2 / tf.Dequantize (mode SCALED), ranges as device operands; the wrappers
    # allocate their results, from torch's caching allocator after the first call
    from bladedisc_amd import tf_quant as TQ
    mn1, mx1 = torch.full((), -4.0, device="cuda"), torch.full((), 4.0, device="cuda")
    mnc, mxc = torch.full((cols,), -4.0, device="cuda"), torch.full((cols,), 4.0, device="cuda")
    tf_cases = (("tf_quantize_v2_scaled_per_tensor", lambda: TQ.quantize_v2(x, mn1, mx1, mode="SCALED")),
                ("tf_quantize_v2_scaled_last_axis", lambda: TQ.quantize_v2(x, mnc, mxc, mode="SCALED", axis=1)),
                ("tf_dequantize_scaled_per_tensor", lambda: TQ.dequantize(q, mn1, mx1, mode="SCALED")))
    for _, fn in tf_cases:
        for _ in range(3):
            fn()
    for name, fn in tf_cases:
        _, ev = time_steps(torch, fn, reps, 3)
        gbps = nbytes * reps / ev / 1e9
        out[name] = {"GB/s": round(gbps, 1), "frac_of_hbm_peak": round(gbps / PEAK_HBM_GBPS, 4),
                     "shape": [rows, cols], "bytes_per_elem": 5}
    # quantize -> dequantize in one pass: 4 bytes read + 4 written per element
    for _ in range(3):
        K.fake_quant(x, s1, z1, out=f)
    for name, fn in (("fake_quant_per_tensor", lambda: K.fake_quant(x, s1, z1, out=f)),
                     ("fake_quant_per_channel_last_axis", lambda: K.fake_quant(x, sc, zc, axis=1, out=f))):
        _, ev = time_steps(torch, fn, reps, 3)
        gbps = 8.0 * rows * cols * reps / ev / 1e9
        out[name] = {"GB/s": round(gbps, 1), "frac_of_hbm_peak": round(gbps / PEAK_HBM_GBPS, 4),
                     "shape": [rows, cols], "bytes_per_elem": 8}
    # 256-entry table over an int8 tensor: 1 byte read + 1 written per element
    table = torch.arange(256, dtype=torch.int16, device="cuda").to(torch.uint8).view(torch.int8)
    q2 = torch.empty_like(q)
    for _ in range(3):
        K.lut8(q, table, out=q2)
    _, ev = time_steps(torch, lambda: K.lut8(q, table, out=q2), reps, 3)
    gbps = 2.0 * rows * cols * reps / ev / 1e9
    out["lut8"] = {"GB/s": round(gbps, 1), "frac_of_hbm_peak": round(gbps / PEAK_HBM_GBPS, 4),
                   "shape": [rows, cols], "bytes_per_elem": 2}
    del x, q, f, q2
    # smaller activations (they fit the 256 MB last-level cache; launches captured in a graph)
    small = {}
    for shape in ((16, 768), (1000, 768), (4096, 768), (16384, 768), (32, 56, 56, 64),
                  (4096, 4096), (16384, 4096)):
        n = 1
        for d in shape:
            n *= d
        xs = torch.randn(shape, device="cuda")
        qs = torch.empty(shape, dtype=torch.int8, device="cuda")
        fs = torch.empty(shape, device="cuda")
        cs = torch.full((shape[-1],), 0.05, device="cuda")
        czs = torch.zeros(shape[-1], dtype=torch.int32, device="cuda")
        ax = len(shape) - 1
        row = {}
        for name, fn in (("q_tensor", lambda: K.quantize(xs, s1, z1, out=qs)),
                         ("dq_tensor", lambda: K.dequantize(qs, s1, z1, out=fs)),
                         ("q_last_axis", lambda: K.quantize(xs, cs, czs, axis=ax, out=qs)),
                         ("dq_last_axis", lambda: K.dequantize(qs, cs, czs, axis=ax, out=fs))):
            t = time_graph(torch, [FnCall(fn)], launches=20, replays=5)
            row[name] = {"us": round(t * 1e6, 2), "GB/s": round(5.0 * n / t / 1e9, 1)}
        small["x".join(str(d) for d in shape)] = row
    out["quantize_dequantize_shapes"] = small
    if which == "qdq":
        return out
    # weight-only quantized linear (f16 activations x uint8 weights, per-channel scale and zero
    # point): bound by the weight bytes for small M, by the f16 matrix cores (2.5 PFLOP/s) above
    wo = {}
    for (k, n, ms) in ((768, 3072, (1, 16, 128, 1024, 4096)), (4096, 4096, (1, 16, 64, 128, 1024, 4096)),
                       (8192, 8192, (1, 16, 64))):
        wq = torch.randint(0, 256, (n, k), dtype=torch.uint8, device="cuda")
        sc = (torch.rand(n, device="cuda") * 0.02 + 0.002).half()
        zp = torch.full((n,), 128, dtype=torch.int32, device="cuda")
        for m in ms:
            xh = torch.randn((m, k), device="cuda").half()
            oh = torch.empty((m, n), dtype=torch.float16, device="cuda")
            t = time_graph(torch, [FnCall(lambda: K.weight_only_qgemm(xh, wq, sc, zp, out=oh))])
            byts, flops = 2.0 * m * k + n * k + 2.0 * m * n + 6.0 * n, 2.0 * m * n * k
            wo["M%d_K%d_N%d" % (m, k, n)] = {
                "us": round(t * 1e6, 2), "us_fastest_replay": round(t.fastest * 1e6, 2),
                "GB/s": round(byts / t / 1e9, 1), "TFLOP/s": round(flops / t / 1e12, 1),
                "roofline_frac": round(max(byts / t / 1e9 / PEAK_HBM_GBPS,
                                           flops / t / 1e12 / 2500.0), 4)}
    out["weight_only_qgemm_f16_u8"] = wo
    # the same with f32 activations, the type of the reference's own test of the pattern: they
    # enter the f16 matrix cores as hi + lo halves, twice the MFMAs (the fraction is of the
    # nominal flops against the f16 peak)
    wo32 = {}
    k, n = 4096, 4096
    wq = torch.randint(0, 256, (n, k), dtype=torch.uint8, device="cuda")
    sc = torch.rand(n, device="cuda") * 0.02 + 0.002
    zp = torch.full((n,), 128, dtype=torch.int32, device="cuda")
    for m in (16, 128, 4096):
        xf = torch.randn((m, k), device="cuda")
        of = torch.empty((m, n), dtype=torch.float32, device="cuda")
        t = time_graph(torch, [FnCall(lambda: K.weight_only_qgemm(xf, wq, sc, zp, out=of))])
        byts, flops = 4.0 * m * k + n * k + 4.0 * m * n + 8.0 * n, 2.0 * m * n * k
        wo32["M%d_K%d_N%d" % (m, k, n)] = {
            "us": round(t * 1e6, 2), "us_fastest_replay": round(t.fastest * 1e6, 2),
            "GB/s": round(byts / t / 1e9, 1), "TFLOP/s": round(flops / t / 1e12, 1),
            "roofline_frac": round(max(byts / t / 1e9 / PEAK_HBM_GBPS,
                                       flops / t / 1e12 / 2500.0), 4)}
    out["weight_only_qgemm_f32_u8"] = wo32
    out["configs"] = config_reports(torch, K)
    # yardstick: the ROCm library int8 GEMM behind torch._int_mm (int32 output, no
    # epilogue) on the headline shape and data distribution -- a library, not the reference
    try:
        a = torch.randint(-127, 128, (4096, 4096), dtype=torch.int8, device="cuda")
        w = torch.randint(-127, 128, (4096, 4096), dtype=torch.int8, device="cuda")
        wt = w.t()
        o32 = torch.empty((4096, 4096), dtype=torch.int32, device="cuda")
        call = GemmCall(torch, a, w, None, None, None, None, 0, 0, o32)
        # both warmed up to the GPU's steady clocks and timed alternately, best of two
        n = 200
        ev = ev2 = float("inf")
        for _ in range(2):
            ev = min(ev, time_steps(torch, lambda: torch._int_mm(a, wt), n, 300)[1])
            ev2 = min(ev2, time_steps(torch, call, n, 300)[1])
        out["rocm_library_int_mm_4096_s32"] = {
            "library_us": round(ev / n * 1e6, 2), "library_TOPS": round(2.0 * 4096 ** 3 / (ev / n) / 1e12, 1),
            "dq8_qgemm_acc_s32_us": round(ev2 / n * 1e6, 2),
            "dq8_qgemm_acc_s32_TOPS": round(2.0 * 4096 ** 3 / (ev2 / n) / 1e12, 1)}
    except Exception as exc:  # the yardstick is optional
        out["rocm_library_int_mm_4096_s32"] = {"error": str(exc)[:200]}
    return out


def two_stream(torch, args, ops, da, dw, dsx, dsw, dso, dbias, out):
    side = [torch.cuda.Stream(), torch.cuda.Stream()]
    out2 = torch.empty_like(out)
    calls2 = []
    for st, o in zip(side, (out, out2)):
        with torch.cuda.stream(st):
            calls2.append(GemmCall(torch, da, dw, dsx, dsw, dso, dbias, 2, 2, o))
    for i in range(2 * args.warmup):
        calls2[i % 2]()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        calls2[i % 2]()
    torch.cuda.synchronize()
    wall2 = time.perf_counter() - t0
    return {"value": round(ops * args.steps / wall2 / 1e12, 2), "unit": "TOPS",
            "ms_per_step": round(wall2 / args.steps * 1e3, 5),
            "note": "same GEMM, launches alternating over two HIP streams"}


def single_workload(torch, args):
    """One configuration of the dynamic-M sweep or one convolution, launched back to back on
    the current stream (pre-warm, warm-up steps, then exactly --steps timed launches): the
    command a profiler is attached to for these shapes.  Prints its own JSON line."""
    import numpy as np
    import oracle as O
    from bladedisc_amd import baseline_configs as cfg
    from bladedisc_amd import kernels as K
    dev = lambda v: torch.from_numpy(np.ascontiguousarray(v)).cuda()  # noqa: E731
    f1 = lambda v: dev(np.array([v], np.float32))                     # noqa: E731
    kind, _, what = args.workload.partition(":")
    if kind == "gemm":
        m, k, n = (int(v) for v in what.split("x"))
        c = cfg.config2(m, k, n)
        o = torch.empty((m, n), dtype=torch.int8, device="cuda")
        a_q, w_q = dev(c["a_q"]), dev(c["w_q"])
        if args.operands == "uniform":
            a_q = torch.randint(-127, 128, (m, k), dtype=torch.int8, device="cuda")
            w_q = torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda")
        elif args.operands in ("ones", "zeros"):
            fill = 1 if args.operands == "ones" else 0
            a_q = torch.full((m, k), fill, dtype=torch.int8, device="cuda")
            w_q = torch.full((n, k), fill, dtype=torch.int8, device="cuda")
        call = GemmCall(torch, a_q, w_q, f1(c["sx"]), dev(c["sw"]), f1(c["so"]), None, 1, 0, o)
        ops, byts = 2.0 * m * n * k, m * k + n * k + m * n + 4 * n
        name = "int8 qgemm M=%d K=%d N=%d, requant to int8 (E1), operands: %s" % (m, k, n, args.operands)
    elif kind == "conv":
        conv = {c["name"]: c for c in cfg.RESNET_CONVS}[what]
        c = cfg.config4(conv)
        nb, h, w_, ci, co, kk = (conv[t] for t in ("nb", "h", "w", "ci", "co", "k"))
        pad4, md, osh = O.conv_attrs((nb, h, w_, ci), (co, kk, kk, ci), "NHWC", [1, 1, 1, 1],
                                     [1, 1, 1, 1], "EXPLICIT",
                                     explicit_paddings=[0, 0, conv["pad"], conv["pad"],
                                                        conv["pad"], conv["pad"], 0, 0])
        md[:12] = O.NHWC_OHWI_METADATA
        xq, wq = dev(c["x_q"]), dev(c["w_q"])
        sx, sw, so = f1(c["sx"]), dev(c["sw"]), f1(c["so"])
        o = torch.empty(tuple(osh), dtype=torch.int8, device="cuda")
        call = lambda: K.qconv2d(xq, wq, pad4, md, osh, K.EPI_REQUANT_CPU, sx=sx, sw=sw,  # noqa: E731
                                 so=so, out=o)
        mg, kg = nb * osh[1] * osh[2], kk * kk * ci
        ops, byts = 2.0 * mg * co * kg, nb * h * w_ * ci + co * kg + mg * co + 4 * co
        name = "int8 NHWC conv %s, batch %d, requant to int8 (E1)" % (what, nb)
    elif kind == "layer":
        # one layer of the ResNet-50 sweep, named as in the report: HxHxCI_KxKxCO_sS
        names = {"%dx%dx%d_%dx%dx%d_s%d" % (h, h, ci, kk, kk, co, s_): (h, ci, co, kk, s_, pd)
                 for h, ci, co, kk, s_, pd in cfg.RESNET50_LAYERS}
        if what not in names:
            raise SystemExit("bench.py: --workload layer:NAME, NAME one of %s" % ", ".join(names))
        h, ci, co, kk, stride, pd = names[what]
        ho = (h + 2 * pd - kk) // stride + 1
        gen = torch.Generator(device="cuda")
        gen.manual_seed(4)
        xf = torch.randn((32, h, h, ci), device="cuda", generator=gen).clamp_min_(0)
        xq = torch.round(xf * (127.0 / xf.max())).to(torch.int8)
        wf = torch.randn((co, kk, kk, ci), device="cuda", generator=gen)
        wq = torch.round(wf * (127.0 / wf.abs().amax(dim=(1, 2, 3), keepdim=True))).to(torch.int8)
        md = list(O.NHWC_OHWI_METADATA) + [stride, stride, 1, 1, 1]
        osh = [32, ho, ho, co]
        sx, so = f1(0.02), f1(20.0)
        sw = torch.rand(co, device="cuda", generator=gen) * 0.049 + 0.001
        o = torch.empty(tuple(osh), dtype=torch.int8, device="cuda")
        call = lambda: K.qconv2d(xq, wq, [pd] * 4, md, osh, K.EPI_REQUANT_CPU, sx=sx, sw=sw,  # noqa: E731
                                 so=so, out=o)
        ops = 2.0 * 32 * ho * ho * co * kk * kk * ci
        byts = xq.numel() + wq.numel() + o.numel() + 4 * co
        name = "int8 NHWC conv %s (ResNet-50 sweep), batch 32, requant to int8 (E1)" % what
    elif kind == "wo":
        # weight-only quantized linear: f16 activations x uint8 weights [N,K]
        m, k, n = (int(v) for v in what.split("x"))
        wq = torch.randint(0, 256, (n, k), dtype=torch.uint8, device="cuda")
        sc = (torch.rand(n, device="cuda") * 0.02 + 0.002).half()
        zp = torch.full((n,), 128, dtype=torch.int32, device="cuda")
        xh = torch.randn((m, k), device="cuda").half()
        oh = torch.empty((m, n), dtype=torch.float16, device="cuda")
        call = lambda: K.weight_only_qgemm(xh, wq, sc, zp, out=oh)  # noqa: E731
        ops, byts = 2.0 * m * n * k, 2.0 * m * k + n * k + 2.0 * m * n + 6.0 * n
        name = "weight-only qgemm M=%d K=%d N=%d, f16 x uint8 (roofline against the f16 peak)" % (m, k, n)
    elif kind == "qlinear":
        # quantize -> qgemm (E1, f32 bias) -> dequantize of f32 activations as one launch
        m, k, n = (int(v) for v in what.split("x"))
        x = torch.randn((m, k), device="cuda")
        wq = torch.randint(-127, 128, (n, k), dtype=torch.int8, device="cuda")
        sx, so = f1(0.03), f1(0.5)
        sw = torch.rand(n, device="cuda") * 0.05 + 0.001
        bias = torch.randn(n, device="cuda")
        o = torch.empty((m, n), device="cuda")
        call = lambda: K.qlinear_f32(x, wq, K.EPI_REQUANT_CPU_DEQUANT_F32, sx, sw, so,  # noqa: E731
                                     bias=bias, out=o)
        ops, byts = 2.0 * m * n * k, 4.0 * m * k + n * k + 4.0 * m * n + 8 * n
        name = "quantized linear on f32 activations, one launch, M=%d K=%d N=%d" % (m, k, n)
    else:
        raise SystemExit("bench.py: unknown --workload %r" % args.workload)
    pre_launches, pre_s = prewarm(torch, call, args.prewarm_ms * 1e-3) if args.prewarm_ms > 0 \
        else (0, 0.0)
    wall, ev = time_steps(torch, call, args.steps, args.warmup)
    r = roof(ops, byts, ev / args.steps)
    if kind == "wo":      # f16 matrix cores: 2.5 PFLOP/s
        r["roofline_frac"] = round(max(r["TOPS"] / 2500.0, r["GB/s"] / PEAK_HBM_GBPS), 4)
    print(json.dumps({
        "metric": "int8 TOPS" if kind != "wo" else "f16 TFLOP/s", "value": round(ops * args.steps / wall / 1e12, 2), "unit": "TOPS",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 5),
        "prewarm": {"ms": round(pre_s * 1e3, 1), "launches": pre_launches},
        "higher_is_better": True, "dtype": "int8", "data": "synthetic",
        "config": {"workload": name},
        "roofline": {"bound": "mfma" if r["TOPS"] / PEAK_INT8_TOPS >= r["GB/s"] / PEAK_HBM_GBPS
                     else "hbm", "kernel_us": r["us"], "TOPS": r["TOPS"], "GB/s": r["GB/s"],
                     "frac": r["roofline_frac"], "ops_per_launch": ops,
                     "algorithmic_bytes": byts}}))


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
    if args.workload != "headline":
        single_workload(torch, args)
        return

    size = args.size
    a, w, sx, sw, so, bias_q = make_problem(torch, size)
    d = lambda v: torch.from_numpy(v).cuda()  # noqa: E731
    import numpy as np
    da, dw = d(a), d(w)
    dsx, dsw, dso = d(np.array([sx])), d(sw), d(np.array([so]))
    dbias = d(bias_q)
    out = torch.empty((size, size), dtype=torch.int8, device="cuda")
    # REQUANT_GPU epilogue (2) with an f32 bias (kind 2): out = sat8(rne(os[n]*acc + b[n]))
    call = GemmCall(torch, da, dw, dsx, dsw, dso, dbias, 2, 2, out)

    pre_launches, pre_s = prewarm(torch, call, args.prewarm_ms * 1e-3) if args.prewarm_ms > 0 \
        else (0, 0.0)
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

    from bladedisc_amd import _lib
    kernel_name = _lib.lib().dq8_qgemm_kernel_name(size, size, size, 1).decode()
    traffic, traffic_note = measured_traffic(size, kernel_name)

    result = {
        "metric": "int8 qgemm TOPS (M=%d,K=N=%d)" % (size, size),
        "value": round(tops, 2),
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "prewarm": {"ms": round(pre_s * 1e3, 1), "launches": pre_launches,
                    "note": "untimed launches of the same kernel before the warm-up steps, "
                            "until the clocks have settled"},
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
            "operand_values": "uniform integers in [-127,127]",
        },
        "roofline": {
            "bound": "mfma",
            "achieved": round(achieved, 2),
            "peak": PEAK_INT8_TOPS,
            "unit": "TOP/s",
            "frac": round(achieved / PEAK_INT8_TOPS, 4),
            "traffic": traffic,
            "traffic_source": traffic_note,
            "kernel": kernel_name,
            "algorithmic_bytes": 3 * size * size + 8 * size,
            "kernel_us": round(kernel_s * 1e6, 2),
            "ops_per_launch": ops,
        },
    }
    # Independent batches need not queue behind each other: with the launches alternating
    # over two streams (two output buffers) the tail of one GEMM (epilogue, write-back,
    # completion) overlaps the head of the next.  Reported next to the headline, which
    # stays the single-stream figure.
    if not args.no_two_stream:
        result["two_stream_throughput"] = two_stream(torch, args, ops, da, dw, dsx, dsw, dso, dbias, out)

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(a, w, sx, sw, so, bias_q)
    else:
        result["cpu_baseline"] = None
    if not args.no_extra:
        result["extra"] = extras(torch, args.steps, args.warmup, args.extras)
        # the second size BASELINE's roofline configuration names, next to the headline
        big = result["extra"].get("configs", {}).get("3_large_square_8192_fused_bias_requant")
        if big:
            result["headline_8192"] = {
                "metric": "int8 qgemm TOPS (M=8192,K=N=8192)", "value": big["TOPS"],
                "unit": "TOPS", "kernel_us": big["us"],
                "roofline": {"bound": "mfma", "achieved": big["TOPS"], "peak": PEAK_INT8_TOPS,
                             "unit": "TOP/s", "frac": round(big["TOPS"] / PEAK_INT8_TOPS, 4)},
                "kernel": _lib.lib().dq8_qgemm_kernel_name(8192, 8192, 8192, 1).decode()}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
