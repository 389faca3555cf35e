"""GPU tests of the drop-in boundary: every quantized entry is called through
tao_ral_call_impl by its mangled name with compiler-style packed arguments and
compared bit-for-bit with the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    from bladedisc_amd import ral, ral_ops
    ctx = ral.RalContext(stream=torch.cuda.current_stream().cuda_stream)
    yield ctx, ral, ral_ops
    torch.cuda.synchronize()
    ctx.close()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def problem(seed, m, n, k):
    rng = np.random.default_rng(seed)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(a, w)
    sx = np.float32(rng.uniform(0.01, 0.03))
    sw = rng.uniform(0.001, 0.05, n).astype(np.float32)
    so = np.float32(np.std(acc * float(sx) * float(sw.mean())) / 40.0)
    return rng, a, w, acc, sx, sw, so


def f1(v):
    return dev(np.array([v], np.float32))


@pytest.mark.parametrize("m,n,k", [(64, 768, 768), (1000, 3072, 768), (7, 40, 48)])
def test_ral_qgemm_per_tensor_and_per_channel(rt, m, n, k):
    ctx, ral, ops = rt
    rng, a, w, acc, sx, sw, so = problem(m + n, m, n, k)
    with ctx.execution() as ex:
        got = ops.qgemm(ex, dev(a), dev(w), f1(sx), dev(sw), f1(so))
        np.testing.assert_array_equal(host(got), O.requant_cpu(acc, sx, sw, so))
        got = ops.qgemm(ex, dev(a), dev(w), f1(sx), f1(sw[0]), f1(so))
        np.testing.assert_array_equal(host(got), O.requant_cpu(acc, sx, sw[:1], so))
        # [K,N] weights (tp_b = false), as the CPU-style graphs pass them
        got = ops.qgemm(ex, dev(a), dev(w.T.copy()), f1(sx), dev(sw), f1(so), tp_b=False,
                        weight_is_const=False)   # per-call transpose through driver scratch
        np.testing.assert_array_equal(host(got), O.requant_cpu(acc, sx, sw, so))


def test_ral_qgemm_known_answer_gpu_case(rt, golden):
    """The reference's (disabled) GPU test: 32x64x128, expect 128.0 after dequantize."""
    ctx, ral, ops = rt
    case = golden["qgemm"][1]
    with ctx.execution() as ex:
        x = torch.full((case["m"], case["k"]), case["x"], device="cuda")
        z = torch.zeros(1, dtype=torch.int32, device="cuda")
        qx = ops.quantize(ex, x, f1(case["sx"]), z)
        w = torch.full((case["k"], case["n"]), case["w"], device="cuda")
        qw = ops.quantize(ex, w, f1(case["sw"]), z)
        out = ops.qgemm(ex, qx, qw, f1(case["sx"]), f1(case["sw"]), f1(case["so"]), tp_b=False)
        f = ops.dequantize(ex, out, f1(case["so"]), z)
        assert (host(f) == case["expect_f32"]).all()


@pytest.mark.parametrize("rank", [2, 3])
@pytest.mark.parametrize("bias_kind", ["s8", "f32"])
def test_ral_pdll_qgemm_gpu_signature(rt, rank, bias_kind):
    ctx, ral, ops = rt
    m, n, k = 96, 256, 320
    rng, a, w, acc, sx, sw, so = problem(rank * 10 + len(bias_kind), m, n, k)
    if bias_kind == "s8":
        bias = rng.integers(-128, 128, n).astype(np.int8)
        want = O.requant_gpu(acc, sx, sw[:1], so, bias_i8=bias)
    else:
        bias = (rng.standard_normal(n) * 10).astype(np.float32)
        want = O.requant_gpu(acc, sx, sw[:1], so, bias_f32=bias)
    x = a if rank == 2 else a.reshape(4, 24, k)
    with ctx.execution() as ex:
        got = ops.pdll_qgemm_gpu(ex, dev(x), dev(w), dev(bias), f1(sx), f1(sw[0]), f1(so))
        assert tuple(got.shape) == tuple(x.shape[:-1]) + (n,)
        np.testing.assert_array_equal(host(got).reshape(m, n), want)


def test_ral_pdll_qgemm_per_channel_merged_qkv(rt):
    """Three per-tensor linears sharing an input, merged into one per-channel call
    (disc_quantized_dot_merge.cc): equals the three separate results."""
    ctx, ral, ops = rt
    m, k, n1 = 128, 768, 768
    rng = np.random.default_rng(99)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    ws = [rng.integers(-128, 128, (n1, k), dtype=np.int8) for _ in range(3)]
    bs = [rng.integers(-128, 128, n1).astype(np.int8) for _ in range(3)]
    sx = np.float32(0.02)
    sws = [np.float32(s) for s in (0.011, 0.023, 0.017)]
    sos = [np.float32(s) for s in (18.0, 33.0, 25.0)]
    parts = []
    for w, b, sw, so in zip(ws, bs, sws, sos):
        acc, _ = O.gemm_s32_fast(a, w)
        parts.append(O.requant_gpu(acc, sx, sw, so, bias_i8=b))
    want = np.concatenate(parts, axis=1)
    w_cat = np.concatenate(ws, axis=0)
    b_cat = np.concatenate(bs)
    sx_n = np.full(3 * n1, sx, np.float32)
    sw_n = np.repeat(np.array(sws, np.float32), n1)
    so_n = np.repeat(np.array(sos, np.float32), n1)
    with ctx.execution() as ex:
        got = ops.pdll_qgemm_per_channel(ex, dev(a), dev(w_cat), dev(b_cat), dev(sx_n),
                                         dev(sw_n), dev(so_n))
        np.testing.assert_array_equal(host(got), want)


@pytest.mark.parametrize("bias_kind", ["none", "f32", "s32"])
@pytest.mark.parametrize("rank", [2, 4])
def test_ral_pdll_qgemm_cpu_style_signature(rt, bias_kind, rank):
    ctx, ral, ops = rt
    m, n, k = 64, 768, 768
    rng, a, w, acc, sx, sw, so = problem(len(bias_kind) + rank, m, n, k)
    bias = b32 = None
    if bias_kind == "f32":
        bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
        b32 = O.bias_f32_to_s32(bias, sx, sw)
    elif bias_kind == "s32":
        bias = b32 = rng.integers(-100000, 100000, n).astype(np.int32)
    want = O.requant_cpu(acc, sx, sw, so, b32=b32, zo=3)
    x = a if rank == 2 else a.reshape(2, 4, 8, k)
    w_kn = dev(w.T.copy())
    # constant weights are cached by address for the life of a context (as the
    # reference caches pre-packed weights), so this test owns its context
    ctx = ral.RalContext(stream=torch.cuda.current_stream().cuda_stream)
    with ctx.execution() as ex:
        for _ in range(2):   # second call hits the packed-weight cache
            got = ops.pdll_qgemm_cpu_style(ex, dev(x), w_kn, dev(bias) if bias is not None else None,
                                           f1(sx), dev(sw), f1(so), zo=3)
            np.testing.assert_array_equal(host(got).reshape(m, n), want)
        got = ops.pdll_qgemm_cpu_style(ex, dev(x), dev(w), dev(bias) if bias is not None else None,
                                       f1(sx), dev(sw), f1(so), zo=3, transpose_b=True)
        np.testing.assert_array_equal(host(got).reshape(m, n), want)
    torch.cuda.synchronize()
    ctx.close()


def test_ral_pdll_qgemm_cpu_style_zero_points(rt):
    """Asymmetric input (one zero point) and a uniform weight zero point through the
    CPU-signature entry: acc = sum (a - z_x)(w - z_w), the oneDNN semantics of the
    reference's CPU entries; a weight zero-point vector that is not uniform is refused."""
    ctx, ral, ops = rt
    m, n, k = 200, 768, 768
    rng = np.random.default_rng(91)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    sx = np.float32(0.02)
    sw = rng.uniform(0.001, 0.02, n).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.5).astype(np.float32)
    ctx = ral.RalContext(stream=torch.cuda.current_stream().cuda_stream)
    with ctx.execution() as ex:
        for zx, zw in ((17, 0), (-100, 4)):
            acc = O.gemm_s32(a, w, tp_b=True, zx=zx, zw=zw)
            so = np.float32(np.std(acc * (sx * sw.mean())) / 40)
            want = O.requant_cpu(acc, sx, sw, so, b32=O.bias_f32_to_s32(bias, sx, sw), zo=-6)
            got = ops.pdll_qgemm_cpu_style(ex, dev(a), dev(w), dev(bias), f1(sx), dev(sw), f1(so),
                                           zo=-6, transpose_b=True, zx=zx, zw=zw)
            np.testing.assert_array_equal(host(got), want)
            got = ops.pdll_qgemm_cpu_style(ex, dev(a), dev(w.T.copy()), dev(bias), f1(sx), dev(sw),
                                           f1(so), zo=-6, transpose_b=False, zx=zx, zw=zw)
            np.testing.assert_array_equal(host(got), want)
        zw_vec = np.zeros(n, np.int32)
        zw_vec[5] = 1
        with pytest.raises(ral.RalError, match="per-channel weight zero points"):
            ops.pdll_qgemm_cpu_style(ex, dev(a), dev(w), dev(bias), f1(sx), dev(sw), f1(np.float32(1)),
                                     transpose_b=True, zw=zw_vec)
    torch.cuda.synchronize()
    ctx.close()


def test_ral_pdll_qgemm_rejects_nonzero_input_zero_point(rt):
    ctx, ral, ops = rt
    with ctx.execution() as ex:
        a = ex.new_args()
        x = torch.zeros((4, 16), dtype=torch.int8, device="cuda")
        w = torch.zeros((8, 16), dtype=torch.int8, device="cuda")
        b = torch.zeros(8, dtype=torch.int8, device="cuda")
        s = torch.ones(1, device="cuda")
        a.tensor(x).tensor(w).tensor(b)
        a.tensor(s, rank0=True).host_array(np.array([5], np.int32), rank0=True)
        a.tensor(s, rank0=True).host_array(np.array([0], np.int32), rank0=True)
        a.tensor(s, rank0=True).host_array(np.array([0], np.int32), rank0=True)
        a.blob(ral.encode_attr({}))
        a.result_memref("i8", 2)
        with pytest.raises(ral.RalError, match="zero point"):
            ex.call("ral_pdll_qgemm", "gpu", a)


@pytest.mark.parametrize("rank", [2, 3])
@pytest.mark.parametrize("tp_b", [True, False])
def test_ral_pdll_qgemm_fused_and_qlinear(rt, rank, tp_b):
    """The fused entries (they have no counterpart among the reference's): each must give, bit
    for bit, what the separate entries give -- ral_pdll_qgemm then ral_dequantize [then an f32
    add and a clamp at zero], a table lookup on the int8 result, and ral_quantize ->
    ral_pdll_qgemm -> ral_dequantize for ral_pdll_qlinear, in its one-launch form (few rows) and
    its two-launch form (many).  (The weights here are torch tensors whose addresses torch hands
    out again, so they are not declared constants: a [K,N] weight is re-laid out per call.)"""
    ctx, ral, ops = rt
    from bladedisc_amd import kernels as K
    for m, n, k in ((48, 96, 256), (600, 768, 768)):
        rng, a, w, acc, sx, sw, so = problem(900 + m + rank, m, n, k)
        bias = rng.standard_normal(n).astype(np.float32)
        shape = (m,) if rank == 2 else (2, m // 2)
        xq = dev(a.reshape(*shape, k))
        wd = dev(w if tp_b else np.ascontiguousarray(w.T))
        z1 = dev(np.zeros(1, np.int32))
        with ctx.execution() as ex:
            base_q = ops.pdll_qgemm_cpu_style(ex, xq, wd, dev(bias), f1(sx), dev(sw), f1(so),
                                              transpose_b=tp_b, weight_is_const=False)
            want_q = O.requant_cpu(acc, sx, sw, so, b32=O.bias_f32_to_s32(bias, sx, sw))
            np.testing.assert_array_equal(host(base_q).reshape(m, n), want_q)
            base_f = ops.dequantize(ex, base_q, f1(so), z1)
            got = ops.pdll_qgemm_fused(ex, xq, wd, dev(bias), f1(sx), dev(sw), f1(so), transpose_b=tp_b, weight_is_const=False)
            assert got.dtype == torch.float32 and tuple(got.shape) == shape + (n,)
            np.testing.assert_array_equal(host(got), host(base_f))
            np.testing.assert_array_equal(host(got).reshape(m, n), O.dequantize(want_q, so, 0))
            resid = dev(rng.standard_normal(shape + (n,)).astype(np.float32))
            for relu in (False, True):
                got = ops.pdll_qgemm_fused(ex, xq, wd, dev(bias), f1(sx), dev(sw), f1(so),
                                           transpose_b=tp_b, weight_is_const=False, residual=resid, relu=relu)
                want = host(base_f) + host(resid)
                if relu:
                    want = np.where(want < 0, np.float32(0), want)
                np.testing.assert_array_equal(host(got), want)
            table = K.activation_table(torch.nn.functional.gelu, f1(so), z1, f1(np.float32(0.02)), z1)
            got = ops.pdll_qgemm_fused(ex, xq, wd, dev(bias), f1(sx), dev(sw), f1(so),
                                       transpose_b=tp_b, weight_is_const=False, table=table)
            assert got.dtype == torch.int8
            np.testing.assert_array_equal(host(got), host(K.lut8(base_q, table)))
            # quantize -> qgemm -> dequantize on f32 activations
            x = (a.astype(np.float32) * sx + rng.uniform(-0.4, 0.4, a.shape).astype(np.float32) * sx)
            x = x.reshape(*shape, k)
            xq2 = ops.quantize(ex, dev(x), f1(sx), z1)
            want2 = ops.dequantize(ex, ops.pdll_qgemm_cpu_style(ex, xq2, wd, dev(bias), f1(sx), dev(sw),
                                                                f1(so), transpose_b=tp_b, weight_is_const=False), f1(so), z1)
            got2 = ops.pdll_qlinear(ex, dev(x), wd, dev(bias), f1(sx), dev(sw), f1(so), transpose_b=tp_b, weight_is_const=False)
            np.testing.assert_array_equal(host(got2), host(want2))
            acc2 = O.gemm_s32(O.quantize(x.reshape(m, k), sx, 0), w, tp_b=True)
            ref2 = O.dequantize(O.requant_cpu(acc2, sx, sw, so, b32=O.bias_f32_to_s32(bias, sx, sw)), so, 0)
            np.testing.assert_array_equal(host(got2).reshape(m, n), ref2)


def _wo_tolerance(want, bound, k, dtype):
    return bound * (k * 2.0 ** -24 + 2.0 ** -20) + \
        (np.abs(want) + bound * 2.0 ** -12) * (2.0 ** -10 if dtype == torch.float16 else 2.0 ** -22)


def _persistent(ral, ex, a):
    """A device buffer from the context's alloc_persistent holding `a`: what ral_const hands a
    program for a constant."""
    a = np.ascontiguousarray(a)
    ptr = ex.alloc_persistent(a.nbytes)
    t = ral.device_view(ptr, a.shape, torch.uint8)
    t.copy_(torch.from_numpy(a))
    return t


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("with_bias,k,n", [(False, 96, 72), (True, 96, 72), (True, 1280, 200)])
def test_ral_pdll_weight_only_qgemm(rt, dtype, with_bias, k, n):
    """The weight-only entry by its mangled name, as the pattern calls it: rank-3 activations,
    uint8 weight [K,N] with zero points 128 (quant range 0..255), per-channel scale, optional
    bias.  The weight is a constant of the context (alloc_persistent), so its [N,K] copy is
    cached: a second call with other activations must agree too.  The deep case (80 rows,
    k = 1280) is one the f16 kernels split over k, with the partial sums in scratch from the
    context's pool.  Tolerance: the f32 accumulation bound of the kernel tests."""
    ctx, ral, ops = rt
    rng = np.random.default_rng(31 + int(with_bias) + k)
    npdt = np.float16 if dtype == torch.float16 else np.float32
    b, s = 2, 40
    w = rng.integers(0, 256, (n, k), dtype=np.uint8)
    zp = np.full(n, 128, np.int32)
    scale = rng.uniform(0.002, 0.02, n).astype(npdt)
    bias = rng.standard_normal(n).astype(npdt) if with_bias else None
    with ctx.execution() as ex:
        w_kn = _persistent(ral, ex, w.T)
        for rep in range(2):
            x = rng.standard_normal((b, s, k)).astype(npdt)
            got = ops.pdll_weight_only_qgemm(ex, dev(x), w_kn, dev(scale), dev(zp),
                                             dev(bias) if with_bias else None)
            assert got.dtype == dtype and tuple(got.shape) == (b, s, n)
            want, bound = O.weight_only_qgemm(x.reshape(-1, k), w, scale, zp, bias)
            err = np.abs(host(got).astype(np.float64).reshape(-1, n) - want)
            assert (err <= _wo_tolerance(want, bound, k, dtype)).all(), rep


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("m,k,n", [(80, 1280, 200), (3, 64, 4), (300, 256, 1024)])
def test_ral_pdll_weight_only_qgemm_takes_the_compiler_reordered_constant(rt, dtype, m, k, n):
    """What the unchanged compiler emits for a constant ui8 weight: the bytes permuted by its
    layout pass and `weight_should_be_reordered = false`
    (R tao_compiler/mlir/disc/transforms/disc_transform_weight_data_layout_for_weight_only_gemm.cc
    :362-410).  The result must be bit-identical to the plain [K,N] weight with the attribute
    true, cached (constant) or not."""
    from oracle import weight_layout_oracle as WL
    ctx, ral, ops = rt
    rng = np.random.default_rng(5 * m + k + n)
    npdt = np.float16 if dtype == torch.float16 else np.float32
    w_kn = rng.integers(0, 256, (k, n), dtype=np.uint8)
    reordered = WL.forward(w_kn)
    zp = rng.integers(100, 156, n).astype(np.int32)
    scale = rng.uniform(0.002, 0.02, n).astype(npdt)
    bias = rng.standard_normal(n).astype(npdt)
    x = dev(rng.standard_normal((1, m, k)).astype(npdt))
    with ctx.execution() as ex:
        plain_const = _persistent(ral, ex, w_kn)
        reordered_const = _persistent(ral, ex, reordered)
        args = (dev(scale), dev(zp), dev(bias))
        for rep in range(2):                                        # second call: from the cache
            got = host(ops.pdll_weight_only_qgemm(ex, x, reordered_const, *args, reorder=False))
            want = host(ops.pdll_weight_only_qgemm(ex, x, plain_const, *args, reorder=True))
            np.testing.assert_array_equal(got.view(np.uint8), want.view(np.uint8))
        # the same weight as the result of another operator (pool memory: not cached)
        want2 = host(ops.pdll_weight_only_qgemm(ex, x, dev(w_kn), *args, reorder=True))
        np.testing.assert_array_equal(want2.view(np.uint8), want.view(np.uint8))
        ref, bound = O.weight_only_qgemm(host(x).reshape(-1, k), np.ascontiguousarray(w_kn.T),
                                         scale, zp, bias)
        err = np.abs(got.astype(np.float64).reshape(-1, n) - ref)
        assert (err <= _wo_tolerance(ref, bound, k, dtype)).all()


def test_ral_pdll_weight_only_qgemm_reordered_shape_outside_the_pass_domain(rt):
    """K % 64 != 0 or N % 4 != 0: the compiler's pass indexes out of bounds there, so what it
    would leave is not a permutation of the weight; the entry says so."""
    ctx, ral, ops = rt
    with ctx.execution() as ex:
        x = torch.zeros((1, 4, 96), dtype=torch.float16, device="cuda")
        w = torch.zeros((96, 72), dtype=torch.uint8, device="cuda")
        sc = torch.ones(72, dtype=torch.float16, device="cuda")
        zp = torch.zeros(72, dtype=torch.int32, device="cuda")
        with pytest.raises(ral.RalError, match="K % 64 == 0"):
            ops.pdll_weight_only_qgemm(ex, x, w, sc, zp, None, reorder=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_ral_pdll_weight_only_qgemm_weight_that_is_not_a_constant(rt, dtype):
    """`weight_should_be_reordered = true` reaches the runtime exactly when the weight is not a
    constant the layout pass could match -- e.g. the result of an mhlo.transpose, in memory the
    allocator reuses.  Two same-shaped weights at one address, one after the other (the buffer
    rewritten in place, and a buffer freed to the context's pool and handed out again), must each
    give their own result."""
    ctx, ral, ops = rt
    rng = np.random.default_rng(77)
    npdt = np.float16 if dtype == torch.float16 else np.float32
    m, k, n = 48, 192, 136
    scale = dev(rng.uniform(0.002, 0.02, n).astype(npdt))
    zp = dev(np.full(n, 128, np.int32))
    x = rng.standard_normal((1, m, k)).astype(npdt)
    ws = [rng.integers(0, 256, (k, n), dtype=np.uint8) for _ in range(3)]

    def check(got, w_kn):
        want, bound = O.weight_only_qgemm(x.reshape(-1, k), np.ascontiguousarray(w_kn.T),
                                          host(scale), host(zp), None)
        err = np.abs(host(got).astype(np.float64).reshape(-1, n) - want)
        assert (err <= _wo_tolerance(want, bound, k, dtype)).all()

    with ctx.execution() as ex:
        buf = dev(ws[0])
        check(ops.pdll_weight_only_qgemm(ex, dev(x), buf, scale, zp), ws[0])
        buf.copy_(torch.from_numpy(ws[1]))                       # same address, new contents
        check(ops.pdll_weight_only_qgemm(ex, dev(x), buf, scale, zp), ws[1])
        # a pool buffer released and handed out again for the next layer's weight
        addrs = []
        for w_kn in ws[1:]:
            ptr = ex.alloc(k * n)
            addrs.append(ptr)
            t = ral.device_view(ptr, (k, n), torch.uint8)
            t.copy_(torch.from_numpy(w_kn))
            got = ops.pdll_weight_only_qgemm(ex, dev(x), t, scale, zp)
            check(got, w_kn)
            torch.cuda.synchronize()
            ex.dealloc(ptr)
        assert addrs[0] == addrs[1], "the pool was expected to hand the same buffer out again"


@pytest.mark.parametrize("nb,h,ci,co,k,stride,pad", [(2, 14, 64, 64, 3, 1, 1), (2, 7, 256, 128, 1, 1, 0),
                                                      (1, 9, 32, 16, 3, 2, 1), (2, 30, 3, 64, 7, 2, 3),
                                                      # 3 x 3 on 128 channels: 32-channel slices of
                                                      # the kernel that keeps the filter in registers
                                                      (3, 28, 128, 128, 3, 1, 1)])
def test_ral_qconv(rt, nb, h, ci, co, k, stride, pad):
    ctx, ral, ops = rt
    rng = np.random.default_rng(h + ci)
    x = rng.integers(-128, 128, (nb, h, h, ci), dtype=np.int8)
    w = rng.integers(-128, 128, (co, k, k, ci), dtype=np.int8)
    ho = (h + 2 * pad - k) // stride + 1
    md = list(O.NHWC_OHWI_METADATA) + [stride, stride, 1, 1, 1]
    padding = [pad] * 4
    acc = O.conv_s32(x, w, padding, md, [nb, ho, ho, co])
    sx = np.float32(0.02)
    sw = rng.uniform(0.001, 0.05, co).astype(np.float32)
    so = np.float32(np.std(acc * float(sx) * float(sw.mean())) / 40.0)
    want = O.requant_cpu(acc.reshape(-1, co), sx, sw, so).reshape(nb, ho, ho, co)
    out = torch.empty((nb, ho, ho, co), dtype=torch.int8, device="cuda")
    with ctx.execution() as ex:
        ops.qconv(ex, dev(x), dev(w), padding, md, f1(sx), dev(sw), f1(so), out)
        np.testing.assert_array_equal(host(out), want)
        # the older entry without zero-point operands gives the same bits
        out2 = torch.empty_like(out)
        ops.qconv_s8_s8_s8(ex, dev(x), dev(w), padding, md, f1(sx), dev(sw), f1(so), out2)
        np.testing.assert_array_equal(host(out2), want)


@pytest.mark.parametrize("fmt,padding,k,stride,dil", [("NHWC", "SAME", 3, 1, 1), ("NHWC", "VALID", 3, 2, 2),
                                                      ("NHWC", "SAME", 1, 1, 1), ("NCHW", "SAME", 3, 1, 1),
                                                      ("NHWC", "EXPLICIT", 3, 1, 1)])
def test_ral_pdll_qconv2d(rt, fmt, padding, k, stride, dil):
    ctx, ral, ops = rt
    rng = np.random.default_rng(k * 10 + stride + len(padding))
    nb, h, w_, ci, co = 2, 14, 12, 32, 48
    x = rng.integers(-128, 128, (nb, h, w_, ci) if fmt == "NHWC" else (nb, ci, h, w_), dtype=np.int8)
    wt = rng.integers(-128, 128, (co, k, k, ci), dtype=np.int8)
    explicit = [0, 0, 1, 2, 2, 0, 0, 0] if padding == "EXPLICIT" else []
    sp = [1, stride, stride, 1] if fmt == "NHWC" else [1, 1, stride, stride]
    dl = [1, dil, dil, 1] if fmt == "NHWC" else [1, 1, dil, dil]
    pad4, md, out_shape = O.conv_attrs(x.shape, wt.shape, fmt, sp, dl, padding,
                                       explicit_paddings=explicit)
    acc = O.conv_s32(x, wt, pad4, md, out_shape)
    sx = np.float32(0.02)
    sw = rng.uniform(0.001, 0.05, co).astype(np.float32)
    so = np.float32(np.std(acc * float(sx) * float(sw.mean())) / 40.0)
    ch_axis = 3 if fmt == "NHWC" else 1
    acc2 = np.ascontiguousarray(np.moveaxis(acc, ch_axis, -1))
    want = np.moveaxis(O.requant_cpu(acc2.reshape(-1, co), sx, sw, so, zo=3).reshape(acc2.shape),
                       -1, ch_axis)
    with ctx.execution() as ex:
        got = ops.pdll_qconv2d(ex, dev(x), dev(wt), f1(sx), dev(sw), f1(so), data_format=fmt,
                               strides=sp, dilations=dl, padding=padding,
                               explicit_paddings=explicit, zo=3)
        assert list(got.shape) == list(out_shape)
        np.testing.assert_array_equal(host(got), want)


@pytest.mark.parametrize("rank", [2, 3, 4])
@pytest.mark.parametrize("bias", [False, True])
def test_ral_pdll_qgemm_per_tensor_signature_uses_the_fixed_point_stage(rt, rank, bias):
    """The per-tensor ral_pdll_qgemm signatures exist in the reference only in the AArch64
    build, on Arm Compute Library's multiplier-and-shift output stage
    (common_context_impl_quantization.cc:747-1187, registered :1689-1695): mirrored on gpu
    with the same stage, bit-exact against its restatement; config 1 sizes."""
    if bias and rank == 4:
        pytest.skip("the reference registers the s32-bias form for ranks 2 and 3 only")
    ctx, ral, ops = rt
    rng = np.random.default_rng(40 + rank)
    lead = {2: (64,), 3: (4, 16), 4: (2, 2, 16)}[rank]
    k, n = 768, 768
    x = rng.integers(-128, 128, lead + (k,), dtype=np.int8)
    w_kn = rng.integers(-128, 128, (k, n), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(x.reshape(-1, k), np.ascontiguousarray(w_kn.T))
    sx, sw = np.float32(0.02), np.float32(0.011)
    so = np.float32(np.std(acc * float(sx) * float(sw)) / 40.0)
    b32 = rng.integers(-100000, 100000, n).astype(np.int32) if bias else None
    want = O.requant_fixedpoint(acc, sx, np.array([sw]), so, b32=b32, zo=2).reshape(lead + (n,))
    with ctx.execution() as ex:
        # (weight_is_const would let the context cache the repacked weight by its address,
        # and these test tensors come and go)
        got = ops.pdll_qgemm_per_tensor(ex, dev(x), dev(w_kn), dev(b32) if bias else None, f1(sx),
                                        f1(sw), f1(so), zo=2, weight_is_const=False)
        assert list(got.shape) == list(lead + (n,))
        np.testing.assert_array_equal(host(got), want)
    # a different rounding from the float stage of the per-channel signatures, one step at most
    flt = O.requant_cpu(acc, sx, np.array([sw]), so, b32=b32, zo=2).reshape(lead + (n,))
    assert np.max(np.abs(flt.astype(np.int32) - want.astype(np.int32))) <= 1


def test_shared_signatures_switch_to_the_fixed_point_stage(rt, monkeypatch):
    """ral_qgemm with per-channel weight scales, ral_qconv and ral_pdll_qconv2d have one
    signature and two CPU implementations in the reference (oneDNN's float post-ops on x86,
    Arm Compute Library's fixed-point stage on AArch64): DISC_GPU_REQUANT_FIXEDPOINT=1 selects
    the second here.  Known answers of the reference's AArch64 tests (12.0, 108.0) and seeded
    tensors against the oracle."""
    ctx, ral, ops = rt
    monkeypatch.setenv("DISC_GPU_REQUANT_FIXEDPOINT", "1")
    rng = np.random.default_rng(99)
    # -- ral_qgemm, per channel
    m, k, n = 100, 400, 136
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(a, w)
    sx = np.float32(0.02)
    sw = rng.uniform(0.001, 0.05, n).astype(np.float32)
    so = np.float32(np.std(acc * float(sx) * float(sw.mean())) / 40.0)
    with ctx.execution() as ex:
        got = ops.qgemm(ex, dev(a), dev(w), f1(sx), dev(sw), f1(so))
        np.testing.assert_array_equal(host(got), O.requant_fixedpoint(acc, sx, sw, so))
    # -- ral_qconv: 3x3, 25 channels of (-72)(-51) -> 108 (quantized_conv2d.cc cases 2, 3)
    x = np.full((1, 5, 5, 25), -72, np.int8)
    wt = np.full((4, 3, 3, 25), -51, np.int8)
    md = list(O.NHWC_OHWI_METADATA) + [1, 1, 1, 1, 1]
    out = torch.empty((1, 3, 3, 4), dtype=torch.int8, device="cuda")
    with ctx.execution() as ex:
        ops.qconv(ex, dev(x), dev(wt), [0, 0, 0, 0], md, f1(8.333333e-3),
                  dev(np.full(4, 1.568627e-2, np.float32)), f1(1.0), out)
        assert np.all(host(out) == 108)
    # -- ral_pdll_qconv2d on seeded tensors, SAME padding, with an output zero point
    nb, h, w_, ci, co = 2, 14, 12, 32, 48
    x = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
    wt = rng.integers(-128, 128, (co, 3, 3, ci), dtype=np.int8)
    pad4, md, out_shape = O.conv_attrs(x.shape, wt.shape, "NHWC", [1, 1, 1, 1], [1, 1, 1, 1], "SAME")
    acc = O.conv_s32(x, wt, pad4, md, out_shape)
    sw = rng.uniform(0.001, 0.05, co).astype(np.float32)
    so = np.float32(np.std(acc * float(sx) * float(sw.mean())) / 40.0)
    want = O.requant_fixedpoint(acc.reshape(-1, co), sx, sw, so, zo=3).reshape(acc.shape)
    with ctx.execution() as ex:
        got = ops.pdll_qconv2d(ex, dev(x), dev(wt), f1(sx), dev(sw), f1(so), zo=3)
        np.testing.assert_array_equal(host(got), want)
    # ... and back: without the switch the float stage answers
    monkeypatch.delenv("DISC_GPU_REQUANT_FIXEDPOINT")
    with ctx.execution() as ex:
        got = ops.pdll_qconv2d(ex, dev(x), dev(wt), f1(sx), dev(sw), f1(so), zo=3)
        np.testing.assert_array_equal(
            host(got), O.requant_cpu(acc.reshape(-1, co), sx, sw, so, zo=3).reshape(acc.shape))


def test_ral_pdll_qconv2d_rejects_bad_attrs(rt):
    ctx, ral, ops = rt
    x = torch.zeros((1, 4, 4, 16), dtype=torch.int8, device="cuda")
    w = torch.zeros((16, 3, 3, 16), dtype=torch.int8, device="cuda")
    own = ral.RalContext()
    try:
        with own.execution() as ex:
            with pytest.raises(ral.RalError, match="padding must be"):
                ops.pdll_qconv2d(ex, x, w, f1(1.0), dev(np.ones(16, np.float32)), f1(1.0),
                                 padding="FULL")
    finally:
        own.close()


@pytest.mark.parametrize("shape,axis", [((64, 768), None), ((64, 768), 1), ((768, 768), 0),
                                        ((2, 14, 14, 64), 3)])
def test_ral_quantize_dequantize(rt, shape, axis):
    ctx, ral, ops = rt
    rng = np.random.default_rng(len(shape))
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    n = 1 if axis is None else shape[axis]
    scale = rng.uniform(0.02, 0.08, n).astype(np.float32)
    zp = rng.integers(-3, 4, n).astype(np.int32)
    with ctx.execution() as ex:
        q = ops.quantize(ex, dev(x), dev(scale), dev(zp), axis=axis)
        want = O.quantize(x, scale, zp, axis=axis)
        np.testing.assert_array_equal(host(q), want)
        f = ops.dequantize(ex, q, dev(scale), dev(zp), axis=axis)
        np.testing.assert_array_equal(host(f), O.dequantize(want, scale, zp, axis=axis))


@pytest.mark.parametrize("name,code,store", [("int16", None, torch.int16), ("uint16", "ui16", torch.int16),
                                             ("int32", None, torch.int32), ("uint32", "ui32", torch.int32)])
def test_ral_quantize_dequantize_wide_types(rt, name, code, store):
    ctx, ral, ops = rt
    rng = np.random.default_rng(11)
    info = np.iinfo(name)
    x = (rng.standard_normal((33, 20)) * 30).astype(np.float32)
    scale = rng.uniform(0.002, 0.01, 20).astype(np.float32)
    zp = rng.integers(0, 40, 20).astype(np.int32)
    with ctx.execution() as ex:
        q = ops.quantize(ex, dev(x), dev(scale), dev(zp), axis=1, qmin=int(info.min),
                         qmax=int(info.max), dtype=store, code=code)
        want = O.quantize(x, scale, zp, axis=1, qmin=int(info.min), qmax=int(info.max), dtype=np.dtype(name))
        np.testing.assert_array_equal(host(q).view(name), want)
        f = ops.dequantize(ex, q, dev(scale), dev(zp), axis=1, code=code)
        np.testing.assert_array_equal(host(f), O.dequantize(want, scale, zp, axis=1))


def test_host_memory_entries_of_the_cpu_device(rt):
    """What a program compiled for the gpu uses for its host-placed values (shape tensors):
    alloc / dealloc / inc_ref on the cpu device with reference counting, persistent and raw
    allocations, memset and memcpy (cpu_context_impl.cc:105-255, cpu_driver.cc:29-35)."""
    import ctypes as C
    ctx, ral, ops = rt

    def call(ex, name, codes_values, ret=None):
        a = ral.Args().ctx(ex.handle)
        for code, v in codes_values:
            a.scalar(code, v)
        r = a.result_scalar(ret) if ret else None
        ex.call(name, "cpu", a)
        return r.value if ret else None

    with ctx.execution() as ex:
        p = call(ex, "alloc", [("i64", 64)], "pvoid")
        q = call(ex, "alloc", [("i64", 0)], "pvoid")            # zero bytes still gives a buffer
        assert p and q and p != q and p % 64 == 0
        call(ex, "ral_cpu_memset", [("pvoid", p), ("i32", 7), ("i64", 64)])
        assert bytes((C.c_uint8 * 64).from_address(p)) == b"\x07" * 64
        src = (C.c_int64 * 4)(11, 22, 33, 44)
        call(ex, "ral_cpu_memcpy", [("pvoid", C.addressof(src)), ("pvoid", p), ("i64", 32)])
        assert list((C.c_int64 * 4).from_address(p)) == [11, 22, 33, 44]
        # a second memref over the same host buffer: one more reference
        a = ral.Args().ctx(ex.handle).scalar("pvoid", 0).memref("i64", p, [4])
        alias = a.result_memref("i64", 1)
        ex.call("inc_ref", "cpu", a)
        assert alias.data == p and alias.sizes[0] == 4
        # ... and a reshaped one ([4] -> [2, 2], shape operand on the host): a third
        shp = np.array([2, 2], np.int64)
        a = ral.Args().ctx(ex.handle).scalar("pvoid", 0).memref("i64", p, [4])
        a.host_array(shp)
        view = a.result_memref("i64", 2)
        ex.call("inc_ref", "cpu", a)
        assert view.data == p and list(view.sizes) == [2, 2] and list(view.strides) == [2, 1]
        call(ex, "dealloc", [("pvoid", p)])
        call(ex, "dealloc", [("pvoid", p)])                     # two references gone
        assert list((C.c_int64 * 4).from_address(p)) == [11, 22, 33, 44]   # still alive
        call(ex, "dealloc", [("pvoid", p)])                     # the last one: released
        call(ex, "dealloc", [("pvoid", q)])
        call(ex, "dealloc", [("pvoid", 0)])                     # null: ignored
        # persistent host memory survives dealloc and the execution
        keep = call(ex, "ral_cpu_alloc_persistent", [("i64", 16)], "pvoid")
        (C.c_int32 * 4).from_address(keep)[:] = [1, 2, 3, 4]
        call(ex, "dealloc", [("pvoid", keep)])
        # an alias of something the execution never saw is an error
        a = ral.Args().ctx(ex.handle).scalar("pvoid", 0).memref("i64", C.addressof(src), [4])
        a.result_memref("i64", 1)
        with pytest.raises(ral.RalError, match="not known"):
            ex.call("inc_ref", "cpu", a)
        leaked = call(ex, "alloc", [("i64", 128)], "pvoid")     # returned with the execution
        assert leaked
    with ctx.execution() as ex:
        assert list((C.c_int32 * 4).from_address(keep)) == [1, 2, 3, 4]
        a = ral.Args().ctx(ex.handle).scalar("pvoid", 0).memref("i32", keep, [4])
        a.result_memref("i32", 1)
        ex.call("inc_ref", "cpu", a)                            # persistent: pinned, never freed
        call(ex, "dealloc", [("pvoid", keep)])
        call(ex, "dealloc", [("pvoid", keep)])
        assert list((C.c_int32 * 4).from_address(keep)) == [1, 2, 3, 4]


def test_driver_alloc_copy_roundtrip_and_pool_reuse(rt):
    ctx, ral, ops = rt
    import ctypes as C
    with ctx.execution() as ex:
        p1 = ex.alloc(1000)
        assert p1
        src = np.arange(250, dtype=np.int32)
        dst = np.zeros(250, np.int32)
        a = ral.Args().ctx(ex.handle).scalar("pvoid", 0).scalar("pvoid", src.ctypes.data)
        a.scalar("pvoid", p1).scalar("i64", 1000)
        ex.call("h2d_", "gpu", a)
        a = ral.Args().ctx(ex.handle).scalar("pvoid", 0).scalar("pvoid", p1)
        a.scalar("pvoid", dst.ctypes.data).scalar("i64", 1000)
        ex.call("d2h_", "gpu", a)
        ex.sync()
        np.testing.assert_array_equal(dst, src)
        ex.dealloc(p1)
        p2 = ex.alloc(900)        # same size class (1024) -> the pooled block comes back
        assert p2 == p1
        ex.dealloc(p2)
        a = ral.Args().ctx(ex.handle).scalar("pvoid", 0)
        r = a.result_scalar("pvoid")
        ex.call("ral_gpu_as_cu_stream", "gpu", a)
        assert (r.value or 0) == torch.cuda.current_stream().cuda_stream
        del C


def test_concurrent_executions_on_one_context(rt):
    """One Context serves several ExecutionContexts from different threads
    (ral/ral_context.h:52-58 in the reference): registry lookups, the attribute cache,
    the packed-weight cache and the allocator are shared.  Every thread checks its own
    results against the oracle."""
    import threading
    ctx, ral, ops = rt
    rng = np.random.default_rng(99)
    k, n = 256, 192
    w_kn = rng.integers(-128, 128, (k, n), dtype=np.int8)           # [K,N]: goes through the pack cache
    sw = rng.uniform(0.001, 0.05, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    sx, so = np.float32(0.02), np.float32(0.5)
    d_w, d_sw, d_bias = dev(w_kn), dev(sw), dev(bias)
    b32 = O.bias_f32_to_s32(bias, float(sx), sw)
    errors = []

    def worker(tid):
        try:
            r = np.random.default_rng(tid)
            for it in range(12):
                m = int(r.integers(1, 300))
                a = r.integers(-128, 128, (m, k), dtype=np.int8)
                with ctx.execution() as ex:
                    got = ops.pdll_qgemm_cpu_style(ex, dev(a), d_w, d_bias, f1(sx), d_sw, f1(so),
                                                   transpose_b=False, weight_is_const=True)
                    torch.cuda.synchronize()
                    acc = O.gemm_s32(a, w_kn)
                    want = O.requant_cpu(acc, float(sx), sw, float(so), b32=b32)
                    if not np.array_equal(got.cpu().numpy(), want):
                        errors.append("thread %d iteration %d (m=%d) differs" % (tid, it, m))
        except Exception as exc:  # noqa: BLE001
            errors.append("thread %d: %r" % (tid, exc))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


_PROFILE_CHILD = r"""
import numpy as np, torch
from bladedisc_amd import ral, ral_ops as ops
ctx = ral.RalContext(stream=torch.cuda.current_stream().cuda_stream)
d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
f1 = lambda v: d(np.array([v], np.float32))
rng = np.random.default_rng(0)
a = rng.integers(-128, 128, (96, 256), dtype=np.int8)
w = rng.integers(-128, 128, (128, 256), dtype=np.int8)
out = torch.empty((96, 128), dtype=torch.int8, device="cuda")
x = rng.integers(-128, 128, (2, 8, 8, 32), dtype=np.int8)
k = rng.integers(-128, 128, (16, 3, 3, 32), dtype=np.int8)
co = torch.empty((2, 8, 8, 16), dtype=torch.int8, device="cuda")
with ctx.execution() as ex:
    ops.qgemm(ex, d(a), d(w), f1(0.02), f1(0.01), f1(3.0), out, tp_b=True)
    ops.qconv(ex, d(x), d(k), [1, 1, 1, 1], [0, 3, 1, 2, 3, 0, 1, 2, 0, 3, 1, 2, 1, 1, 1, 1, 1],
              f1(0.02), d(np.full(16, 0.01, np.float32)), f1(3.0), co)
torch.cuda.synchronize()
print("checksum", int(out.to(torch.int32).sum()), int(co.to(torch.int32).sum()))
ctx.close()
"""


def test_profile_mode_logs_the_reference_fields():
    """DISC_GPU_ENABLE_PROFILE=1: each GEMM / convolution entry logs sizes, "Math Ops", "Bytes",
    bandwidth and rate (the fields of the reference's DISC_CPU_ENABLE_PROFILE dump), and the
    results are the same as without it.  The switch is read once per process, hence the
    child processes."""
    import os
    import re
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    runs = {}
    for flag in ("1", "0"):
        env = dict(os.environ, DISC_GPU_ENABLE_PROFILE=flag, PYTHONPATH=root)
        r = subprocess.run([sys.executable, "-c", _PROFILE_CHILD], env=env, capture_output=True,
                           text=True, timeout=110)
        assert r.returncode == 0, r.stderr[-2000:]
        runs[flag] = r
    log = runs["1"].stderr + runs["1"].stdout
    assert "ral_qgemm (gpu):" in log and "ral_qconv (gpu):" in log
    assert re.search(r"m = 96\s+n = 128\s+k = 256", log)
    assert "Math Ops = %d" % (2 * 96 * 128 * 256) in log
    assert "Bytes = %d" % (96 * 256 + 256 * 128 + 96 * 128) in log
    assert "Math Ops = %d" % (2 * 2 * 8 * 8 * 16 * 3 * 3 * 32) in log       # the convolution
    assert re.search(r"Elapsed = [0-9.e+-]+ us", log) and "Bandwidth = " in log and "GOPS = " in log
    quiet = runs["0"].stderr + runs["0"].stdout
    assert "Math Ops" not in quiet
    line = [l for l in runs["1"].stdout.splitlines() if l.startswith("checksum")]
    assert line and line == [l for l in runs["0"].stdout.splitlines() if l.startswith("checksum")]
