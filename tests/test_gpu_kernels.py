"""GPU parity tests of the raw kernel C ABI against the CPU oracle (bit-exact for
int32/int8 results; 1e-5 relative for f32 outputs)."""
import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from bladedisc_amd import kernels
    return kernels


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def gemm_variants(K, k):
    """All variant ids of the GEMM."""
    return [i for i, nm in enumerate(K.variant_names())
            if not nm.startswith(("direct3x3_", "stream"))]


def make_scales(rng, n, per_channel=True):
    sx = np.float32(rng.uniform(0.01, 0.03))
    sw = rng.uniform(0.001, 0.05, n if per_channel else 1).astype(np.float32)
    return sx, sw


def pick_so(acc, sx, sw):
    """Output scale putting the results at about 40 LSB rms (few saturate)."""
    s = float(np.std(acc.astype(np.float64) * (float(sx) * sw.astype(np.float64).mean())))
    return np.float32(max(s, 1e-6) / 40.0)


# ------------------------------------------------------------------ MFMA layout
def test_mfma_operand_and_result_layouts(K):
    rng = np.random.default_rng(0)
    a = rng.integers(-128, 128, (32, 32), dtype=np.int8)   # row i, k contiguous
    b = rng.integers(-128, 128, (32, 32), dtype=np.int8)   # column j, k contiguous
    a16 = rng.integers(-128, 128, (16, 64), dtype=np.int8)
    b16 = rng.integers(-128, 128, (16, 64), dtype=np.int8)
    d32, d16 = K.mfma_probe(dev(a), dev(b), dev(a16), dev(b16))
    np.testing.assert_array_equal(host(d32), a.astype(np.int32) @ b.astype(np.int32).T)
    np.testing.assert_array_equal(host(d16), a16.astype(np.int32) @ b16.astype(np.int32).T)


# ------------------------------------------------------------------------ qgemm
SHAPES = [(1, 768, 768), (16, 768, 768), (64, 768, 768), (128, 3072, 768), (1000, 768, 3072),
          (257, 130, 64), (33, 36, 16), (300, 260, 1040), (512, 512, 512), (5, 7, 48),
          # contraction lengths that are not a multiple of 16: padded into the scratch
          (4, 71, 25), (300, 260, 1041), (1000, 768, 777), (64, 64, 1), (2048, 1024, 15)]


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_qgemm_acc_s32_all_variants(K, m, n, k):
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    want, _ = O.gemm_s32_fast(a, w)
    da, dw = dev(a), dev(w)
    for v in gemm_variants(K, k):
        got = host(K.qgemm(da, dw, K.EPI_ACC_S32, variant=v))
        np.testing.assert_array_equal(got, want, err_msg=K.variant_names()[v])
    np.testing.assert_array_equal(host(K.qgemm(da, dw, K.EPI_ACC_S32)), want)


@pytest.mark.parametrize("m,n,k", [(64, 768, 768), (1000, 768, 3072), (257, 130, 64), (4096, 768, 768)])
@pytest.mark.parametrize("bias", ["none", "s32", "f32"])
def test_qgemm_requant_cpu(K, m, n, k, bias):
    rng = np.random.default_rng(m + n + k + len(bias))
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(a, w)
    sx, sw = make_scales(rng, n)
    so = pick_so(acc, sx, sw)
    b32 = bias_t = None
    if bias == "s32":
        b32 = rng.integers(-200000, 200000, n).astype(np.int32)
        bias_t = dev(b32)
    elif bias == "f32":
        bf = (rng.standard_normal(n) * 10 * so).astype(np.float32)
        b32 = O.bias_f32_to_s32(bf, sx, sw)
        bias_t = dev(bf)
    want = O.requant_cpu(acc, sx, sw, so, b32=b32)
    for v in [-1] + gemm_variants(K, k):
        got = host(K.qgemm(dev(a), dev(w), K.EPI_REQUANT_CPU, sx=dev(np.array([sx])), sw=dev(sw),
                           so=dev(np.array([so])), bias=bias_t, variant=v))
        np.testing.assert_array_equal(got, want, err_msg="variant %d" % v)
    sat = np.mean((want == 127) | (want == -128))
    assert sat < 0.5, "degenerate test: %.2f saturated" % sat


@pytest.mark.parametrize("m,n,k", [
    (4133, 4109, 272),     # 17 x 17 tiles of 256 x 256: more tiles than compute units, not a multiple of 8
    (4096, 4300, 144),     # 16 x 17 = 272 tiles: dealt per XCD; two k tiles, the second ragged
    (5000, 3840, 128),     # 20 x 20 tiles of 256 x 192 / 20 x 15 of 256 x 256; one k tile
    (16384, 1536, 400),    # three and four rounds of the two big tile shapes
])
def test_qgemm_persistent_variants_walk_many_tiles(K, m, n, k):
    """The persistent kernels with several output tiles per workgroup: ragged last tiles in
    M, N and K, tile counts that do and do not divide over the XCDs, all epilogue families
    (int8 with and without additive terms, int32, f32), and the heuristic's own pick at these
    sizes -- bit-exact against the oracle."""
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(a, w)
    sx, sw = make_scales(rng, n)
    so = pick_so(acc, sx, sw)
    bf = (rng.standard_normal(n) * 10 * so).astype(np.float32)
    b32 = O.bias_f32_to_s32(bf, sx, sw)
    want_plain = O.requant_cpu(acc, sx, sw, so)
    want_bias = O.requant_cpu(acc, sx, sw, so, b32=b32, zo=3)
    want_f32 = O.dequant_acc(acc, sx, sw, bias=bf)
    da, dw = dev(a), dev(w)
    dsx, dsw, dso = dev(np.array([sx])), dev(sw), dev(np.array([so]))
    names = K.variant_names()
    persistent = [i for i, nm in enumerate(names) if nm.startswith("persist_")]
    assert len(persistent) >= 2
    for v in [-1] + persistent:
        tag = names[v] if v >= 0 else "heuristic"
        got = host(K.qgemm(da, dw, K.EPI_REQUANT_CPU, sx=dsx, sw=dsw, so=dso, variant=v))
        np.testing.assert_array_equal(got, want_plain, err_msg=tag)
        got = host(K.qgemm(da, dw, K.EPI_REQUANT_CPU, sx=dsx, sw=dsw, so=dso, bias=dev(bf), zo=3,
                           variant=v))
        np.testing.assert_array_equal(got, want_bias, err_msg=tag)
        np.testing.assert_array_equal(host(K.qgemm(da, dw, K.EPI_ACC_S32, variant=v)), acc, err_msg=tag)
        got = host(K.qgemm(da, dw, K.EPI_DEQUANT_F32, sx=dsx, sw=dsw, bias=dev(bf), variant=v))
        assert np.array_equal(got.view(np.uint32), want_f32.view(np.uint32)), tag
        # requant -> dequantize in one epilogue (f32 result) and the E2 form with its f32 bias
        got = host(K.qgemm(da, dw, K.EPI_REQUANT_CPU_DEQUANT_F32, sx=dsx, sw=dsw, so=dso, bias=dev(bf),
                           zo=3, variant=v))
        want = O.dequantize(want_bias, np.array([so], np.float32), np.array([3], np.int32))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), tag
        got = host(K.qgemm(da, dw, K.EPI_REQUANT_GPU, sx=dsx, sw=dsw, so=dso, bias=dev(bf), variant=v))
        np.testing.assert_array_equal(got, O.requant_gpu(acc, sx, sw, so, bias_f32=bf), err_msg=tag)


@pytest.mark.parametrize("m,n,k", [(64, 768, 768), (1000, 768, 3072), (257, 130, 64), (5, 7, 48),
                                   (4096, 768, 768), (300, 260, 1041)])
@pytest.mark.parametrize("bias", ["none", "s32"])
def test_qgemm_requant_fixedpoint(K, m, n, k, bias):
    """The integer output stage of the reference's AArch64 path (multiplier + shift) in every
    kernel variant, per-channel and per-tensor weight scales, with and without an output zero
    point, multipliers below and above one -- bit-exact against the oracle's restatement."""
    rng = np.random.default_rng(m + 5 * n + k + len(bias))
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(a, w)
    sx, sw = make_scales(rng, n)
    so = pick_so(acc, sx, sw)
    b32 = rng.integers(-200000, 200000, n).astype(np.int32) if bias == "s32" else None
    bias_t = dev(b32) if b32 is not None else None
    cases = [(sw, so, 0), (sw, so, -5), (sw[:1], so, 0),
             (sw, np.float32(so * 1e-5), 7)]          # multipliers above one: left shifts, saturation
    for swv, sov, zo in cases:
        want = O.requant_fixedpoint(acc, sx, swv, sov, b32=b32, zo=zo)
        for v in [-1] + gemm_variants(K, k):
            if K.variant_names()[v].startswith("persist_") and v >= 0:
                # (the persistent kernels leave this stage out and say so when forced)
                with pytest.raises(RuntimeError, match="persistent"):
                    K.qgemm(dev(a), dev(w), K.EPI_REQUANT_FIXEDPOINT, sx=dev(np.array([sx])),
                            sw=dev(swv), so=dev(np.array([sov], np.float32)), bias=bias_t, zo=zo,
                            variant=v)
                continue
            got = host(K.qgemm(dev(a), dev(w), K.EPI_REQUANT_FIXEDPOINT, sx=dev(np.array([sx])),
                               sw=dev(swv), so=dev(np.array([sov], np.float32)), bias=bias_t, zo=zo,
                               variant=v))
            np.testing.assert_array_equal(got, want, err_msg="variant %d zo %d" % (v, zo))
    want = O.requant_fixedpoint(acc, sx, sw, so, b32=b32)
    sat = np.mean((want == 127) | (want == -128))
    assert sat < 0.5, "degenerate test: %.2f saturated" % sat
    # it is a different rounding from the float stage, not the same numbers by another route
    other = O.requant_cpu(acc, sx, sw, so, b32=b32)
    assert np.max(np.abs(other.astype(np.int32) - want.astype(np.int32))) <= 1


@pytest.mark.parametrize("m,n,k", [(64, 768, 768), (1000, 768, 3072), (257, 132, 64), (5, 16, 48),
                                   (4096, 768, 768), (3072, 3072, 768), (300, 260, 96)])
def test_qgemm_fused_operators_equal_the_separate_ones(K, m, n, k):
    """Operators fused behind a quantized GEMM -- dequantize -> +residual (f32 or int8) ->
    ReLU -> quantize, dequantize -> +residual -> f32, and a 256-entry table on the int8
    result -- give the bits of the chain of separate library calls (qgemm, dq8_dequantize, an
    f32 add, a clamp at zero, dq8_quantize, dq8_lut8), for every epilogue family."""
    rng = np.random.default_rng(11 * m + n + k)
    a = dev(rng.integers(-128, 128, (m, k), dtype=np.int8))
    w = dev(rng.integers(-128, 128, (n, k), dtype=np.int8))
    acc, _ = O.gemm_s32_fast(host(a), host(w))
    sx, sw = make_scales(rng, n)
    so = pick_so(acc, sx, sw)
    dsx, dsw, dso = dev(np.array([sx])), dev(sw), dev(np.array([so], np.float32))
    bias = dev((rng.standard_normal(n) * 10 * so).astype(np.float32))
    b32 = dev(rng.integers(-100000, 100000, n).astype(np.int32))
    rf = dev((rng.standard_normal((m, n)) * 40 * so).astype(np.float32))
    rq = dev(rng.integers(-128, 128, (m, n), dtype=np.int8))
    rs, rz = dev(np.array([so * 1.7], np.float32)), 4
    s2, z2 = dev(np.array([so * 1.3], np.float32)), -7
    zero = torch.zeros(1, dtype=torch.int32, device="cuda")
    table = dev(rng.integers(-128, 128, 256, dtype=np.int8))

    def unfused(q, zo, resid, relu, requant):
        y = K.dequantize(q, dso, torch.full((1,), zo, dtype=torch.int32, device="cuda"))
        r = resid if resid.dtype == torch.float32 else \
            K.dequantize(resid, rs, torch.full((1,), rz, dtype=torch.int32, device="cuda"))
        t = y + r
        if relu:
            t = torch.where(t < 0, torch.zeros_like(t), t)
        if not requant:
            return t
        return K.quantize(t, s2, torch.full((1,), z2, dtype=torch.int32, device="cuda"))

    stages = [(K.EPI_REQUANT_CPU, K.EPI_REQUANT_CPU_DEQUANT_F32, bias, 3),
              (K.EPI_REQUANT_GPU, K.EPI_REQUANT_GPU_DEQUANT_F32, bias, 0),
              (K.EPI_REQUANT_FIXEDPOINT, None, b32, -2)]
    for epi, epi_f32, b, zo in stages:
        q = K.qgemm(a, w, epi, sx=dsx, sw=dsw, so=dso, bias=b, zo=zo)
        for resid in (rf, rq):
            for relu in (False, True):
                kw = dict(residual=resid, relu=relu)
                if resid.dtype == torch.int8:
                    kw.update(residual_scale=rs, residual_zp=rz)
                got = K.qgemm(a, w, epi, sx=dsx, sw=dsw, so=dso, bias=b, zo=zo,
                              post=K.make_postops(out_scale=s2, out_zp=z2, **kw))
                assert torch.equal(got, unfused(q, zo, resid, relu, True)), (epi, resid.dtype, relu)
                if epi_f32 is not None:
                    got = K.qgemm(a, w, epi_f32, sx=dsx, sw=dsw, so=dso, bias=b, zo=zo,
                                  post=K.make_postops(**kw))
                    want = unfused(q, zo, resid, relu, False)
                    assert torch.equal(got.view(torch.int32), want.view(torch.int32)), \
                        (epi_f32, resid.dtype, relu)
        got = K.qgemm(a, w, epi, sx=dsx, sw=dsw, so=dso, bias=b, zo=zo,
                      post=K.make_postops(table=table))
        assert torch.equal(got, K.lut8(q, table)), epi
    # what the API refuses
    with pytest.raises(RuntimeError, match="out_scale"):
        K.qgemm(a, w, K.EPI_REQUANT_CPU, sx=dsx, sw=dsw, so=dso, post=K.make_postops(residual=rf))
    with pytest.raises(RuntimeError, match="requantising"):
        K.qgemm(a, w, K.EPI_ACC_S32, post=K.make_postops(table=table))
    with pytest.raises(RuntimeError, match="no residual"):
        K.qgemm(a, w, K.EPI_REQUANT_CPU, sx=dsx, sw=dsw, so=dso,
                post=K.make_postops(table=table, residual=rf, out_scale=s2))
    assert zero.item() == 0


@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("bias", ["none", "f32", "s8"])
def test_qgemm_requant_gpu(K, per_channel, bias):
    m, n, k = 200, 384, 512
    rng = np.random.default_rng(17 + per_channel)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(a, w)
    ns = n if per_channel else 1
    sx = rng.uniform(0.01, 0.03, ns).astype(np.float32)
    sw = rng.uniform(0.001, 0.05, ns).astype(np.float32)
    so = (np.full(ns, pick_so(acc, sx.mean(), sw)) * rng.uniform(0.9, 1.1, ns)).astype(np.float32)
    bf = bi = bias_t = None
    if bias == "f32":
        bf = (rng.standard_normal(n) * 10).astype(np.float32)
        bias_t = dev(bf)
    elif bias == "s8":
        bi = rng.integers(-128, 128, n).astype(np.int8)
        bias_t = dev(bi)
    want = O.requant_gpu(acc, sx, sw, so, bias_f32=bf, bias_i8=bi)
    for v in [-1] + gemm_variants(K, k):
        got = host(K.qgemm(dev(a), dev(w), K.EPI_REQUANT_GPU, sx=dev(sx), sw=dev(sw), so=dev(so),
                           bias=bias_t, variant=v))
        np.testing.assert_array_equal(got, want, err_msg="variant %d" % v)


@pytest.mark.parametrize("m,n,k", [(64, 768, 768), (1000, 768, 3072), (257, 130, 64), (3072, 3072, 768),
                                   (5, 130, 784)])
@pytest.mark.parametrize("form", ["cpu_f32", "cpu_s32_zo", "gpu_s8", "gpu_none"])
def test_qgemm_requant_then_dequantize_in_one_epilogue(K, m, n, k, form):
    """Epilogues 4 / 5: the f32 result must equal, bit for bit, dequantize applied to the int8
    result of the requant epilogue -- against the oracle's two functions and against the two
    separate GPU kernels."""
    rng = np.random.default_rng(m * 7 + n + k + len(form))
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(a, w)
    sx, sw = make_scales(rng, n)
    so = pick_so(acc, sx, sw)
    zo = 0
    t = lambda v: dev(np.array([v], np.float32))
    if form.startswith("cpu"):
        epi, fused = K.EPI_REQUANT_CPU, K.EPI_REQUANT_CPU_DEQUANT_F32
        if form == "cpu_f32":
            bf = (rng.standard_normal(n) * 10 * so).astype(np.float32)
            bias_t, b32 = dev(bf), O.bias_f32_to_s32(bf, sx, sw)
        else:
            b32 = rng.integers(-200000, 200000, n).astype(np.int32)
            bias_t, zo = dev(b32), 5
        q_want = O.requant_cpu(acc, sx, sw, so, b32=b32, zo=zo)
    else:
        epi, fused = K.EPI_REQUANT_GPU, K.EPI_REQUANT_GPU_DEQUANT_F32
        bi = rng.integers(-128, 128, n).astype(np.int8) if form == "gpu_s8" else None
        bias_t = dev(bi) if bi is not None else None
        q_want = O.requant_gpu(acc, np.array([sx], np.float32), sw, np.array([so], np.float32),
                               bias_i8=bi)
    want = O.dequantize(q_want, np.array([so], np.float32), np.array([zo], np.int32))
    sov, zov = t(so), dev(np.array([zo], np.int32))
    for v in [-1] + gemm_variants(K, k):
        got = K.qgemm(dev(a), dev(w), fused, sx=t(sx), sw=dev(sw), so=sov, bias=bias_t, zo=zo,
                      variant=v)
        assert got.dtype == torch.float32
        two = K.dequantize(K.qgemm(dev(a), dev(w), epi, sx=t(sx), sw=dev(sw), so=sov, bias=bias_t,
                                   zo=zo, variant=v), sov, zov)
        assert torch.equal(got, two), "variant %d" % v
        assert np.array_equal(host(got).view(np.uint32), want.view(np.uint32)), "variant %d" % v
    # a per-channel output scale is refused
    with pytest.raises(RuntimeError, match="per-tensor"):
        K.qgemm(dev(a), dev(w), fused, sx=t(sx), sw=dev(sw), so=dev(np.full(n, so, np.float32)),
                bias=bias_t, zo=zo)


def test_qgemm_dequant_f32(K):
    m, n, k = 64, 768, 768
    rng = np.random.default_rng(5)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(a, w)
    sx, sw = make_scales(rng, n)
    bias = rng.standard_normal(n).astype(np.float32)
    want = O.dequant_acc(acc, sx, sw, bias)
    exact = acc.astype(np.float64) * (np.float64(sx) * sw.astype(np.float64)) + bias
    for v in [-1] + gemm_variants(K, k):
        got = host(K.qgemm(dev(a), dev(w), K.EPI_DEQUANT_F32, sx=dev(np.array([sx])), sw=dev(sw),
                           bias=dev(bias), variant=v))
        np.testing.assert_array_equal(got, want)
        # tolerance stated by the task for dequantized outputs: 1e-5 relative
        np.testing.assert_allclose(got, exact, rtol=1e-5, atol=1e-5 * np.abs(exact).max())


@pytest.mark.parametrize("tp_a,tp_b", [(0, 0), (1, 0), (1, 1)])
def test_qgemm_transposed_operands(K, tp_a, tp_b):
    m, n, k = 96, 200, 320
    rng = np.random.default_rng(31)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (k, n), dtype=np.int8)
    want = O.gemm_s32(a, w)
    a_in = a.T.copy() if tp_a else a
    w_in = w.T.copy() if tp_b else w
    for v in [-1, 0, 2]:
        got = host(K.qgemm(dev(a_in), dev(w_in), K.EPI_ACC_S32, tp_a=bool(tp_a), tp_b=bool(tp_b),
                           variant=v))
        np.testing.assert_array_equal(got, want)


def test_qgemm_ragged_k_stays_on_the_mfma_kernels(K):
    """K % 16 != 0: with the scratch dq8_qgemm_workspace_bytes asks for, the operands are
    padded and the MFMA kernels run (every layout, zero points, every epilogue); the result
    is the oracle's, and it is not the generic kernel's speed."""
    import time
    rng = np.random.default_rng(77)
    m, n, k = 1000, 520, 777
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    for tp_a, tp_b, zx, zw in [(0, 1, 0, 0), (1, 0, 0, 0), (0, 0, 5, 0), (1, 1, -9, 4)]:
        acc = O.gemm_s32(a, w, tp_b=True, zx=zx, zw=zw)
        a_in = np.ascontiguousarray(a.T) if tp_a else a
        w_in = w if tp_b else np.ascontiguousarray(w.T)
        kw = dict(tp_a=bool(tp_a), tp_b=bool(tp_b), zx=zx, zw=zw)
        np.testing.assert_array_equal(host(K.qgemm(dev(a_in), dev(w_in), K.EPI_ACC_S32, **kw)), acc)
        sx, sw = make_scales(rng, n)
        so = pick_so(acc, sx, sw)
        bias = (rng.standard_normal(n) * 3).astype(np.float32)
        want = O.requant_cpu(acc, sx, sw, so, b32=O.bias_f32_to_s32(bias, sx, sw))
        got = host(K.qgemm(dev(a_in), dev(w_in), K.EPI_REQUANT_CPU, sx=dev(np.array([sx])),
                           sw=dev(sw), so=dev(np.array([so])), bias=dev(bias), **kw))
        np.testing.assert_array_equal(got, want)
    # speed: 4096 x 4096 x 4095 would take the generic kernel seconds
    big = 4096
    ab = torch.randint(-128, 128, (big, big - 1), dtype=torch.int8, device="cuda")
    wb = torch.randint(-128, 128, (big, big - 1), dtype=torch.int8, device="cuda")
    out = K.qgemm(ab, wb, K.EPI_ACC_S32)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = K.qgemm(ab, wb, K.EPI_ACC_S32)
    torch.cuda.synchronize()
    assert time.perf_counter() - t0 < 0.01
    rows = [0, 1234, big - 1]
    want = O.gemm_s32(ab[rows].cpu().numpy(), wb.cpu().numpy(), tp_b=True)
    np.testing.assert_array_equal(out[rows].cpu().numpy(), want)


def test_qgemm_zero_points_generic(K):
    m, n, k = 17, 19, 23
    rng = np.random.default_rng(3)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    want = O.gemm_s32(a, w, tp_b=True, zx=3, zw=-4)
    got = host(K.qgemm(dev(a), dev(w), K.EPI_ACC_S32, zx=3, zw=-4))
    np.testing.assert_array_equal(got, want)
    with pytest.raises(RuntimeError):
        K.qgemm(dev(a), dev(w), K.EPI_ACC_S32, zx=3, variant=2)


@pytest.mark.parametrize("m,n,k,tp_a,tp_b,zx,zw", [
    (64, 768, 768, 0, 1, 7, 0), (300, 130, 400, 0, 1, -128, 0), (33, 48, 64, 0, 1, 5, -3),
    (256, 512, 1040, 0, 0, 100, 0), (100, 96, 128, 1, 1, 127, 2), (1, 768, 3072, 0, 1, 11, 0),
    (1000, 768, 768, 0, 1, -77, 9),
    # one shape per pipelined tile: 256x256 and 128x128 on eight waves, 256x64, 64x64 with K split
    (4096, 2560, 128, 0, 1, 9, -4), (2048, 2048, 256, 0, 1, -128, 127), (16384, 64, 128, 0, 1, 3, 1),
    (256, 256, 2048, 0, 1, 100, -100), (4100, 2570, 4096, 0, 1, 1, 0),
])
def test_qgemm_zero_points_on_the_mfma_path(K, m, n, k, tp_a, tp_b, zx, zw):
    """Asymmetric operands stay on the MFMA kernels when the caller provides the scratch for
    the correction vectors (the accumulators start at them): every epilogue equals the oracle's direct sum of (a - zx)(w - zw);
    without the scratch the generic kernel gives the same result."""
    rng = np.random.default_rng(m + n + k + zx)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc = O.gemm_s32(a, w, tp_b=True, zx=zx, zw=zw)
    a_in = np.ascontiguousarray(a.T) if tp_a else a
    w_in = w if tp_b else np.ascontiguousarray(w.T)
    kw = dict(tp_a=bool(tp_a), tp_b=bool(tp_b), zx=zx, zw=zw)
    got = host(K.qgemm(dev(a_in), dev(w_in), K.EPI_ACC_S32, **kw))
    np.testing.assert_array_equal(got, acc)
    got0 = host(K.qgemm(dev(a_in), dev(w_in), K.EPI_ACC_S32, variant=0, **kw))   # generic
    np.testing.assert_array_equal(got0, acc)
    sx, sw = make_scales(rng, n)
    so = pick_so(acc, sx, sw)
    bias = (rng.standard_normal(n) * 3).astype(np.float32)
    dsx, dsw, dso = dev(np.array([sx])), dev(sw), dev(np.array([so]))
    b32 = O.bias_f32_to_s32(bias, sx, sw)
    want = O.requant_cpu(acc, sx, sw, so, b32=b32, zo=5)
    got = host(K.qgemm(dev(a_in), dev(w_in), K.EPI_REQUANT_CPU, sx=dsx, sw=dsw, so=dso,
                       bias=dev(bias), zo=5, **kw))
    np.testing.assert_array_equal(got, want)
    want = O.requant_gpu(acc, sx, sw, so, bias_f32=bias)
    got = host(K.qgemm(dev(a_in), dev(w_in), K.EPI_REQUANT_GPU, sx=dsx, sw=dsw, so=dso,
                       bias=dev(bias), **kw))
    np.testing.assert_array_equal(got, want)
    want = O.dequant_acc(acc, sx, sw, bias=bias)
    got = host(K.qgemm(dev(a_in), dev(w_in), K.EPI_DEQUANT_F32, sx=dsx, sw=dsw, bias=dev(bias), **kw))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)


def test_qgemm_zero_points_full_size_property(K):
    """4096^3 with an input zero point: the result equals the symmetric result of
    the shifted problem computed another way -- acc(a - zx, w) = acc(a, w) - zx * colsum(w)
    -- with both sides from the GPU in int32 and the column sums from numpy."""
    n = 4096
    g = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randint(-128, 128, (n, n), dtype=torch.int8, device="cuda", generator=g)
    w = torch.randint(-128, 128, (n, n), dtype=torch.int8, device="cuda", generator=g)
    sym = K.qgemm(a, w, K.EPI_ACC_S32)
    asym = K.qgemm(a, w, K.EPI_ACC_S32, zx=37)
    colsum = w.to(torch.int32).sum(dim=1)
    assert torch.equal(asym, sym - 37 * colsum[None, :])


def test_qgemm_known_answers(K, golden):
    for case in golden["qgemm"]:
        m, k, n = case["m"], case["k"], case["n"]
        qx = np.full((m, k), case["qx"], np.int8)
        qw = np.full((k, n), case["qw"], np.int8)   # [K,N] as the CPU callers hand it
        sw = np.full(n if case["per_channel"] else 1, case["sw"], np.float32)
        out = host(K.qgemm(dev(qx), dev(qw), K.EPI_REQUANT_CPU, tp_b=False,
                           sx=dev(np.array([case["sx"]], np.float32)), sw=dev(sw),
                           so=dev(np.array([case["so"]], np.float32))))
        assert (out == case["q_out"]).all(), case["src"]
        f = host(K.dequantize(dev(out), dev(np.array([case["so"]], np.float32)),
                              dev(np.array([0], np.int32))))
        assert (f == case["expect_f32"]).all()


def test_qgemm_empty_and_k0(K):
    a = torch.empty((0, 64), dtype=torch.int8, device="cuda")
    w = torch.zeros((32, 64), dtype=torch.int8, device="cuda")
    assert K.qgemm(a, w, K.EPI_ACC_S32).shape == (0, 32)
    a = torch.empty((8, 0), dtype=torch.int8, device="cuda")
    w = torch.empty((32, 0), dtype=torch.int8, device="cuda")
    out = host(K.qgemm(a, w, K.EPI_ACC_S32))
    assert out.shape == (8, 32) and (out == 0).all()


def test_qgemm_output_zero_point_and_saturation(K):
    acc_vals = np.array([[0, 1000, -1000, 127 * 127 * 64]], np.int32)
    a = np.zeros((1, 64), np.int8)
    w = np.zeros((4, 64), np.int8)
    a[0, :] = 127
    w[1, :16] = 1; w[1, 16] = -16 + 8  # noqa: E702
    # simpler: check against the oracle on random data with zo != 0
    rng = np.random.default_rng(8)
    a = rng.integers(-128, 128, (40, 64), dtype=np.int8)
    w = rng.integers(-128, 128, (52, 64), dtype=np.int8)
    acc = O.gemm_s32(a, w, tp_b=True)
    sx, sw = np.float32(0.02), rng.uniform(0.001, 0.05, 52).astype(np.float32)
    so = np.float32(0.05)   # small: many values saturate on both sides
    want = O.requant_cpu(acc, sx, sw, so, zo=7)
    got = host(K.qgemm(dev(a), dev(w), K.EPI_REQUANT_CPU, sx=dev(np.array([sx])), sw=dev(sw),
                       so=dev(np.array([so])), zo=7))
    np.testing.assert_array_equal(got, want)
    assert (want == 127).any() and (want == -128).any()
    del acc_vals


# --------------------------------------------------------------- quantize/dequant
@pytest.mark.parametrize("shape,axis", [((1000, 768), None), ((64, 768), 1), ((768, 768), 0),
                                        ((4, 56, 56, 64), 3), ((3, 5, 7), 1), ((1001,), None),
                                        ((130, 260), 1), ((2, 6, 10), 0), ((4096, 4096), 1)])
@pytest.mark.parametrize("round_mode", [0, 1])
def test_quantize_dequantize_parity(K, shape, axis, round_mode):
    rng = np.random.default_rng(len(shape) * 100 + (axis or 0))
    x = (rng.standard_normal(shape) * 2).astype(np.float32)
    flat = x.reshape(-1)
    flat[: min(64, flat.size)] = (np.arange(min(64, flat.size)) - 32 + 0.5) * 0.05  # ties
    n = 1 if axis is None else shape[axis]
    scale = rng.uniform(0.02, 0.08, n).astype(np.float32)
    scale[0] = 0.05
    zp = rng.integers(-3, 4, n).astype(np.int32)
    want = O.quantize(x, scale, zp, axis=axis, round_mode=round_mode)
    got = host(K.quantize(dev(x), dev(scale), dev(zp), axis=axis, round_mode=round_mode))
    np.testing.assert_array_equal(got, want)
    want_f = O.dequantize(want, scale, zp, axis=axis)
    got_f = host(K.dequantize(dev(want), dev(scale), dev(zp), axis=axis))
    np.testing.assert_array_equal(got_f, want_f)


@pytest.mark.parametrize("shape,axis", [((1000, 768), None), ((1003,), None), ((64, 768), 1), ((768, 768), 0),
                                        ((2, 3, 4, 5), 1), ((32, 8, 8, 64), 3), ((33, 52), 1), ((5, 7), 1)])
@pytest.mark.parametrize("round_mode", [0, 1])
@pytest.mark.parametrize("unsigned", [False, True])
def test_fake_quant_equals_quantize_then_dequantize(K, shape, axis, round_mode, unsigned):
    """dq8_fake_quant against the oracle's quantize -> dequantize and against the two GPU
    kernels, bit for bit (ties, saturation, non-zero zero points, in place)."""
    rng = np.random.default_rng(len(shape) * 31 + shape[0] + round_mode + 2 * unsigned)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    flat = x.reshape(-1)
    flat[::7] = np.round(flat[::7] * 4) / 8          # plenty of exact halves after scaling by 1/0.125
    flat[::11] = 1e9
    nq = shape[axis] if axis is not None else 1
    scale = np.full(nq, 0.125, np.float32) if nq == 1 else rng.choice([0.125, 0.25, 0.1], nq).astype(np.float32)
    zp = rng.integers(-10, 11, nq).astype(np.int32) + (128 if unsigned else 0)
    qmin, qmax = (0, 255) if unsigned else (-128, 127)
    dt = np.uint8 if unsigned else np.int8
    want = O.dequantize(O.quantize(x, scale, zp, axis=axis, qmin=qmin, qmax=qmax,
                                   round_mode=round_mode, dtype=dt), scale, zp, axis=axis)
    dx, ds, dz = dev(x), dev(scale), dev(zp)
    got = K.fake_quant(dx, ds, dz, axis=axis, qmin=qmin, qmax=qmax, round_mode=round_mode)
    assert np.array_equal(host(got).view(np.uint32), want.view(np.uint32))
    two = K.dequantize(K.quantize(dx, ds, dz, axis=axis, qmin=qmin, qmax=qmax, round_mode=round_mode,
                                  dtype=torch.uint8 if unsigned else torch.int8), ds, dz, axis=axis)
    assert torch.equal(got.view(torch.int32), two.view(torch.int32))
    K.fake_quant(dx, ds, dz, axis=axis, qmin=qmin, qmax=qmax, round_mode=round_mode, out=dx)   # in place
    assert torch.equal(dx.view(torch.int32), got.view(torch.int32))
    # idempotent on its own output
    again = K.fake_quant(got, ds, dz, axis=axis, qmin=qmin, qmax=qmax, round_mode=round_mode)
    assert torch.equal(again, got)


def test_quantize_golden_vectors(K, golden):
    """Every vector of disc-fold-quantize.mlir, all six quantized types (the unsigned 16 / 32
    bit results come back as bits in the signed torch dtype of the same width)."""
    seen = set()
    for case in golden["quantize_fold"]:
        x = np.array(case["x"], np.float32)
        got = host(K.quantize(dev(x), dev(np.array(case["scale"], np.float32)),
                              dev(np.array(case["zp"], np.int32)), axis=case["axis"],
                              qmin=case["qmin"], qmax=case["qmax"], round_mode=case["round_mode"],
                              dtype=case["dtype"]))
        np.testing.assert_array_equal(got.view(case["dtype"]), np.array(case["expect"], case["dtype"]),
                                      err_msg=case["src"])
        seen.add(case["dtype"])
    assert seen == {"int8", "uint8", "int16", "uint16", "int32", "uint32"}


@pytest.mark.parametrize("name", ["int16", "uint16", "int32", "uint32"])
@pytest.mark.parametrize("axis", [None, 0, 1])
def test_quantize_dequantize_wide_types(K, name, axis):
    """16- and 32-bit quantized types against the oracle: values that land inside the range,
    on both limits and beyond them (the conversion of the clamped value saturates), both
    rounding modes, per tensor and per channel; dequantize back."""
    rng = np.random.default_rng(len(name) + (axis or 0) * 7)
    npdt = np.dtype(name)
    info = np.iinfo(npdt)
    shape = (37, 24)
    nq = 1 if axis is None else shape[axis]
    scale = rng.uniform(0.001, 0.01, nq).astype(np.float32)
    zp = rng.integers(-50, 50, nq).astype(np.int32) if info.min < 0 else rng.integers(0, 100, nq).astype(np.int32)
    span = float(info.max) * float(scale.mean())
    x = (rng.standard_normal(shape) * span * 0.6).astype(np.float32)
    x[0, :4] = [span * 4, -span * 4, span, -span]
    for rm in (0, 1):
        want = O.quantize(x, scale, zp, axis=axis, qmin=int(info.min), qmax=int(info.max),
                          round_mode=rm, dtype=npdt)
        got = K.quantize(dev(x), dev(scale), dev(zp), axis=axis, qmin=int(info.min),
                         qmax=int(info.max), round_mode=rm, dtype=name)
        np.testing.assert_array_equal(host(got).view(npdt), want)
        assert (want == info.max).any() and (want == info.min).any()
    back = K.dequantize(got, dev(scale), dev(zp), axis=axis, dtype=name)
    want_f = O.dequantize(want, scale, zp, axis=axis)
    assert np.array_equal(host(back).view(np.uint32), want_f.view(np.uint32))


@pytest.mark.parametrize("name", ["int8", "uint8", "int16"])
def test_quantize_f16_input_is_the_f32_path_on_the_widened_values(K, name):
    """Half-precision input (an extension: the reference's lowering takes f32 only) is widened
    exactly and then quantized by the f32 steps."""
    rng = np.random.default_rng(3)
    npdt = np.dtype(name)
    info = np.iinfo(npdt)
    x16 = (rng.standard_normal((50, 33)) * 3).astype(np.float16)
    scale = rng.uniform(0.01, 0.05, 33).astype(np.float32)
    zp = np.full(33, int((int(info.min) + int(info.max) + 1) // 2), np.int32)
    want = O.quantize(x16.astype(np.float32), scale, zp, axis=1, qmin=int(info.min),
                      qmax=int(info.max), dtype=npdt)
    got = K.quantize(dev(x16), dev(scale), dev(zp), axis=1, qmin=int(info.min), qmax=int(info.max),
                     dtype=name)
    np.testing.assert_array_equal(host(got).view(npdt), want)


def test_quantize_unaligned_and_uint8(K):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(4099) * 50).astype(np.float32)
    base = dev(np.concatenate([[0.0], x]).astype(np.float32))
    xv = base[1:]                                      # 4-byte aligned only
    scale, zp = np.array([0.5], np.float32), np.array([128], np.int32)
    want = O.quantize(x, scale, zp, qmin=0, qmax=255, dtype=np.uint8)
    out = torch.empty(4099, dtype=torch.uint8, device="cuda")
    K.quantize(xv, dev(scale), dev(zp), qmin=0, qmax=255, dtype=torch.uint8, out=out)
    np.testing.assert_array_equal(host(out), want)
    got_f = host(K.dequantize(dev(want), dev(scale), dev(zp)))
    np.testing.assert_array_equal(got_f, O.dequantize(want, scale, zp))


def test_quantize_empty(K):
    x = torch.empty((0, 8), device="cuda")
    s = torch.ones(1, device="cuda")
    z = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert K.quantize(x, s, z).shape == (0, 8)


# ------------------------------------------------------------------------- table
@pytest.mark.parametrize("n", [0, 1, 15, 16, 17, 4099, 1 << 20])
def test_lut8_matches_numpy_take(K, n):
    rng = np.random.default_rng(n)
    table = rng.integers(-128, 128, 256, dtype=np.int8)
    q = rng.integers(-128, 128, n, dtype=np.int8)
    want = table[q.view(np.uint8)]
    got = K.lut8(dev(q), dev(table))
    np.testing.assert_array_equal(host(got), want)
    if n > 20:
        base = dev(np.concatenate([[0], q]).astype(np.int8))
        view = base[1:]                                      # 1-byte aligned only
        np.testing.assert_array_equal(host(K.lut8(view, dev(table))), want)
        buf = dev(q)
        K.lut8(buf, dev(table), out=buf)                     # in place
        np.testing.assert_array_equal(host(buf), want)
    u = rng.integers(0, 256, max(n, 1), dtype=np.uint8)
    tu = rng.integers(0, 256, 256, dtype=np.uint8)
    np.testing.assert_array_equal(host(K.lut8(dev(u), dev(tu))), tu[u])


def test_activation_table_equals_the_operator_chain(K):
    """table[q] = quantize(f(dequantize(q))) built from the kernels themselves: a lookup
    equals running the three operators, for an asymmetric input and output."""
    rng = np.random.default_rng(2)
    q = dev(rng.integers(-128, 128, (300, 77), dtype=np.int8))
    s_in, z_in = dev(np.array([0.037], np.float32)), dev(np.array([-11], np.int32))
    s_out, z_out = dev(np.array([0.021], np.float32)), dev(np.array([7], np.int32))
    for fn in (torch.nn.functional.gelu, torch.tanh, torch.relu):
        table = K.activation_table(fn, s_in, z_in, s_out, z_out)
        chain = K.quantize(fn(K.dequantize(q, s_in, z_in)), s_out, z_out)
        assert torch.equal(K.lut8(q, table), chain)
        # and the oracle's view of it for one function with exact float32 semantics
    table = host(K.activation_table(torch.relu, s_in, z_in, s_out, z_out))
    allq = np.arange(256, dtype=np.uint8).view(np.int8)
    deq = O.dequantize(allq, np.float32(0.037), np.array([-11], np.int32))
    want = O.quantize(np.maximum(deq, 0), np.float32(0.021), np.array([7], np.int32))
    np.testing.assert_array_equal(table, want)


def test_qgemm_library_choice_on_random_shapes(K):
    """Seeded sweep over what decides the kernel of a GEMM -- rows from one to 16384, contraction
    lengths and channel counts that are and are not multiples of the tiles, transposed operands,
    zero points, every epilogue and bias kind: whatever the library picks gives the bytes
    (the floats, to 1e-6 relative) of the generic kernel, which the tests above pin to the
    oracle."""
    rng = np.random.default_rng(20260702)
    gen = K.variant_names().index("generic")
    done = 0
    for case in range(400):
        r = rng.random()
        if r < 0.5:
            m = int(rng.integers(1, 300))
            k = int(rng.choice([64, 128, 768, 1024, 3072, 4096, int(rng.integers(1, 3000))]))
            n = int(rng.choice([16, 64, 768, 3072, 4096, int(rng.integers(1, 2000))]))
        elif r < 0.92:
            m = int(rng.integers(300, 5000))
            k = int(rng.choice([128, 256, 768, 2304, int(rng.integers(1, 1500))]))
            n = int(rng.choice([64, 256, 768, 1024, 3072, int(rng.integers(1, 1500))]))
        else:
            m, k, n = int(rng.choice([8192, 16384, 12000])), int(rng.choice([768, 512])), int(rng.choice([768, 3072, 1000]))
        tp_b, tp_a = bool(rng.random() < 0.8), bool(rng.random() < 0.1)
        a = dev(rng.integers(-128, 128, (k, m) if tp_a else (m, k), dtype=np.int8))
        w = dev(rng.integers(-128, 128, (n, k) if tp_b else (k, n), dtype=np.int8))
        epi = int(rng.choice([K.EPI_ACC_S32, K.EPI_REQUANT_CPU, K.EPI_REQUANT_CPU, K.EPI_REQUANT_GPU, K.EPI_REQUANT_GPU,
                              K.EPI_DEQUANT_F32, K.EPI_REQUANT_CPU_DEQUANT_F32, K.EPI_REQUANT_GPU_DEQUANT_F32]))
        kw = dict(tp_a=tp_a, tp_b=tp_b)
        so = np.float32(0.02 * 0.025 * 74.0 * 74.0 * np.sqrt(k) / 40.0)
        if epi != K.EPI_ACC_S32:
            kw.update(sx=dev(np.array([0.02], np.float32)), so=dev(np.array([so])),
                      sw=dev(rng.uniform(0.001, 0.05, n if rng.random() < 0.8 else 1).astype(np.float32)))
        bk = int(rng.integers(0, 3))
        cpu_kind = epi in (K.EPI_REQUANT_CPU, K.EPI_REQUANT_CPU_DEQUANT_F32)
        gpu_kind = epi in (K.EPI_REQUANT_GPU, K.EPI_REQUANT_GPU_DEQUANT_F32)
        if cpu_kind and bk == 1:
            kw.update(bias=dev((rng.standard_normal(n) * 3 * so).astype(np.float32)))
        if cpu_kind and bk == 2:
            kw.update(bias=dev(rng.integers(-100000, 100000, n).astype(np.int32)))
        if gpu_kind and bk == 1:
            kw.update(bias=dev((rng.standard_normal(n) * 30).astype(np.float32)))
        if gpu_kind and bk == 2:
            kw.update(bias=dev(rng.integers(-128, 128, n, dtype=np.int8)))
        if epi == K.EPI_DEQUANT_F32 and bk:
            kw.update(bias=dev(rng.standard_normal(n).astype(np.float32)))
        kw.update(zx=int(rng.integers(-5, 5)) if rng.random() < 0.15 else 0,
                  zw=int(rng.integers(-5, 5)) if rng.random() < 0.1 else 0,
                  zo=int(rng.integers(-10, 10)) if epi == K.EPI_REQUANT_CPU else 0)
        got = K.qgemm(a, w, epi, **kw)
        want = K.qgemm(a, w, epi, variant=gen, **kw)
        tag = "case %d: %dx%dx%d, epilogue %d, bias kind %d, transposes %d %d, zero points %d %d %d" % (
            case, m, k, n, epi, bk, tp_a, tp_b, kw["zx"], kw["zw"], kw["zo"])
        if got.dtype == torch.float32:
            assert torch.allclose(got, want, rtol=1e-6, atol=0), tag
        else:
            assert torch.equal(got, want), tag
        done += 1
    assert done == 400


# ------------------------------------------------------------------------- conv
CONVS = [  # nb, h, w, ci, co, k, stride, pad, dil
    (2, 30, 30, 3, 64, 7, 2, 3, 1),      # an RGB first layer: channels padded into scratch
    (1, 9, 9, 20, 24, 3, 1, 1, 1),
    (2, 14, 14, 64, 64, 3, 1, 1, 1),
    (2, 9, 11, 32, 48, 3, 2, 1, 1),
    (1, 8, 8, 16, 16, 3, 1, 2, 2),
    (3, 7, 7, 256, 128, 1, 1, 0, 1),
    (2, 6, 6, 5, 6, 3, 1, 1, 1),      # Ci % 16 != 0 -> generic kernel
    (4, 28, 28, 64, 64, 3, 1, 1, 1),  # K = 576: a partial last k tile, several tiles of rows
    (2, 15, 13, 48, 80, 3, 2, 1, 2),  # ragged everything, K = 432
    # the direct 3x3 kernels: every channel count they take, images of one tile and of
    # several with a ragged last one, ragged Co, no / one / two pixels of padding
    (3, 20, 18, 32, 40, 3, 1, 1, 1),
    (2, 30, 30, 128, 136, 3, 1, 1, 1),
    (2, 12, 10, 256, 64, 3, 1, 0, 1),
    (1, 33, 17, 64, 200, 3, 1, 2, 1),
    (1, 36, 36, 256, 64, 3, 1, 1, 1),  # a patch of 107 KiB: LDS addresses beyond 128 KiB
    (1, 6, 150, 64, 64, 3, 1, 1, 1),   # a wide image: tiles of 256 pixels span 2-3 rows
    # 1 x 1 filters with a stride: the library runs them as a GEMM over the pixels they read
    (3, 14, 14, 256, 512, 1, 2, 0, 1),
    (2, 9, 11, 48, 80, 1, 2, 0, 1),    # odd image sizes, K = 48, ragged Co
    (5, 28, 28, 128, 256, 1, 2, 0, 1),  # several row tiles, images ending inside a tile
    (1, 7, 5, 512, 1024, 1, 3, 0, 1),
]


@pytest.mark.parametrize("nb,h,w_,ci,co,k,stride,pad,dil", CONVS)
def test_qconv_parity(K, nb, h, w_, ci, co, k, stride, pad, dil):
    rng = np.random.default_rng(nb * h + ci + co + k)
    x = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
    wt = rng.integers(-128, 128, (co, k, k, ci), dtype=np.int8)
    ho = (h + 2 * pad - dil * (k - 1) - 1) // stride + 1
    wo = (w_ + 2 * pad - dil * (k - 1) - 1) // stride + 1
    md = list(O.NHWC_OHWI_METADATA) + [stride, stride, dil, dil, 1]
    padding = [pad, pad, pad, pad]
    out_shape = [nb, ho, wo, co]
    acc = O.conv_s32(x, wt, padding, md, out_shape)
    names = K.variant_names()
    variants = [-1, 0] + ([i for i, nm in enumerate(names) if nm.startswith(("mfma_", "pipe_", "dual_"))]
                          if ci % 16 == 0 else [])
    if k == 3 and stride == 1 and dil == 1 and ci in (32, 64, 128, 256):
        for i, nm in enumerate(names):
            if not nm.startswith("direct3x3_"):
                continue
            try:      # (a tile whose input patch does not fit the LDS for this shape is refused)
                K.qconv2d(dev(x), dev(wt), padding, md, out_shape, K.EPI_ACC_S32, variant=i)
                variants.append(i)
            except RuntimeError as exc:
                assert "fits the LDS" in str(exc) and nm == "direct3x3_512x64", (nm, exc)
    for v in variants:
        got = host(K.qconv2d(dev(x), dev(wt), padding, md, out_shape, K.EPI_ACC_S32, variant=v))
        np.testing.assert_array_equal(got, acc, err_msg="variant %d" % v)
    sx, sw = make_scales(rng, co)
    so = pick_so(acc, sx, sw)
    want = O.requant_cpu(acc.reshape(-1, co), sx, sw, so).reshape(out_shape)
    for v in variants:
        got = host(K.qconv2d(dev(x), dev(wt), padding, md, out_shape, K.EPI_REQUANT_CPU,
                             sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])), variant=v))
        np.testing.assert_array_equal(got, want, err_msg="variant %d" % v)
    # the integer output stage of the reference's AArch64 convolution, with an s32 bias
    b32 = rng.integers(-100000, 100000, co).astype(np.int32)
    want_fx = O.requant_fixedpoint(acc.reshape(-1, co), sx, sw, so, b32=b32, zo=-2).reshape(out_shape)
    for v in variants:
        got = host(K.qconv2d(dev(x), dev(wt), padding, md, out_shape, K.EPI_REQUANT_FIXEDPOINT,
                             sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])),
                             bias=dev(b32), zo=-2, variant=v))
        np.testing.assert_array_equal(got, want_fx, err_msg="fixed-point, variant %d" % v)
    # requant -> dequantize in the convolution's epilogue: the bits of dequantize(requant)
    want_f = O.dequantize(want, np.array([so], np.float32), np.array([0], np.int32))
    for v in variants:
        got = host(K.qconv2d(dev(x), dev(wt), padding, md, out_shape, K.EPI_REQUANT_CPU_DEQUANT_F32,
                             sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])), variant=v))
        assert got.dtype == np.float32
        assert np.array_equal(got.view(np.uint32), want_f.view(np.uint32)), "variant %d" % v


@pytest.mark.parametrize("nb,h,w_,ci,co,k,pad", [(2, 14, 14, 64, 256, 1, 0), (1, 28, 28, 128, 128, 3, 1),
                                                 (2, 9, 11, 48, 72, 3, 1), (1, 7, 7, 24, 40, 1, 0),
                                                 # the kernel with the input patch resident in LDS
                                                 (64, 32, 32, 32, 32, 3, 1), (32, 56, 56, 64, 64, 3, 1)])
def test_qconv_fused_residual_relu_quantize(K, nb, h, w_, ci, co, k, pad):
    """The tail of a ResNet block in the convolution's epilogue: dequantize -> + the block's
    int8 input (its own scale and zero point) -> ReLU -> quantize gives the bits of the
    separate library calls; so does an f32 residual with an f32 result, and a table."""
    rng = np.random.default_rng(h * 31 + ci + co)
    x = dev(rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8))
    wt = dev(rng.integers(-128, 128, (co, k, k, ci), dtype=np.int8))
    md = list(O.NHWC_OHWI_METADATA) + [1, 1, 1, 1, 1]
    padding = [pad] * 4
    out_shape = [nb, h, w_, co]
    acc = O.conv_s32(host(x), host(wt), padding, md, out_shape)
    sx, sw = make_scales(rng, co)
    so = pick_so(acc, sx, sw)
    sc = dict(sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so], np.float32)))
    bias = dev((rng.standard_normal(co) * 10 * so).astype(np.float32))
    q = K.qconv2d(x, wt, padding, md, out_shape, K.EPI_REQUANT_CPU, bias=bias, zo=2, **sc)
    zi = lambda v: torch.full((1,), v, dtype=torch.int32, device="cuda")  # noqa: E731
    y = K.dequantize(q, sc["so"], zi(2))
    rq = dev(rng.integers(-128, 128, out_shape, dtype=np.int8))
    rs, rz = dev(np.array([so * 0.8], np.float32)), -5
    s2, z2 = dev(np.array([so * 1.1], np.float32)), -128
    t = y + K.dequantize(rq, rs, zi(rz))
    t = torch.where(t < 0, torch.zeros_like(t), t)
    want = K.quantize(t, s2, zi(z2))
    got = K.qconv2d(x, wt, padding, md, out_shape, K.EPI_REQUANT_CPU, bias=bias, zo=2, **sc,
                    post=K.make_postops(residual=rq, residual_scale=rs, residual_zp=rz,
                                        relu=True, out_scale=s2, out_zp=z2))
    assert torch.equal(got, want)
    rf = dev((rng.standard_normal(out_shape) * 40 * so).astype(np.float32))
    got = K.qconv2d(x, wt, padding, md, out_shape, K.EPI_REQUANT_CPU_DEQUANT_F32, bias=bias, zo=2,
                    **sc, post=K.make_postops(residual=rf))
    assert torch.equal(got.view(torch.int32), (y + rf).view(torch.int32))
    table = dev(rng.integers(-128, 128, 256, dtype=np.int8))
    got = K.qconv2d(x, wt, padding, md, out_shape, K.EPI_REQUANT_CPU, bias=bias, zo=2, **sc,
                    post=K.make_postops(table=table))
    assert torch.equal(got, K.lut8(q, table))


def test_qconv_1x1_with_many_tiles_keeps_the_fixed_point_stage_and_fused_operators(K):
    """A 1x1 convolution runs as a plain GEMM over the pixels; with several rounds of tiles the
    plain GEMM would take its persistent kernels, which carry neither the fixed-point stage nor
    fused operators -- the dispatch has to stay on the kernels that do."""
    rng = np.random.default_rng(5)
    nb, h, ci, co = 32, 56, 64, 256                      # 100352 x 64 -> 256: 392 tiles of 256 x 256, two rounds
    x = dev(rng.integers(-128, 128, (nb, h, h, ci), dtype=np.int8))
    wt = dev(rng.integers(-128, 128, (co, 1, 1, ci), dtype=np.int8))
    md = list(O.NHWC_OHWI_METADATA) + [1, 1, 1, 1, 1]
    osh = [nb, h, h, co]
    acc, _ = O.gemm_s32_fast(host(x).reshape(-1, ci), host(wt).reshape(co, ci))
    sx, sw = make_scales(rng, co)
    so = pick_so(acc, sx, sw)
    sc = dict(sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so], np.float32)))
    b32 = rng.integers(-1000, 1000, co).astype(np.int32)
    want = O.requant_fixedpoint(acc, sx, sw, so, b32=b32, zo=1).reshape(osh)
    got = K.qconv2d(x, wt, [0] * 4, md, osh, K.EPI_REQUANT_FIXEDPOINT, bias=dev(b32), zo=1, **sc)
    np.testing.assert_array_equal(host(got), want)
    table = dev(rng.integers(-128, 128, 256, dtype=np.int8))
    q = K.qconv2d(x, wt, [0] * 4, md, osh, K.EPI_REQUANT_CPU, **sc)
    np.testing.assert_array_equal(host(q), O.requant_cpu(acc, sx, sw, so).reshape(osh))
    got = K.qconv2d(x, wt, [0] * 4, md, osh, K.EPI_REQUANT_CPU, **sc, post=K.make_postops(table=table))
    assert torch.equal(got, K.lut8(q, table))
    # the same through the GEMM entry
    a2, w2 = x.reshape(-1, ci), wt.reshape(co, ci)
    got = K.qgemm(a2, w2, K.EPI_REQUANT_FIXEDPOINT, bias=dev(b32), zo=1, **sc)
    np.testing.assert_array_equal(host(got), want.reshape(-1, co))
    got = K.qgemm(a2, w2, K.EPI_REQUANT_CPU, **sc, post=K.make_postops(table=table))
    assert torch.equal(got, K.lut8(q, table).reshape(-1, co))


def test_qconv_direct_random_shapes(K):
    """Seeded sweep for the kernels that keep the input patch in LDS: image sizes that make
    tiles start and end anywhere in a row, every channel count, ragged output channels,
    asymmetric padding, both tile shapes, two epilogues -- bit-exact against the oracle."""
    rng = np.random.default_rng(20250117)
    names = K.variant_names()
    direct = [i for i, nm in enumerate(names) if nm.startswith("direct3x3_")]
    for case in range(24):
        nb = int(rng.integers(1, 4))
        h = int(rng.integers(3, 40))
        w_ = int(rng.integers(3, 70))
        ci = int(rng.choice([32, 64, 128, 256]))
        co = int(rng.choice([8, 17, 64, 72, 130]))
        pad = [int(v) for v in rng.integers(0, 3, 4)]          # top, bottom, left, right
        ho, wo = h + pad[0] + pad[1] - 2, w_ + pad[2] + pad[3] - 2
        if ho < 1 or wo < 1 or (ho + 10) * (wo + 2) * ci > 120 * 1024:
            continue
        x = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
        wt = rng.integers(-128, 128, (co, 3, 3, ci), dtype=np.int8)
        md = list(O.NHWC_OHWI_METADATA) + [1, 1, 1, 1, 1]
        out_shape = [nb, ho, wo, co]
        acc = O.conv_s32(x, wt, pad, md, out_shape)
        sx, sw = make_scales(rng, co)
        so = pick_so(acc, sx, sw)
        want = O.requant_cpu(acc.reshape(-1, co), sx, sw, so).reshape(out_shape)
        tag = "case %d: %dx%dx%dx%d -> %d pad %s" % (case, nb, h, w_, ci, co, pad)
        for v in direct:
            got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_ACC_S32, variant=v))
            np.testing.assert_array_equal(got, acc, err_msg=tag + " variant %d" % v)
            got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU,
                                 sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])),
                                 variant=v))
            np.testing.assert_array_equal(got, want, err_msg=tag + " variant %d" % v)



def test_qconv_strided_pointwise_rows_are_pixels(K):
    """1 x 1 filters with unequal strides, and with fused operators, on the path that finds each
    GEMM row's input pixel once and then runs the plain GEMM's loop: against the oracle, the
    implicit-GEMM kernel and the separate calls."""
    rng = np.random.default_rng(20260618)
    names = K.variant_names()
    pipe128 = names.index("pipe_128x128x128")
    for nb, h, w_, ci, co, sh, sw_ in [(2, 13, 17, 64, 96, 2, 1), (3, 16, 9, 128, 200, 1, 2), (1, 30, 31, 32, 64, 3, 2),
                                      (16, 28, 28, 256, 512, 2, 2), (4, 56, 56, 64, 128, 2, 2)]:
        x = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
        wt = rng.integers(-128, 128, (co, 1, 1, ci), dtype=np.int8)
        ho, wo = (h - 1) // sh + 1, (w_ - 1) // sw_ + 1
        md = list(O.NHWC_OHWI_METADATA) + [sh, sw_, 1, 1, 1]
        out_shape, pad = [nb, ho, wo, co], [0, 0, 0, 0]
        acc = O.conv_s32(x, wt, pad, md, out_shape)
        tag = "%dx%dx%dx%d -> %d, strides %d %d" % (nb, h, w_, ci, co, sh, sw_)
        np.testing.assert_array_equal(host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_ACC_S32)), acc,
                                      err_msg=tag)
        sx, sw = make_scales(rng, co)
        so = pick_so(acc, sx, sw)
        sc = dict(sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])))
        bf = (rng.standard_normal(co) * 30).astype(np.float32)
        got = K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_GPU, bias=dev(bf), **sc)
        np.testing.assert_array_equal(host(got), O.requant_gpu(acc.reshape(-1, co), sx, sw, so, bias_f32=bf).reshape(out_shape),
                                      err_msg=tag)
        assert torch.equal(got, K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_GPU, bias=dev(bf),
                                          variant=pipe128, **sc)), tag
        plain = K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU, **sc)
        res = dev(rng.standard_normal(out_shape).astype(np.float32) * 300)
        s2, z1 = dev(np.array([7.0], np.float32)), torch.zeros(1, dtype=torch.int32, device="cuda")
        fused = K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU, **sc,
                          post=K.make_postops(residual=res, relu=True, out_scale=s2, out_zp=-3))
        t = torch.clamp_min(K.dequantize(plain, sc["so"], z1) + res, 0.0)
        assert torch.equal(fused, K.quantize(t, s2, torch.full((1,), -3, dtype=torch.int32, device="cuda"))), tag


def test_qconv_library_choice_on_random_shapes(K):
    """Seeded sweep over what decides the kernel of a convolution -- channel counts with and
    without a register-filter instance, 1 x 1 to 7 x 7 filters, strides, paddings, batch and
    image sizes from one pixel tile to many, ragged output channels, every int8 epilogue and
    bias kind: whatever the library picks gives the bytes of the generic kernel (one thread
    per result; pinned to the oracle by the tests above)."""
    rng = np.random.default_rng(20260507)
    gen = K.variant_names().index("generic")
    md0 = list(O.NHWC_OHWI_METADATA)
    done = 0
    for case in range(500):
        ci = int(rng.choice([3, 4, 16, 32, 64, 64, 128, 128, 256, 256, 512]))
        k = int(rng.choice([7, 3, 5])) if ci <= 4 else int(rng.choice([1, 1, 1, 3, 3, 2]))
        s = int(rng.choice([1, 1, 1, 2]))
        pad = int(rng.choice([0, k // 2, 1 if k > 1 else 0]))
        big = rng.random() < 0.3
        nb = int(rng.integers(1, 40 if big else 6))
        lo, hi = max(k - 2 * pad, 1), 30 if big else 60
        h, w_ = int(rng.integers(lo, hi)), int(rng.integers(lo, hi))
        if ci <= 4:
            h, w_ = 3 * h + 7, 3 * w_ + 7
        co = int(rng.choice([16, 32, 48, 64, 80, 128, 144, 208, 256, 512, 1024, int(rng.integers(1, 300))]))
        ho, wo = (h + 2 * pad - k) // s + 1, (w_ + 2 * pad - k) // s + 1
        if ho < 1 or wo < 1 or nb * ho * wo * co > 3e7 or nb * h * w_ * ci > 3e7:
            continue
        x = dev(rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8))
        wt = dev(rng.integers(-128, 128, (co, k, k, ci), dtype=np.int8))
        out_shape, md = [nb, ho, wo, co], md0 + [s, s, 1, 1, 1]
        so = np.float32(0.02 * 0.025 * 74.0 * 74.0 * np.sqrt(k * k * ci) / 40.0)
        kw = dict(sx=dev(np.array([0.02], np.float32)), sw=dev(rng.uniform(0.001, 0.05, co).astype(np.float32)),
                  so=dev(np.array([so])))
        kind, epi = int(rng.integers(0, 4)), K.EPI_REQUANT_CPU
        if kind == 1:
            kw.update(bias=dev((rng.standard_normal(co) * 3 * so).astype(np.float32)), zo=int(rng.integers(-10, 10)))
        elif kind == 2:
            kw.update(bias=dev(rng.integers(-100000, 100000, co).astype(np.int32)))
        elif kind == 3:
            epi = K.EPI_REQUANT_GPU
            kw.update(bias=dev((rng.standard_normal(co) * 30).astype(np.float32)))
        got = K.qconv2d(x, wt, [pad] * 4, md, out_shape, epi, **kw)
        want = K.qconv2d(x, wt, [pad] * 4, md, out_shape, epi, variant=gen, **kw)
        assert torch.equal(got, want), "case %d: %dx%dx%dx%d, %dx%d stride %d pad %d -> %d, bias kind %d" % (
            case, nb, h, w_, ci, k, k, s, pad, co, kind)
        done += 1
    assert done > 400


def test_qconv_stream_variant(K):
    """The 3 x 3 kernel (64 or 128 input channels) that keeps the filter in registers: images whose pixel
    tiles start and end anywhere in a row, one to many tiles per image, ragged and several
    64-channel slices of output channels, asymmetric padding, both int8 epilogues with every
    bias kind they take and an output zero point -- bit-exact against the oracle; then what it
    must refuse."""
    rng = np.random.default_rng(20260311)
    sv = K.variant_names().index("stream")
    md = list(O.NHWC_OHWI_METADATA) + [1, 1, 1, 1, 1]
    shapes = [(2, 56, 56, 64, 64, [1, 1, 1, 1]), (1, 3, 3, 64, 16, [1, 1, 1, 1]), (3, 9, 7, 64, 80, [0, 0, 0, 0]),
              (1, 6, 150, 64, 64, [1, 1, 1, 1]), (1, 33, 17, 64, 208, [2, 0, 1, 2]),
              (5, 28, 28, 64, 128, [1, 1, 1, 1]), (1, 112, 112, 64, 64, [1, 1, 1, 1]),
              (40, 14, 14, 64, 64, [0, 2, 2, 0]),
              # 128 input channels: 32-channel slices, several slices per pixel tile
              (3, 28, 28, 128, 128, [1, 1, 1, 1]), (1, 5, 4, 128, 16, [1, 1, 1, 1]),
              (2, 17, 33, 128, 80, [0, 2, 2, 1]), (9, 14, 14, 128, 256, [1, 1, 1, 1]),
              (1, 56, 56, 128, 48, [1, 1, 1, 1])]
    for nb, h, w_, ci, co, pad in shapes:
        ho, wo = h + pad[0] + pad[1] - 2, w_ + pad[2] + pad[3] - 2
        x = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
        wt = rng.integers(-128, 128, (co, 3, 3, ci), dtype=np.int8)
        out_shape = [nb, ho, wo, co]
        acc = O.conv_s32(x, wt, pad, md, out_shape)
        sx, sw = make_scales(rng, co)
        so = pick_so(acc, sx, sw)
        scales = dict(sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])))
        tag = "%dx%dx%dx%d -> %d pad %s" % (nb, h, w_, ci, co, pad)
        a2 = acc.reshape(-1, co)
        # E1: plain, f32 bias (folded to s32 as the library does) with an output zero point, s32 bias
        got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU, variant=sv, **scales))
        np.testing.assert_array_equal(got, O.requant_cpu(a2, sx, sw, so).reshape(out_shape), err_msg=tag)
        bf = (rng.standard_normal(co) * 40 * so).astype(np.float32)
        b32 = O.bias_f32_to_s32(bf, sx, sw)
        got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU, bias=dev(bf), zo=3,
                             variant=sv, **scales))
        np.testing.assert_array_equal(got, O.requant_cpu(a2, sx, sw, so, b32=b32, zo=3).reshape(out_shape),
                                      err_msg=tag + " f32 bias")
        bi = rng.integers(-2000000, 2000000, co).astype(np.int32)
        got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU, bias=dev(bi), zo=-5,
                             variant=sv, **scales))
        np.testing.assert_array_equal(got, O.requant_cpu(a2, sx, sw, so, b32=bi, zo=-5).reshape(out_shape),
                                      err_msg=tag + " s32 bias")
        # E2: f32 bias in output units, int8 bias
        bo = (rng.standard_normal(co) * 30).astype(np.float32)
        got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_GPU, bias=dev(bo),
                             variant=sv, **scales))
        np.testing.assert_array_equal(got, O.requant_gpu(a2, sx, sw, so, bias_f32=bo).reshape(out_shape),
                                      err_msg=tag + " E2 f32 bias")
        b8 = rng.integers(-128, 128, co, dtype=np.int8)
        got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_GPU, bias=dev(b8),
                             variant=sv, **scales))
        np.testing.assert_array_equal(got, O.requant_gpu(a2, sx, sw, so, bias_i8=b8).reshape(out_shape),
                                      err_msg=tag + " E2 s8 bias")
        # the library's own choice for this shape gives the same bytes
        auto = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_GPU, bias=dev(b8), **scales))
        np.testing.assert_array_equal(auto, got, err_msg=tag + " heuristic")
    # operators fused behind the convolution run in this kernel too (the library picks it for
    # these shapes): residual (+ ReLU) + quantize and a table, against the separate calls
    for nb, h, w_, ci, co in [(2, 56, 56, 64, 64), (3, 28, 28, 128, 128), (1, 9, 11, 64, 80)]:
        x = dev(rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8))
        wt = dev(rng.integers(-128, 128, (co, 3, 3, ci), dtype=np.int8))
        out_shape = [nb, h, w_, co]
        sc = dict(sx=dev(np.array([0.02], np.float32)), sw=dev(rng.uniform(0.001, 0.05, co).astype(np.float32)),
                  so=dev(np.array([9.0], np.float32)))
        plain = K.qconv2d(x, wt, [1, 1, 1, 1], md, out_shape, K.EPI_REQUANT_CPU, **sc)
        z1 = torch.zeros(1, dtype=torch.int32, device="cuda")
        res = dev(rng.standard_normal(out_shape).astype(np.float32) * 300)
        s2 = dev(np.array([7.0], np.float32))
        for relu in (False, True):
            fused = K.qconv2d(x, wt, [1, 1, 1, 1], md, out_shape, K.EPI_REQUANT_CPU, **sc,
                              post=K.make_postops(residual=res, relu=relu, out_scale=s2, out_zp=-3))
            t = K.dequantize(plain, sc["so"], z1) + res
            if relu:
                t = torch.clamp_min(t, 0.0)
            want = K.quantize(t, s2, torch.full((1,), -3, dtype=torch.int32, device="cuda"))
            assert torch.equal(fused, want), (nb, h, w_, ci, co, relu)
        table = K.activation_table(torch.nn.functional.gelu, sc["so"], z1, s2, z1)
        fused = K.qconv2d(x, wt, [1, 1, 1, 1], md, out_shape, K.EPI_REQUANT_CPU, **sc,
                          post=K.make_postops(table=table))
        assert torch.equal(fused, K.lut8(plain, table))
    # refusals: 4-byte results, other channel counts and filters, strides
    x = dev(rng.integers(-128, 128, (1, 8, 8, 64), dtype=np.int8))
    wt = dev(rng.integers(-128, 128, (64, 3, 3, 64), dtype=np.int8))
    with pytest.raises(RuntimeError, match="streaming variant"):
        K.qconv2d(x, wt, [1, 1, 1, 1], md, [1, 8, 8, 64], K.EPI_ACC_S32, variant=sv)
    one = dev(np.array([0.01], np.float32))
    x32 = dev(rng.integers(-128, 128, (1, 8, 8, 32), dtype=np.int8))
    w32 = dev(rng.integers(-128, 128, (64, 3, 3, 32), dtype=np.int8))
    with pytest.raises(RuntimeError, match="streaming variant"):
        K.qconv2d(x32, w32, [1, 1, 1, 1], md, [1, 8, 8, 64], K.EPI_REQUANT_CPU, sx=one, sw=one, so=one, variant=sv)
    md2 = list(O.NHWC_OHWI_METADATA) + [2, 2, 1, 1, 1]
    with pytest.raises(RuntimeError, match="streaming variant"):
        K.qconv2d(x, wt, [1, 1, 1, 1], md2, [1, 4, 4, 64], K.EPI_REQUANT_CPU, sx=one, sw=one, so=one, variant=sv)


def test_qconv_stream_16_channels(K):
    """4 x 4 filters on 16 channels (what a 7 x 7 stride-2 stem becomes after space to depth) in
    the kernel that keeps the filter in registers: an MFMA step's 32 bytes of k are two
    neighbouring patch pixels.  Bit-exact against the oracle, forced and as the library's choice,
    and the stem itself (3 channels, stride 2) through the library against the oracle."""
    rng = np.random.default_rng(20260413)
    sv = K.variant_names().index("stream")
    md = list(O.NHWC_OHWI_METADATA) + [1, 1, 1, 1, 1]
    for nb, h, w_, co, pad in [(2, 115, 115, 64, [0, 0, 0, 0]), (1, 9, 12, 80, [1, 2, 0, 3]),
                               (3, 30, 31, 16, [0, 0, 0, 0]), (1, 131, 67, 96, [3, 0, 1, 1]),
                               (9, 20, 20, 64, [0, 0, 0, 0])]:
        ho, wo = h + pad[0] + pad[1] - 3, w_ + pad[2] + pad[3] - 3
        x = rng.integers(-128, 128, (nb, h, w_, 16), dtype=np.int8)
        wt = rng.integers(-128, 128, (co, 4, 4, 16), dtype=np.int8)
        out_shape = [nb, ho, wo, co]
        acc = O.conv_s32(x, wt, pad, md, out_shape)
        sx, sw = make_scales(rng, co)
        so = pick_so(acc, sx, sw)
        scales = dict(sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])))
        tag = "%dx%dx%dx16 -> %d pad %s" % (nb, h, w_, co, pad)
        a2 = acc.reshape(-1, co)
        bi = rng.integers(-200000, 200000, co).astype(np.int32)
        got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU, bias=dev(bi), zo=-5,
                             variant=sv, **scales))
        np.testing.assert_array_equal(got, O.requant_cpu(a2, sx, sw, so, b32=bi, zo=-5).reshape(out_shape),
                                      err_msg=tag + " s32 bias")
        bo = (rng.standard_normal(co) * 30).astype(np.float32)
        got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_GPU, bias=dev(bo),
                             variant=sv, **scales))
        np.testing.assert_array_equal(got, O.requant_gpu(a2, sx, sw, so, bias_f32=bo).reshape(out_shape),
                                      err_msg=tag + " E2 f32 bias")
        auto = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_GPU, bias=dev(bo), **scales))
        np.testing.assert_array_equal(auto, got, err_msg=tag + " heuristic")
    # the stem: 7 x 7, stride 2, padding 3, three channels
    md2 = list(O.NHWC_OHWI_METADATA) + [2, 2, 1, 1, 1]
    for nb, h in [(2, 224), (1, 97)]:
        ho = (h + 6 - 7) // 2 + 1
        x = rng.integers(-128, 128, (nb, h, h, 3), dtype=np.int8)
        wt = rng.integers(-128, 128, (64, 7, 7, 3), dtype=np.int8)
        out_shape = [nb, ho, ho, 64]
        acc = O.conv_s32(x, wt, [3, 3, 3, 3], md2, out_shape)
        sx, sw = make_scales(rng, 64)
        so = pick_so(acc, sx, sw)
        got = host(K.qconv2d(dev(x), dev(wt), [3, 3, 3, 3], md2, out_shape, K.EPI_REQUANT_CPU,
                             sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so]))))
        np.testing.assert_array_equal(got, O.requant_cpu(acc.reshape(-1, 64), sx, sw, so).reshape(out_shape),
                                      err_msg="stem %d x %d" % (nb, h))


def test_qconv_stream_pointwise(K):
    """1 x 1 filters on 64 to 256 input channels in the kernel that keeps the filter in registers
    (a GEMM over the pixels with a short k): pixel counts that are and are not a multiple of 16
    (one long row of pixels cut anywhere, or tiles per image), one pixel tile to many, tiles
    that end inside a block of 32 pixels, ragged channel slices, both slice widths of the
    64-channel filter, every bias kind of the int8 epilogues, fused operators -- bit-exact
    against the oracle and against the library's choice; then what it must refuse."""
    rng = np.random.default_rng(20260412)
    names = K.variant_names()
    sv = names.index("stream")
    md = list(O.NHWC_OHWI_METADATA) + [1, 1, 1, 1, 1]
    pad = [0, 0, 0, 0]
    shapes = [(8, 56, 56, 64, 256), (2, 56, 56, 64, 64), (4, 28, 28, 128, 512), (3, 7, 7, 128, 2048),
              (1, 4, 4, 128, 16), (5, 9, 7, 64, 208), (1, 1, 48, 64, 80), (7, 13, 3, 128, 144),
              (2, 23, 5, 128, 96), (1, 56, 56, 128, 64), (1, 1, 16, 64, 16), (3, 5, 11, 64, 400),
              (1, 1, 33, 64, 48), (16, 112, 112, 64, 64), (1, 300, 301, 128, 128),
              # 256 input channels: 64-channel slices, one round of workgroups and several
              (32, 14, 14, 256, 1024), (3, 9, 7, 256, 208), (2, 56, 56, 256, 64), (1, 5, 3, 256, 16)]
    for nb, h, w_, ci, co in shapes:
        x = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
        wt = rng.integers(-128, 128, (co, 1, 1, ci), dtype=np.int8)
        out_shape = [nb, h, w_, co]
        acc = x.reshape(-1, ci).astype(np.int32) @ wt.reshape(co, ci).astype(np.int32).T
        sx, sw = make_scales(rng, co)
        so = pick_so(acc, sx, sw)
        scales = dict(sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])))
        tag = "%dx%dx%dx%d -> %d" % (nb, h, w_, ci, co)
        for v in (sv,):
            got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU, variant=v, **scales))
            np.testing.assert_array_equal(got, O.requant_cpu(acc, sx, sw, so).reshape(out_shape), err_msg=tag)
            bf = (rng.standard_normal(co) * 40 * so).astype(np.float32)
            b32 = O.bias_f32_to_s32(bf, sx, sw)
            got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU, bias=dev(bf), zo=3,
                                 variant=v, **scales))
            np.testing.assert_array_equal(got, O.requant_cpu(acc, sx, sw, so, b32=b32, zo=3).reshape(out_shape),
                                          err_msg=tag + " f32 bias")
            bi = rng.integers(-2000000, 2000000, co).astype(np.int32)
            got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU, bias=dev(bi), zo=-5,
                                 variant=v, **scales))
            np.testing.assert_array_equal(got, O.requant_cpu(acc, sx, sw, so, b32=bi, zo=-5).reshape(out_shape),
                                          err_msg=tag + " s32 bias")
            bo = (rng.standard_normal(co) * 30).astype(np.float32)
            got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_GPU, bias=dev(bo),
                                 variant=v, **scales))
            np.testing.assert_array_equal(got, O.requant_gpu(acc, sx, sw, so, bias_f32=bo).reshape(out_shape),
                                          err_msg=tag + " E2 f32 bias")
            b8 = rng.integers(-128, 128, co, dtype=np.int8)
            got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_GPU, bias=dev(b8),
                                 variant=v, **scales))
            np.testing.assert_array_equal(got, O.requant_gpu(acc, sx, sw, so, bias_i8=b8).reshape(out_shape),
                                          err_msg=tag + " E2 s8 bias")
            auto = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_GPU, bias=dev(b8), **scales))
            np.testing.assert_array_equal(auto, got, err_msg=tag + " heuristic")
    # fused operators: residual (+ ReLU) + quantize and a table, against the separate calls
    for nb, h, w_, ci, co in [(32, 28, 28, 64, 256), (2, 28, 28, 128, 512), (1, 9, 11, 64, 80), (40, 56, 56, 128, 128),
                              (8, 14, 14, 256, 1024)]:   # fused on 256 channels: the GEMM tiles' result
        x = dev(rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8))
        wt = dev(rng.integers(-128, 128, (co, 1, 1, ci), dtype=np.int8))
        out_shape = [nb, h, w_, co]
        sc = dict(sx=dev(np.array([0.02], np.float32)), sw=dev(rng.uniform(0.001, 0.05, co).astype(np.float32)),
                  so=dev(np.array([4.0], np.float32)))
        z1 = torch.zeros(1, dtype=torch.int32, device="cuda")
        res = dev(rng.standard_normal(out_shape).astype(np.float32) * 300)
        s2 = dev(np.array([7.0], np.float32))
        plain = K.qconv2d(x, wt, pad, md, out_shape, K.EPI_REQUANT_CPU, variant=sv, **sc)
        for relu in (False, True):
            fused = K.qconv2d(x, wt, pad, md, out_shape, K.EPI_REQUANT_CPU, **sc,
                              post=K.make_postops(residual=res, relu=relu, out_scale=s2, out_zp=-3))
            t = K.dequantize(plain, sc["so"], z1) + res
            if relu:
                t = torch.clamp_min(t, 0.0)
            want = K.quantize(t, s2, torch.full((1,), -3, dtype=torch.int32, device="cuda"))
            assert torch.equal(fused, want), (nb, h, w_, ci, co, relu)
        table = K.activation_table(torch.nn.functional.gelu, sc["so"], z1, s2, z1)
        fused = K.qconv2d(x, wt, pad, md, out_shape, K.EPI_REQUANT_CPU, **sc,
                          post=K.make_postops(table=table))
        assert torch.equal(fused, K.lut8(plain, table)), (nb, h, w_, ci, co)
    # refusals: channel counts without an instance, strides, 4-byte results
    one = dev(np.array([0.01], np.float32))
    for ci, v in ((32, sv), (512, sv)):
        x = dev(rng.integers(-128, 128, (1, 8, 8, ci), dtype=np.int8))
        wt = dev(rng.integers(-128, 128, (64, 1, 1, ci), dtype=np.int8))
        with pytest.raises(RuntimeError, match="streaming variant"):
            K.qconv2d(x, wt, pad, md, [1, 8, 8, 64], K.EPI_REQUANT_CPU, sx=one, sw=one, so=one, variant=v)
    x = dev(rng.integers(-128, 128, (1, 8, 8, 64), dtype=np.int8))
    wt = dev(rng.integers(-128, 128, (64, 1, 1, 64), dtype=np.int8))
    with pytest.raises(RuntimeError, match="streaming variant"):
        K.qconv2d(x, wt, pad, md, [1, 8, 8, 64], K.EPI_ACC_S32, variant=sv)
    md2 = list(O.NHWC_OHWI_METADATA) + [2, 2, 1, 1, 1]
    with pytest.raises(RuntimeError, match="streaming variant"):
        K.qconv2d(x, wt, pad, md2, [1, 4, 4, 64], K.EPI_REQUANT_CPU, sx=one, sw=one, so=one, variant=sv)


def test_qconv_direct_other_filter_sizes(K):
    """The same kernels on filters other than 3 x 3 (up to 7 x 7, rectangular ones too) and on
    16 channels with an even filter width, where an MFMA step's 32 bytes of k are two
    neighbouring patch pixels (the stride-1 form of a stem convolution after space to depth):
    bit-exact against the oracle for every tile shape that accepts the problem."""
    rng = np.random.default_rng(20260303)
    names = K.variant_names()
    direct = [i for i, nm in enumerate(names) if nm.startswith("direct3x3_")]
    ran = 0
    for (nb, h, w_, ci, co, kh, kw, pad) in [
            (2, 20, 30, 32, 64, 5, 5, [2, 2, 2, 2]), (1, 16, 16, 64, 40, 7, 7, [3, 3, 3, 3]),
            (2, 12, 25, 32, 64, 1, 3, [0, 0, 1, 1]), (1, 18, 18, 128, 17, 2, 2, [0, 1, 0, 1]),
            (2, 35, 35, 16, 64, 4, 4, [0, 0, 0, 0]), (3, 19, 40, 16, 48, 2, 2, [1, 0, 0, 1]),
            (1, 60, 115, 16, 64, 4, 4, [0, 0, 0, 0]), (1, 14, 14, 16, 8, 3, 6, [1, 1, 2, 3])]:
        ho, wo = h + pad[0] + pad[1] - kh + 1, w_ + pad[2] + pad[3] - kw + 1
        x = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
        wt = rng.integers(-128, 128, (co, kh, kw, ci), dtype=np.int8)
        md = list(O.NHWC_OHWI_METADATA) + [1, 1, 1, 1, 1]
        out_shape = [nb, ho, wo, co]
        acc = O.conv_s32(x, wt, pad, md, out_shape)
        sx, sw = make_scales(rng, co)
        so = pick_so(acc, sx, sw)
        want = O.requant_cpu(acc.reshape(-1, co), sx, sw, so).reshape(out_shape)
        tag = "%dx%dx%dx%d -> %d, %dx%d pad %s" % (nb, h, w_, ci, co, kh, kw, pad)
        for v in direct:
            try:
                got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_ACC_S32, variant=v))
            except RuntimeError as exc:
                assert "fits the LDS" in str(exc), (tag, names[v], exc)
                continue
            ran += 1
            np.testing.assert_array_equal(got, acc, err_msg=tag + " " + names[v])
            got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_REQUANT_CPU,
                                 sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])),
                                 variant=v))
            np.testing.assert_array_equal(got, want, err_msg=tag + " " + names[v])
        got = host(K.qconv2d(dev(x), dev(wt), pad, md, out_shape, K.EPI_ACC_S32))
        np.testing.assert_array_equal(got, acc, err_msg=tag + " auto")
    assert ran >= 20
    # 16 channels and an odd filter width: no layout for that
    x = rng.integers(-128, 128, (1, 8, 8, 16), dtype=np.int8)
    wt = rng.integers(-128, 128, (8, 3, 3, 16), dtype=np.int8)
    md = list(O.NHWC_OHWI_METADATA) + [1, 1, 1, 1, 1]
    for v in direct:
        with pytest.raises(RuntimeError, match="direct variants"):
            K.qconv2d(dev(x), dev(wt), [1] * 4, md, [1, 8, 8, 8], K.EPI_ACC_S32, variant=v)


def test_qconv_direct_variants_refuse_what_they_cannot_run(K):
    """A named direct-convolution variant fails with an error, not a wrong result, on a
    filter of a single tap or a stride other than 1, on a channel count it has no layout for, and on an image
    row too wide for its patch to fit the LDS; the automatic choice runs all of them."""
    names = K.variant_names()
    direct = [i for i, nm in enumerate(names) if nm.startswith("direct3x3_")]
    assert direct
    rng = np.random.default_rng(5)
    cases = [  # nb, h, w, ci, co, k, stride
        (1, 8, 8, 64, 64, 1, 1),
        (1, 9, 9, 64, 64, 3, 2),
        (1, 8, 8, 48, 64, 3, 1),
        (1, 4, 300, 256, 64, 3, 1),
    ]
    for nb, h, w_, ci, co, k, stride in cases:
        pad = k // 2
        x = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
        wt = rng.integers(-128, 128, (co, k, k, ci), dtype=np.int8)
        ho = (h + 2 * pad - k) // stride + 1
        wo = (w_ + 2 * pad - k) // stride + 1
        md = list(O.NHWC_OHWI_METADATA) + [stride, stride, 1, 1, 1]
        out_shape = [nb, ho, wo, co]
        for v in direct:
            with pytest.raises(RuntimeError, match="direct variants"):
                K.qconv2d(dev(x), dev(wt), [pad] * 4, md, out_shape, K.EPI_ACC_S32, variant=v)
        got = host(K.qconv2d(dev(x), dev(wt), [pad] * 4, md, out_shape, K.EPI_ACC_S32))
        np.testing.assert_array_equal(got, O.conv_s32(x, wt, [pad] * 4, md, out_shape))


def test_qconv_nchw_oihw_generic(K):
    rng = np.random.default_rng(77)
    x = rng.integers(-128, 128, (2, 4, 6, 6), dtype=np.int8)       # NCHW
    wt = rng.integers(-128, 128, (3, 4, 3, 3), dtype=np.int8)      # OIHW
    md = [0, 1, 2, 3, 1, 0, 2, 3, 0, 1, 2, 3, 1, 1, 1, 1, 1]
    acc = O.conv_s32(x, wt, [1, 1, 1, 1], md, [2, 3, 6, 6])
    got = host(K.qconv2d(dev(x), dev(wt), [1, 1, 1, 1], md, [2, 3, 6, 6], K.EPI_ACC_S32))
    np.testing.assert_array_equal(got, acc)


@pytest.mark.parametrize("nb,ci,h,w_,co,k,stride,pad,dil", [(2, 32, 14, 14, 48, 3, 1, 1, 1), (3, 24, 9, 11, 40, 3, 2, 1, 1),
                                                         (1, 64, 28, 28, 64, 1, 1, 0, 1), (2, 16, 12, 12, 20, 3, 1, 2, 2)])
def test_qconv_nchw_oihw_on_the_mfma_path(K, nb, ci, h, w_, co, k, stride, pad, dil):
    """NCHW x OIHW -> NCHW with scratch: tensors re-laid out as NHWC / OHWI, MFMA kernels, result
    turned back -- the same bits as the oracle and as the generic kernel without scratch, for
    every epilogue family (int8, int32 and f32 results)."""
    rng = np.random.default_rng(ci + co + h)
    x = rng.integers(-128, 128, (nb, ci, h, w_), dtype=np.int8)
    wt = rng.integers(-128, 128, (co, ci, k, k), dtype=np.int8)
    ho = (h + 2 * pad - dil * (k - 1) - 1) // stride + 1
    wo = (w_ + 2 * pad - dil * (k - 1) - 1) // stride + 1
    md = [0, 1, 2, 3, 1, 0, 2, 3, 0, 1, 2, 3, stride, stride, dil, dil, 1]
    padding, osh = [pad] * 4, [nb, co, ho, wo]
    acc = O.conv_s32(x, wt, padding, md, osh)
    for ws in (True, False):
        got = host(K.qconv2d(dev(x), dev(wt), padding, md, osh, K.EPI_ACC_S32, workspace=ws))
        np.testing.assert_array_equal(got, acc)
    sx, sw = make_scales(rng, co)
    so = pick_so(acc, sx, sw)
    sc = dict(sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so], np.float32)))
    per_c = lambda a: np.moveaxis(a, 1, -1).reshape(-1, co)                      # noqa: E731
    back = lambda a: np.moveaxis(a.reshape(nb, ho, wo, co), -1, 1)               # noqa: E731
    want = back(O.requant_cpu(per_c(acc), sx, sw, so))
    got = host(K.qconv2d(dev(x), dev(wt), padding, md, osh, K.EPI_REQUANT_CPU, **sc))
    np.testing.assert_array_equal(got, want)
    b32 = rng.integers(-100000, 100000, co).astype(np.int32)
    want = back(O.requant_fixedpoint(per_c(acc), sx, sw, so, b32=b32, zo=3))
    got = host(K.qconv2d(dev(x), dev(wt), padding, md, osh, K.EPI_REQUANT_FIXEDPOINT, bias=dev(b32),
                         zo=3, **sc))
    np.testing.assert_array_equal(got, want)
    got_f = host(K.qconv2d(dev(x), dev(wt), padding, md, osh, K.EPI_REQUANT_CPU_DEQUANT_F32, **sc))
    want_f = O.dequantize(back(O.requant_cpu(per_c(acc), sx, sw, so)), np.array([so], np.float32),
                          np.array([0], np.int32))
    assert np.array_equal(got_f.view(np.uint32), want_f.view(np.uint32))


@pytest.mark.parametrize("nb,ci,h,w_,co,k,pads", [(2, 3, 32, 32, 64, 7, (3, 3, 3, 3)), (1, 3, 17, 23, 20, 7, (3, 2, 2, 3)),
                                                 (3, 1, 12, 12, 16, 3, (1, 1, 1, 1)), (2, 4, 15, 14, 33, 5, (2, 2, 2, 2)),
                                                 (1, 2, 9, 9, 8, 2, (0, 0, 0, 0)), (2, 3, 8, 8, 64, 3, (0, 1, 0, 1)),
                                                 (1, 3, 4, 4, 8, 7, (3, 3, 3, 3))])
def test_qconv_stride2_few_channels_space_to_depth(K, nb, ci, h, w_, co, k, pads):
    """Stride-2 convolutions of images with at most 4 channels (the 7 x 7 stem of a vision
    network): with scratch they run as a stride-1 convolution of the space-to-depth image on
    the MFMA kernels -- the same bits as the oracle and as the path without scratch; odd and
    even filter sizes, asymmetric padding, odd image sizes, an image so small that the
    space-to-depth copy is larger than the padded one, NCHW x OIHW on top."""
    rng = np.random.default_rng(ci * 100 + k + h)
    x = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
    wt = rng.integers(-128, 128, (co, k, k, ci), dtype=np.int8)
    ho = (h + pads[0] + pads[1] - k) // 2 + 1
    wo = (w_ + pads[2] + pads[3] - k) // 2 + 1
    md = list(O.NHWC_OHWI_METADATA) + [2, 2, 1, 1, 1]
    padding, osh = list(pads), [nb, ho, wo, co]
    acc = O.conv_s32(x, wt, padding, md, osh)
    for ws in (True, False):
        got = host(K.qconv2d(dev(x), dev(wt), padding, md, osh, K.EPI_ACC_S32, workspace=ws))
        np.testing.assert_array_equal(got, acc)
    sx, sw = make_scales(rng, co)
    so = pick_so(acc, sx, sw)
    sc = dict(sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so], np.float32)))
    want = O.requant_cpu(acc.reshape(-1, co), sx, sw, so).reshape(osh)
    got = host(K.qconv2d(dev(x), dev(wt), padding, md, osh, K.EPI_REQUANT_CPU, **sc))
    np.testing.assert_array_equal(got, want)
    # the PyTorch layouts: NCHW x OIHW -> NCHW
    md_t = [0, 1, 2, 3, 1, 0, 2, 3, 0, 1, 2, 3, 2, 2, 1, 1, 1]
    x_t, w_t = np.ascontiguousarray(np.moveaxis(x, -1, 1)), np.ascontiguousarray(np.moveaxis(wt, -1, 1))
    got = host(K.qconv2d(dev(x_t), dev(w_t), padding, md_t, [nb, co, ho, wo], K.EPI_REQUANT_CPU, **sc))
    np.testing.assert_array_equal(got, np.moveaxis(want, -1, 1))


def test_qconv_known_answers(K, golden):
    for case in golden["qconv"]:
        if case["data_format"] != "NHWC":
            continue
        x = np.full(case["in_shape"], case["x"], np.float32)
        w = np.full(case["w_hwio"], case["w"], np.float32)
        co = w.shape[3]
        sw = np.full(co, case["sw"], np.float32)
        qx = O.quantize(x, case["sx"], 0)
        qw = np.ascontiguousarray(O.quantize(w, sw, np.zeros(co, np.int32), axis=3).transpose(3, 0, 1, 2))
        pad, md, out_shape = O.conv_attrs(qx.shape, qw.shape, "NHWC", case["strides"],
                                          case["dilations"], case["padding"])
        out = host(K.qconv2d(dev(qx), dev(qw), pad, md, out_shape, K.EPI_REQUANT_CPU,
                             sx=dev(np.array([case["sx"]], np.float32)), sw=dev(sw),
                             so=dev(np.array([case["so"]], np.float32))))
        if case["padding"] == "VALID" or case["w_hwio"][0] == 1 or case["x"] == 0.0:
            assert (out.astype(np.float32) * case["so"] == case["expect_f32"]).all(), case["src"]


@pytest.mark.parametrize("m,n,k,pad", [(300, 200, 256, 64), (17, 48, 1040, 16), (1000, 768, 768, 128)])
def test_qgemm_strided_rows_all_variants(K, m, n, k, pad):
    """Operands and output that are column slices of wider buffers (row stride > row
    length): the kernels must neither read the gap as data nor write into it."""
    rng = np.random.default_rng(m + n + k)
    a_full = rng.integers(-128, 128, (m, k + pad), dtype=np.int8)
    w_full = rng.integers(-128, 128, (n, k + 2 * pad), dtype=np.int8)
    a, w = a_full[:, :k], w_full[:, pad:pad + k]
    acc, _ = O.gemm_s32_fast(np.ascontiguousarray(a), np.ascontiguousarray(w))
    sx, sw = make_scales(rng, n)
    so = pick_so(acc, sx, sw)
    want = O.requant_cpu(acc, sx, sw, so)
    da, dw = dev(a_full)[:, :k], dev(w_full)[:, pad:pad + k]
    for v in [-1] + gemm_variants(K, k):
        out_full = torch.full((m, n + pad), 77, dtype=torch.int8, device="cuda")
        K.qgemm(da, dw, K.EPI_REQUANT_CPU, sx=dev(np.array([sx])), sw=dev(sw),
                so=dev(np.array([so])), out=out_full[:, :n], variant=v)
        got = host(out_full)
        np.testing.assert_array_equal(got[:, :n], want, err_msg="variant %d" % v)
        assert (got[:, n:] == 77).all(), "variant %d wrote past the row" % v


@pytest.mark.parametrize("m,n,k,ldo", [(300, 200, 256, 208), (1000, 100, 768, 112), (513, 72, 128, 80),
                                       (4100, 1000, 768, 1008), (260, 328, 512, 336)])
def test_qgemm_ragged_channels_in_16_byte_aligned_rows(K, m, n, k, ldo):
    """Output rows that take 16-byte stores (aligned buffer, row stride a multiple of 16) while
    the channel count is not a multiple of 16: the last chunk of a row is written byte by byte,
    and nothing lands in the columns behind it -- every variant, both int8 epilogues."""
    rng = np.random.default_rng(m * 7 + n)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(a, w)
    sx, sw = make_scales(rng, n)
    so = pick_so(acc, sx, sw)
    bias = rng.standard_normal(n).astype(np.float32) * 5
    want1 = O.requant_cpu(acc, sx, sw, so)
    want2 = O.requant_gpu(acc, sx, sw, so, bias_f32=bias)
    da, dw = dev(a), dev(w)
    scales = dict(sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])))
    for v in [-1] + gemm_variants(K, k):
        for epi, want, b in ((K.EPI_REQUANT_CPU, want1, None), (K.EPI_REQUANT_GPU, want2, dev(bias))):
            out_full = torch.full((m, ldo), 77, dtype=torch.int8, device="cuda")
            K.qgemm(da, dw, epi, bias=b, out=out_full[:, :n], variant=v, **scales)
            got = host(out_full)
            np.testing.assert_array_equal(got[:, :n], want, err_msg="variant %d epilogue %d" % (v, epi))
            assert (got[:, n:] == 77).all(), "variant %d wrote past the row" % v


def test_qgemm_random_shapes_epilogues_variants(K):
    """Seeded sweep over ragged shapes, every epilogue / bias kind and every kernel
    variant (heuristic included), bit-exact against the oracle."""
    rng = np.random.default_rng(20240611)
    choices = [-1] + gemm_variants(K, 16)
    for case in range(80):
        m = int(rng.choice([1, 2, 7, 16, 31, 33, 64, 100, 129, 255, 300, 513, 1000]))
        n = int(rng.choice([1, 3, 16, 17, 48, 64, 65, 130, 256, 300, 768]))
        k = int(rng.choice([16, 32, 48, 64, 112, 128, 144, 256, 400, 768, 1040]))
        a = rng.integers(-128, 128, (m, k), dtype=np.int8)
        w = rng.integers(-128, 128, (n, k), dtype=np.int8)
        acc, _ = O.gemm_s32_fast(a, w)
        sx, sw = make_scales(rng, n, per_channel=bool(rng.integers(0, 2)))
        so = pick_so(acc, sx, np.broadcast_to(sw, (n,)))
        v = choices[int(rng.integers(0, len(choices)))]
        epi = int(rng.integers(0, 4))
        tag = "case %d: %dx%dx%d variant %d epilogue %d" % (case, m, n, k, v, epi)
        da, dw = dev(a), dev(w)
        dsx, dsw, dso = dev(np.array([sx])), dev(sw), dev(np.array([so]))
        if epi == 0:
            got = host(K.qgemm(da, dw, K.EPI_ACC_S32, variant=v))
            np.testing.assert_array_equal(got, acc, err_msg=tag)
        elif epi == 1:
            kind = int(rng.integers(0, 3))
            bias = [None, rng.integers(-5000, 5000, n).astype(np.int32),
                    rng.standard_normal(n).astype(np.float32)][kind]
            b32 = bias if kind != 2 else O.bias_f32_to_s32(bias, float(sx), np.broadcast_to(sw, (n,)))
            zo = int(rng.integers(-5, 6))
            want = O.requant_cpu(acc, float(sx), sw, float(so), b32=b32, zo=zo)
            got = host(K.qgemm(da, dw, K.EPI_REQUANT_CPU, sx=dsx, sw=dsw, so=dso,
                               bias=None if bias is None else dev(bias), zo=zo, variant=v))
            np.testing.assert_array_equal(got, want, err_msg=tag)
        elif epi == 2:
            kind = int(rng.integers(0, 3))
            bias = [None, rng.standard_normal(n).astype(np.float32) * 5,
                    rng.integers(-128, 128, n, dtype=np.int8)][kind]
            want = O.requant_gpu(acc, sx, sw, so, bias_f32=bias if kind == 1 else None,
                                 bias_i8=bias if kind == 2 else None)
            got = host(K.qgemm(da, dw, K.EPI_REQUANT_GPU, sx=dsx, sw=dsw, so=dso,
                               bias=None if bias is None else dev(bias), variant=v))
            np.testing.assert_array_equal(got, want, err_msg=tag)
        else:
            bias = rng.standard_normal(n).astype(np.float32) if rng.integers(0, 2) else None
            want = O.dequant_acc(acc, float(sx), sw, bias=bias)
            got = host(K.qgemm(da, dw, K.EPI_DEQUANT_F32, sx=dsx, sw=dsw,
                               bias=None if bias is None else dev(bias), variant=v))
            np.testing.assert_array_equal(got, want, err_msg=tag)


def test_requant_nan_and_inf_scales_saturate_like_the_oracle(K):
    """A NaN or infinite per-channel factor: NaN results go to -128, infinities
    saturate by sign, on every kernel family and both requant epilogues."""
    rng = np.random.default_rng(11)
    m, n, k = 130, 256, 256
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    acc, _ = O.gemm_s32_fast(a, w)
    sx = np.float32(0.02)
    sw = rng.uniform(0.001, 0.05, n).astype(np.float32)
    sw[3] = np.nan
    sw[7] = np.inf
    sw[200] = -np.inf
    so = np.float32(2.0)
    bias = rng.standard_normal(n).astype(np.float32)
    with np.errstate(all="ignore"):
        want_gpu = O.requant_gpu(acc, sx, sw, so, bias_f32=bias)
        want_cpu = O.requant_cpu(acc, sx, sw, so)
    assert (want_gpu[:, 3] == -128).all()
    for v in gemm_variants(K, k):
        got = host(K.qgemm(dev(a), dev(w), K.EPI_REQUANT_GPU, sx=dev(np.array([sx])), sw=dev(sw),
                           so=dev(np.array([so])), bias=dev(bias), variant=v))
        np.testing.assert_array_equal(got, want_gpu, err_msg="variant %d" % v)
        got = host(K.qgemm(dev(a), dev(w), K.EPI_REQUANT_CPU, sx=dev(np.array([sx])), sw=dev(sw),
                           so=dev(np.array([so])), variant=v))
        np.testing.assert_array_equal(got, want_cpu, err_msg="variant %d" % v)


def test_bad_arguments_fail_loudly(K):
    a = torch.zeros((4, 16), dtype=torch.int8, device="cuda")
    w = torch.zeros((4, 32), dtype=torch.int8, device="cuda")
    with pytest.raises(ValueError):
        K.qgemm(a, w, K.EPI_ACC_S32)
    w = torch.zeros((4, 16), dtype=torch.int8, device="cuda")
    with pytest.raises(RuntimeError):
        K.qgemm(a, w, K.EPI_REQUANT_CPU)          # scales missing
    with pytest.raises(RuntimeError):
        K.qgemm(a, w, K.EPI_ACC_S32, variant=99)
    # limits are checked before any pointer is touched
    from bladedisc_amd import _lib
    L = _lib.lib()
    import ctypes as C
    big = C.c_int64(1 << 31)
    one = C.c_int64(1)
    st = L.dq8_qgemm(None, one, None, one, None, big, one, big, one, 0, 1, 0, None, 0, None, one,
                     None, one, None, one, 0, 0, 0, None, C.c_size_t(0), None)
    assert st != 0 and b"2^31" in L.dq8_last_error()
    st = L.dq8_qgemm(None, one, None, one, None, one, C.c_int64(-1), one, one, 0, 1, 0, None, 0,
                     None, one, None, one, None, one, 0, 0, 0, None, C.c_size_t(0), None)
    assert st != 0 and b"negative" in L.dq8_last_error()


@pytest.mark.parametrize("m,k,n", [(64, 768, 768), (1, 768, 768), (16, 768, 3072), (33, 3072, 768),
                                   (128, 768, 768), (7, 80, 24), (50, 1024, 200), (32, 768, 2304)])
@pytest.mark.parametrize("epi_name", ["REQUANT_CPU", "REQUANT_GPU", "REQUANT_CPU_DEQUANT_F32",
                                      "DEQUANT_F32", "ACC_S32"])
def test_qlinear_f32_equals_quantize_then_qgemm(K, m, k, n, epi_name):
    """The one-launch quantized linear on f32 activations against the oracle's quantize ->
    gemm -> epilogue and against the library's own two operators: the same bits.  Activations
    include exact rounding ties (multiples of scale / 2), values beyond the int8 range, zeros,
    and infinities; both rounding modes.  (A NaN activation is compared between the two forms of
    the library only: the reference leaves its quantized value undefined.)"""
    rng = np.random.default_rng(m + k + n)
    sx = np.float32(rng.uniform(0.01, 0.05))
    x = rng.standard_normal((m, k)).astype(np.float32)
    ties = rng.integers(-300, 300, x.shape).astype(np.float32) * np.float32(0.5) * sx
    x = np.where(rng.random(x.shape) < 0.1, ties, x).astype(np.float32)
    x.flat[0] = 0.0
    if x.size > 8:
        x.flat[3], x.flat[4] = np.inf, -np.inf
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    sw = rng.uniform(0.001, 0.05, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    epi = getattr(K, "EPI_" + epi_name)
    for round_mode in (K.ROUND_HALF_TO_EVEN, K.ROUND_HALF_AWAY_FROM_ZERO):
        xq = O.quantize(x, sx, 0, round_mode=round_mode)
        acc = O.gemm_s32(xq, w, tp_b=True)
        so = pick_so(acc, sx, sw)
        b = None if epi_name == "ACC_S32" else bias
        got = K.qlinear_f32(dev(x), dev(w), epi, dev(np.array([sx])), dev(sw), dev(np.array([so])),
                            bias=dev(b) if b is not None else None, round_mode=round_mode)
        dxq = K.quantize(dev(x), dev(np.array([sx])), dev(np.zeros(1, np.int32)), round_mode=round_mode)
        np.testing.assert_array_equal(host(dxq), xq)
        two = K.qgemm(dxq, dev(w), epi, sx=dev(np.array([sx])), sw=dev(sw), so=dev(np.array([so])),
                      bias=dev(b) if b is not None else None)
        np.testing.assert_array_equal(host(got).view(np.uint8), host(two).view(np.uint8))
        if x.size > 8:
            xn = x.copy()
            xn.flat[6] = np.nan
            args = (dev(w), epi, dev(np.array([sx])), dev(sw), dev(np.array([so])))
            got_n = K.qlinear_f32(dev(xn), *args, bias=dev(b) if b is not None else None,
                                  round_mode=round_mode)
            xnq = K.quantize(dev(xn), dev(np.array([sx])), dev(np.zeros(1, np.int32)), round_mode=round_mode)
            two_n = K.qgemm(xnq, dev(w), epi, sx=args[2], sw=args[3], so=args[4],
                            bias=dev(b) if b is not None else None)
            np.testing.assert_array_equal(host(got_n).view(np.uint8), host(two_n).view(np.uint8))
        if epi_name == "REQUANT_CPU":
            want = O.requant_cpu(acc, sx, sw, so, b32=O.bias_f32_to_s32(bias, sx, sw))
        elif epi_name == "REQUANT_GPU":
            want = O.requant_gpu(acc, sx, sw, so, bias_f32=bias)
        elif epi_name == "ACC_S32":
            want = acc
        else:
            continue
        np.testing.assert_array_equal(host(got), want)


def test_qlinear_f32_refuses_more_rows_than_it_pays_for(K):
    n, k = 768, 768
    rows = K.qlinear_f32_fused_max_rows(n, k)
    assert 64 <= rows <= 4096 and K.qlinear_f32_fused_max_rows(n, 100) == 0
    x = torch.zeros((rows + 1, k), device="cuda")
    w = torch.zeros((n, k), dtype=torch.int8, device="cuda")
    one = torch.ones(1, device="cuda")
    with pytest.raises(RuntimeError, match="fused_max_rows"):
        K.qlinear_f32(x, w, K.EPI_ACC_S32, one)


def _weight_only_case(rng, m, k, n, dtype, signed):
    npdt = np.float16 if dtype == torch.float16 else np.float32
    x = rng.standard_normal((m, k)).astype(npdt)
    if signed:
        w = rng.integers(-128, 128, (n, k), dtype=np.int8)
        zp = rng.integers(-8, 9, n).astype(np.int32)
    else:
        w = rng.integers(0, 256, (n, k), dtype=np.uint8)
        zp = rng.integers(118, 139, n).astype(np.int32)
    scale = rng.uniform(0.002, 0.02, n).astype(npdt)
    bias = rng.standard_normal(n).astype(npdt)
    return x, w, scale, zp, bias


def _weight_only_check(got, x, w, scale, zp, bias, dtype):
    """|error| <= accumulation bound: products are exact in f32 (half activations; f32 ones
    enter as two halves, 2^-21 relative -- or 2^-25 absolute per activation where the low
    half is a subnormal half, i.e. for |x| < 1/8), the f32 accumulation of K terms adds
    K * 2^-24 of sum |x||w|, then one rounding to the output type."""
    want, bound = O.weight_only_qgemm(x, w, scale, zp, bias)
    k = x.shape[1]
    tol = bound * (k * 2.0 ** -24 + 2.0 ** -20) + 1e-30
    if dtype == torch.float32:
        _, wsum = O.weight_only_qgemm(np.ones((1, k), np.float32), w, scale, zp, None)
        tol = tol + wsum * 2.0 ** -25
    tol = tol + (np.abs(want) + bound * 2.0 ** -12) * (2.0 ** -10 if dtype == torch.float16 else 2.0 ** -22)
    err = np.abs(host(got).astype(np.float64) - want)
    assert (err <= tol).all(), "max excess %.3g at %s" % (float((err - tol).max()),
                                                          np.unravel_index(np.argmax(err - tol), err.shape))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("k,n", [(768, 768), (768, 3072), (3072, 768)])
@pytest.mark.parametrize("m", [1, 16, 128, 1024])
def test_weight_only_qgemm_bert_linears(K, m, k, n, dtype):
    """Weight-only quantized linear on the BERT-base shapes: uint8 weights with per-channel
    scale and zero point near 128 (the reference pattern's quantization), bias, f16 and f32
    activations, every kernel form (small-M, both tile shapes)."""
    rng = np.random.default_rng(m * 7 + k + n)
    x, w, scale, zp, bias = _weight_only_case(rng, m, k, n, dtype, signed=False)
    got = K.weight_only_qgemm(dev(x), dev(w), dev(scale), dev(zp), dev(bias))
    assert got.dtype == dtype and tuple(got.shape) == (m, n)
    _weight_only_check(got, x, w, scale, zp, bias, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("m", [2, 24, 200])
def test_weight_only_qgemm_zero_points_at_the_documented_extremes(K, dtype, signed, m):
    """Zero points at both ends of the documented range (uint8 weights [-1024, 1024], int8
    weights [-1152, 896]), odd values next to the ends included: the kernels' half 1024 + zp
    (+ 128) is exact there, so the usual accumulation bound holds."""
    k, n = 256, 96
    rng = np.random.default_rng(m + int(signed))
    x, w, scale, _, bias = _weight_only_case(rng, m, k, n, dtype, signed)
    lo, hi = (-1152, 896) if signed else (-1024, 1024)
    ends = np.array([lo, lo + 1, lo + 3, hi - 3, hi - 1, hi], np.int32)
    zp = ends[rng.integers(0, len(ends), n)]
    zp[:len(ends)] = ends
    scale = (scale / 8).astype(scale.dtype)              # keeps f16 results finite
    got = K.weight_only_qgemm(dev(x), dev(w), dev(scale), dev(zp), dev(bias))
    _weight_only_check(got, x, w, scale, zp, bias, dtype)


@pytest.mark.parametrize("k,n", [(64, 4), (128, 8), (192, 20), (1280, 200), (4096, 4096),
                                 (11008, 4096)])
def test_weight_only_undo_compiler_layout(K, k, n):
    """The inverse of the compiler's constant-weight permutation
    (R tao_compiler/mlir/disc/transforms/disc_transform_weight_data_layout_for_weight_only_gemm.cc
    :54-300, :362-370), bit for bit against the oracle's restatement of the four functions."""
    from oracle import weight_layout_oracle as WL
    w_kn = np.random.default_rng(k + n).integers(0, 256, (k, n), dtype=np.uint8)
    got = K.weight_only_undo_compiler_layout(dev(WL.forward(w_kn)))
    assert tuple(got.shape) == (n, k)
    np.testing.assert_array_equal(host(got), w_kn.T)


def test_weight_only_undo_compiler_layout_refuses_shapes_outside_the_pass_domain(K):
    for k, n in [(96, 8), (64, 6)]:
        with pytest.raises(RuntimeError, match="K % 64 == 0"):
            K.weight_only_undo_compiler_layout(torch.zeros((k, n), dtype=torch.uint8, device="cuda"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_weight_only_qgemm_layouts_and_ragged_shapes(K, dtype):
    """[K,N] weights as the custom call passes them (with and without the scratch for the
    transpose), int8 weights, no bias / no zero points, shapes that leave partial tiles, a k
    depth that is not a multiple of 32, and the shapes the alignment rules send to the
    kernel without them (the reference's own test uses K = 3, N = 5)."""
    rng = np.random.default_rng(77)
    for (m, k, n) in [(2, 3, 5), (33, 48, 40), (200, 80, 136), (1, 16, 1), (70, 2064, 100),
                      (130, 40, 260), (5, 1000, 33),
                      # enough 128 x 128 tiles for the kernel that stages both operands in LDS:
                      # ragged last tiles in M and N, k depths off a multiple of 64
                      (1500, 80, 1100), (1290, 208, 1300), (9, 4112, 40),
                      # a full round of 256 x 256 tiles (ragged last row and column of tiles,
                      # XCD-ordered) and of 256 x 128 tiles
                      (4000, 144, 4090), (2000, 80, 4090)]:
        for signed in (False, True):
            x, w, scale, zp, bias = _weight_only_case(rng, m, k, n, dtype, signed)
            got = K.weight_only_qgemm(dev(x), dev(w), dev(scale), dev(zp), dev(bias))
            _weight_only_check(got, x, w, scale, zp, bias, dtype)
            w_kn = np.ascontiguousarray(w.T)
            for ws in (True, False):
                got = K.weight_only_qgemm(dev(x), dev(w_kn), dev(scale), dev(zp), None, tp_b=False,
                                          workspace=ws)
                _weight_only_check(got, x, w, scale, zp, None, dtype)
            got = K.weight_only_qgemm(dev(x), dev(w), dev(scale))
            _weight_only_check(got, x, w, scale, None, None, dtype)
    # small-magnitude f32 activations: the low halves are subnormal, the absolute term of the
    # bound takes over
    if dtype == torch.float32:
        x, w, scale, zp, bias = _weight_only_case(rng, 40, 256, 96, dtype, False)
        x = (x * 1e-4).astype(np.float32)
        got = K.weight_only_qgemm(dev(x), dev(w), dev(scale), dev(zp), None)
        _weight_only_check(got, x, w, scale, zp, None, dtype)
    # strided activations (a column slice of a wider tensor)
    x, w, scale, zp, bias = _weight_only_case(rng, 64, 64, 96, dtype, False)
    wide = dev(np.concatenate([x, x], axis=1))
    got = K.weight_only_qgemm(wide[:, :64], dev(w), dev(scale), dev(zp), dev(bias))
    _weight_only_check(got, x, w, scale, zp, bias, dtype)
    empty = K.weight_only_qgemm(dev(x[:0]), dev(w), dev(scale), dev(zp), dev(bias))
    assert tuple(empty.shape) == (0, 96)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_weight_only_qgemm_one_or_two_rows(K, dtype):
    """One or two activation rows (three or four against narrow weights): the row-streaming
    kernel on the vector ALUs (k depths that end inside a wave's 1 KiB step and inside a group
    of steps, N that ends inside a workgroup's 8 channels, signed weights, strided activations,
    no bias / zero points), and a k depth whose rows do not fit the LDS, which the matrix-core
    kernels take."""
    rng = np.random.default_rng(1234)
    for (m, k, n, signed) in [(1, 16, 1, False), (1, 768, 3072, False), (1, 4096, 100, True),
                              (2, 2064, 77, False), (1, 8192 + 48, 19, False), (2, 8192, 64, True),
                              (1, 1024 * 5 + 16, 9, False), (1, 40000, 24, False), (2, 20000, 24, False),
                              (3, 3072, 768, False), (4, 2064, 77, True), (4, 8192 + 48, 1024, False),
                              (3, 16384, 20, False), (4, 2048, 1030, False)]:
        x, w, scale, zp, bias = _weight_only_case(rng, m, k, n, dtype, signed)
        got = K.weight_only_qgemm(dev(x), dev(w), dev(scale), dev(zp), dev(bias))
        _weight_only_check(got, x, w, scale, zp, bias, dtype)
        wide = dev(np.concatenate([x, x], axis=1))
        got = K.weight_only_qgemm(wide[:, :k], dev(w), dev(scale))
        _weight_only_check(got, x, w, scale, None, None, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_weight_only_qgemm_small_m_staged_through_lds(K, dtype):
    """5 .. 32 rows against deep weights: the kernel that stages both operands through
    wave-private LDS (16 and 32 staged rows; k depths that end inside a unit of 64 and inside
    a group of three units; N that ends inside a workgroup's 32 channels; signed weights; few
    rows against 8192 channels and more, where it starts at five rows whatever the depth).
    With f32 activations it ends at 16 rows and the tiled kernel takes the rest."""
    rng = np.random.default_rng(99)
    for (m, k, n, signed) in [(12, 2048, 96, False), (16, 3072, 768, False), (17, 2064, 100, True),
                              (32, 4096, 330, False), (5, 6160, 72, True), (9, 8192, 64, False),
                              (31, 2048 + 16 * 9, 40, False), (7, 2048, 8200, False)]:
        x, w, scale, zp, bias = _weight_only_case(rng, m, k, n, dtype, signed)
        got = K.weight_only_qgemm(dev(x), dev(w), dev(scale), dev(zp), dev(bias))
        _weight_only_check(got, x, w, scale, zp, bias, dtype)
        # strided activations and no bias / zero points
        wide = dev(np.concatenate([x, x], axis=1))
        got = K.weight_only_qgemm(wide[:, :k], dev(w), dev(scale))
        _weight_only_check(got, x, w, scale, None, None, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_weight_only_qgemm_split_over_k(K, dtype):
    """M between the skinny kernels' range and the sizes whose tiles fill the chip: the launch
    is split over k (f32 partial sums in the scratch, a reduction launch behind the GEMM).
    Ragged M, N and k ranges, N that is not a multiple of 4 (scalar reduction), with and
    without the scratch (without it the unsplit kernels run), the same bits on every call, and
    a caller-owned scratch that is reused."""
    import bladedisc_amd._lib as _lib
    L = _lib.lib()
    rng = np.random.default_rng(4242)
    code = 1 if dtype == torch.float16 else 0
    split_seen = 0
    for (m, k, n) in [(33, 1024, 256), (64, 3072, 768), (100, 2064, 130), (128, 4096, 1024),
                      (200, 1040, 333), (512, 2048, 640), (48, 1536, 4096)]:
        x, w, scale, zp, bias = _weight_only_case(rng, m, k, n, dtype, signed=False)
        plain = L.dq8_weight_only_qgemm_workspace_bytes(n, k, 1)
        need = L.dq8_weight_only_qgemm_workspace_bytes_ex(m, n, k, 1, code)
        assert plain == 0 and need % (4 * m * n) == 0
        split_seen += need > 0
        args = (dev(x), dev(w), dev(scale), dev(zp), dev(bias))
        got = K.weight_only_qgemm(*args)
        _weight_only_check(got, x, w, scale, zp, bias, dtype)
        again = K.weight_only_qgemm(*args)
        assert torch.equal(got, again)
        unsplit = K.weight_only_qgemm(*args, workspace=False)
        _weight_only_check(unsplit, x, w, scale, zp, bias, dtype)
        if need:
            ws = torch.empty(need + 4096, dtype=torch.uint8, device="cuda")
            ws.fill_(0xff)                                   # (NaN patterns: nothing may leak)
            assert torch.equal(K.weight_only_qgemm(*args, workspace=ws), got)
            assert torch.equal(K.weight_only_qgemm(*args, workspace=ws), got)
            # a scratch that is too small for the partial sums: the unsplit kernels
            assert torch.equal(K.weight_only_qgemm(*args, workspace=ws[:need - 16]), unsplit)
        # [K,N] weights: the transposed copy and the partial sums share the scratch
        got_kn = K.weight_only_qgemm(dev(x), dev(np.ascontiguousarray(w.T)), dev(scale), dev(zp),
                                     dev(bias), tp_b=False)
        assert torch.equal(got_kn, got)
    assert split_seen >= 5


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_weight_only_qgemm_few_rounds_of_small_tiles(K, dtype):
    """Above 32 rows while the tiles are a few rounds of the chip: 64 x 64 tiles on four waves
    (or 128 x 128), over the whole k range where a split is not estimated to pay -- shallow k,
    ragged M and N, a k range that is not a multiple of the 64-deep tile, M on both sides of
    the tile sizes."""
    import bladedisc_amd._lib as _lib
    L = _lib.lib()
    rng = np.random.default_rng(5151)
    code = 1 if dtype == torch.float16 else 0
    unsplit_seen = 0
    for (m, k, n) in [(33, 16, 64), (40, 256, 1024), (64, 272, 100), (65, 768, 3072),
                      (128, 768, 768), (129, 528, 200), (300, 1024, 4096), (700, 784, 1000),
                      (1000, 768, 3072)]:
        x, w, scale, zp, bias = _weight_only_case(rng, m, k, n, dtype, signed=bool(m & 1))
        unsplit_seen += L.dq8_weight_only_qgemm_workspace_bytes_ex(m, n, k, 1, code) == 0
        args = (dev(x), dev(w), dev(scale), dev(zp), dev(bias))
        got = K.weight_only_qgemm(*args)
        _weight_only_check(got, x, w, scale, zp, bias, dtype)
        assert torch.equal(K.weight_only_qgemm(*args), got)
        _weight_only_check(K.weight_only_qgemm(*args, workspace=False), x, w, scale, zp, bias, dtype)
    assert unsplit_seen >= 5


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_weight_only_qgemm_strided_rows_in_and_out(K, dtype):
    """Activation and result rows that are slices of wider buffers (ldx > K, ldo > N), one shape
    per kernel family (row-streaming, 16-channel, staged, 64 x 64 tiles unsplit and split over
    k, 128-row and 256-row tiles): right results, and nothing written outside the slice."""
    rng = np.random.default_rng(5)
    for (m, k, n) in [(1, 4096, 100), (4, 3072, 768), (8, 768, 200), (8, 2048, 8200),
                      (24, 2064, 300), (40, 4096, 520), (100, 784, 200), (300, 1024, 1000),
                      (64, 8192, 264), (1000, 768, 3072), (2100, 256, 520)]:
        x, w, scale, zp, bias = _weight_only_case(rng, m, k, n, dtype, False)
        wide = dev(np.concatenate([x, x], axis=1))
        frame = torch.full((m, n + 24), 7.0, dtype=dtype, device="cuda")
        out = frame[:, 8:8 + n]
        K.weight_only_qgemm(wide[:, :k], dev(w), dev(scale), dev(zp), dev(bias), out=out)
        _weight_only_check(out, x, w, scale, zp, bias, dtype)
        assert bool((frame[:, :8] == 7).all()) and bool((frame[:, 8 + n:] == 7).all())


def test_weight_only_dispatch_sweep_stays_within_the_accumulation_bound(K):
    """Seeded sweep over what the launcher's choice depends on -- rows from 1 to several rounds
    of tiles, k from one 16-chunk to 9000, narrow to wide weights, both activation types,
    signed and unsigned weights: whichever kernel the rules and the cost estimate land on,
    the result stays within the accumulation bound of the oracle."""
    rng = np.random.default_rng(20260202)
    ms = [1, 2, 3, 4, 5, 8, 9, 12, 16, 17, 24, 31, 32, 33, 48, 64, 65, 100, 128, 129, 200, 256,
          300, 512, 700, 1100]
    cases = []
    for m in ms:
        for _ in range(2):
            k = 16 * int(rng.integers(1, 560))
            n = int(rng.integers(1, 3000))
            while m * k * n > 1.2e9:
                n = max(1, n // 2)
            cases.append((m, k, n))
    # few rows against wide weights, deep k against narrow ones
    cases += [(5, 2048, 8200), (11, 2064, 9000), (24, 2048, 8192), (4, 8192, 1000),
              (3, 2048, 1024), (24, 1536, 1536), (40, 8192, 520), (2100, 256, 4100)]
    for i, (m, k, n) in enumerate(cases):
        dtype = torch.float16 if i % 2 == 0 else torch.float32
        x, w, scale, zp, bias = _weight_only_case(rng, m, k, n, dtype, signed=bool(i % 3 == 0))
        got = K.weight_only_qgemm(dev(x), dev(w), dev(scale), dev(zp), dev(bias))
        _weight_only_check(got, x, w, scale, zp, bias, dtype)


def test_multi_kernel_paths_replay_from_a_captured_graph(K):
    """The paths that are several launches -- a weight-only GEMM split over k (GEMM, then the
    reduction), a stem convolution through space to depth (two re-layouts, then the
    convolution) -- captured into one HIP graph with caller-owned scratch and replayed with
    other work in between: every replay gives the eager result, also after the inputs change."""
    import bladedisc_amd._lib as _lib
    L = _lib.lib()
    rng = np.random.default_rng(808)
    m, k, n = 128, 2048, 512
    x, w, scale, zp, bias = _weight_only_case(rng, m, k, n, torch.float16, False)
    xd, wd, sd, zd, bd = dev(x), dev(w), dev(scale), dev(zp), dev(bias)
    need = L.dq8_weight_only_qgemm_workspace_bytes_ex(m, n, k, 1, 1)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = torch.empty((m, n), dtype=torch.float16, device="cuda")
    ci, co, h = 3, 32, 40
    cx = dev(rng.integers(-128, 128, (2, h, h, ci), dtype=np.int8))
    cw = dev(rng.integers(-128, 128, (co, 7, 7, ci), dtype=np.int8))
    md = list(O.NHWC_OHWI_METADATA) + [2, 2, 1, 1, 1]
    osh = [2, h // 2, h // 2, co]
    cout = torch.empty(tuple(osh), dtype=torch.int32, device="cuda")

    def run():
        K.weight_only_qgemm(xd, wd, sd, zd, bd, out=out, workspace=ws)
        K.qconv2d(cx, cw, [3, 3, 3, 3], md, osh, K.EPI_ACC_S32, out=cout)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run()
    for rep in range(4):
        if rep == 2:                                       # new inputs in the captured buffers
            xd.copy_(dev(rng.standard_normal((m, k)).astype(np.float16)))
            cx.copy_(dev(rng.integers(-128, 128, (2, h, h, ci), dtype=np.int8)))
        out.zero_()
        cout.zero_()
        ws.fill_(0xff)
        graph.replay()
        torch.cuda.synchronize()
        got, cgot = out.clone(), cout.clone()
        want = K.weight_only_qgemm(xd, wd, sd, zd, bd)
        cwant = K.qconv2d(cx, cw, [3, 3, 3, 3], md, osh, K.EPI_ACC_S32)
        assert torch.equal(got, want), rep
        assert torch.equal(cgot, cwant), rep


def test_dispatch_sweep_agrees_with_the_generic_kernel(K):
    """Seeded sweep over what the library's own choice of kernel depends on -- M from one row
    to several rounds of the largest tiles, N, K, the epilogue family, fused operators -- with
    the scalar generic kernel (variant 0, itself pinned against the oracle above) as the
    yardstick on the same device buffers: every combination must give the same bits, whichever
    kernel the heuristic lands on (row-streaming for one or two rows against deep weights,
    small-M, 64 / 128 / 256-wide tiles, persistent forms)."""
    rng = np.random.default_rng(20260101)
    ms = [1, 7, 16, 31, 33, 100, 500, 1000, 2100, 4096, 9000, 20000]
    cases = 0
    # (m, n, k): three random (n, k) per m, then one and two rows against rows of 2048 of k and
    # more, with k ending inside a wave's step and N inside a workgroup's channels, then few
    # rows against weights wide enough for the tiled kernel to take them, then k deep enough
    # for the split over four wave groups
    shapes = [(m, None, None) for m in ms for _ in range(3)] + \
             [(1, 100, 3072), (2, 9, 2048), (1, 40, 8208), (2, 130, 4112),
              (3, 14400, 2048), (9, 9250, 2064), (16, 9216, 2048), (8, 9216, 2048),
              (40, 1000, 8192), (100, 520, 8208),
              # the small-M kernel's range above 32 rows: one, two and four row tiles per
              # workgroup, ragged N and k, partial last row tile
              (64, 776, 784), (130, 40, 3088), (256, 768, 768), (200, 24, 2064),
              (64, 4096, 4096), (33, 4104, 4096), (250, 72, 1040)]
    for m, n_fixed, k_fixed in shapes:
        if True:
            n = n_fixed or int(rng.choice([16, 48, 64, 136, 768, 1024, 2304, 3072]))
            k = k_fixed or int(rng.choice([16, 64, 144, 768, 1040, 3072]))
            if m * n * k > 2.2e10:
                k = 64
            a = dev(rng.integers(-128, 128, (m, k), dtype=np.int8))
            w = dev(rng.integers(-128, 128, (n, k), dtype=np.int8))
            sx = dev(np.array([rng.uniform(0.01, 0.03)], np.float32))
            sw = dev(rng.uniform(0.001, 0.05, n).astype(np.float32))
            so = dev(np.array([float(np.sqrt(k)) * 0.02 * 0.025 * 5400 / 40.0], np.float32))
            bf = dev((rng.standard_normal(n) * 3).astype(np.float32))
            b32 = dev(rng.integers(-20000, 20000, n).astype(np.int32))
            table = dev(rng.integers(-128, 128, 256, dtype=np.int8))
            resid = dev(rng.integers(-128, 128, (m, n), dtype=np.int8))
            rs = dev(np.array([0.05], np.float32))
            s2 = dev(np.array([0.07], np.float32))
            sc = dict(sx=sx, sw=sw, so=so)
            plans = [
                (K.EPI_ACC_S32, {}, None),
                (K.EPI_REQUANT_CPU, dict(bias=bf, zo=2, **sc), None),
                (K.EPI_REQUANT_GPU, dict(bias=bf, **sc), None),
                (K.EPI_DEQUANT_F32, dict(sx=sx, sw=sw, bias=bf), None),
                (K.EPI_REQUANT_CPU_DEQUANT_F32, dict(bias=bf, zo=2, **sc), None),
                (K.EPI_REQUANT_FIXEDPOINT, dict(bias=b32, zo=-1, **sc), None),
                (K.EPI_REQUANT_CPU, dict(bias=bf, **sc), dict(table=table)),
                (K.EPI_REQUANT_GPU, dict(bias=bf, **sc),
                 dict(residual=resid, residual_scale=rs, residual_zp=3, relu=True, out_scale=s2, out_zp=-4)),
            ]
            for epi, kw, post in plans:
                if post is None:
                    want = K.qgemm(a, w, epi, variant=0, **kw)
                    got = K.qgemm(a, w, epi, **kw)
                else:
                    # (fused operators go with the library's own choice: the yardstick is the chain
                    # of separate calls on the generic kernel's result)
                    q = K.qgemm(a, w, epi, variant=0, **kw)
                    if "table" in post:
                        want = K.lut8(q, table)
                    else:
                        zero = torch.zeros(1, dtype=torch.int32, device="cuda")
                        t = K.dequantize(q, so, zero) + K.dequantize(
                            resid, rs, torch.full((1,), 3, dtype=torch.int32, device="cuda"))
                        t = torch.where(t < 0, torch.zeros_like(t), t)
                        want = K.quantize(t, s2, torch.full((1,), -4, dtype=torch.int32, device="cuda"))
                    got = K.qgemm(a, w, epi, post=K.make_postops(**post), **kw)
                assert got.dtype == want.dtype
                same = torch.equal(got.view(torch.int32) if got.dtype == torch.float32 else got,
                                   want.view(torch.int32) if want.dtype == torch.float32 else want)
                assert same, (m, n, k, epi, post)
                cases += 1
    assert cases == len(shapes) * 8


def test_conv_dispatch_sweep_agrees_with_the_generic_kernel(K):
    """The same for convolutions: batch, image size, channel counts (multiples of 16 and not),
    filter, stride, padding and dilation drawn from a seeded generator; the library's choice
    (direct 3x3 kernels, implicit GEMM tiles, 1x1 as a plain GEMM, channel padding through the
    scratch) against the generic kernel, for the int8, int32, f32 and fixed-point results and a
    fused table."""
    rng = np.random.default_rng(20260102)
    cases = 0
    shapes = []
    for _ in range(30):
        nb = int(rng.choice([1, 2, 8, 32, 70]))
        h = int(rng.choice([7, 14, 28, 33, 56]))
        w_ = int(rng.choice([7, 14, 28, 30, 56]))
        ci = int(rng.choice([3, 16, 24, 32, 64, 128, 256]))
        co = int(rng.choice([16, 40, 64, 128, 256]))
        k = int(rng.choice([1, 3, 3, 5]))
        stride = int(rng.choice([1, 1, 2]))
        dil = int(rng.choice([1, 1, 2]))
        pad = int(rng.integers(0, 3))
        shapes.append((nb, h, w_, ci, co, k, stride, dil, pad))
    # k deep enough for the 64 x 64 tiles to split it over four wave groups
    shapes += [(8, 7, 7, 1024, 256, 3, 1, 1, 1), (1, 10, 10, 1040, 70, 3, 1, 1, 0)]
    for (nb, h, w_, ci, co, k, stride, dil, pad) in shapes:
        ho = (h + 2 * pad - dil * (k - 1) - 1) // stride + 1
        wo = (w_ + 2 * pad - dil * (k - 1) - 1) // stride + 1
        if ho <= 0 or wo <= 0 or nb * ho * wo * co * k * k * ci > 6e10:
            continue
        x = dev(rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8))
        wt = dev(rng.integers(-128, 128, (co, k, k, ci), dtype=np.int8))
        md = list(O.NHWC_OHWI_METADATA) + [stride, stride, dil, dil, 1]
        padding, osh = [pad] * 4, [nb, ho, wo, co]
        sc = dict(sx=dev(np.array([0.02], np.float32)), sw=dev(rng.uniform(0.001, 0.05, co).astype(np.float32)),
                  so=dev(np.array([float(np.sqrt(k * k * ci)) * 0.02 * 0.025 * 5400 / 40.0], np.float32)))
        b32 = dev(rng.integers(-20000, 20000, co).astype(np.int32))
        table = dev(rng.integers(-128, 128, 256, dtype=np.int8))
        for epi, kw in ((K.EPI_ACC_S32, {}), (K.EPI_REQUANT_CPU, dict(zo=1, **sc)),
                        (K.EPI_REQUANT_CPU_DEQUANT_F32, sc), (K.EPI_REQUANT_FIXEDPOINT, dict(bias=b32, **sc))):
            want = K.qconv2d(x, wt, padding, md, osh, epi, variant=0, **kw)
            got = K.qconv2d(x, wt, padding, md, osh, epi, **kw)
            v = (lambda t: t.view(torch.int32) if t.dtype == torch.float32 else t)
            assert torch.equal(v(got), v(want)), (nb, h, w_, ci, co, k, stride, pad, dil, epi)
            cases += 1
        q = K.qconv2d(x, wt, padding, md, osh, K.EPI_REQUANT_CPU, variant=0, **sc)
        got = K.qconv2d(x, wt, padding, md, osh, K.EPI_REQUANT_CPU, **sc, post=K.make_postops(table=table))
        assert torch.equal(got, K.lut8(q, table)), (nb, h, w_, ci, co, k, stride, pad, dil)
    assert cases >= 80
