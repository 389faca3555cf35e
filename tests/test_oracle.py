"""Pins the CPU oracle: reference golden vectors, known-answer cases, and what the
mathematics fixes (brute force, numpy int64 products, float64 closed forms)."""
import numpy as np
import pytest

import oracle as O


# ----------------------------------------------------------------- quantize
def test_quantize_fold_golden_vectors(golden):
    """disc-fold-quantize.mlir: the folder's double arithmetic, every dtype."""
    for case in golden["quantize_fold"]:
        x = np.array(case["x"], np.float32)
        got = O.quantize(x, case["scale"], case["zp"], axis=case["axis"],
                         qmin=case["qmin"], qmax=case["qmax"],
                         round_mode=case["round_mode"],
                         dtype=np.dtype(case["dtype"]), fold=True)
        np.testing.assert_array_equal(got, np.array(case["expect"], case["dtype"]),
                                      err_msg=case["src"])


def test_quantize_runtime_f32_matches_golden_for_8_and_16_bit(golden):
    """The runtime decomposition (f32 divide/add/round/clamp) must give the same
    vectors wherever qmin/qmax are exactly representable in f32."""
    for case in golden["quantize_fold"]:
        if case["dtype"] in ("int32", "uint32"):
            continue
        x = np.array(case["x"], np.float32)
        got = O.quantize(x, case["scale"], case["zp"], axis=case["axis"],
                         qmin=case["qmin"], qmax=case["qmax"],
                         round_mode=case["round_mode"],
                         dtype=np.dtype(case["dtype"]), fold=False)
        np.testing.assert_array_equal(got, np.array(case["expect"], case["dtype"]),
                                      err_msg=case["src"])


def test_quantize_edge_values(golden):
    """quantize_v2.cc edge vector: 1.25/1.75 exercise rounding, -255/500 saturation."""
    x = np.array(golden["quantize_v2_edge_values"]["x"], np.float32)
    got = O.quantize(x, 1.0, 0)
    np.testing.assert_array_equal(got, [-128, 0, 1, 1, 2, 64, 127, 127])
    got = O.quantize(x, 0.5, 0, round_mode=O.ROUND_HALF_AWAY_FROM_ZERO)
    # x/0.5 = -510, 0, 2, 2.5, 3.5, 128, 254, 1000 -> away-from-zero: 3, 4
    np.testing.assert_array_equal(got, [-128, 0, 2, 3, 4, 127, 127, 127])
    got = O.quantize(x, 0.5, 0, round_mode=O.ROUND_HALF_TO_EVEN)
    np.testing.assert_array_equal(got, [-128, 0, 2, 2, 4, 127, 127, 127])


def test_quantize_is_true_division_not_reciprocal():
    """x/scale and x*(1/scale) differ at ties; the reference divides."""
    rng = np.random.default_rng(0)
    scale = np.float32(0.0473)
    # construct x = (k+0.5)*scale rounded to f32: a near-tie for every k
    k = np.arange(-120, 120, dtype=np.float32)
    x = ((k + np.float32(0.5)) * scale).astype(np.float32)
    got = O.quantize(x, scale, 0)
    want = np.clip(np.rint((x / scale).astype(np.float32)), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(got, want)
    recip = np.clip(np.rint(x * (np.float32(1) / scale)), -128, 127).astype(np.int8)
    assert (recip != want).any(), "probe vector no longer separates the two"
    del rng


@pytest.mark.parametrize("axis", [None, 0, 1, 2])
def test_quantize_per_channel_vs_numpy(axis):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 7, 6)).astype(np.float32) * 3
    n = 1 if axis is None else x.shape[axis]
    scale = rng.uniform(0.01, 0.1, n).astype(np.float32)
    zp = rng.integers(-5, 5, n).astype(np.int32)
    shape = [1, 1, 1]
    if axis is not None:
        shape[axis] = n
    s = scale.reshape(shape)
    z = zp.reshape(shape).astype(np.float32)
    want = np.clip(np.rint((x / s).astype(np.float32) + z), -128, 127).astype(np.int8)
    got = O.quantize(x, scale, zp, axis=axis)
    np.testing.assert_array_equal(got, want)
    # dequantize: (q - zp) * scale with an integer subtract
    dq = O.dequantize(got, scale, zp, axis=axis)
    want_dq = ((got.astype(np.int32) - zp.reshape(shape)).astype(np.float32) * s)
    np.testing.assert_array_equal(dq, want_dq.astype(np.float32))


def test_dequantize_uint8():
    q = np.array([[0, 10, 255]], np.uint8)
    got = O.dequantize(q, 0.5, 10)
    np.testing.assert_array_equal(got, [[-5.0, 0.0, 122.5]])


# -------------------------------------------------------------------- qgemm
@pytest.mark.parametrize("tp_a,tp_b", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_gemm_s32_vs_int64(tp_a, tp_b):
    rng = np.random.default_rng(7)
    m, k, n = 9, 37, 11
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (k, n), dtype=np.int8)
    zx, zw = 3, -2
    want = (a.astype(np.int64) - zx) @ (w.astype(np.int64) - zw)
    got = O.gemm_s32(a.T.copy() if tp_a else a, w.T.copy() if tp_b else w,
                     tp_a=tp_a, tp_b=tp_b, zx=zx, zw=zw)
    np.testing.assert_array_equal(got, want.astype(np.int32))


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (4, 4, 64), (5, 7, 63), (13, 9, 200),
                                   (8, 12, 768), (3, 5, 65)])
def test_gemm_fast_equals_plain(m, n, k):
    rng = np.random.default_rng(m * 1000 + n * 10 + k)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    want = a.astype(np.int64) @ w.astype(np.int64).T
    got, threads = O.gemm_s32_fast(a, w)
    assert threads >= 1
    np.testing.assert_array_equal(got, want.astype(np.int32))


def test_gemm_fast_extreme_values():
    """-128 * -128 * K must not overflow the a+128 trick."""
    k = 4096
    a = np.full((4, k), -128, np.int8)
    w = np.full((4, k), -128, np.int8)
    got, _ = O.gemm_s32_fast(a, w)
    assert (got == 128 * 128 * k).all()
    a[:] = 127
    got, _ = O.gemm_s32_fast(a, w)
    assert (got == -127 * 128 * k).all()


def test_gemm_mismatched_contraction_dim():
    with pytest.raises(ValueError):
        O.gemm_s32(np.zeros((2, 3), np.int8), np.zeros((4, 5), np.int8))


def test_qgemm_known_answers(golden):
    """quantized_matmul.cc: 4x25x71 -> 12.0; GPU per-tensor 32x64x128 -> 128.0."""
    for case in golden["qgemm"]:
        m, k, n = case["m"], case["k"], case["n"]
        x = np.full((m, k), case["x"], np.float32)
        w = np.full((k, n), case["w"], np.float32)
        sw = np.full(n if case["per_channel"] else 1, case["sw"], np.float32)
        qx = O.quantize(x, case["sx"], 0)
        qw = O.quantize(w, sw, np.zeros_like(sw, np.int32),
                        axis=1 if case["per_channel"] else None)
        assert (qx == case["qx"]).all() and (qw == case["qw"]).all()
        acc = O.gemm_s32(qx, qw)
        assert (acc == case["acc"]).all()
        for out in (O.requant_cpu(acc, case["sx"], sw, case["so"]),
                    O.requant_gpu(acc, case["sx"], sw[:1], case["so"])):
            assert (out == case["q_out"]).all()
            f = O.dequantize(out, case["so"], 0)
            assert (f == case["expect_f32"]).all(), case["src"]


def test_requant_cpu_closed_form_and_order():
    """E1 = (acc + b32) * os: distinguishes the order from acc*os + b32*os and from
    acc*os + b32 on constructed values; checked against exact rational arithmetic."""
    from fractions import Fraction
    rng = np.random.default_rng(11)
    m, n = 64, 48
    acc = rng.integers(-300000, 300000, (m, n)).astype(np.int32)
    b32 = rng.integers(-50000, 50000, n).astype(np.int32)
    sx = np.float32(0.021)
    sw = rng.uniform(0.001, 0.05, n).astype(np.float32)
    so = np.float32(0.37)
    got = O.requant_cpu(acc, sx, sw, so, b32=b32)
    os_ = ((sx * sw).astype(np.float32) / so).astype(np.float32)
    # the sum acc+b32 is exact in f32 only below 2^24: emulate f32 rounding
    s = (acc.astype(np.float32) + b32.astype(np.float32)).astype(np.float32)
    d = (s * os_[None, :]).astype(np.float32)
    want = np.clip(np.rint(d), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(got, want)
    # and the f32 pipeline stays within half an LSB + 2^-10 of the exact value
    for i in range(0, m, 9):
        for j in range(0, n, 7):
            exact = (Fraction(int(acc[i, j])) + int(b32[j])) * Fraction(float(os_[j]))
            if -128 < exact < 127:
                assert abs(Fraction(int(got[i, j])) - exact) <= Fraction(1, 2) + Fraction(1, 1024)


def test_requant_cpu_output_zero_point_and_saturation():
    acc = np.array([[0, 1000, -1000, 10**9, -10**9]], np.int32)
    out = O.requant_cpu(acc, 1.0, np.float32(0.1), 1.0, zo=5)
    np.testing.assert_array_equal(out, [[5, 105, -95, 127, -128]])


def test_requant_ties_round_half_to_even():
    # os = 0.5 exactly: acc odd -> x.5 ties
    acc = np.array([[1, 3, 5, -1, -3, -5, 7]], np.int32)
    out = O.requant_cpu(acc, 1.0, np.float32(0.5), 1.0)
    np.testing.assert_array_equal(out, [[0, 2, 2, 0, -2, -2, 4]])
    out = O.requant_gpu(acc, 1.0, np.float32(0.5), 1.0)
    np.testing.assert_array_equal(out, [[0, 2, 2, 0, -2, -2, 4]])


def test_bias_f32_to_s32():
    sx = np.float32(0.02)
    sw = np.array([0.01, 0.05, 0.001], np.float32)
    bias = np.array([0.5, -0.25, 1e9], np.float32)
    got = O.bias_f32_to_s32(bias, sx, sw)
    bs = np.float32(1.0) / (sx * sw).astype(np.float32)
    want = np.rint((bias * bs).astype(np.float32).astype(np.float64))
    want = np.clip(want, -2**31, 2147483520).astype(np.int64)
    np.testing.assert_array_equal(got.astype(np.int64), want)
    assert got[2] == 2147483520  # saturates at the largest float below 2^31


def test_requant_gpu_per_channel_and_bias():
    rng = np.random.default_rng(5)
    m, n = 17, 23
    acc = rng.integers(-200000, 200000, (m, n)).astype(np.int32)
    sx = rng.uniform(0.01, 0.03, n).astype(np.float32)
    sw = rng.uniform(0.001, 0.05, n).astype(np.float32)
    so = rng.uniform(0.2, 0.5, n).astype(np.float32)
    bi8 = rng.integers(-128, 128, n).astype(np.int8)
    alpha = ((sx * sw).astype(np.float32) / so).astype(np.float32)
    d = (alpha[None, :] * acc.astype(np.float32)).astype(np.float32)
    d = (d + bi8.astype(np.float32)[None, :]).astype(np.float32)
    want = np.clip(np.rint(d), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(O.requant_gpu(acc, sx, sw, so, bias_i8=bi8), want)
    bf = rng.standard_normal(n).astype(np.float32) * 10
    d = (alpha[None, :] * acc.astype(np.float32)).astype(np.float32)
    d = (d + bf[None, :]).astype(np.float32)
    want = np.clip(np.rint(d), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(O.requant_gpu(acc, sx, sw, so, bias_f32=bf), want)


def test_dequant_acc_within_1e5_of_float64():
    rng = np.random.default_rng(9)
    acc = rng.integers(-10**6, 10**6, (8, 16)).astype(np.int32)
    sw = rng.uniform(0.001, 0.05, 16).astype(np.float32)
    bias = rng.standard_normal(16).astype(np.float32)
    got = O.dequant_acc(acc, 0.02, sw, bias)
    want = acc.astype(np.float64) * (np.float64(np.float32(0.02)) * sw.astype(np.float64)) + bias
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())


# --------------------------------------------------------------------- conv
def _hwio_to_ohwi(w):
    return np.ascontiguousarray(np.transpose(w, (3, 0, 1, 2)))


def test_conv_known_answers(golden):
    for case in golden["qconv"]:
        fmt = case["data_format"]
        x = np.full(case["in_shape"], case["x"], np.float32)
        w = np.full(case["w_hwio"], case["w"], np.float32)
        co = w.shape[3]
        sw = np.full(co, case["sw"], np.float32)
        qx = O.quantize(x, case["sx"], 0)
        qw = _hwio_to_ohwi(O.quantize(w, sw, np.zeros(co, np.int32), axis=3))
        pad, md, out_shape = O.conv_attrs(qx.shape, qw.shape, fmt, case["strides"],
                                          case["dilations"], case["padding"])
        assert out_shape == case["out_shape"], case["src"]
        acc = O.conv_s32(qx, qw, pad, md, out_shape)
        ch_axis = fmt.index("C")
        acc2 = np.moveaxis(acc, ch_axis, -1).reshape(-1, co)
        q = O.requant_cpu(acc2, case["sx"], sw, case["so"])
        f = O.dequantize(q, case["so"], 0)
        if case["padding"] == "VALID" or case["w_hwio"][0] == 1 or case["x"] == 0.0:
            assert (f == case["expect_f32"]).all(), case["src"]


def test_conv_layout_probe(golden):
    c = golden["qconv_layout_probe"]
    x = np.array(c["x"], np.float32).reshape(c["in_shape"])
    w = np.array(c["w_hwio"], np.float32).reshape(c["w_hwio_shape"])
    qx = O.quantize(x, c["sx"], 0)
    qw = _hwio_to_ohwi(O.quantize(w, [c["sw"]], [0], axis=3))
    pad, md, out_shape = O.conv_attrs(qx.shape, qw.shape, "NHWC", c["strides"],
                                      c["dilations"], c["padding"])
    assert out_shape == c["out_shape"]
    acc = O.conv_s32(qx, qw, pad, md, out_shape)
    assert (acc == 0).all()


def test_conv_metadata_matches_lowering_test():
    """disc-lower-to-library-call.mlir:472-475 expects, for NHWC x OHWI,
    {0,3,1,2, 3,0,1,2, 0,3,1,2, strides, dilations, const}."""
    pad, md, out = O.conv_attrs([2, 8, 8, 16], [4, 3, 3, 16], "NHWC", [1, 2, 2, 1],
                                [1, 1, 1, 1], "SAME", weight_is_const=True)
    assert md == [0, 3, 1, 2, 3, 0, 1, 2, 0, 3, 1, 2, 2, 2, 1, 1, 1]
    assert pad == [0, 1, 0, 1] and out == [2, 4, 4, 4]
    pad, md, out = O.conv_attrs([2, 16, 8, 8], [4, 3, 3, 16], "NCHW", [1], [1],
                                "EXPLICIT", explicit_paddings=[1, 1, 2, 2])
    assert md[:4] == [0, 1, 2, 3] and pad == [1, 1, 2, 2] and out == [2, 4, 8, 10]


@pytest.mark.parametrize("stride,dil,pad", [(1, 1, 1), (2, 1, 0), (1, 2, 2), (2, 2, 1)])
def test_conv_equals_im2col_gemm(stride, dil, pad):
    """Textbook identity: conv = im2col + matmul (independent numpy im2col)."""
    rng = np.random.default_rng(stride * 100 + dil * 10 + pad)
    nb, h, w_, ci, co, kh, kw = 2, 9, 7, 5, 6, 3, 3
    x = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
    wt = rng.integers(-128, 128, (co, kh, kw, ci), dtype=np.int8)
    ho = (h + 2 * pad - dil * (kh - 1) - 1) // stride + 1
    wo = (w_ + 2 * pad - dil * (kw - 1) - 1) // stride + 1
    md = list(O.NHWC_OHWI_METADATA) + [stride, stride, dil, dil, 1]
    got = O.conv_s32(x, wt, [pad, pad, pad, pad], md, [nb, ho, wo, co])
    xp = np.zeros((nb, h + 2 * pad, w_ + 2 * pad, ci), np.int64)
    xp[:, pad:pad + h, pad:pad + w_, :] = x
    cols = np.zeros((nb, ho, wo, kh, kw, ci), np.int64)
    for r in range(kh):
        for q in range(kw):
            cols[:, :, :, r, q, :] = xp[:, r * dil:r * dil + stride * ho:stride,
                                        q * dil:q * dil + stride * wo:stride, :]
    want = cols.reshape(-1, kh * kw * ci) @ wt.reshape(co, -1).astype(np.int64).T
    np.testing.assert_array_equal(got.reshape(-1, co), want.astype(np.int32))


def test_conv_nchw_oihw_layout_via_metadata():
    rng = np.random.default_rng(21)
    x = rng.integers(-128, 128, (2, 6, 6, 4), dtype=np.int8)        # NHWC
    wt = rng.integers(-128, 128, (3, 3, 3, 4), dtype=np.int8)       # OHWI
    md_nhwc = list(O.NHWC_OHWI_METADATA) + [1, 1, 1, 1, 1]
    ref = O.conv_s32(x, wt, [1, 1, 1, 1], md_nhwc, [2, 6, 6, 3])
    x2 = np.ascontiguousarray(x.transpose(0, 3, 1, 2))              # NCHW
    w2 = np.ascontiguousarray(wt.transpose(0, 3, 1, 2))             # OIHW
    md = [0, 1, 2, 3, 1, 0, 2, 3, 0, 1, 2, 3, 1, 1, 1, 1, 1]
    got = O.conv_s32(x2, w2, [1, 1, 1, 1], md, [2, 3, 6, 6])
    np.testing.assert_array_equal(got.transpose(0, 2, 3, 1), ref)


def test_requant_cpu_tie_margin_audit():
    """E1's order of float operations lives in a library that is absent from the
    reference checkout.  This audit bounds what a different order could change: on
    the single-linear benchmark inputs, the alternative evaluation orders differ from
    E1 only where the pre-rounding value sits next to a .5 tie."""
    from bladedisc_amd import baseline_configs as C
    c = C.config1()
    x_q = O.quantize(c["x"], c["sx"], 0)
    acc = O.gemm_s32(x_q, c["w_q"], tp_b=True)
    sx, sw, so, bias = np.float32(c["sx"]), c["sw"], np.float32(c["so"]), c["bias"]
    b32 = O.bias_f32_to_s32(bias, float(sx), sw)
    base = O.requant_cpu(acc, float(sx), sw, float(so), b32=b32).astype(np.int32)
    f = np.float32
    os_ = ((sx * sw).astype(f) / so).astype(f)
    pre = ((acc.astype(f) + b32.astype(f)).astype(f) * os_).astype(f)
    assert np.array_equal(np.clip(np.rint(pre), -128, 127).astype(np.int32), base)
    dist_to_tie = np.abs(np.abs(pre - np.floor(pre)) - 0.5)
    # (a) distribute the scale over the sum: acc*os + b32*os
    alt_a = ((acc.astype(f) * os_).astype(f) + (b32.astype(f) * os_).astype(f)).astype(f)
    # (b) dequantize first, add the real-valued bias, divide by the output scale
    alt_b = (((acc.astype(f) * (sx * sw).astype(f)).astype(f) + bias).astype(f) / so).astype(f)
    for alt, margin in ((alt_a, 2.0 ** -10), (alt_b, 2.0 ** -10 + float(os_.max()))):
        q = np.clip(np.rint(alt), -128, 127).astype(np.int32)
        differs = q != base
        assert np.abs(q - base).max() <= 1
        assert np.all(dist_to_tie[differs] < margin)
        assert differs.mean() < 0.01


def test_requant_cpu_agrees_with_library_quantized_linear_away_from_ties():
    """Cross-check of E1 against library routines of this image (PyTorch's CPU quantized
    linear on its qnnpack, fbgemm and oneDNN-3 engines) -- not the reference, whose oneDNN 2.x
    is absent, but independent implementations of the same contract: int32 accumulate, bias
    quantized to int32 with scale s_x s_w[n], one multiplication by s_x s_w[n] / s_o, round to
    nearest even, saturate.  They must agree with the oracle wherever the exact pre-rounding
    value is further than 2^-10 from a rounding tie (the margin of the audit above), and never
    differ by more than one step."""
    torch = pytest.importorskip("torch")
    engines = [e for e in torch.backends.quantized.supported_engines if e in ("qnnpack", "fbgemm", "onednn")]
    if not engines:
        pytest.skip("no CPU quantized engine in this torch build")
    rng = np.random.default_rng(0)
    saved = torch.backends.quantized.engine
    checked = 0
    try:
        for m, k, n in [(64, 256, 128), (128, 768, 768), (33, 100, 77)]:
            x_q = rng.integers(-128, 128, (m, k), dtype=np.int8)
            w_q = rng.integers(-128, 128, (n, k), dtype=np.int8)
            sx = np.float32(rng.uniform(0.01, 0.03))
            sw = rng.uniform(0.001, 0.05, n).astype(np.float32)
            acc = O.gemm_s32(x_q, w_q, tp_b=True)
            so = np.float32(np.std(acc * float(sx) * float(sw.mean())) / 40)
            bias = (rng.standard_normal(n) * 3 * so).astype(np.float32)
            b32 = O.bias_f32_to_s32(bias, sx, sw)
            want = O.requant_cpu(acc, sx, sw, so, b32=b32)
            exact = (acc.astype(np.float64) + b32.astype(np.float64)[None, :]) * \
                (np.float64(sx) * sw.astype(np.float64) / np.float64(so))[None, :]
            near_tie = np.abs(exact - np.floor(exact) - 0.5) < 2.0 ** -10
            for eng in engines:
                torch.backends.quantized.engine = eng
                # these engines take unsigned activations: the same values with zero point 128
                xq = torch._make_per_tensor_quantized_tensor(
                    torch.from_numpy((x_q.astype(np.int16) + 128).astype(np.uint8)), float(sx), 128)
                wq = torch._make_per_channel_quantized_tensor(
                    torch.from_numpy(w_q), torch.from_numpy(sw.astype(np.float64)),
                    torch.zeros(n, dtype=torch.int64), 0)
                packed = torch.ops.quantized.linear_prepack(wq, torch.from_numpy(bias))
                y = torch.ops.quantized.linear(xq, packed, float(so), 128)
                got = y.int_repr().numpy().astype(np.int16) - 128
                differs = got != want
                assert np.abs(got - want).max() <= 1, eng
                assert not (differs & ~near_tie).any(), eng
                checked += int((~near_tie).sum())
    finally:
        torch.backends.quantized.engine = saved
    assert checked > 100000


def test_conv_oracle_agrees_with_library_quantized_conv2d():
    """The convolution geometry (padding, stride, dilation, NHWC x OHWI) and its requant against
    PyTorch's CPU quantized conv2d on the fbgemm and qnnpack engines (libraries of this image,
    not the reference): equal wherever the pre-rounding value is further than 2^-10 from a tie,
    within one step elsewhere."""
    torch = pytest.importorskip("torch")
    engines = [e for e in torch.backends.quantized.supported_engines if e in ("qnnpack", "fbgemm")]
    if not engines:
        pytest.skip("no CPU quantized engine in this torch build")
    rng = np.random.default_rng(1)
    saved = torch.backends.quantized.engine
    try:
        for nb, h, w_, ci, co, k, stride, pad, dil in [(2, 14, 14, 32, 48, 3, 1, 1, 1), (1, 9, 11, 16, 24, 3, 2, 1, 1),
                                                       (1, 12, 12, 8, 16, 3, 1, 2, 2), (2, 7, 7, 64, 32, 1, 1, 0, 1)]:
            x_q = rng.integers(-128, 128, (nb, h, w_, ci), dtype=np.int8)
            wt = rng.integers(-128, 128, (co, k, k, ci), dtype=np.int8)
            ho = (h + 2 * pad - dil * (k - 1) - 1) // stride + 1
            wo = (w_ + 2 * pad - dil * (k - 1) - 1) // stride + 1
            md = list(O.NHWC_OHWI_METADATA) + [stride, stride, dil, dil, 1]
            acc = O.conv_s32(x_q, wt, [pad] * 4, md, [nb, ho, wo, co])
            sx = np.float32(0.02)
            sw = rng.uniform(0.001, 0.05, co).astype(np.float32)
            so = np.float32(np.std(acc * float(sx) * float(sw.mean())) / 40)
            want = O.requant_cpu(acc.reshape(-1, co), sx, sw, so).reshape(nb, ho, wo, co)
            exact = acc.astype(np.float64) * (np.float64(sx) * sw.astype(np.float64) / np.float64(so))
            near_tie = np.abs(exact - np.floor(exact) - 0.5) < 2.0 ** -10
            for eng in engines:
                torch.backends.quantized.engine = eng
                xu = torch.from_numpy((x_q.astype(np.int16) + 128).astype(np.uint8))
                xq = torch._make_per_tensor_quantized_tensor(
                    xu.permute(0, 3, 1, 2).contiguous(memory_format=torch.channels_last), float(sx), 128)
                wq = torch._make_per_channel_quantized_tensor(
                    torch.from_numpy(wt).permute(0, 3, 1, 2).contiguous(),
                    torch.from_numpy(sw.astype(np.float64)), torch.zeros(co, dtype=torch.int64), 0)
                packed = torch.ops.quantized.conv2d_prepack(wq, None, [stride, stride], [pad, pad],
                                                            [dil, dil], 1)
                y = torch.ops.quantized.conv2d(xq, packed, float(so), 128)
                got = y.int_repr().permute(0, 2, 3, 1).numpy().astype(np.int16) - 128
                assert got.shape == want.shape
                assert np.abs(got - want).max() <= 1, eng
                assert not ((got != want) & ~near_tie).any(), eng
    finally:
        torch.backends.quantized.engine = saved


# ---------------------------------------------------------------- fixed-point requantisation
# Pins for the restatement of Arm Compute Library's QUANTIZE_DOWN_FIXEDPOINT output stage (the
# reference's AArch64 entries, common_context_impl_quantization.cc:671-679, 865-872, 1083-1090).
# The library is not in the reference tree, so the pins are what the arithmetic fixes: the two
# rounding primitives against exact rationals, the multiplier decomposition against exact
# equality, the whole stage against an independent evaluation in exact arithmetic, the
# reference's 12.0 / 108.0 closed forms, saturation and left shifts.
def _floor_div(a, b):
    return a // b


def test_sqrdmulh_is_round_half_up_of_the_doubled_high_half():
    from fractions import Fraction
    import math
    rng = np.random.default_rng(5)
    cases = [(0, 0), (1, 1 << 30), (-1, 1 << 30), (3, 1 << 30), (-3, 1 << 30), (5, 1 << 29),
             (-5, 1 << 29), (2**31 - 1, 2**31 - 1), (-2**31, 2**31 - 1), (-2**31, -2**31),
             (-2**31, 1 << 30), (12345, -(1 << 30))]
    cases += [(int(a), int(b)) for a, b in zip(rng.integers(-2**31, 2**31, 2000),
                                               rng.integers(-2**31, 2**31, 2000))]
    for a, b in cases:
        exact = Fraction(a * b, 1 << 31)                 # the doubled product's high half
        want = math.floor(exact + Fraction(1, 2))        # ties toward +infinity
        want = min(want, 2**31 - 1)                      # only -2^31 * -2^31 saturates
        assert O.sqrdmulh(a, b) == want, (a, b)
    assert O.sqrdmulh(-3, 1 << 30) == -1                 # -1.5 -> -1: not half away from zero


def test_rounding_divide_by_pow2_rounds_half_away_from_zero():
    from fractions import Fraction
    import math
    rng = np.random.default_rng(6)
    xs = [0, 1, -1, 2, -2, 3, -3, 5, -5, 6, -6, 2**31 - 1, -2**31] + \
        [int(v) for v in rng.integers(-2**31, 2**31, 500)]
    for x in xs:
        for e in (0, 1, 2, 3, 7, 16, 30, 31):
            q = Fraction(x, 1 << e)
            fl = math.floor(q)
            frac = q - fl
            if frac > Fraction(1, 2) or (frac == Fraction(1, 2) and x > 0):
                want = fl + 1
            else:
                want = fl
            assert O.rounding_divide_by_pow2(x, e) == want, (x, e)


def test_fixedpoint_multiplier_represents_the_binary32_value_exactly():
    from fractions import Fraction
    rng = np.random.default_rng(7)
    vals = [1.3071891e-4, 0.5, 0.25, 0.75, 1.0, 1.5, 2.0, 3.999, 1e-5, 0.99999994, 123.456]
    vals += list(np.exp(rng.uniform(np.log(1e-6), np.log(64.0), 500)))
    for v in vals:
        f = np.float32(v)
        m0, sh = O.fixedpoint_multiplier(float(f))
        assert (1 << 30) <= m0 < (1 << 31), (v, m0)
        assert Fraction(m0, 1 << 31) / (Fraction(2) ** sh) == Fraction(float(f)), (v, m0, sh)
    assert O.fixedpoint_multiplier(0.0) == (0, 0)
    assert O.fixedpoint_multiplier(0.5) == (1 << 30, 0)
    assert O.fixedpoint_multiplier(1.0) == (1 << 30, -1)     # a left shift


def _stage_exact(v, mult_f32, zo):
    """The output stage evaluated independently in exact arithmetic: the high-half product
    rounded half up, then the power-of-two division rounded half away from zero."""
    from fractions import Fraction
    import math
    m = Fraction(float(np.float32(mult_f32)))
    e = 0
    q = m
    while q >= 1:
        q /= 2
        e += 1
    while 0 < q < Fraction(1, 2):
        q *= 2
        e -= 1
    m0 = int(q * (1 << 31))                       # exact: q has 24 significant bits
    shift = -e
    if shift < 0:
        v = ((v << -shift) + 2**31) % 2**32 - 2**31      # vmulq_n_s32 wraps
        v = math.floor(Fraction(v * m0, 1 << 31) + Fraction(1, 2))
    else:
        h = math.floor(Fraction(v * m0, 1 << 31) + Fraction(1, 2))
        qq = Fraction(h, 1 << shift)
        fl = math.floor(qq)
        v = fl + 1 if (qq - fl > Fraction(1, 2) or (qq - fl == Fraction(1, 2) and h > 0)) else fl
    return int(min(127, max(-128, v + zo)))


def test_requant_fixedpoint_known_answers_and_exact_stage():
    # the reference's AArch64 closed forms: 25 x (-72)(-51) -> 12, nine taps of it -> 108
    # (disc/tests/tensorflow_ops/quantized_matmul.cc:26-55, disc/tests/pdll/quantized_conv2d.cc)
    sx, sw, so = np.float32(8.333333e-3), np.float32(1.568627e-2), np.float32(1.0)
    acc = np.array([[91800, 826200, 0, -91800, -826200]], np.int32)
    got = O.requant_fixedpoint(acc, sx, np.array([sw] * 5, np.float32), so)
    np.testing.assert_array_equal(got, [[12, 108, 0, -12, -108]])
    # random accumulators, per-channel scales (right shifts), bias and zero point
    rng = np.random.default_rng(8)
    m, n = 37, 29
    acc = rng.integers(-3_000_000, 3_000_000, (m, n)).astype(np.int32)
    acc[0, :5] = [2**31 - 1, -2**31, 0, 1, -1]
    b32 = rng.integers(-100000, 100000, n).astype(np.int32)
    sx = np.float32(0.02)
    swv = rng.uniform(0.001, 0.05, n).astype(np.float32)
    so = np.float32(0.7)
    got = O.requant_fixedpoint(acc, sx, swv, so, b32=b32, zo=-3)
    for i in range(m):
        for j in range(n):
            mult = np.float32(np.float32(sx * swv[j]) / so)
            v = int(acc[i, j]) + int(b32[j])
            v = (v + 2**31) % 2**32 - 2**31
            assert got[i, j] == _stage_exact(v, mult, -3), (i, j)
    # within one step of the real-valued product wherever nothing saturates
    real = (acc.astype(np.float64) + b32) * (np.float64(sx) * swv.astype(np.float64) / np.float64(so)) - 3
    inside = np.abs(real) < 126
    assert np.all(np.abs(got.astype(np.float64) - real)[inside] <= 0.5 + 1e-3)
    # multipliers of one and more: left shifts, saturation on both sides
    # (the pre-multiplication by 2^-shift wraps like the library's vmulq_n_s32: 2^30 * 2 is
    # -2^31, which the last two columns show)
    acc = np.array([[1, -1, 50, -50, 100, -100, 2**28, -2**28, 2**30, -2**30]], np.int32)
    for mult in (1.0, 1.5, 2.0, 3.25):
        got = O.requant_fixedpoint(acc, np.float32(mult), np.ones(10, np.float32), np.float32(1.0))
        want = [_stage_exact(int(v), mult, 0) for v in acc[0]]
        np.testing.assert_array_equal(got[0], want, err_msg=str(mult))
        assert got[0, 6] == 127 and got[0, 7] == -128
    got = O.requant_fixedpoint(acc, np.float32(1.0), np.ones(10, np.float32), np.float32(1.0))
    assert got[0, 8] == -128 and got[0, 9] == -128


def test_weight_only_qgemm_is_linear_on_the_fake_quantized_weight():
    """The weight-only oracle against the model the reference's pattern matches
    (test_quantization.py:501-523): F.linear on torch.fake_quantize_per_channel_affine(weight)
    with quant range [0, 255], zero point 128 -- a library cross-check on the CPU that pins the
    sign of the zero point, the channel axis and the place of the scale."""
    import torch
    rng = np.random.default_rng(5)
    n, k, m = 5, 3, 7
    w = torch.from_numpy(rng.standard_normal((n, k)).astype(np.float32))
    scale = torch.from_numpy(rng.uniform(0.005, 0.03, n).astype(np.float32))
    zp = torch.from_numpy(rng.integers(100, 156, n).astype(np.int32))
    bias = torch.from_numpy(rng.standard_normal(n).astype(np.float32))
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32))
    fq = torch.fake_quantize_per_channel_affine(w, scale, zp, 0, 0, 255)
    want = torch.nn.functional.linear(x, fq, bias).numpy()
    q = torch.clamp(torch.round(w / scale[:, None]) + zp[:, None], 0, 255).to(torch.uint8).numpy()
    got, bound = O.weight_only_qgemm(x.numpy(), q, scale.numpy(), zp.numpy(), bias.numpy())
    assert got.shape == (m, n) and (bound >= np.abs(got - bias.numpy()[None]) - 1e-9).all()
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-6 * float(bound.max()) + 1e-6)
    # no zero points / no bias: plain matmul on the scaled integers
    got2, _ = O.weight_only_qgemm(x.numpy(), q, scale.numpy())
    np.testing.assert_allclose(got2, x.numpy().astype(np.float64) @ (q.astype(np.float64) * scale.numpy().astype(np.float64)[:, None]).T,
                               rtol=1e-12)
