"""Parity of the five benchmark configurations at their full sizes: the HIP path
against the CPU oracle on the same seeded inputs.  Integer and int8 results bit-exact,
fp32 results within 1e-5 relative."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
import oracle as O  # noqa: E402

pytestmark = pytest.mark.gpu

REL_TOL_F32 = 1e-5


@pytest.fixture(scope="module")
def K():
    from bladedisc_amd import kernels
    return kernels


@pytest.fixture(scope="module")
def C():
    from bladedisc_amd import baseline_configs
    return baseline_configs


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def f1(v):
    return dev(np.array([v], np.float32))


def test_config1_single_quantized_linear(K, C):
    c = C.config1()
    z1 = torch.zeros(1, dtype=torch.int32, device="cuda")
    # quantize on the GPU, bit-exact against the oracle
    x_q = K.quantize(dev(c["x"]), f1(c["sx"]), z1)
    ref_xq = O.quantize(c["x"], c["sx"], 0)
    assert np.array_equal(x_q.cpu().numpy(), ref_xq)
    # E1 with f32 bias -> int8
    y_q = K.qgemm(x_q, dev(c["w_q"]), K.EPI_REQUANT_CPU, sx=f1(c["sx"]), sw=dev(c["sw"]),
                  so=f1(c["so"]), bias=dev(c["bias"]))
    acc = O.gemm_s32(ref_xq, c["w_q"], tp_b=True)
    b32 = O.bias_f32_to_s32(c["bias"], float(c["sx"]), c["sw"])
    ref_yq = O.requant_cpu(acc, float(c["sx"]), c["sw"], float(c["so"]), b32=b32)
    assert np.array_equal(y_q.cpu().numpy(), ref_yq)
    assert 0 < np.abs(ref_yq).max() <= 127 and (np.abs(ref_yq) == 127).mean() < 0.01
    # dequantized fp32 output
    y = K.dequantize(y_q, f1(c["so"]), z1).cpu().numpy()
    ref_y = O.dequantize(ref_yq, c["so"], 0)
    np.testing.assert_allclose(y, ref_y, rtol=REL_TOL_F32, atol=0)
    # and it approximates the fp32 linear to quantisation accuracy
    assert np.abs(y - c["y_fp32"]).max() < 4 * float(c["so"])
    # the whole chain as one launch (quantize on load, dequantize in the epilogue): the same bits
    y1 = K.qlinear_f32(dev(c["x"]), dev(c["w_q"]), K.EPI_REQUANT_CPU_DEQUANT_F32, f1(c["sx"]),
                       dev(c["sw"]), f1(c["so"]), bias=dev(c["bias"])).cpu().numpy()
    np.testing.assert_array_equal(y1, ref_y)
    yq1 = K.qlinear_f32(dev(c["x"]), dev(c["w_q"]), K.EPI_REQUANT_CPU, f1(c["sx"]), dev(c["sw"]),
                        f1(c["so"]), bias=dev(c["bias"])).cpu().numpy()
    np.testing.assert_array_equal(yq1, ref_yq)
    # E3: int32 accumulators dequantized directly, against a float64 closed form
    y3 = K.qgemm(x_q, dev(c["w_q"]), K.EPI_DEQUANT_F32, sx=f1(c["sx"]), sw=dev(c["sw"]),
                 bias=dev(c["bias"])).cpu().numpy()
    ref3 = acc.astype(np.float64) * (np.float64(c["sx"]) * c["sw"].astype(np.float64)) + c["bias"]
    np.testing.assert_allclose(y3, ref3, rtol=REL_TOL_F32, atol=1e-6)
    np.testing.assert_array_equal(y3, O.dequant_acc(acc, float(c["sx"]), c["sw"], bias=c["bias"]))


@pytest.mark.parametrize("k,n", [(768, 768), (768, 3072), (3072, 768)])
@pytest.mark.parametrize("m", [1, 16, 128, 1000, 4096, 16384])
def test_config2_dynamic_m_sweep(K, C, m, k, n):
    c = C.config2(m, k, n)
    y_q = K.qgemm(dev(c["a_q"]), dev(c["w_q"]), K.EPI_REQUANT_CPU, sx=f1(c["sx"]),
                  sw=dev(c["sw"]), so=f1(c["so"]))
    acc, _ = O.gemm_s32_fast(c["a_q"], c["w_q"])
    ref = O.requant_cpu(acc, float(c["sx"]), c["sw"], float(c["so"]))
    assert np.array_equal(y_q.cpu().numpy(), ref)
    assert np.abs(ref).max() > 32          # the output scale is not degenerate


@pytest.mark.parametrize("size", [4096, 8192])
def test_config3_large_square(K, C, size):
    c = C.config3(size)
    a, w = dev(c["a_q"]), dev(c["w_q"])
    acc_ref, _ = O.gemm_s32_fast(c["a_q"], c["w_q"])
    # int32 accumulators
    acc = K.qgemm(a, w, K.EPI_ACC_S32)
    assert np.array_equal(acc.cpu().numpy(), acc_ref)
    del acc
    # fused f32 bias + requant (E2), the benchmark's epilogue
    y = K.qgemm(a, w, K.EPI_REQUANT_GPU, sx=f1(c["sx"]), sw=dev(c["sw"]), so=f1(c["so"]),
                bias=dev(c["bias_q"]))
    ref = O.requant_gpu(acc_ref, c["sx"], c["sw"], c["so"], bias_f32=c["bias_q"])
    assert np.array_equal(y.cpu().numpy(), ref)
    sat = float(((ref == 127) | (ref == -128)).mean())
    assert 0.001 < sat < 0.10, "saturated fraction %.4f: output scale degenerate" % sat
    # E1 with an int32 bias
    b32 = np.rint(c["bias_q"] * 1000).astype(np.int32)
    y1 = K.qgemm(a, w, K.EPI_REQUANT_CPU, sx=f1(c["sx"]), sw=dev(c["sw"]), so=f1(c["so"]),
                 bias=dev(b32))
    ref1 = O.requant_cpu(acc_ref, float(c["sx"]), c["sw"], float(c["so"]), b32=b32)
    assert np.array_equal(y1.cpu().numpy(), ref1)


def _im2col(x, k, stride, pad):
    nb, h, w, ci = x.shape
    xp = np.zeros((nb, h + 2 * pad, w + 2 * pad, ci), np.int8)
    xp[:, pad:pad + h, pad:pad + w] = x
    ho = (h + 2 * pad - k) // stride + 1
    wo = (w + 2 * pad - k) // stride + 1
    cols = np.empty((nb, ho, wo, k, k, ci), np.int8)
    for i in range(k):
        for j in range(k):
            cols[:, :, :, i, j] = xp[:, i:i + stride * ho:stride, j:j + stride * wo:stride]
    return cols.reshape(nb * ho * wo, k * k * ci), ho, wo


@pytest.mark.parametrize("idx", [0, 1, 2])
def test_config4_resnet_convs(K, C, idx):
    conv = C.RESNET_CONVS[idx]
    c = C.config4(conv)
    nb, h, w_, ci, co, k = (conv[x] for x in ("nb", "h", "w", "ci", "co", "k"))
    pad4, md, out_shape = O.conv_attrs((nb, h, w_, ci), (co, k, k, ci), "NHWC", [1, 1, 1, 1],
                                       [1, 1, 1, 1], "EXPLICIT",
                                       explicit_paddings=[0, 0, conv["pad"], conv["pad"],
                                                          conv["pad"], conv["pad"], 0, 0])
    md[:12] = O.NHWC_OHWI_METADATA
    y = K.qconv2d(dev(c["x_q"]), dev(c["w_q"]), pad4, md, out_shape, K.EPI_REQUANT_CPU,
                  sx=f1(c["sx"]), sw=dev(c["sw"]), so=f1(c["so"]))
    # oracle at full size: im2col (a textbook identity, itself checked against the
    # direct convolution loop in the CPU tests) + the multi-threaded int8 GEMM
    cols, ho, wo = _im2col(c["x_q"], k, conv["stride"], conv["pad"])
    assert [nb, ho, wo, co] == list(out_shape)
    acc, _ = O.gemm_s32_fast(cols, c["w_q"].reshape(co, -1))
    ref = O.requant_cpu(acc, float(c["sx"]), c["sw"], float(c["so"])).reshape(out_shape)
    assert np.array_equal(y.cpu().numpy(), ref)
    assert np.abs(ref).max() > 32
    # a slice through the direct convolution loop as well
    small = O.conv_s32(c["x_q"][:1], c["w_q"], pad4, md, [1, ho, wo, co])
    assert np.array_equal(small.reshape(-1, co), acc[:ho * wo])


def test_resnet50_layer_sweep(K, C):
    """Every distinct convolution of ResNet-50 (the layers bench.py times next to config 4), at
    batch 4 so that each goes to the kernel its full-size form goes to or a neighbour of it:
    bit-exact against im2col + the oracle's int8 GEMM, with an s32 bias and an output zero
    point."""
    rng = np.random.default_rng(50)
    for h, ci, co, k, stride, pad in C.RESNET50_LAYERS:
        nb = 4
        x = rng.integers(-128, 128, (nb, h, h, ci), dtype=np.int8)
        wt = rng.integers(-128, 128, (co, k, k, ci), dtype=np.int8)
        cols, ho, wo = _im2col(x, k, stride, pad)
        acc, _ = O.gemm_s32_fast(cols, wt.reshape(co, -1))
        sw = rng.uniform(0.001, 0.05, co).astype(np.float32)
        sx = 0.02
        so = float(np.abs(acc * (sx * sw)).max() / 200.0)
        bi = rng.integers(-20000, 20000, co).astype(np.int32)
        md = list(O.NHWC_OHWI_METADATA) + [stride, stride, 1, 1, 1]
        out_shape = [nb, ho, wo, co]
        y = K.qconv2d(dev(x), dev(wt), [pad] * 4, md, out_shape, K.EPI_REQUANT_CPU, sx=f1(sx), sw=dev(sw),
                      so=f1(so), bias=dev(bi), zo=2)
        ref = O.requant_cpu(acc, sx, sw, so, b32=bi, zo=2).reshape(out_shape)
        assert np.array_equal(y.cpu().numpy(), ref), (h, ci, co, k, stride)


@pytest.mark.parametrize("seq", [32, 128, 384])
@pytest.mark.parametrize("backend", ["raw", "ral"])
def test_config5_bert_layer(C, seq, backend):
    from bladedisc_amd import bert_layer as B
    from bladedisc_amd import ral
    weights = C.config5_weights()
    tokens = C.config5_tokens(8, seq)
    ctx = ex = None
    if backend == "ral":
        ctx = ral.RalContext()
        ex = ctx.execution()
        be = B.RalBackend(ex)
    else:
        be = B.RawBackend()
    try:
        layer = B.QuantBertLayer(weights, be)
        h = layer.embed(tokens)
        layer.calibrate(h)
        rec = {}
        out = layer.forward(h, rec)
        ref_fp32 = layer.forward_fp32(h)
        torch.cuda.synchronize()
        # every quantized operator, on the tensors the layer actually fed it
        for name in B.LINEARS:
            r = rec[name]
            sx = float(layer.s_in[name].cpu()[0])
            so = float(layer.s_out[name].cpu()[0])
            sw = layer.sw[name].cpu().numpy()
            x_q = O.quantize(r["x"].cpu().numpy(), sx, 0)
            assert np.array_equal(r["x_q"].cpu().numpy(), x_q), name
            acc, _ = O.gemm_s32_fast(x_q, layer.w_q[name].cpu().numpy())
            b32 = O.bias_f32_to_s32(layer.fb[name], sx, sw)
            y_q = O.requant_cpu(acc, sx, sw, so, b32=b32)
            assert np.array_equal(r["y_q"].cpu().numpy(), y_q), name
            np.testing.assert_allclose(r["y"].cpu().numpy(), O.dequantize(y_q, so, 0),
                                       rtol=REL_TOL_F32, atol=0)
        # the quantized layer tracks the fp32 layer (LayerNorm output, unit variance)
        err = (out - ref_fp32).abs()
        assert float(err.mean()) < 0.05 and float(err.max()) < 1.0
    finally:
        if ex is not None:
            ex.close()
            ctx.close()


@pytest.mark.parametrize("seq", [32, 384])
def test_config5_bert_layer_gelu_as_table_is_bit_identical(C, seq):
    """dequantize -> GELU -> quantize between the two FFN linears as one table lookup on the
    int8 tensor: same int8 input to the second linear, same layer output, bit for bit."""
    from bladedisc_amd import bert_layer as B
    layer = B.QuantBertLayer(C.config5_weights(), B.RawBackend())
    h = layer.embed(C.config5_tokens(8, seq))
    layer.calibrate(h)
    rec_a, rec_b = {}, {}
    want = layer.forward(h, rec_a)
    layer.fuse_gelu = True
    got = layer.forward(h, rec_b)
    torch.cuda.synchronize()
    assert torch.equal(rec_b["ffn1"]["y_q"], rec_a["ffn1"]["y_q"])
    assert torch.equal(rec_b["ffn2"]["x_q"], rec_a["ffn2"]["x_q"])
    assert torch.equal(got, want)
    # the table really bends the values (GELU is not the identity on this range)
    t = layer.gelu_table.cpu().numpy().astype(np.int32)
    assert t.min() <= 0 and t.max() > 50 and (t[128:] <= 0).all()     # negatives map near 0-


@pytest.mark.parametrize("seq", [32, 384])
@pytest.mark.parametrize("fuse_gelu", [False, True])
def test_config5_bert_layer_dequantize_in_the_gemm_epilogue_is_bit_identical(C, seq, fuse_gelu):
    """Each linear whose int8 result is only dequantized writes the dequantized f32 from its
    epilogue: the f32 tensors and the layer output keep their bits."""
    from bladedisc_amd import bert_layer as B
    layer = B.QuantBertLayer(C.config5_weights(), B.RawBackend(), fuse_gelu=fuse_gelu)
    h = layer.embed(C.config5_tokens(8, seq))
    layer.calibrate(h)
    rec_a, rec_b = {}, {}
    want = layer.forward(h, rec_a)
    layer.fuse_dequant = True
    got = layer.forward(h, rec_b)
    torch.cuda.synchronize()
    for name in ("qkv", "out", "ffn2"):
        assert rec_b[name]["y_q"] is None
        assert torch.equal(rec_b[name]["y"].view(torch.int32), rec_a[name]["y"].view(torch.int32))
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))


@pytest.mark.parametrize("seq", [32, 384])
def test_config5_bert_layer_operators_in_the_gemm_epilogues_are_bit_identical(C, seq):
    """The residual additions behind the attention output and FFN2 and the GELU table behind
    FFN1 run in the producing GEMM's epilogue: the int8 input of FFN2, the two pre-LayerNorm
    sums and the layer output keep their bits."""
    from bladedisc_amd import bert_layer as B
    layer = B.QuantBertLayer(C.config5_weights(), B.RawBackend())
    h = layer.embed(C.config5_tokens(8, seq))
    layer.calibrate(h)
    rec_a, rec_b = {}, {}
    want = layer.forward(h, rec_a)
    layer.fuse_epilogue = layer.fuse_gelu = layer.fuse_dequant = True
    got = layer.forward(h, rec_b)
    torch.cuda.synchronize()
    assert torch.equal(rec_b["ffn2"]["x_q"], rec_a["ffn2"]["x_q"])
    pre1 = h.reshape(-1, h.shape[-1]) + rec_a["out"]["y"]
    assert torch.equal(rec_b["out"]["y_plus_residual"].view(torch.int32), pre1.view(torch.int32))
    pre2 = rec_a["ffn1"]["x"] + rec_a["ffn2"]["y"]
    assert torch.equal(rec_b["ffn2"]["y_plus_residual"].view(torch.int32), pre2.view(torch.int32))
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))


@pytest.mark.parametrize("backend", ["raw", "ral"])
@pytest.mark.parametrize("fused", [False, True, "epilogue"])
def test_config5_bert_layer_graph_replays_match_eager(C, fused, backend):
    """The captured layer against eager execution: several replays, with eager work and
    synchronisations in between, each compared bit for bit; also with the GELU table and the
    dequantize-in-epilogue forms switched on.  Through the RAL entries as well (the plugin
    path): their results come from the context's pool, so nothing is allocated while
    capturing, and the fused forms are the ral_pdll_qgemm_fused entries."""
    from bladedisc_amd import bert_layer as B
    from bladedisc_amd import ral
    ctx = ex = ex2 = stream = None
    if backend == "ral":
        stream = torch.cuda.Stream()
        ctx = ral.RalContext(stream=stream.cuda_stream)
        ex = ctx.execution()
        be = B.RalBackend(ex)
    else:
        be = B.RawBackend()
    try:
        layer = B.QuantBertLayer(C.config5_weights(), be, fuse_gelu=bool(fused),
                                 fuse_dequant=bool(fused), fuse_epilogue=fused == "epilogue")
        h0 = layer.embed(C.config5_tokens(8, 32))
        layer.calibrate(h0)
        replay, static_in, static_out = layer.capture(h0, stream=stream)
        if backend == "ral":          # eager passes from here on run in another execution
            ex2 = ctx.execution()
            be.ex = ex2
        for i in range(4):
            h = layer.embed(C.config5_tokens(8, 32) if i == 0 else
                            np.roll(C.config5_tokens(8, 32), i, axis=1))
            if stream is not None:
                stream.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(stream):
                    want = layer.forward(h)               # eager work between the replays
            else:
                want = layer.forward(h)
            torch.cuda.synchronize()
            static_in.copy_(h)
            torch.cuda.synchronize()
            replay()
            torch.cuda.synchronize()
            assert torch.equal(static_out, want), "replay %d differs from eager" % i
    finally:
        torch.cuda.synchronize()
        for e in (ex2, ex):
            if e is not None:
                e.close()
        if ctx is not None:
            ctx.close()
