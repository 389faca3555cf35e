"""End to end against PyTorch's eager fake-quantized linear, the way the reference's own
end-to-end tests check the compiled int8 path
(R/pytorch_blade/tests/disc/pdl/test_e2e/test_quantization.py: a model of
fake_quantize(x) -> linear(fake_quantize(w), bias) -> fake_quantize, the scales 0.1 / 0.3 /
0.2 and shapes of its cases, ranks 2 to 4, bias none / f32 / int32-quantized, per-tensor and
per-channel weights).  Here the left-hand side is quantize -> ral_pdll_qgemm -> dequantize
through the runtime ABI.  The eager model accumulates in float32, the kernels in int32, so
results may differ where the float sum lands on the other side of a rounding tie: the
reference's GPU variant of this test allows one output step (atol = output scale), and so
does this one -- and only there: with these scales (s_x s_w / s_o = 0.15) one accumulator
value in twenty is an exact tie, so wherever the exact pre-rounding value (from an int64
product, in float64) is not within 1e-4 of a half-integer the two sides must agree exactly."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

S_X, S_W, S_O = 0.1, 0.3, 0.2          # the reference cases' scales


@pytest.fixture(scope="module")
def rt():
    from bladedisc_amd import ral, ral_ops
    ctx = ral.RalContext(stream=torch.cuda.current_stream().cuda_stream)
    yield ctx, ral, ral_ops
    torch.cuda.synchronize()
    ctx.close()


def t1(v, dtype=torch.float32):
    return torch.tensor([v], dtype=dtype, device="cuda")


def eager(x, w, bias, sw, per_channel):
    """The reference test's Model.forward."""
    x = torch.fake_quantize_per_tensor_affine(x, S_X, 0, -128, 127)
    if per_channel:
        z = torch.zeros(sw.numel(), dtype=torch.int32, device="cuda")
        w = torch.fake_quantize_per_channel_affine(w, sw, z, 0, -128, 127)
    else:
        w = torch.fake_quantize_per_tensor_affine(w, S_W, 0, -128, 127)
    y = torch.nn.functional.linear(x, w, bias=bias)
    return torch.fake_quantize_per_tensor_affine(y, S_O, 0, -128, 127)


def check(got, want, exact, margin=1e-4):
    """exact: float64 value of (acc + bias terms) / s_o before rounding; the two sides must
    agree wherever that is further than `margin` from a half-integer."""
    diff = (got - want).abs().double()
    assert float(diff.max()) <= S_O * 1.0001, "more than one output step apart"
    frac = (exact - torch.floor(exact) - 0.5).abs()
    away_from_tie = (frac > margin) & (exact.abs() < 127)
    assert bool((diff[away_from_tie] == 0).all()), "differs away from a rounding tie"
    assert float(away_from_tie.double().mean()) > 0.7


def pre_round(x_q, w_q, sw, bias_f64):
    """(sum x_q w_q) s_x s_w[n] / s_o + bias / s_o in float64 from an exact integer product."""
    acc = x_q.reshape(-1, x_q.shape[-1]).cpu().long() @ w_q.cpu().long().T
    t = acc.double() * (S_X / S_O) * sw.cpu().double()[None, :]
    if bias_f64 is not None:
        t = t + bias_f64.cpu().double()[None, :] / S_O
    return t.cuda()


@pytest.mark.parametrize("shape", [(1, 64), (1, 2, 64), (1, 2, 3, 64), (37, 64)])
@pytest.mark.parametrize("bias_kind", ["none", "f32", "s32"])
@pytest.mark.parametrize("per_channel", [False, True])
def test_cpu_signature_entry_against_eager_fake_quant(rt, shape, bias_kind, per_channel):
    ctx, ral, ops = rt
    from bladedisc_amd import kernels as K
    g = torch.Generator(device="cuda").manual_seed(
        1000 * len(shape) + 100 * shape[0] + 10 * ["none", "f32", "s32"].index(bias_kind) + per_channel)
    x = torch.randn(shape, device="cuda", generator=g)
    w = torch.randn((64, 64), device="cuda", generator=g)
    sw = (torch.rand(64, device="cuda", generator=g) * 0.2 + 0.2) if per_channel \
        else torch.full((64,), S_W, device="cuda")
    bias = None
    if bias_kind != "none":
        bias = torch.randn(64, device="cuda", generator=g)
    bias_model = bias
    if bias_kind == "s32":
        # the reference quantizes the bias to int32 with scale s_x * s_w and feeds the
        # integers (test_quantization.py: bias_scale = input_scale * weight_scale)
        bs = S_X * sw
        zb = torch.zeros(64, dtype=torch.int32, device="cuda")
        bias_model = torch.fake_quantize_per_channel_affine(bias, bs, zb, 0, -2 ** 31, 2 ** 31 - 1)
        bias = torch.round(bias / bs).to(torch.int32)
    want = eager(x, w, bias_model, sw, per_channel)

    z1 = torch.zeros(1, dtype=torch.int32, device="cuda")
    zc = torch.zeros(64, dtype=torch.int32, device="cuda")
    w_q = K.quantize(w, sw, zc, axis=0)
    with ctx.execution() as ex:
        x_q = ops.quantize(ex, x, t1(S_X), z1)
        y_q = ops.pdll_qgemm_cpu_style(ex, x_q, w_q, bias, t1(S_X), sw, t1(S_O), transpose_b=True)
        got = ops.dequantize(ex, y_q, t1(S_O), z1)
        torch.cuda.synchronize()
        assert tuple(got.shape) == tuple(shape[:-1]) + (64,)
        exact = pre_round(x_q, w_q, sw, bias_model)
        # An f32 bias reaches the accumulator as an integer (oneDNN's bias reorder with
        # scale 1 / (s_x s_w), which the entry mirrors) while the eager model adds the float:
        # the two pre-rounding values differ by up to half a bias step, s_x s_w / (2 s_o).
        margin = float((S_X * sw.max() / (2 * S_O)).item()) + 1e-3 if bias_kind == "f32" else 1e-4
        check(got.reshape(-1, 64), want.reshape(-1, 64), exact, margin)


@pytest.mark.parametrize("shape", [(1, 64), (4, 5, 64)])
@pytest.mark.parametrize("bias_kind", ["f32", "i8"])
def test_gpu_signature_entry_against_eager_fake_quant(rt, shape, bias_kind):
    """The reference's gpu entries take the bias already in output units: bias / s_o as f32
    or quantize(bias, s_o) as int8 (its PDLL patterns insert that conversion)."""
    ctx, ral, ops = rt
    from bladedisc_amd import kernels as K
    g = torch.Generator(device="cuda").manual_seed(len(shape) * 7 + len(bias_kind))
    x = torch.randn(shape, device="cuda", generator=g)
    w = torch.randn((64, 64), device="cuda", generator=g)
    bias = torch.randn(64, device="cuda", generator=g)
    z1 = torch.zeros(1, dtype=torch.int32, device="cuda")
    if bias_kind == "i8":
        bias_op = K.quantize(bias, t1(S_O), z1)
        bias_model = bias_op.float() * S_O
    else:
        bias_op = bias / S_O
        bias_model = bias
    sw = torch.full((64,), S_W, device="cuda")
    want = eager(x, w, bias_model, sw, False)
    w_q = K.quantize(w, t1(S_W), z1)
    with ctx.execution() as ex:
        x_q = ops.quantize(ex, x, t1(S_X), z1)
        y_q = ops.pdll_qgemm_gpu(ex, x_q, w_q, bias_op, t1(S_X), t1(S_W), t1(S_O))
        got = ops.dequantize(ex, y_q, t1(S_O), z1)
        torch.cuda.synchronize()
        exact = pre_round(x_q, w_q, sw, bias_model)
        check(got.reshape(-1, 64), want.reshape(-1, 64), exact)


@pytest.mark.parametrize("shape,s_o", [((512, 512), 0.05), ((8, 512, 512), 0.1)])
def test_reference_gpu_cases_512(rt, shape, s_o):
    """The two GPU cases of the reference's end-to-end test (test_quantization.py:356-460):
    512 x 512 weights, inputs [512, 512] and [8, 512, 512], f32 bias, output scale 0.05 /
    0.1, checked the way it checks them -- within one output step (atol = output scale) --
    and, more strictly, equal wherever the exact pre-rounding value is neither saturated nor
    within 0.02 of a rounding tie (the eager model sums 512 products in float32)."""
    ctx, ral, ops = rt
    from bladedisc_amd import kernels as K
    g = torch.Generator(device="cuda").manual_seed(len(shape))
    x = torch.randn(shape, device="cuda", generator=g)
    w = torch.randn((512, 512), device="cuda", generator=g)
    bias = torch.randn(512, device="cuda", generator=g)
    z1 = torch.zeros(1, dtype=torch.int32, device="cuda")
    xf = torch.fake_quantize_per_tensor_affine(x, S_X, 0, -128, 127)
    wf = torch.fake_quantize_per_tensor_affine(w, S_W, 0, -128, 127)
    want = torch.fake_quantize_per_tensor_affine(torch.nn.functional.linear(xf, wf, bias=bias),
                                                 s_o, 0, -128, 127)
    w_q = K.quantize(w, t1(S_W), z1)
    with ctx.execution() as ex:
        x_q = ops.quantize(ex, x, t1(S_X), z1)
        y_q = ops.pdll_qgemm_gpu(ex, x_q, w_q, bias / s_o, t1(S_X), t1(S_W), t1(s_o))
        got = ops.dequantize(ex, y_q, t1(s_o), z1)
        torch.cuda.synchronize()
    assert tuple(got.shape) == tuple(shape)
    diff = (got - want).abs().double().reshape(-1, 512)
    assert float(diff.max()) <= s_o * 1.0001
    acc = (x_q.reshape(-1, 512).to(torch.float64) @ w_q.to(torch.float64).T)      # exact: < 2^53
    exact = acc * (S_X * S_W / s_o) + bias.double()[None, :] / s_o
    frac = (exact - torch.floor(exact) - 0.5).abs()
    clear = (frac > 0.02) & (exact.abs() < 127)
    assert bool((diff[clear] == 0).all())
    assert float(clear.double().mean()) > 0.05        # (most outputs saturate with these scales)
    assert float((diff == 0).double().mean()) > 0.99
