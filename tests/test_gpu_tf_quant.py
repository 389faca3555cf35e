"""tf.QuantizeV2 / tf.Dequantize on the GPU against the oracle's restatement of the reference's
lowering (tao_compiler/mlir/disc/transforms/lower_tf.cc:307-654): bit-exact outputs and
ranges, on the reference's own test inputs (disc/tests/tensorflow_ops/quantize_v2.cc,
dequantize.cc), on seeded tensors over the three access patterns, and at full size.
"""
import numpy as np
import pytest
import torch

from oracle import tf_quant_oracle as tfo

pytestmark = pytest.mark.gpu

EDGE = [-255.0, 0.0, 1.0, 1.25, 1.75, 64.0, 127.0, 500.0]


def dev(a):
    a = np.asarray(a)
    return torch.from_numpy(np.ascontiguousarray(a) if a.ndim else a.copy()).cuda()


def same_bits(got, want):
    got = got.cpu().numpy()
    assert got.dtype == want.dtype and got.shape == want.shape
    assert np.array_equal(got.view(np.uint8 if got.itemsize == 1 else np.uint32),
                          want.view(np.uint8 if want.itemsize == 1 else np.uint32))


def test_reference_min_first_vector():
    from bladedisc_amd import tf_quant
    x = np.array([0.0, 1.0, 1.25, 1.75, 127.0, 255.0, 500.0] * 2, np.float32).reshape(2, 7)
    q, lo, hi = tf_quant.quantize_v2(dev(x), dev(np.float32(0)), dev(np.float32(255)),
                                     mode="MIN_FIRST")
    assert q.cpu().reshape(-1).tolist() == [-128, -127, -127, -126, -1, 127, 127] * 2
    assert float(lo) == 0.0 and float(hi) == 255.0


def test_reference_scaled_vectors():
    from bladedisc_amd import tf_quant
    x = np.array([EDGE[i % 8] for i in range(120)], np.float32).reshape(2, 3, 4, 5)
    q, lo, hi = tf_quant.quantize_v2(dev(x), dev(np.float32(-255)), dev(np.float32(127)),
                                     mode="SCALED")
    assert q.cpu().reshape(-1, 8).tolist() == [[-128, 0, 1, 1, 1, 32, 64, 127]] * 15
    wq, wlo, whi = tfo.quantize_v2_scaled(x, -255.0, 127.0)
    same_bits(q, wq)
    same_bits(lo, wlo)
    same_bits(hi, whi)
    mn = np.array([-255.0, -510.0, -765.0], np.float32)
    mx = np.array([127.0, 254.0, 381.0], np.float32)
    q, lo, hi = tf_quant.quantize_v2(dev(x), dev(mn), dev(mx), mode="SCALED", axis=1)
    wq, wlo, whi = tfo.quantize_v2_scaled(x, mn, mx, axis=1)
    same_bits(q, wq)
    same_bits(lo, wlo)
    same_bits(hi, whi)


def test_reference_dequantize_vectors():
    from bladedisc_amd import tf_quant
    vals = [-127, -128, 127, 0, 1, 3, 12, -34]
    q = np.array([vals[i % 8] for i in range(120)], np.int8).reshape(2, 3, 4, 5)
    y = tf_quant.dequantize(dev(q), dev(np.float32(-255)), dev(np.float32(127)), mode="SCALED")
    same_bits(y, tfo.dequantize_scaled(q, -255.0, 127.0))
    mn = np.array([-255.0, -255.0 * 0.2, -255.0 * 0.3], np.float32)
    mx = np.array([127.0, 127.0 * 0.2, 127.0 * 0.3], np.float32)
    y = tf_quant.dequantize(dev(q), dev(mn), dev(mx), mode="SCALED", axis=1)
    same_bits(y, tfo.dequantize_scaled(q, mn, mx, axis=1))


SHAPES = [
    ((4096,), -1), ((1003,), -1), ((7, 9, 11), -1), ((1, 1), -1),
    ((64, 768), 1), ((33, 52), 1), ((5, 7), 1), ((17, 3), 1),          # channel = last axis
    ((8, 6, 64), 1), ((2, 5, 12), 0), ((3, 4, 7), 1), ((6, 10), 0),    # rows / scalar
    ((2, 3, 4, 5), 1), ((2, 3, 4, 5), 3), ((32, 8, 8, 64), 3),
]


@pytest.mark.parametrize("signed", [True, False])
@pytest.mark.parametrize("narrow", [False, True])
@pytest.mark.parametrize("shape,axis", SHAPES)
def test_scaled_matches_oracle(shape, axis, narrow, signed):
    from bladedisc_amd import tf_quant
    rng = np.random.default_rng(abs(hash((shape, axis, narrow, signed))) % (1 << 31))
    x = (rng.normal(0, 1, shape) * rng.choice([0.01, 1.0, 30.0])).astype(np.float32)
    x.reshape(-1)[:: max(1, x.size // 17)] = 0.0
    if axis == -1:
        mn = np.float32(rng.uniform(-3, 0.5))
        mx = np.float32(rng.uniform(-0.5, 3))
    else:
        nch = shape[axis]
        mn = rng.uniform(-3, 0.5, nch).astype(np.float32)
        mx = rng.uniform(-0.5, 3, nch).astype(np.float32)
        mn[0], mx[0] = 0.0, 0.0                      # a degenerate range
        if nch > 1:
            mn[1], mx[1] = 0.25, 2.0                 # one-sided
    T = torch.int8 if signed else torch.uint8
    q, lo, hi = tf_quant.quantize_v2(dev(x), dev(mn), dev(mx), T=T, mode="SCALED",
                                     narrow_range=narrow, axis=axis)
    wq, wlo, whi = tfo.quantize_v2_scaled(x, mn, mx, signed=signed, narrow_range=narrow, axis=axis)
    same_bits(lo, np.asarray(wlo, np.float32))
    same_bits(hi, np.asarray(whi, np.float32))
    same_bits(q, wq)
    y = tf_quant.dequantize(q, lo, hi, mode="SCALED", narrow_range=narrow, axis=axis)
    same_bits(y, tfo.dequantize_scaled(wq, wlo, whi, narrow_range=narrow, axis=axis))


@pytest.mark.parametrize("signed", [True, False])
@pytest.mark.parametrize("shape", [(4096,), (1003,), (3, 5, 7), (64, 768)])
def test_min_first_matches_oracle(shape, signed):
    from bladedisc_amd import tf_quant
    rng = np.random.default_rng(len(shape) * 131 + shape[0] + signed)
    x = rng.normal(0, 40, shape).astype(np.float32)
    for mn, mx, emr in [(-51.0, 51.0, 0.01), (0.0, 255.0, 0.01), (-3.0, 200.0, 0.01),
                        (5.0, 5.0, 0.5), (-100.0, -100.0, 0.01)]:
        q, lo, hi = tf_quant.quantize_v2(dev(x), dev(np.float32(mn)), dev(np.float32(mx)),
                                         T=torch.int8 if signed else torch.uint8,
                                         mode="MIN_FIRST", ensure_minimum_range=emr)
        wq, wlo, whi = tfo.quantize_v2_min_first(x, mn, mx, signed=signed,
                                                 ensure_minimum_range=emr)
        same_bits(q, wq)
        assert float(lo) == float(wlo) and float(hi) == float(whi)


def test_forms_the_reference_does_not_lower_are_refused():
    from bladedisc_amd import tf_quant
    x = torch.zeros(8, device="cuda")
    r = torch.zeros((), device="cuda")
    with pytest.raises(NotImplementedError, match="MIN_COMBINED"):
        tf_quant.quantize_v2(x, r, r)
    with pytest.raises(NotImplementedError, match="HALF_TO_EVEN"):
        tf_quant.quantize_v2(x, r, r, mode="SCALED", round_mode="HALF_TO_EVEN")
    with pytest.raises(NotImplementedError, match="MIN_FIRST with an axis"):
        tf_quant.quantize_v2(x, r.reshape(1).expand(8), r.reshape(1).expand(8), mode="MIN_FIRST",
                             axis=0)
    with pytest.raises(NotImplementedError, match="MIN_FIRST"):
        tf_quant.dequantize(x.to(torch.int8), r, r, mode="MIN_FIRST")
    with pytest.raises(ValueError, match="one entry per slice"):
        tf_quant.quantize_v2(x.reshape(2, 4), torch.zeros(3, device="cuda"),
                             torch.zeros(3, device="cuda"), mode="SCALED", axis=1)
    empty = torch.zeros((0, 4), device="cuda")
    q, lo, hi = tf_quant.quantize_v2(empty, r - 1, r + 1, mode="SCALED")
    assert q.shape == (0, 4) and float(lo) == pytest.approx(-128 / 127) and float(hi) == 1.0


def test_full_size_round_trip_and_oracle_slices():
    """[16384, 4096] f32: per tensor and per channel along the last axis.  The oracle checks
    seeded slices; the whole tensor is checked through the round trip (dequantize returns
    the clamped input to within half a step) and by re-quantizing the result (idempotence)."""
    from bladedisc_amd import tf_quant
    g = torch.Generator(device="cuda").manual_seed(99)
    x = torch.randn(16384, 4096, device="cuda", generator=g)
    mn = x.amin().reshape(())
    mx = x.amax().reshape(())
    q, lo, hi = tf_quant.quantize_v2(x, mn, mx, mode="SCALED")
    y = tf_quant.dequantize(q, lo, hi, mode="SCALED")
    step = float(torch.maximum(lo / -128.0, hi / 127.0))
    assert float((y - torch.clamp(x, lo, hi)).abs().max()) <= step * 0.5001
    q2, _, _ = tf_quant.quantize_v2(y, lo, hi, mode="SCALED")
    assert torch.equal(q, q2)
    rows = [0, 1, 4097, 16383]
    wq, _, _ = tfo.quantize_v2_scaled(x[rows].cpu().numpy(), mn.cpu().numpy(), mx.cpu().numpy())
    assert np.array_equal(q[rows].cpu().numpy(), wq)

    mnc = x.amin(dim=0)
    mxc = x.amax(dim=0)
    q, lo, hi = tf_quant.quantize_v2(x, mnc, mxc, mode="SCALED", axis=1)
    wq, wlo, whi = tfo.quantize_v2_scaled(x[rows].cpu().numpy(), mnc.cpu().numpy(),
                                          mxc.cpu().numpy(), axis=1)
    assert np.array_equal(q[rows].cpu().numpy(), wq)
    same_bits(lo, wlo)
    y = tf_quant.dequantize(q, lo, hi, mode="SCALED", axis=1)
    stepc = torch.maximum(lo / -128.0, hi / 127.0)
    assert bool(((y - torch.maximum(torch.minimum(x, hi), lo)).abs() <= stepc * 0.5001).all())
