"""Pins oracle/tf_quant_oracle.py (the reference's lowering of tf.QuantizeV2 / tf.Dequantize,
tao_compiler/mlir/disc/transforms/lower_tf.cc:307-654) with known answers.

The inputs are the ones of the reference's own tests (disc/tests/tensorflow_ops/
quantize_v2.cc, dequantize.cc), which compare against a TensorFlow run and hold no output
values; the expected outputs below are derived from the definitions of the modes in float64
(none of the cases sits on a rounding tie, so the rounding mode does not enter).
"""
import math

import numpy as np
import pytest

from oracle import tf_quant_oracle as tfo

EDGE = [-255.0, 0.0, 1.0, 1.25, 1.75, 64.0, 127.0, 500.0]      # quantize_v2.cc:78-79


def edge_tensor():
    n = 2 * 3 * 4 * 5
    return np.array([EDGE[i % 8] for i in range(n)], np.float32).reshape(2, 3, 4, 5)


def test_adjusted_range_closed_forms():
    # already contains zero and is wide enough: unchanged
    lo, hi = tfo.adjust_min_max_range(-255.0, 127.0)
    assert (lo, hi) == (-255.0, 127.0)
    # one-sided positive range is extended down to zero
    lo, hi = tfo.adjust_min_max_range(3.0, 10.0)
    assert (lo, hi) == (0.0, 10.0)
    # one-sided negative range: max becomes max(0, min + eps) = 0
    lo, hi = tfo.adjust_min_max_range(-8.0, -2.0)
    assert (lo, hi) == (-8.0, 0.0)
    # degenerate range: widened by ensure_minimum_range * max(|min|, |max|, 1)
    lo, hi = tfo.adjust_min_max_range(0.0, 0.0)
    assert lo == 0.0 and hi == np.float32(0.01)
    lo, hi = tfo.adjust_min_max_range(-200.0, -200.0, ensure_minimum_range=0.5)
    assert lo == -200.0 and hi == 0.0           # -200 + 100 < 0
    lo, hi = tfo.adjust_min_max_range(50.0, 50.0, ensure_minimum_range=0.5)
    assert lo == 0.0 and hi == 50.0             # 0 + 25 < 50


def test_min_first_reference_vector():
    # quantize_v2.cc:24-40: range 0 .. 255 -> factor 1, bias round(0) - (-128) = 128
    x = np.array([0.0, 1.0, 1.25, 1.75, 127.0, 255.0, 500.0] * 2, np.float32).reshape(2, 7)
    q, lo, hi = tfo.quantize_v2_min_first(x, 0.0, 255.0)
    want = [-128, -127, -127, -126, -1, 127, 127] * 2
    assert q.dtype == np.int8 and q.reshape(-1).tolist() == want
    assert (lo, hi) == (0.0, 255.0)


def test_min_first_factor_is_range_over_255():
    # lower_tf.cc:416-423 multiplies by (max - min) / 255; with the range -51 .. 51 that is
    # 0.4, and the bias is round(-51 * 0.4) + 128 = 108
    x = np.array([-300.0, -10.0, 0.0, 3.0, 10.0, 100.0], np.float32)
    q, lo, hi = tfo.quantize_v2_min_first(x, -51.0, 51.0)
    want = [max(-128, min(127, round(v * 0.4) - 108)) for v in x.tolist()]
    assert want == [-128, -112, -108, -107, -104, -68]
    assert q.tolist() == want
    qu, _, _ = tfo.quantize_v2_min_first(x, -51.0, 51.0, signed=False)
    assert qu.dtype == np.uint8
    assert qu.tolist() == [max(0, min(255, round(v * 0.4) + 20)) for v in x.tolist()]


def expected_scaled(values, mn, mx, min_q=-128.0, max_q=127.0):
    sf = min(min_q / mn if mn * min_q > 0 else math.inf, max_q / mx if mx * max_q > 0 else math.inf)
    out = []
    for v in values:
        v = min(max(v, min_q / sf), max_q / sf)
        t = v * sf
        assert abs(abs(t - math.floor(t)) - 0.5) > 1e-3     # no tie among the cases
        out.append(int(round(t)))
    return out, min_q / sf, max_q / sf


def test_scaled_scalar_reference_vector():
    # quantize_v2.cc:132-148: range -255 .. 127 -> factor min(128/255, 1) = 128/255
    q, lo, hi = tfo.quantize_v2_scaled(edge_tensor(), -255.0, 127.0)
    want, wlo, whi = expected_scaled(EDGE, -255.0, 127.0)
    assert want == [-128, 0, 1, 1, 1, 32, 64, 127]
    assert q.reshape(-1, 8).tolist() == [want] * 15
    assert lo == pytest.approx(wlo, rel=1e-6) and hi == pytest.approx(whi, rel=1e-6)


def test_scaled_per_channel_reference_vector():
    # quantize_v2.cc:76-93: axis 1 with ranges (-255 c, 127 c), c = 1, 2, 3
    x = edge_tensor()
    mn = np.array([-255.0, -510.0, -765.0], np.float32)
    mx = np.array([127.0, 254.0, 381.0], np.float32)
    q, lo, hi = tfo.quantize_v2_scaled(x, mn, mx, axis=1)
    assert lo.shape == (3,) and hi.shape == (3,)
    for c in range(3):
        want_tab, wlo, whi = expected_scaled(EDGE, float(mn[c]), float(mx[c]))
        want = np.array([want_tab[EDGE.index(float(v))] for v in x[:, c].reshape(-1)])
        assert np.array_equal(q[:, c].reshape(-1), want)
        assert lo[c] == pytest.approx(wlo, rel=1e-6) and hi[c] == pytest.approx(whi, rel=1e-6)
    assert expected_scaled(EDGE, -765.0, 381.0)[0] == [-43, 0, 0, 0, 0, 11, 21, 84]


def test_scaled_narrow_range_one_sided_and_unsigned():
    # narrow_range: the lowest code is -127, so a symmetric range maps onto -127 .. 127
    q, lo, hi = tfo.quantize_v2_scaled(np.array([-10.0, -1.0, 0.26, 1.0, 10.0], np.float32), -1.0, 1.0,
                                       narrow_range=True)
    assert q.tolist() == [-127, -127, 33, 127, 127] and (lo, hi) == (-1.0, 1.0)
    # without it the positive side decides: factor 127, min_out = -128 / 127
    q, lo, hi = tfo.quantize_v2_scaled(np.array([-10.0, -1.0, 1.0], np.float32), -1.0, 1.0)
    assert q.tolist() == [-128, -127, 127] and hi == 1.0 and lo == np.float32(-128.0) / np.float32(127.0)
    # a range that starts at zero takes its factor from the positive side alone
    q, lo, hi = tfo.quantize_v2_scaled(np.array([-3.0, 0.0, 1.0, 2.0, 5.0], np.float32), 0.0, 2.0)
    assert q.tolist() == [-128, 0, 64, 127, 127]            # 63.5 would be a tie: 1 * 63.5
    # unsigned output: codes 0 .. 255, negative inputs clamp to 0
    q, lo, hi = tfo.quantize_v2_scaled(np.array([-3.0, 0.0, 0.3, 1.0, 5.0], np.float32), 0.0, 1.0,
                                       signed=False)
    assert q.dtype == np.uint8 and q.tolist() == [0, 0, 76, 255, 255] and (lo, hi) == (0.0, 1.0)


def test_dequantize_reference_vectors():
    # dequantize.cc:24-133: factor max(min / -128, max / 127)
    vals = [-127, -128, 127, 0, 1, 3, 12, -34]
    n = 2 * 3 * 4 * 5
    q = np.array([vals[i % 8] for i in range(n)], np.int8).reshape(2, 3, 4, 5)
    y = tfo.dequantize_scaled(q, -255.0, 127.0)
    sf = max(255.0 / 128.0, 1.0)
    assert np.allclose(y, q.astype(np.float64) * sf, rtol=1e-6, atol=0)
    mn = np.array([-255.0, -255.0 * 0.2, -255.0 * 0.3], np.float32)
    mx = np.array([127.0, 127.0 * 0.2, 127.0 * 0.3], np.float32)
    y = tfo.dequantize_scaled(q, mn, mx, axis=1)
    for c, k in enumerate((1.0, 0.2, 0.3)):
        assert np.allclose(y[:, c], q[:, c].astype(np.float64) * (255.0 * k / 128.0), rtol=1e-6, atol=0)
    # narrow range: -127 is the lowest code the minimum maps to
    assert tfo.dequantize_factor(-127.0, 100.0, narrow_range=True) == 1.0
    # unsigned input: only the maximum enters
    yu = tfo.dequantize_scaled(np.array([0, 51, 255], np.uint8), -7.0, 5.1)
    assert np.allclose(yu, [0.0, 1.02, 5.1], rtol=1e-6)


def test_quantize_then_dequantize_returns_the_grid():
    rng = np.random.default_rng(7)
    x = rng.normal(0, 1, 4096).astype(np.float32)
    q, lo, hi = tfo.quantize_v2_scaled(x, x.min(), x.max())
    y = tfo.dequantize_scaled(q, lo, hi)
    step = float(tfo.dequantize_factor(lo, hi))
    assert np.max(np.abs(y - np.clip(x, lo, hi))) <= step * 0.5001
