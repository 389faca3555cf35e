"""Pins the oracle's restatement of the reference observers' qparams arithmetic
(tools/torch_quant/torch_quant/observer.py:134-163, 221-224, 312-319) with closed forms,
each chosen so that a plausible slip (127 for 127.5, a missing eps floor, the wrong sign or
rounding of the zero point, a clamp left out) fails it."""
import numpy as np
import pytest

from oracle import observer_oracle as OB


def test_quant_ranges():
    assert OB.calc_quant_min_max(8, True) == (-128, 127)
    assert OB.calc_quant_min_max(8, False) == (0, 255)
    assert OB.calc_quant_min_max(32, True) == (-2 ** 31, 2 ** 31 - 1)


def test_symmetric_scale_divides_by_half_the_range():
    # (q_max - q_min) / 2 = 127.5 for qint8, not 127
    s, z = OB.calculate_qparams(-1.0, 2.55, -128, 127, symmetric=True)
    assert s == np.float32(np.float32(2.55) / np.float32(127.5)) and z == 0
    # the larger magnitude wins, whichever side it is on
    s, _ = OB.calculate_qparams(-5.1, 1.0, -128, 127, symmetric=True)
    assert s == np.float32(np.float32(5.1) / np.float32(127.5))
    # a range that does not contain zero is extended to it (min_neg / max_pos)
    s, _ = OB.calculate_qparams(1.0, 2.55, -128, 127, symmetric=True)
    assert s == np.float32(np.float32(2.55) / np.float32(127.5))


def test_scale_floor_is_float32_eps():
    s, z = OB.calculate_qparams(0.0, 0.0, -128, 127, symmetric=True)
    assert s == np.finfo(np.float32).eps and z == 0
    s, z = OB.calculate_qparams(0.0, 0.0, 0, 255, symmetric=False)
    assert s == np.finfo(np.float32).eps and z == 0


def test_affine_zero_point():
    # [-1, 3] on quint8: scale 4/255, zp = 0 - round(-1 / scale) = round(63.75) = 64
    s, z = OB.calculate_qparams(-1.0, 3.0, 0, 255, symmetric=False)
    assert s == np.float32(np.float32(4.0) / np.float32(255.0)) and z == 64
    # qint8: zp = -128 - round(-1/scale) = -128 + 64 = -64
    s, z = OB.calculate_qparams(-1.0, 3.0, -128, 127, symmetric=False)
    assert z == -64
    # round-half-to-even: [-2.5, 252.5] on quint8 -> scale exactly 1, min/scale = -2.5 -> -2
    s, z = OB.calculate_qparams(-2.5, 252.5, 0, 255, symmetric=False)
    assert s == 1.0 and z == 2
    s, z = OB.calculate_qparams(-3.5, 251.5, 0, 255, symmetric=False)
    assert s == 1.0 and z == 4
    # an all-positive range is extended to zero: zp = q_min
    s, z = OB.calculate_qparams(2.0, 5.1, 0, 255, symmetric=False)
    assert s == np.float32(np.float32(5.1) / np.float32(255.0)) and z == 0
    # an all-negative one puts the zero point at q_max (255 - 0 clamps nothing, -(-255) = 255)
    s, z = OB.calculate_qparams(-5.1, -2.0, 0, 255, symmetric=False)
    assert z == 255


def test_per_channel_vectors_and_unsigned_symmetric():
    lo = np.array([-1.0, -0.5, 0.0], np.float32)
    hi = np.array([0.5, 2.0, 0.0], np.float32)
    s, z = OB.calculate_qparams(lo, hi, -128, 127, symmetric=True)
    want = np.maximum(np.array([1.0, 2.0, 0.0], np.float32) / np.float32(127.5),
                      np.finfo(np.float32).eps)
    np.testing.assert_array_equal(s, want)
    np.testing.assert_array_equal(z, [0, 0, 0])
    _, z = OB.calculate_qparams(lo, hi, 0, 255, symmetric=True, unsigned=True)
    np.testing.assert_array_equal(z, [128, 128, 128])


def test_unobserved_state_and_bad_ranges():
    s, z = OB.calculate_qparams(np.float32("inf"), np.float32("-inf"), -128, 127, True)
    assert s == 1.0 and z == 0
    s, z = OB.calculate_qparams(np.zeros(0), np.zeros(0), -128, 127, True)
    assert s == 1.0 and z == 0
    with pytest.raises(AssertionError):
        OB.calculate_qparams(1.0, -1.0, -128, 127, True)


def test_running_min_max_and_bias_scale():
    a = np.array([[1.0, -2.0], [0.5, 3.0]], np.float32)
    b = np.array([[4.0, -1.0], [-7.0, 0.0]], np.float32)
    lo, hi = OB.running_min_max([a, b])
    assert lo == -7.0 and hi == 4.0
    lo, hi = OB.running_min_max([a, b], ch_axis=1)
    np.testing.assert_array_equal(lo, [-7.0, -2.0])
    np.testing.assert_array_equal(hi, [4.0, 3.0])
    lo, hi = OB.running_min_max([a, b], ch_axis=0)
    np.testing.assert_array_equal(lo, [-2.0, -7.0])
    np.testing.assert_array_equal(hi, [4.0, 3.0])
    np.testing.assert_array_equal(OB.bias_scale(np.array([0.5, 0.25], np.float32), np.float32(0.1)),
                                  np.array([0.5, 0.25], np.float32) * np.float32(0.1))
