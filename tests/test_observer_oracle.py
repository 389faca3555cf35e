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


def test_fake_quant_against_torch_fake_quantize():
    """The observers' fake quantization here is quantize -> dequantize as a compiled program
    executes it (x / scale, a true division); the reference's observer calls
    torch.fake_quantize_per_{tensor,channel}_affine (observer.py:203-206), which multiplies
    by 1 / scale.  On the CPU, against torch itself: the two agree wherever x / scale + zp is
    not within a few ulp of a rounding tie, never differ by more than one quantization step,
    and on random data differ on fewer than one element in a thousand."""
    import torch
    import oracle as O
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((64, 96)) * 2).astype(np.float32)
    # per tensor, symmetric int8 and affine uint8
    for (scale, zp, qmin, qmax, dt) in ((0.0173, 0, -128, 127, np.int8), (0.031, 117, 0, 255, np.uint8)):
        q = O.quantize(x, np.float32(scale), zp, qmin=qmin, qmax=qmax, dtype=dt)
        mine = O.dequantize(q, np.float32(scale), zp)
        ref = torch.fake_quantize_per_tensor_affine(torch.from_numpy(x), scale, zp, qmin, qmax).numpy()
        diff = np.abs(mine - ref)
        assert diff.max() <= np.float32(scale) * 1.0001
        t = x.astype(np.float64) / np.float32(scale) + zp
        near_tie = np.abs(np.abs(t - np.floor(t)) - 0.5) < 1e-4
        assert not (diff[~near_tie] > 0).any()
        assert (diff > 0).mean() < 1e-3
    # per channel (axis 0), the weight observers' form
    scale = rng.uniform(0.005, 0.03, 64).astype(np.float32)
    zp = np.zeros(64, np.int32)
    q = O.quantize(x, scale, zp, axis=0)
    mine = O.dequantize(q, scale, zp, axis=0)
    ref = torch.fake_quantize_per_channel_affine(torch.from_numpy(x), torch.from_numpy(scale),
                                                 torch.from_numpy(zp), 0, -128, 127).numpy()
    diff = np.abs(mine - ref)
    assert (diff <= scale[:, None] * 1.0001).all() and (diff > 0).mean() < 1e-3
    # an exact tie where the two really part: x / s is a tie in exact arithmetic, x * (1 / s)
    # need not be
    s = np.float32(0.1)
    xt = (np.arange(1, 200, 2, dtype=np.float32) * np.float32(0.05)).astype(np.float32)
    q = O.quantize(xt, s, 0)
    ref = torch.fake_quantize_per_tensor_affine(torch.from_numpy(xt), float(s), 0, -128, 127).numpy()
    assert np.abs(O.dequantize(q, s, 0) - ref).max() <= s * 1.0001
