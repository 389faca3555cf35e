"""CPU restatement of the calibration arithmetic of the reference's observers
(R = tools/torch_quant/torch_quant/observer.py): test infrastructure only, like the rest of
this package.

Pinned by closed forms (tests/test_observer_oracle.py): every formula here is a handful of
float32 operations on min / max values, so hand-computed cases fix each branch -- symmetric
scale = max(|min|, |max|) / 127.5 for qint8, the eps floor, the affine zero point and its
clamp, the "never observed" default.  The reference file is read, not run.
"""
import numpy as np

EPS = np.finfo(np.float32).eps          # R:107 torch.finfo(torch.float32).eps


def calc_quant_min_max(bit, signed):
    """R:221-224."""
    q_min = -(1 << (bit - 1)) if signed else 0
    q_max = (1 << (bit - 1)) - 1 if signed else (1 << bit) - 1
    return q_min, q_max


def calculate_qparams(min_val, max_val, q_min, q_max, symmetric, unsigned=False):
    """R:134-163 (`Observer._calculate_qparams`) in float32.

    min_val / max_val: scalars or per-channel vectors.  Returns (scale f32, zero_point i32).
    A state that has observed nothing (min = +inf, max = -inf, or empty) gives (1.0, 0)
    (R:37-50, 135-136)."""
    min_val = np.asarray(min_val, np.float32)
    max_val = np.asarray(max_val, np.float32)
    if min_val.size == 0 or max_val.size == 0:
        return np.ones(1, np.float32), np.zeros(1, np.int32)
    if min_val.ndim == 0 and np.isposinf(min_val) and np.isneginf(max_val):
        return np.ones(1, np.float32), np.zeros(1, np.int32)
    if not np.all(min_val <= max_val):
        raise AssertionError("min %s should be less than max %s" % (min_val, max_val))
    min_neg = np.minimum(min_val, np.float32(0))
    max_pos = np.maximum(max_val, np.float32(0))
    zero_point = np.zeros(min_neg.shape, np.int32)
    if symmetric:
        max_pos = np.maximum(-min_neg, max_pos)
        scale = (max_pos / np.float32(float(q_max - q_min) / 2)).astype(np.float32)
        scale = np.maximum(scale, EPS)
        if unsigned:
            zero_point = np.full(min_neg.shape, 128, np.int32)
    else:
        scale = ((max_pos - min_neg) / np.float32(float(q_max - q_min))).astype(np.float32)
        scale = np.maximum(scale, EPS)
        # torch.round is round-half-to-even, as np.rint
        zero_point = (q_min - np.rint(min_neg / scale).astype(np.int32)).astype(np.int32)
        zero_point = np.clip(zero_point, q_min, q_max).astype(np.int32)
    return scale.astype(np.float32), zero_point


def running_min_max(chunks, ch_axis=None):
    """What the observers accumulate over the batches they see: the min and max over all of
    them, per tensor (R:238-241) or per slice along `ch_axis` (R:261-281)."""
    lo = hi = None
    for x in chunks:
        x = np.asarray(x, np.float32)
        if ch_axis is None:
            cur_lo, cur_hi = x.min(), x.max()
        else:
            red = tuple(i for i in range(x.ndim) if i != ch_axis)
            cur_lo, cur_hi = x.min(axis=red), x.max(axis=red)
        lo = cur_lo if lo is None else np.minimum(lo, cur_lo)
        hi = cur_hi if hi is None else np.maximum(hi, cur_hi)
    return np.asarray(lo, np.float32), np.asarray(hi, np.float32)


def bias_scale(w_scale, act_scale):
    """R:312-319 (`BiasObserver`): the bias is quantized to int32 with scale s_w * s_x."""
    return (np.asarray(w_scale, np.float32) * np.asarray(act_scale, np.float32)).astype(np.float32)
