"""CPU restatement of the reference's lowering of TensorFlow's QuantizeV2 and Dequantize
(R = tao_compiler/mlir/disc/transforms/lower_tf.cc): test infrastructure only, like the rest
of this package.

The reference rewrites the two TF ops into chains of elementwise f32 TF ops; this file runs
the same chains in numpy float32, one separately rounded operation per emitted op.
`tf.Round` rounds half to even (TensorFlow's published semantics of the op; its legalization
lives in TensorFlow, which is not part of R), so `np.rint` stands for it even though the
attribute the pattern accepts is called HALF_AWAY_FROM_ZERO (R:346-347, 549-554).

MIN_FIRST follows R:415-444 as written: the factor is (max - min) / 255, the reciprocal of
TensorFlow's own kernel; both agree on the one range the reference tests (0 .. 255).

Pinned by known answers (tests/test_tf_quant_oracle.py): the input vectors and ranges of
R's tests (disc/tests/tensorflow_ops/quantize_v2.cc:24-200, dequantize.cc:24-133) with
outputs derived by hand from the SCALED / MIN_FIRST definitions in float64, the adjusted
ranges in closed form, narrow_range, zero and one-sided ranges, unsigned outputs.
"""
import numpy as np

F = np.float32
FLT_MAX = np.finfo(np.float32).max


def numeric_limits(signed):
    """R:251-290 for 8-bit types: (lowest_quantized, lower_bound_float, upper_bound_float)."""
    return (-128.0, -128.0, 127.0) if signed else (0.0, 0.0, 255.0)


def adjust_min_max_range(min_range, max_range, ensure_minimum_range=0.01):
    """R:365-393 (mirrors tensorflow/core/kernels/quantize_op.cc)."""
    mn = np.asarray(min_range, F)
    mx = np.asarray(max_range, F)
    lo = np.minimum(F(0), mn)
    eps = np.maximum(np.maximum(np.abs(mn), np.abs(mx)), F(1)) * F(ensure_minimum_range)
    hi = (eps + lo).astype(F)
    hi = np.maximum(mx, hi)
    hi = np.maximum(F(0), hi)
    return lo.astype(F), hi.astype(F)


def quantize_v2_min_first(x, min_range, max_range, signed=True, ensure_minimum_range=0.01):
    """R:395-451.  Scalar ranges only (R:338 refuses an axis).  Returns (q, min, max)."""
    x = np.asarray(x, F)
    lowest, lb, ub = numeric_limits(signed)
    lo, hi = adjust_min_max_range(min_range, max_range, ensure_minimum_range)
    rs = ((hi - lo).astype(F) / F(255.0)).astype(F)
    r = np.rint((x * rs).astype(F))
    rms = np.rint((lo * rs).astype(F))
    bias = (rms - F(lowest)).astype(F)
    r = (r - bias).astype(F)
    r = np.minimum(np.maximum(r, F(lb)), F(ub))
    return r.astype(np.int8 if signed else np.uint8), lo, hi


def scaled_factor(min_range, max_range, signed=True, narrow_range=False,
                  ensure_minimum_range=0.01):
    """R:453-538: (scale_factor, min_out, max_out) per range entry."""
    _, lb, ub = numeric_limits(signed)
    lo, hi = adjust_min_max_range(min_range, max_range, ensure_minimum_range)
    min_q = F(lb + (1.0 if narrow_range else 0.0))
    max_q = F(ub)
    adj_lo = (lo - (lo == 0).astype(F) * F(1e-6)).astype(F)
    with np.errstate(divide="ignore", invalid="ignore"):
        sf_lo = (min_q / adj_lo).astype(F)
    sf_lo = np.where((lo * min_q).astype(F) > 0, sf_lo, F(FLT_MAX)).astype(F)
    adj_hi = (hi - (hi == 0).astype(F) * F(1e-6)).astype(F)
    with np.errstate(divide="ignore", invalid="ignore"):
        sf_hi = (max_q / adj_hi).astype(F)
    sf_hi = np.where((hi * max_q).astype(F) > 0, sf_hi, F(FLT_MAX)).astype(F)
    sf = np.minimum(sf_lo, sf_hi).astype(F)
    return sf, (min_q / sf).astype(F), (max_q / sf).astype(F)


def _along(v, axis, rank):
    """R:288-305 `expandValueDims`: a per-channel vector broadcast along `axis`."""
    v = np.asarray(v, F)
    if axis == -1 or v.ndim == 0:
        return v
    return v.reshape(v.shape + (1,) * (rank - 1 - axis))


def quantize_v2_scaled(x, min_range, max_range, signed=True, narrow_range=False, axis=-1,
                       ensure_minimum_range=0.01):
    """R:453-560.  Returns (q, min_out, max_out)."""
    x = np.asarray(x, F)
    sf, lo, hi = scaled_factor(min_range, max_range, signed, narrow_range,
                               ensure_minimum_range)
    r = np.minimum(np.maximum(x, _along(lo, axis, x.ndim)), _along(hi, axis, x.ndim))
    r = np.rint((r * _along(sf, axis, x.ndim)).astype(F))
    return r.astype(np.int8 if signed else np.uint8), lo, hi


def dequantize_factor(min_range, max_range, signed=True, narrow_range=False):
    """R:629-644: the factor TF Dequantize (SCALED) multiplies by."""
    _, lb, ub = numeric_limits(signed)
    mn = np.asarray(min_range, F)
    mx = np.asarray(max_range, F)
    sf = (mx / F(ub)).astype(F)
    if lb != 0.0:
        min_q = F(lb + (1.0 if narrow_range else 0.0))
        sf = np.maximum((mn / min_q).astype(F), sf)
    return sf.astype(F)


def dequantize_scaled(q, min_range, max_range, narrow_range=False, axis=-1):
    """R:602-654.  q: int8 or uint8 array."""
    q = np.asarray(q)
    signed = q.dtype == np.int8
    sf = dequantize_factor(min_range, max_range, signed, narrow_range)
    return (_along(sf, axis, q.ndim) * q.astype(F)).astype(F)
