"""tf.QuantizeV2 and tf.Dequantize on the GPU, with the attributes and the limits of the
reference's lowering (tao_compiler/mlir/disc/transforms/lower_tf.cc:307-654).

The reference rewrites the two ops only in the forms below and leaves every other form
unlowered, which fails its compilation; the same forms raise NotImplementedError here:

  QuantizeV2   mode SCALED (any axis) or MIN_FIRST (axis -1 only); round_mode
               HALF_AWAY_FROM_ZERO (the attribute's name: the op the pattern emits, tf.Round,
               rounds half to even); f32 input and ranges; qint8 / quint8 output
  Dequantize   mode SCALED; qint8 / quint8 input; f32 output
"""
import torch

from . import _lib
from .kernels import _need_cuda, _ptr, _stream, _view3

_MODES = {"SCALED": 0, "MIN_FIRST": 1}


def _params(channels, device):
    nbytes = _lib.lib().dq8_tf_params_bytes(channels)
    return torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes


def _ranges(min_range, max_range, x, axis):
    _need_cuda(x, min_range, max_range)
    if min_range.dtype != torch.float32 or max_range.dtype != torch.float32:
        raise NotImplementedError("range operands must be float32 (lower_tf.cc:325-331)")
    if min_range.shape != max_range.shape:
        raise ValueError("min_range and max_range must have the same shape")
    if axis == -1:
        if min_range.numel() != 1:
            raise ValueError("axis = -1 takes scalar ranges")
        return _view3(tuple(x.shape), None)
    if not 0 <= axis < x.dim():
        raise ValueError("axis %d out of range for rank %d" % (axis, x.dim()))
    outer, nch, inner = _view3(tuple(x.shape), axis)
    if min_range.numel() != nch:
        raise ValueError("ranges must have one entry per slice along axis (%d)" % nch)
    return outer, nch, inner


def quantize_v2(x, min_range, max_range, T=torch.int8, mode="MIN_COMBINED",
                round_mode="HALF_AWAY_FROM_ZERO", narrow_range=False, axis=-1,
                ensure_minimum_range=0.01):
    """Returns (output, output_min, output_max) like the TF op.  x, min_range, max_range:
    device f32 tensors.  The defaults are the TF op's, so `mode` has to be given: its
    default, MIN_COMBINED, is one of the forms the reference does not lower."""
    if T not in (torch.int8, torch.uint8):
        raise NotImplementedError("QuantizeV2: output type %s is not lowered" % T)
    if x.dtype != torch.float32:
        raise NotImplementedError("QuantizeV2: only float32 input is lowered (lower_tf.cc:325)")
    if mode == "MIN_FIRST" and axis != -1:
        raise NotImplementedError("QuantizeV2: MIN_FIRST with an axis (lower_tf.cc:335-338)")
    if mode not in _MODES:
        raise NotImplementedError("QuantizeV2: mode %s is not lowered (lower_tf.cc:344-345)" % mode)
    if round_mode != "HALF_AWAY_FROM_ZERO":
        raise NotImplementedError("QuantizeV2: round_mode %s is not lowered (lower_tf.cc:347-348)"
                                  % round_mode)
    outer, nch, inner = _ranges(min_range, max_range, x, axis)
    x = x.contiguous()
    out = torch.empty(x.shape, dtype=T, device=x.device)
    out_min = torch.empty_like(min_range)
    out_max = torch.empty_like(max_range)
    params, nbytes = _params(nch, x.device)
    st = _lib.lib().dq8_tf_quantize_v2(
        _ptr(x), _ptr(out), 0 if T == torch.int8 else 1, outer, nch, inner,
        _ptr(min_range.contiguous()), _ptr(max_range.contiguous()), _MODES[mode],
        1 if narrow_range else 0, float(ensure_minimum_range), _ptr(out_min), _ptr(out_max),
        _ptr(params), nbytes, _stream())
    _lib.check(st, "dq8_tf_quantize_v2")
    return out, out_min, out_max


def dequantize(q, min_range, max_range, mode="MIN_COMBINED", narrow_range=False, axis=-1):
    """tf.Dequantize: device int8 / uint8 tensor -> f32."""
    if q.dtype not in (torch.int8, torch.uint8):
        raise NotImplementedError("Dequantize: input type %s is not lowered" % q.dtype)
    if mode != "SCALED":
        raise NotImplementedError("Dequantize: mode %s is not lowered (lower_tf.cc:586-590)" % mode)
    outer, nch, inner = _ranges(min_range, max_range, q, axis)
    q = q.contiguous()
    out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    params, nbytes = _params(nch, q.device)
    st = _lib.lib().dq8_tf_dequantize(
        _ptr(q), 0 if q.dtype == torch.int8 else 1, _ptr(out), outer, nch, inner,
        _ptr(min_range.contiguous()), _ptr(max_range.contiguous()), 1 if narrow_range else 0,
        _ptr(params), nbytes, _stream())
    _lib.check(st, "dq8_tf_dequantize")
    return out
