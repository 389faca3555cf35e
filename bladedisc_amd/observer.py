"""Calibration observers of the quantization tool, on the GPU kernels of this library.

The host-side mirror of the reference's observer interface for the quantized path
(tools/torch_quant/torch_quant/observer.py): same class names, constructor arguments,
modes (``observe`` / ``fake_quant``), state (``min_val``, ``max_val``, ``scale``,
``zero_point``) and error behaviour.  What runs on the device:

* the statistic -- running min / max per tensor or per channel -- is ``dq8_minmax`` (the
  reference calls ``torch.aminmax``, observer.py:238, 270-275);
* fake quantization is ``dq8_fake_quant``, ``dq8_quantize`` followed by ``dq8_dequantize`` in
  one pass: the arithmetic a compiled program executes for the observer's qparams (``x / scale`` as a true division;
  ``torch.fake_quantize_per_tensor_affine``, which the reference calls at observer.py:203-206,
  multiplies by ``1 / scale`` and can differ from it in the last bit at ties).

The qparams arithmetic itself (observer.py:134-163) is a handful of float32 operations on
the min / max vectors; it is done with torch on the device that holds the state.
"""
from typing import NamedTuple, Tuple

import torch

from . import kernels as K

DTYPE_TO_BIT_SIGN = {                       # observer.py:213-217
    torch.qint8: (8, True),
    torch.quint8: (8, False),
    torch.qint32: (32, True),
}


def calc_quant_min_max(bit: int, signed: bool) -> Tuple[int, int]:
    """observer.py:221-224."""
    q_min = -(1 << bit - 1) if signed else 0
    q_max = (1 << bit - 1) - 1 if signed else (1 << bit) - 1
    return q_min, q_max


class QParams(NamedTuple):                  # observer.py:29-34
    qscheme: torch.qscheme
    dtype: torch.dtype
    scale: torch.Tensor
    zero_point: torch.Tensor
    ch_axis: int = -1                       # -1: per tensor


def is_per_channel(qscheme):
    return qscheme in (torch.per_channel_symmetric, torch.per_channel_affine)


def is_symmetric(qscheme):
    return qscheme in (torch.per_tensor_symmetric, torch.per_channel_symmetric)


class Observer:
    """Common state and the qparams arithmetic (observer.py:103-209)."""

    def __init__(self, dtype, qscheme, ch_axis=-1, device="cuda"):
        self.dtype = dtype
        self.qscheme = qscheme
        self.bit, self.signed = DTYPE_TO_BIT_SIGN[dtype]
        if self.symmetric and not self.signed:
            raise ValueError('Symmetric quantization requires signed dtype.')
        self.q_min, self.q_max = calc_quant_min_max(self.bit, self.signed)
        self.device = torch.device(device)
        self.eps = torch.tensor(torch.finfo(torch.float32).eps, device=self.device)
        self.observe = True
        self.fake_quant = True
        self.ch_axis = ch_axis
        self.scale = torch.tensor(1.0, device=self.device)
        self.zero_point = torch.tensor(0, dtype=torch.int32, device=self.device)

    @property
    def symmetric(self):
        return is_symmetric(self.qscheme)

    @property
    def per_channel(self):
        return is_per_channel(self.qscheme)

    @property
    def qparams(self):
        return QParams(qscheme=self.qscheme, dtype=self.dtype, scale=self.scale,
                       zero_point=self.zero_point, ch_axis=self.ch_axis)

    def set_mode(self, *, observe: bool, fake_quant: bool):
        self.observe = observe
        self.fake_quant = fake_quant

    def _calculate_qparams(self, min_val, max_val):
        """observer.py:134-163; min_val / max_val are device tensors."""
        if min_val.numel() == 0 or max_val.numel() == 0:
            return (torch.tensor([1.0], device=self.device),
                    torch.tensor([0], dtype=torch.int32, device=self.device))
        if min_val.dim() == 0 or max_val.dim() == 0:
            if min_val == float("inf") and max_val == float("-inf"):
                return (torch.tensor([1.0], device=self.device),
                        torch.tensor([0], dtype=torch.int32, device=self.device))
            assert min_val <= max_val, "min {} should be less than max {}".format(min_val, max_val)
        else:
            assert torch.all(min_val <= max_val), \
                "min {} should be less than max {}".format(min_val, max_val)
        q_min, q_max = self.q_min, self.q_max
        # The divisors are device tensors: tensor / tensor is an IEEE division on the GPU as
        # on the host, whereas torch's GPU kernels turn "tensor / Python scalar" into a
        # multiplication by the reciprocal, which can differ in the last bit.
        half_range = torch.tensor(float(q_max - q_min) / 2, device=self.device)
        full_range = torch.tensor(float(q_max - q_min), device=self.device)
        min_val_neg = torch.min(min_val, torch.zeros_like(min_val))
        max_val_pos = torch.max(max_val, torch.zeros_like(max_val))
        zero_point = torch.zeros(min_val_neg.size(), dtype=torch.int32, device=self.device)
        if self.symmetric:
            max_val_pos = torch.max(-min_val_neg, max_val_pos)
            scale = max_val_pos / half_range
            scale = torch.max(scale, self.eps)
            if self.dtype == torch.quint8:
                zero_point = zero_point.new_full(zero_point.size(), 128)
        else:
            scale = (max_val_pos - min_val_neg) / full_range
            scale = torch.max(scale, self.eps)
            zero_point = q_min - torch.round(min_val_neg / scale).to(torch.int32)
            zero_point = torch.clamp(zero_point, q_min, q_max)
        return scale, zero_point

    def _fake_quant(self, x, scale, zero_point):
        """quantize -> dequantize with the observer's qparams in one GPU kernel (8-bit
        types); the int32 bias grid is evaluated with the same formula in torch."""
        scale = scale.reshape(-1).float()
        zero_point = zero_point.reshape(-1).to(torch.int32)
        axis = self.ch_axis if self.per_channel else None
        if self.bit == 8:
            return K.fake_quant(x, scale, zero_point, axis=axis, qmin=self.q_min, qmax=self.q_max)
        shape = [1] * x.dim()
        if axis is not None:
            shape[axis] = -1
        s, z = scale.reshape(shape), zero_point.reshape(shape).float()
        q = torch.clamp(torch.round(x / s + z), self.q_min, self.q_max)
        return (q - z) * s


class MinMaxObserver(Observer):
    """Per tensor (observer.py:227-248)."""

    def __init__(self, dtype=torch.qint8, qscheme=torch.per_tensor_symmetric, **kwargs):
        super().__init__(dtype, qscheme, **kwargs)
        self.min_val = torch.tensor(float("inf"), device=self.device)
        self.max_val = torch.tensor(float("-inf"), device=self.device)

    def __call__(self, x):
        if self.observe:
            K.minmax(x.detach().float(), self.min_val.reshape(1), self.max_val.reshape(1))
            self.scale, self.zero_point = self._calculate_qparams(self.min_val, self.max_val)
        if self.fake_quant:
            return self._fake_quant(x, self.scale, self.zero_point)
        return x

    forward = __call__


class PerChannelMinMaxObserver(Observer):
    """Per slice along ``ch_axis`` (observer.py:251-297)."""

    def __init__(self, ch_axis=0, dtype=torch.qint8, qscheme=torch.per_channel_symmetric,
                 **kwargs):
        super().__init__(dtype, qscheme, ch_axis, **kwargs)
        self.min_val = torch.tensor([], device=self.device)
        self.max_val = torch.tensor([], device=self.device)
        self.scale = torch.tensor([], device=self.device)
        self.zero_point = torch.tensor([], dtype=torch.int32, device=self.device)

    def __call__(self, x):
        if self.observe:
            if x.numel() == 0:
                return x
            nch = x.shape[self.ch_axis]
            if self.min_val.numel() == 0 or self.max_val.numel() == 0:
                self.min_val = torch.full((nch,), float("inf"), device=self.device)
                self.max_val = torch.full((nch,), float("-inf"), device=self.device)
            K.minmax(x.detach().float(), self.min_val, self.max_val, axis=self.ch_axis)
            self.scale, self.zero_point = self._calculate_qparams(self.min_val, self.max_val)
        if self.fake_quant:
            return self._fake_quant(x, self.scale, self.zero_point)
        return x

    forward = __call__


class BiasObserver(Observer):
    """The bias is quantized to int32 with scale s_w * s_x (observer.py:300-323)."""

    def __init__(self, w_ob, act_ob, **kwargs):
        if w_ob.per_channel or act_ob.per_channel:
            qscheme = torch.per_channel_symmetric
        else:
            qscheme = torch.per_tensor_symmetric
        super().__init__(torch.qint32, qscheme, w_ob.ch_axis, **kwargs)
        self.w_ob = w_ob
        self.act_ob = act_ob

    def __call__(self, x):
        if self.observe:
            self.scale = self.w_ob.scale * self.act_ob.scale
            if self.per_channel:
                self.zero_point = torch.zeros_like(self.scale, dtype=torch.int32)
        if self.fake_quant:
            return self._fake_quant(x, self.scale, self.zero_point)
        return x

    forward = __call__
