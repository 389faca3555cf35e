"""Typed callers of the quantized RAL entries: each packs torch tensors the way the
compiled program would and goes through ``tao_ral_call_impl`` by mangled name.

Operand order of every call is the reference's (disc/transforms/
disc_lower_to_library_call.cc:196-267 for ral_qgemm, :391-421 for ral_qconv, the
PDLL rewrite patterns for ral_pdll_qgemm).
"""
import numpy as np
import torch

from . import ral


def _zp0(a, host):
    """A rank-0 zero point: host int32 (ral_pdll_*) or device int32."""
    if host:
        return a.host_array(np.zeros(1, np.int32), rank0=True)
    z = torch.zeros(1, dtype=torch.int32, device="cuda")
    a._keep.append(z)
    return a.tensor(z, rank0=True)


def qgemm(ex, x, w, sx, sw, so, out=None, tp_a=False, tp_b=True, weight_is_const=False,
          per_channel=None):
    """ral_qgemm: x [M,K] i8, w [N,K] (tp_b) or [K,N]; sx/so one-element device f32
    tensors, sw one-element (per tensor, rank 0) or [N] (per channel, rank 1)."""
    m = x.shape[1] if tp_a else x.shape[0]
    n = w.shape[0] if tp_b else w.shape[1]
    if out is None:
        out = torch.empty((m, n), dtype=torch.int8, device=x.device)
    if per_channel is None:
        per_channel = sw.numel() > 1
    a = ex.new_args().tensor(x).tensor(w)
    a.tensor(sx, rank0=True)
    _zp0(a, host=False)
    if per_channel:
        a.tensor(sw)
        z = torch.zeros(sw.numel(), dtype=torch.int32, device=x.device)
        a._keep.append(z)
        a.tensor(z)
    else:
        a.tensor(sw, rank0=True)
        _zp0(a, host=False)
    a.tensor(so, rank0=True)
    _zp0(a, host=False)
    a.tensor(out)
    a.scalar("i1", tp_a).scalar("i1", tp_b).scalar("i1", weight_is_const)
    ex.call("ral_qgemm", "gpu", a)
    return out


def pdll_qgemm_gpu(ex, x, w_nk, bias, sx, sw, so):
    """ral_pdll_qgemm, gpu signature: rank-2/3 input, weight [N,K], bias int8 or f32
    in output-quantised units, rank-0 device scales, rank-0 host zero points.
    Returns the callee-allocated result as a tensor view."""
    a = ex.new_args().tensor(x).tensor(w_nk).tensor(bias)
    for s in (sx, sw, so):
        a.tensor(s, rank0=True)
        _zp0(a, host=True)
    a.blob(ral.encode_attr({}))
    res = a.result_memref("i8", x.dim())
    ex.call("ral_pdll_qgemm", "gpu", a)
    return ral.memref_to_tensor(res, torch.int8)


def pdll_qgemm_per_channel(ex, x, w_nk, bias_i8, sx_n, sw_n, so_n):
    """ral_pdll_qgemm_per_channel (merged-QKV form): all scales are [N] vectors."""
    n = w_nk.shape[0]
    a = ex.new_args().tensor(x).tensor(w_nk).tensor(bias_i8)
    for s in (sx_n, sw_n, so_n):
        a.tensor(s)
        a.host_array(np.zeros(n, np.int32))
    a.blob(ral.encode_attr({}))
    res = a.result_memref("i8", x.dim())
    ex.call("ral_pdll_qgemm_per_channel", "gpu", a)
    return ral.memref_to_tensor(res, torch.int8)


def pdll_qgemm_cpu_style(ex, x, w, bias, sx, sw_n, so, zo=0, transpose_b=False,
                         weight_is_const=True, zx=0, zw=0):
    """ral_pdll_qgemm with the CPU patterns' signature on the gpu device: weight
    [K,N] unless transpose_b, bias f32 / s32 / None, per-channel weight scale; zx: input
    zero point, zw: weight zero point(s), a value or one per channel (host values)."""
    n = w.shape[0] if transpose_b else w.shape[1]
    a = ex.new_args().tensor(x).tensor(w)
    if bias is not None:
        a.tensor(bias)
    a.tensor(sx, rank0=True)
    a.host_array(np.array([zx], np.int32), rank0=True)
    a.tensor(sw_n)
    a.host_array(np.broadcast_to(np.asarray(zw, np.int32), (sw_n.numel(),)).copy())
    a.tensor(so, rank0=True)
    a.host_array(np.array([zo], np.int32), rank0=True)
    a.blob(ral.encode_attr({"transpose_a": False, "transpose_b": bool(transpose_b),
                            "weight_is_const": bool(weight_is_const),
                            "bias_is_const": True}))
    res = a.result_memref("i8", x.dim())
    ex.call("ral_pdll_qgemm", "gpu", a)
    assert n == res.sizes[x.dim() - 1]
    return ral.memref_to_tensor(res, torch.int8)


def _cpu_style_operands(ex, x, w, bias, sx, sw_n, so, zo):
    a = ex.new_args().tensor(x).tensor(w).tensor(bias)
    a.tensor(sx, rank0=True)
    a.host_array(np.array([0], np.int32), rank0=True)
    a.tensor(sw_n)
    a.host_array(np.zeros(sw_n.numel(), np.int32))
    a.tensor(so, rank0=True)
    a.host_array(np.array([zo], np.int32), rank0=True)
    return a


def pdll_qgemm_fused(ex, x, w, bias, sx, sw_n, so, zo=0, transpose_b=False, weight_is_const=True,
                     residual=None, relu=False, table=None):
    """ral_pdll_qgemm_fused: the CPU-style ral_pdll_qgemm (f32 bias) with the operators that
    follow it taken into the call -- dequantize (f32 result), dequantize + f32 residual
    [+ relu], or a 256-entry table on the int8 result (int8 result)."""
    a = _cpu_style_operands(ex, x, w, bias, sx, sw_n, so, zo)
    if residual is not None:
        a.tensor(residual)
    elif table is not None:
        a.tensor(table.view(torch.uint8))
    a.blob(ral.encode_attr({"transpose_a": False, "transpose_b": bool(transpose_b),
                            "weight_is_const": bool(weight_is_const), "bias_is_const": True,
                            "relu": bool(relu)}))
    int8_out = table is not None
    res = a.result_memref("i8" if int8_out else "f32", x.dim())
    ex.call("ral_pdll_qgemm_fused", "gpu", a)
    return ral.memref_to_tensor(res, torch.int8 if int8_out else torch.float32)


def pdll_qlinear(ex, x_f32, w, bias, sx, sw_n, so, zo=0, transpose_b=False, weight_is_const=True,
                 round_mode=1):
    """ral_pdll_qlinear: quantize -> ral_pdll_qgemm -> dequantize of f32 activations as one
    call; f32 result."""
    a = _cpu_style_operands(ex, x_f32, w, bias, sx, sw_n, so, zo)
    a.blob(ral.encode_attr({"transpose_a": False, "transpose_b": bool(transpose_b),
                            "weight_is_const": bool(weight_is_const), "bias_is_const": True,
                            "round_mode": int(round_mode)}))
    res = a.result_memref("f32", x_f32.dim())
    ex.call("ral_pdll_qlinear", "gpu", a)
    return ral.memref_to_tensor(res, torch.float32)


def pdll_qgemm_per_tensor(ex, x, w, bias_s32, sx, sw, so, zo=0, transpose_b=False,
                          weight_is_const=True):
    """ral_pdll_qgemm with the AArch64 patterns' per-tensor signature on the gpu device
    (fixed-point output stage): weight [K,N] unless transpose_b, bias s32 or None, rank-0
    device scales, rank-0 host zero points."""
    n = w.shape[0] if transpose_b else w.shape[1]
    a = ex.new_args().tensor(x).tensor(w)
    if bias_s32 is not None:
        a.tensor(bias_s32)
    a.tensor(sx, rank0=True)
    _zp0(a, host=True)
    a.tensor(sw, rank0=True)
    _zp0(a, host=True)
    a.tensor(so, rank0=True)
    a.host_array(np.array([zo], np.int32), rank0=True)
    a.blob(ral.encode_attr({"transpose_a": False, "transpose_b": bool(transpose_b),
                            "weight_is_const": bool(weight_is_const),
                            "bias_is_const": True}))
    res = a.result_memref("i8", x.dim())
    ex.call("ral_pdll_qgemm", "gpu", a)
    assert n == res.sizes[x.dim() - 1]
    return ral.memref_to_tensor(res, torch.int8)


def pdll_weight_only_qgemm(ex, x, w_kn, scale, zero_points, bias=None, reorder=True):
    """ral_pdll_weight_only_qgemm: f32 / f16 activations [..., K], uint8 weight [K,N], optional
    bias [N], per-channel scale [N] (activation dtype) and zero point [N] (int32), all on the
    device; `reorder` is the pattern's `weight_should_be_reordered` attribute."""
    code = {torch.float32: "f32", torch.float16: "f16"}[x.dtype]
    a = ex.new_args().tensor(x).tensor(w_kn)
    if bias is not None:
        a.tensor(bias)
    a.tensor(scale).tensor(zero_points)
    a.blob(ral.encode_attr({"weight_should_be_reordered": bool(reorder)}))
    res = a.result_memref(code, x.dim())
    ex.call("ral_pdll_weight_only_qgemm", "gpu", a)
    assert w_kn.shape[1] == res.sizes[x.dim() - 1]
    return ral.memref_to_tensor(res, x.dtype)


def qconv(ex, x, w, padding, metadata, sx, sw_c, so, out):
    """ral_qconv: padding [4] and metadata [17] are host int32 memrefs."""
    a = ex.new_args().tensor(x).tensor(w)
    a.host_array(np.asarray(padding, np.int32))
    a.tensor(sx, rank0=True)
    _zp0(a, host=False)
    a.tensor(sw_c)
    z = torch.zeros(sw_c.numel(), dtype=torch.int32, device=x.device)
    a._keep.append(z)
    a.tensor(z)
    a.tensor(so, rank0=True)
    _zp0(a, host=False)
    a.tensor(out)
    a.host_array(np.asarray(metadata, np.int32))
    ex.call("ral_qconv", "gpu", a)
    return out


def qconv_s8_s8_s8(ex, x, w, padding, metadata, sx, sw_c, so, out):
    """ral_qconv_s8_s8_s8: the older symmetric entry, ral_qconv without zero-point operands."""
    a = ex.new_args().tensor(x).tensor(w)
    a.host_array(np.asarray(padding, np.int32))
    a.tensor(sx, rank0=True)
    a.tensor(sw_c)
    a.tensor(so, rank0=True)
    a.tensor(out)
    a.host_array(np.asarray(metadata, np.int32))
    ex.call("ral_qconv_s8_s8_s8", "gpu", a)
    return out


def pdll_qconv2d(ex, x, w_ohwi, sx, sw_c, so, data_format="NHWC", strides=(1, 1, 1, 1),
                 dilations=(1, 1, 1, 1), padding="SAME", explicit_paddings=(),
                 weight_is_const=True, zo=0):
    """ral_pdll_qconv2d: TensorFlow-style attributes, callee-allocated result."""
    a = ex.new_args().tensor(x).tensor(w_ohwi)
    a.tensor(sx, rank0=True)
    _zp0(a, host=True)
    a.tensor(sw_c)
    a.host_array(np.zeros(sw_c.numel(), np.int32))
    a.tensor(so, rank0=True)
    a.host_array(np.array([zo], np.int32), rank0=True)
    a.blob(ral.encode_attr({"data_format": data_format, "strides": [int(v) for v in strides],
                            "dilations": [int(v) for v in dilations], "padding": padding,
                            "explicit_paddings": [int(v) for v in explicit_paddings],
                            "weight_is_const": bool(weight_is_const)}))
    res = a.result_memref("i8", 4)
    ex.call("ral_pdll_qconv2d", "gpu", a)
    return ral.memref_to_tensor(res, torch.int8)


def conv2d_plan(in_shape, w_shape, data_format, strides, dilations, padding,
                explicit_paddings=(), weight_is_const=True):
    """(padding[4], metadata[17], result_shape[4]) as ral_pdll_qconv2d derives them;
    raises ValueError for malformed attributes.  Host only."""
    import ctypes as C
    L = ral.lib()
    i64 = lambda v: (C.c_int64 * max(len(v), 1))(*[int(t) for t in v])  # noqa: E731
    pad, md, out = (C.c_int32 * 4)(), (C.c_int32 * 17)(), (C.c_int64 * 4)()
    L.disc_ral_conv2d_plan.restype = C.c_int
    rc = L.disc_ral_conv2d_plan(data_format.encode(), i64(strides), len(strides),
                                i64(dilations), len(dilations), padding.encode(),
                                i64(explicit_paddings), len(explicit_paddings),
                                int(weight_is_const), i64(in_shape), i64(w_shape), pad, md, out)
    if rc != 0:
        raise ValueError("malformed convolution attributes")
    return list(pad), list(md), list(out)


def quantize(ex, x, scale, zp, axis=None, qmin=-128, qmax=127, round_mode=1, out=None,
             dtype=torch.int8, code=None):
    """ral_quantize; `code` names the result's element type in the mangled symbol where the
    torch dtype that stores the bits does not ("ui16" / "ui32" in int16 / int32 storage)."""
    if out is None:
        out = torch.empty(x.shape, dtype=dtype, device=x.device)
    a = ex.new_args().tensor(x)
    a.tensor(scale, rank0=axis is None).tensor(zp, rank0=axis is None)
    if code is None:
        a.tensor(out)
    else:
        a.memref(code, out.data_ptr(), list(out.shape), list(out.stride()))
    a.scalar("i64", -1 if axis is None else axis).scalar("i64", qmin).scalar("i64", qmax)
    a.scalar("i64", round_mode)
    ex.call("ral_quantize", "gpu", a)
    return out


def dequantize(ex, q, scale, zp, axis=None, out=None, code=None):
    if out is None:
        out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    a = ex.new_args()
    if code is None:
        a.tensor(q)
    else:
        a.memref(code, q.data_ptr(), list(q.shape), list(q.stride()))
    a.tensor(scale, rank0=axis is None).tensor(zp, rank0=axis is None)
    a.tensor(out)
    a.scalar("i64", -1 if axis is None else axis)
    ex.call("ral_dequantize", "gpu", a)
    return out
