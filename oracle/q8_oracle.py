"""numpy front-end of ``libq8_oracle.so`` (the C restatement in q8_oracle.c).

TEST INFRASTRUCTURE ONLY -- the checker for the HIP kernels and the timed CPU
baseline.  See q8_oracle.h for the reference file:line each function follows.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libq8_oracle.so")

ROUND_HALF_AWAY_FROM_ZERO = 0
ROUND_HALF_TO_EVEN = 1

_KINDS = {
    np.dtype(np.int8): 0,
    np.dtype(np.uint8): 1,
    np.dtype(np.int16): 2,
    np.dtype(np.uint16): 3,
    np.dtype(np.int32): 4,
    np.dtype(np.uint32): 5,
}


def build(force=False):
    """Compile the oracle with the committed Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s",
                               "libq8_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.q8o_gemm_s32_fast.restype = C.c_int
        for name in ("q8o_conv_reorder_dims", "q8o_conv_expand",
                     "q8o_conv_padding", "q8o_conv_explicit_padding",
                     "q8o_conv_metadata"):
            getattr(_lib, name).restype = C.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def _i64(v):
    return C.c_int64(int(v))


def _i64arr(v):
    return (C.c_int64 * len(v))(*[int(x) for x in v])


def _i32arr(v):
    return (C.c_int32 * len(v))(*[int(x) for x in v])


def gemm_s32(a, w, tp_a=False, tp_b=False, zx=0, zw=0):
    """acc = (A - zx) @ (W - zw) in int32.  a: [M,K] ([K,M] if tp_a); w: [K,N]
    ([N,K] if tp_b)."""
    a = _c(a, np.int8)
    w = _c(w, np.int8)
    m, k = (a.shape[1], a.shape[0]) if tp_a else a.shape
    n = w.shape[0] if tp_b else w.shape[1]
    kw = w.shape[1] if tp_b else w.shape[0]
    if k != kw:
        raise ValueError("mismatch contraction dim")
    acc = np.empty((m, n), np.int32)
    lib().q8o_gemm_s32(_p(a), _p(w), _p(acc), _i64(m), _i64(n), _i64(k),
                       C.c_int(int(tp_a)), C.c_int(int(tp_b)),
                       C.c_int32(zx), C.c_int32(zw))
    return acc


def gemm_s32_fast(a, w_nk):
    """Same as gemm_s32(a, w_nk, tp_b=True), multi-threaded.  Returns (acc, threads)."""
    a = _c(a, np.int8)
    w_nk = _c(w_nk, np.int8)
    m, k = a.shape
    n, k2 = w_nk.shape
    if k != k2:
        raise ValueError("mismatch contraction dim")
    acc = np.empty((m, n), np.int32)
    t = lib().q8o_gemm_s32_fast(_p(a), _p(w_nk), _p(acc), _i64(m), _i64(n),
                                _i64(k))
    return acc, t


def bias_f32_to_s32(bias, sx, sw):
    bias = _c(bias, np.float32)
    sw = _c(np.atleast_1d(sw), np.float32)
    out = np.empty(bias.shape, np.int32)
    lib().q8o_bias_f32_to_s32(_p(bias), C.c_float(sx), _p(sw), _i64(sw.size),
                              _p(out), _i64(bias.size))
    return out


def requant_cpu(acc, sx, sw, so, b32=None, zo=0):
    """E1: sat8(rne((f32(acc)+f32(b32)) * ((sx*sw)/so) + zo))."""
    acc = _c(acc, np.int32)
    m, n = acc.shape
    sw = _c(np.atleast_1d(sw), np.float32)
    b = _c(b32, np.int32) if b32 is not None else None
    out = np.empty((m, n), np.int8)
    lib().q8o_requant_cpu(_p(acc), _i64(m), _i64(n), _p(b), C.c_float(sx),
                          _p(sw), _i64(sw.size), C.c_float(so), C.c_int32(zo),
                          _p(out))
    return out


def requant_gpu(acc, sx, sw, so, bias_f32=None, bias_i8=None):
    """E2: sat8(rne((sx*sw/so) * f32(acc) + bias))."""
    acc = _c(acc, np.int32)
    m, n = acc.shape
    sx = _c(np.atleast_1d(sx), np.float32)
    sw = _c(np.atleast_1d(sw), np.float32)
    so = _c(np.atleast_1d(so), np.float32)
    for v in (sx, sw, so):
        if v.size not in (1, n):
            raise ValueError("E2 scales must have 1 or N entries")
    bf = _c(bias_f32, np.float32) if bias_f32 is not None else None
    bi = _c(bias_i8, np.int8) if bias_i8 is not None else None
    out = np.empty((m, n), np.int8)
    lib().q8o_requant_gpu(_p(acc), _i64(m), _i64(n), _p(bf), _p(bi), _p(sx),
                          _i64(sx.size), _p(sw), _i64(sw.size), _p(so),
                          _i64(so.size), _p(out))
    return out


def requant_fixedpoint(acc, sx, sw, so, b32=None, zo=0):
    """The AArch64 path's output stage: (acc + b32[n]) times a fixed-point multiplier and
    shift derived from (sx * sw[n]) / so, plus zo, clamped to int8."""
    acc = _c(acc, np.int32)
    m, n = acc.shape
    sw = _c(np.atleast_1d(sw), np.float32)
    if sw.size not in (1, n):
        raise ValueError("weight scales must have 1 or N entries")
    b = _c(b32, np.int32) if b32 is not None else None
    out = np.empty((m, n), np.int8)
    lib().q8o_requant_fixedpoint(_p(acc), _i64(m), _i64(n), _p(b), C.c_float(sx), _p(sw),
                                 _i64(sw.size), C.c_float(so), C.c_int32(int(zo)), _p(out))
    return out


def fixedpoint_multiplier(multiplier):
    """(M0, shift) of a binary32 multiplier."""
    m0, sh = C.c_int32(), C.c_int32()
    lib().q8o_fixedpoint_multiplier(C.c_float(multiplier), C.byref(m0), C.byref(sh))
    return m0.value, sh.value


def sqrdmulh(a, b):
    f = lib().q8o_sqrdmulh
    f.restype = C.c_int32
    return f(C.c_int32(int(a)), C.c_int32(int(b)))


def rounding_divide_by_pow2(x, exponent):
    f = lib().q8o_rounding_divide_by_pow2
    f.restype = C.c_int32
    return f(C.c_int32(int(x)), C.c_int(int(exponent)))


def finalize_fixedpoint(v, m0, shift, zo=0):
    f = lib().q8o_finalize_fixedpoint
    f.restype = C.c_int8
    return f(C.c_int32(int(v)), C.c_int32(int(m0)), C.c_int32(int(shift)), C.c_int32(int(zo)))


def dequant_acc(acc, sx, sw, bias=None):
    """E3: f32(acc) * (sx*sw[n]) + bias[n]."""
    acc = _c(acc, np.int32)
    m, n = acc.shape
    sw = _c(np.atleast_1d(sw), np.float32)
    b = _c(bias, np.float32) if bias is not None else None
    out = np.empty((m, n), np.float32)
    lib().q8o_dequant_acc(_p(acc), _i64(m), _i64(n), C.c_float(sx), _p(sw),
                          _i64(sw.size), _p(b), _p(out))
    return out


def weight_only_qgemm(x, w_nk, scale, zero_points=None, bias=None):
    """(out, bound) for the weight-only quantized linear the reference's pattern rewrites into
    `ral_pdll_weight_only_qgemm` (pytorch_blade/tests/disc/pdl/pdll_files/gpu/
    weight_only_qgemm.pdll:2-104): matmul(x, dequantize(w)^T) + bias with
    dequantize(w)[n, k] = (w[n, k] - zero_points[n]) * scale[n]
    (torch.fake_quantize_per_channel_affine's dequantized weight, the model of
    pytorch_blade/tests/disc/pdl/test_torchscipt_to_mhlo/test_quantization.py:501-523).
    PARITY UNPINNED beyond this definition: the reference tree holds no runtime implementation
    and no expected values for it.  Computed in float64; `bound[m, n]` = sum_k |x| |w_deq|,
    the quantity accumulation-error tolerances are stated against."""
    x64 = np.asarray(x, np.float64)
    zp = np.zeros(w_nk.shape[0], np.int64) if zero_points is None else np.asarray(zero_points, np.int64)
    wd = (w_nk.astype(np.int64) - zp[:, None]).astype(np.float64) * np.asarray(scale, np.float64)[:, None]
    out = x64 @ wd.T
    if bias is not None:
        out = out + np.asarray(bias, np.float64)[None, :]
    return out, np.abs(x64) @ np.abs(wd).T


def _view3(shape, axis):
    if axis is None:
        return 1, 1, int(np.prod(shape, dtype=np.int64))
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return outer, int(shape[axis]), inner


def quantize(x, scale, zp, axis=None, qmin=-128, qmax=127,
             round_mode=ROUND_HALF_TO_EVEN, dtype=np.int8, fold=False):
    """mhlo_disc.quantize.  axis=None is per-tensor.  fold=True uses the
    compile-time folder's double arithmetic instead of the runtime f32 one."""
    x = _c(x, np.float32)
    scale = _c(np.atleast_1d(scale), np.float32)
    zp = _c(np.atleast_1d(zp), np.int32)
    outer, nch, inner = _view3(x.shape, axis)
    if scale.size != zp.size or scale.size not in (1, nch):
        raise ValueError("scale/zero_point shape")
    out = np.empty(x.shape, dtype)
    fn = lib().q8o_quantize_fold if fold else lib().q8o_quantize_f32
    fn(_p(x), _i64(outer), _i64(nch), _i64(inner), _p(scale), _p(zp),
       _i64(scale.size if axis is not None else 1), _i64(qmin), _i64(qmax),
       C.c_int(round_mode), C.c_int(_KINDS[np.dtype(dtype)]), _p(out))
    return out


def dequantize(q, scale, zp, axis=None):
    q = np.ascontiguousarray(q)
    scale = _c(np.atleast_1d(scale), np.float32)
    zp = _c(np.atleast_1d(zp), np.int32)
    outer, nch, inner = _view3(q.shape, axis)
    out = np.empty(q.shape, np.float32)
    lib().q8o_dequantize(_p(q), C.c_int(_KINDS[q.dtype]), _i64(outer),
                         _i64(nch), _i64(inner), _p(scale), _p(zp),
                         _i64(scale.size if axis is not None else 1), _p(out))
    return out


NHWC_OHWI_METADATA = (0, 3, 1, 2, 3, 0, 1, 2, 0, 3, 1, 2)


def conv_s32(x, w, padding, metadata, out_shape, zx=0, zw=0):
    """int32 conv accumulators; layouts described by the 17-entry metadata."""
    x = _c(x, np.int8)
    w = _c(w, np.int8)
    acc = np.empty(tuple(out_shape), np.int32)
    lib().q8o_conv_s32(_p(x), _i64arr(x.shape), _p(w), _i64arr(w.shape),
                       _i32arr(padding), _i32arr(metadata), _p(acc),
                       _i64arr(out_shape), C.c_int32(zx), C.c_int32(zw))
    return acc


def conv_attrs(in_shape, w_shape, data_format, strides, dilations, padding,
               explicit_paddings=(), weight_is_const=True):
    """TF-style attrs -> (padding[4], metadata[17], out_shape[4]) as
    common_context_impl_quantization.h:27-206 derives them."""
    L = lib()
    reorder = (C.c_int32 * 4)()
    if not L.q8o_conv_reorder_dims(data_format.encode(), reorder):
        raise ValueError("bad data_format")
    st = (C.c_int32 * 2)()
    dl = (C.c_int32 * 2)()
    if not L.q8o_conv_expand(reorder, _i64arr(strides), _i64(len(strides)), st):
        raise ValueError("bad strides")
    if not L.q8o_conv_expand(reorder, _i64arr(dilations), _i64(len(dilations)),
                             dl):
        raise ValueError("bad dilations")
    pad = (C.c_int32 * 4)()
    if padding == "EXPLICIT":
        ok = L.q8o_conv_explicit_padding(reorder, _i64arr(explicit_paddings),
                                         _i64(len(explicit_paddings)), pad)
    else:
        ok = L.q8o_conv_padding(_i64arr(in_shape), _i64arr(w_shape),
                                padding.encode(), reorder, st, dl, pad)
    if not ok:
        raise ValueError("bad padding")
    md = (C.c_int32 * 17)()
    if not L.q8o_conv_metadata(st, dl, reorder, C.c_int(int(weight_is_const)),
                               md):
        raise ValueError("metadata")
    out = (C.c_int64 * 4)()
    L.q8o_conv_result_shape(_i64arr(in_shape), _i64arr(w_shape), reorder, pad,
                            st, dl, out)
    return list(pad), list(md), list(out)
