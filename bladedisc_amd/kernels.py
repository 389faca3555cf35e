"""torch-tensor front-end of the raw kernel C ABI (include/disc_q8.h).

PyTorch only supplies device memory and the current stream here; every function
launches the hand-written HIP kernels in libdisc_q8_ral.so.
"""
import ctypes as C

import torch

from . import _lib

EPI_ACC_S32, EPI_REQUANT_CPU, EPI_REQUANT_GPU, EPI_DEQUANT_F32 = 0, 1, 2, 3
# requant, then dequantize with the per-tensor output scale, in one epilogue
EPI_REQUANT_CPU_DEQUANT_F32, EPI_REQUANT_GPU_DEQUANT_F32 = 4, 5
EPI_REQUANT_FIXEDPOINT = 6
BIAS_NONE, BIAS_S32, BIAS_F32, BIAS_S8 = 0, 1, 2, 3
ROUND_HALF_AWAY_FROM_ZERO, ROUND_HALF_TO_EVEN = 0, 1

_BIAS_KIND = {torch.int32: BIAS_S32, torch.float32: BIAS_F32, torch.int8: BIAS_S8}
_OUT_DTYPE = {EPI_ACC_S32: torch.int32, EPI_REQUANT_CPU: torch.int8,
              EPI_REQUANT_GPU: torch.int8, EPI_DEQUANT_F32: torch.float32,
              EPI_REQUANT_CPU_DEQUANT_F32: torch.float32,
              EPI_REQUANT_GPU_DEQUANT_F32: torch.float32,
              EPI_REQUANT_FIXEDPOINT: torch.int8}


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("expected device tensors")


def _scale(t, device):
    if not torch.is_tensor(t):
        t = torch.tensor(t, dtype=torch.float32, device=device)
    return t.reshape(-1).contiguous().float()


def variant_names():
    """Names of the kernel variants a test can force (from the test-hooks library)."""
    L = _lib.hooks()
    return [L.dq8_qgemm_variant_name(i).decode() for i in range(L.dq8_qgemm_num_variants())]


def _view3(shape, axis):
    n = 1
    for s in shape:
        n *= s
    if axis is None:
        return 1, 1, n
    outer = 1
    for s in shape[:axis]:
        outer *= s
    inner = 1
    for s in shape[axis + 1:]:
        inner *= s
    return outer, shape[axis], inner


# quantized element types: name -> (kind of the C ABI, torch dtype that stores the bits)
QUANT_KINDS = {"int8": (0, torch.int8), "uint8": (1, torch.uint8), "int16": (2, torch.int16),
               "uint16": (3, torch.int16), "int32": (4, torch.int32), "uint32": (5, torch.int32)}


def _quant_kind(dtype):
    if isinstance(dtype, str):
        return QUANT_KINDS[dtype]
    name = str(dtype).replace("torch.", "")
    kind, _ = QUANT_KINDS[name]
    return kind, dtype


def quantize(x, scale, zero_point, axis=None, qmin=-128, qmax=127,
             round_mode=ROUND_HALF_TO_EVEN, dtype=torch.int8, out=None):
    """mhlo_disc.quantize on the GPU.  scale/zero_point: device tensors (f32 / i32); x: f32 or
    f16.  dtype: a torch dtype or one of the names in QUANT_KINDS -- the unsigned 16 / 32 bit
    types are returned in the signed torch dtype of the same width (same bits)."""
    _need_cuda(x, scale, zero_point)
    if x.dtype not in (torch.float32, torch.float16):
        raise TypeError("quantize takes f32 or f16 input")
    x = x.contiguous()
    outer, nch, inner = _view3(tuple(x.shape), axis)
    if out is not None and not isinstance(dtype, str):
        dtype = out.dtype
    kind, store = _quant_kind(dtype)
    if out is None:
        out = torch.empty(x.shape, dtype=store, device=x.device)
    n_q = scale.numel() if axis is not None else 1
    st = _lib.lib().dq8_quantize_ex(_ptr(x), 0 if x.dtype == torch.float32 else 1, _ptr(out), kind,
                                    outer, nch, inner, _ptr(scale), _ptr(zero_point), n_q,
                                    int(qmin), int(qmax), round_mode, _stream())
    _lib.check(st, "dq8_quantize")
    return out


def fake_quant(x, scale, zero_point, axis=None, qmin=-128, qmax=127,
               round_mode=ROUND_HALF_TO_EVEN, out=None):
    """dequantize(quantize(x)) in one pass: f32 -> f32, the same bits as the two calls."""
    _need_cuda(x, scale, zero_point)
    if x.dtype != torch.float32:
        raise TypeError("fake_quant takes float32 tensors")
    x = x.contiguous()
    outer, nch, inner = _view3(tuple(x.shape), axis)
    if out is None:
        out = torch.empty_like(x)
    n_q = scale.numel() if axis is not None else 1
    st = _lib.lib().dq8_fake_quant(_ptr(x), _ptr(out), outer, nch, inner, _ptr(scale),
                                   _ptr(zero_point), n_q, qmin, qmax, round_mode, _stream())
    _lib.check(st, "dq8_fake_quant")
    return out


def minmax(x, min_io, max_io, axis=None, workspace=None):
    """Folds the minimum and maximum of `x` (device f32), per tensor (axis None) or per
    slice along `axis`, into the running values min_io / max_io (device f32, one entry or
    one per channel).  Returns (min_io, max_io)."""
    _need_cuda(x, min_io, max_io)
    if x.dtype != torch.float32 or min_io.dtype != torch.float32 or max_io.dtype != torch.float32:
        raise TypeError("minmax takes float32 tensors")
    x = x.contiguous()
    outer, nch, inner = _view3(tuple(x.shape), axis)
    if min_io.numel() != nch or max_io.numel() != nch:
        raise ValueError("min / max state must have one entry per channel (%d)" % nch)
    L = _lib.lib()
    need = L.dq8_minmax_workspace_bytes(outer, nch, inner)
    if workspace is None or workspace.numel() * workspace.element_size() < need:
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=x.device)
    st = L.dq8_minmax(_ptr(x), outer, nch, inner, _ptr(min_io), _ptr(max_io), _ptr(workspace),
                      workspace.numel() * workspace.element_size(), _stream())
    _lib.check(st, "dq8_minmax")
    return min_io, max_io


def lut8(q, table, out=None):
    """out[i] = table[bit pattern of q[i]] for an int8 / uint8 device tensor; `table` is a
    256-entry device tensor of the output's 8-bit type."""
    _need_cuda(q, table)
    if q.element_size() != 1 or table.element_size() != 1 or table.numel() != 256:
        raise TypeError("lut8 takes 8-bit tensors and a 256-entry table")
    q = q.contiguous()
    if out is None:
        out = torch.empty(q.shape, dtype=table.dtype, device=q.device)
    st = _lib.lib().dq8_lut8(_ptr(q), _ptr(out), q.numel(), _ptr(table), _stream())
    _lib.check(st, "dq8_lut8")
    return out


def weight_only_qgemm(x, w, scale, zero_points=None, bias=None, tp_b=True, out=None,
                      workspace=True):
    """out = x @ ((w - zero_points[:, None]) * scale[:, None]).T + bias for f16 / f32
    activations x [M,K] and 8-bit weights (uint8 or int8) w [N,K] (tp_b) or [K,N]; scale and
    bias have x's dtype, zero_points is int32.  workspace=False withholds the scratch that
    [K,N] weights are transposed into and that a launch split over k keeps its partial sums
    in; a uint8 tensor is used as that scratch."""
    _need_cuda(x, w, scale, zero_points, bias)
    if x.dtype not in (torch.float32, torch.float16):
        raise TypeError("weight_only_qgemm takes f32 or f16 activations")
    if w.dtype not in (torch.uint8, torch.int8) or w.dim() != 2:
        raise TypeError("weight_only_qgemm takes a uint8 / int8 weight matrix")
    if x.dim() != 2 or x.stride(1) != 1:
        x = x.reshape(-1, x.shape[-1]).contiguous()
    w = w.contiguous()
    n, k = (w.shape if tp_b else (w.shape[1], w.shape[0]))
    m = x.shape[0]
    if x.shape[1] != k:
        raise ValueError("contraction dimensions differ")
    scale = scale.to(x.dtype).contiguous()
    bias = bias.to(x.dtype).contiguous() if bias is not None else None
    zero_points = zero_points.to(torch.int32).contiguous() if zero_points is not None else None
    if out is None:
        out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    L = _lib.lib()
    if isinstance(workspace, torch.Tensor):
        ws, ws_bytes = workspace, workspace.numel() * workspace.element_size()
    else:
        ws_bytes = L.dq8_weight_only_qgemm_workspace_bytes_ex(
            m, n, k, int(tp_b), 0 if x.dtype == torch.float32 else 1) if workspace else 0
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    st = L.dq8_weight_only_qgemm(_ptr(x), 0 if x.dtype == torch.float32 else 1, x.stride(0),
                                 _ptr(w), int(w.dtype == torch.int8), w.stride(0), int(tp_b),
                                 _ptr(scale), _ptr(zero_points), _ptr(bias), _ptr(out),
                                 out.stride(0), m, n, k, _ptr(ws), ws_bytes, _stream())
    _lib.check(st, "dq8_weight_only_qgemm")
    return out


def weight_only_undo_compiler_layout(reordered_kn):
    """[K,N] uint8 bytes as the reference's compiler leaves a constant weight-only weight
    (`weight_should_be_reordered = false`) -> the dense [N,K] weight matrix."""
    _need_cuda(reordered_kn)
    if reordered_kn.dtype != torch.uint8 or reordered_kn.dim() != 2:
        raise TypeError("weight_only_undo_compiler_layout takes a uint8 [K,N] tensor")
    r = reordered_kn.contiguous()
    k, n = r.shape
    out = torch.empty((n, k), dtype=torch.uint8, device=r.device)
    st = _lib.lib().dq8_weight_only_undo_compiler_layout(_ptr(r), _ptr(out), k, n, _stream())
    _lib.check(st, "dq8_weight_only_undo_compiler_layout")
    return out


def activation_table(fn, s_in, z_in, s_out, z_out, in_dtype=torch.int8, out_dtype=torch.int8,
                     device="cuda"):
    """The table of  q -> quantize(fn(dequantize(q, s_in, z_in)), s_out, z_out)  for every
    8-bit q, built with the same dequantize / quantize kernels a chain of separate operators
    would run, so that  lut8(q, table)  equals that chain bit for bit.  s_*: one-element
    device f32 tensors, z_*: one-element device i32 tensors; fn: a torch elementwise function.
    Entry i belongs to the input whose bit pattern is i."""
    bits = torch.arange(256, dtype=torch.int16, device=device).to(torch.uint8)
    q = bits.view(in_dtype) if in_dtype != torch.uint8 else bits
    y = fn(dequantize(q, s_in, z_in))
    qmin, qmax = (-128, 127) if out_dtype == torch.int8 else (0, 255)
    return quantize(y, s_out, z_out, qmin=qmin, qmax=qmax, dtype=out_dtype)


def dequantize(q, scale, zero_point, axis=None, out=None, dtype=None):
    """mhlo_disc.dequantize on the GPU; dtype names the quantized type where q's torch dtype
    does not (the unsigned 16 / 32 bit types, see QUANT_KINDS)."""
    _need_cuda(q, scale, zero_point)
    q = q.contiguous()
    outer, nch, inner = _view3(tuple(q.shape), axis)
    if out is None:
        out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    kind, _ = _quant_kind(dtype if dtype is not None else q.dtype)
    n_q = scale.numel() if axis is not None else 1
    st = _lib.lib().dq8_dequantize_ex(_ptr(q), kind, _ptr(out), outer, nch, inner, _ptr(scale),
                                      _ptr(zero_point), n_q, _stream())
    _lib.check(st, "dq8_dequantize")
    return out


def make_postops(residual=None, residual_scale=None, residual_zp=0, relu=False, out_scale=None,
                 out_zp=0, table=None):
    """dq8_postops_t for the operators fused behind a quantized GEMM / convolution; returns
    (struct, objects to keep alive).  residual: f32 or int8 device tensor of the output's
    shape (int8: with residual_scale, a one-element device tensor, and residual_zp);
    out_scale: one-element device tensor of the quantize that follows (int8 results);
    table: 256-entry int8 / uint8 device tensor."""
    po = _lib.PostOps()
    keep = []
    if residual is not None:
        if residual.stride(-1) != 1:
            residual = residual.contiguous()
        r2 = residual.reshape(-1, residual.shape[-1]) if residual.is_contiguous() else residual
        po.residual = r2.data_ptr()
        po.residual_kind = 1 if residual.dtype == torch.float32 else 2
        po.ldr = r2.stride(0)
        keep.append(r2)
        if residual_scale is not None:
            po.residual_scale = residual_scale.data_ptr()
            keep.append(residual_scale)
        po.residual_zp = int(residual_zp)
    po.relu = int(bool(relu))
    if out_scale is not None:
        po.out_scale = out_scale.data_ptr()
        keep.append(out_scale)
    po.out_zp = int(out_zp)
    if table is not None:
        po.table = table.data_ptr()
        keep.append(table)
    return po, keep


def qgemm(a, w, epilogue, sx=None, sw=None, so=None, bias=None, tp_a=False, tp_b=True,
          zx=0, zw=0, zo=0, variant=-1, out=None, post=None):
    """int8 GEMM with a fused epilogue.  a: [M,K] ([K,M] if tp_a); w: [N,K] if tp_b
    else [K,N]; scales are device f32 tensors with 1 or N entries."""
    _need_cuda(a, w, bias)
    L = _lib.lib()
    # rows may be strided (leading dimension > row length); elements must be dense
    if a.dim() != 2 or a.stride(1) != 1:
        a = a.contiguous()
    if w.dim() != 2 or w.stride(1) != 1:
        w = w.contiguous()
    m, k = (a.shape[1], a.shape[0]) if tp_a else a.shape
    n = w.shape[0] if tp_b else w.shape[1]
    kw = w.shape[1] if tp_b else w.shape[0]
    if k != kw:
        raise ValueError("mismatch contraction dim")
    dev = a.device
    if out is None:
        out = torch.empty((m, n), dtype=_OUT_DTYPE[epilogue], device=dev)
    sx = _scale(sx, dev) if sx is not None else None
    sw = _scale(sw, dev) if sw is not None else None
    so = _scale(so, dev) if so is not None else None
    bias_kind = BIAS_NONE if bias is None else _BIAS_KIND[bias.dtype]
    # with zero points and the heuristic this includes the two correction vectors of the
    # MFMA path; a forced generic variant (0) needs none of it
    ws_bytes = (L.dq8_qgemm_workspace_bytes_zp(m, n, k, int(tp_a), int(tp_b), zx, zw)
                if variant == -1 else L.dq8_qgemm_workspace_bytes(m, n, k, int(tp_a), int(tp_b)))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    args = (_ptr(a), max(a.stride(0), a.shape[1]), _ptr(w), max(w.stride(0), w.shape[1]),
            _ptr(out), out.stride(0) if m else n,
            m, n, k, int(tp_a), int(tp_b), epilogue, _ptr(bias), bias_kind,
            _ptr(sx), sx.numel() if sx is not None else 0,
            _ptr(sw), sw.numel() if sw is not None else 0,
            _ptr(so), so.numel() if so is not None else 0,
            zx, zw, zo, _ptr(ws), ws_bytes)
    if post is not None:
        if variant != -1:
            raise ValueError("fused operators go with the library's own choice of kernel")
        po, keep = post if isinstance(post, tuple) else (post, None)
        st = L.dq8_qgemm_fused(*args, C.byref(po), _stream())
    elif variant == -1:
        st = L.dq8_qgemm(*args, _stream())
    else:       # a forced kernel variant: the tests' entry point, in the test-hooks library
        L = _lib.hooks()
        st = L.dq8_qgemm_variant(variant, *args, _stream())
    _lib.check(st, "dq8_qgemm", L)
    return out


def qlinear_f32_fused_max_rows(n, k):
    return int(_lib.lib().dq8_qlinear_f32_fused_max_rows(n, k))


def qlinear_f32(x, w, epilogue, sx, sw=None, so=None, bias=None, zo=0,
                round_mode=ROUND_HALF_TO_EVEN, out=None):
    """quantize(x; sx, zero point 0) -> qgemm(., w [N,K]) with the given epilogue, one launch,
    for a few rows of f32 activations x [M,K]; the same bits as quantize followed by qgemm."""
    _need_cuda(x, w, bias)
    L = _lib.lib()
    if x.dim() != 2 or x.stride(1) != 1:
        x = x.reshape(-1, x.shape[-1]).contiguous()
    if w.dim() != 2 or w.stride(1) != 1:
        w = w.contiguous()
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k:
        raise ValueError("mismatch contraction dim")
    dev = x.device
    if out is None:
        out = torch.empty((m, n), dtype=_OUT_DTYPE[epilogue], device=dev)
    sx = _scale(sx, dev)
    sw = _scale(sw, dev) if sw is not None else None
    so = _scale(so, dev) if so is not None else None
    bias_kind = BIAS_NONE if bias is None else _BIAS_KIND[bias.dtype]
    st = L.dq8_qlinear_f32(_ptr(x), max(x.stride(0), k), _ptr(w), max(w.stride(0), k), _ptr(out),
                           out.stride(0) if m else n, m, n, k, epilogue, _ptr(bias), bias_kind,
                           _ptr(sx), _ptr(sw), sw.numel() if sw is not None else 0,
                           _ptr(so), so.numel() if so is not None else 0, zo, round_mode, _stream())
    _lib.check(st, "dq8_qlinear_f32")
    return out


NHWC_OHWI = (0, 3, 1, 2, 3, 0, 1, 2, 0, 3, 1, 2)


def qconv2d(x, w, padding, metadata, out_shape, epilogue, sx=None, sw=None, so=None,
            bias=None, zo=0, variant=-1, out=None, workspace=True, post=None):
    """int8 convolution; layouts/strides/dilations from the 17-entry ral_qconv
    metadata, padding = (top, bottom, left, right).  workspace=False withholds the scratch
    that keeps channel counts off a multiple of 16 on the MFMA kernels."""
    _need_cuda(x, w, bias)
    L = _lib.lib()
    x = x.contiguous()
    w = w.contiguous()
    dev = x.device
    if out is None:
        out = torch.empty(tuple(out_shape), dtype=_OUT_DTYPE[epilogue], device=dev)
    sx = _scale(sx, dev) if sx is not None else None
    sw = _scale(sw, dev) if sw is not None else None
    so = _scale(so, dev) if so is not None else None
    bias_kind = BIAS_NONE if bias is None else _BIAS_KIND[bias.dtype]
    i64x4 = C.c_int64 * 4
    md = (C.c_int32 * 17)(*metadata)
    ws_bytes = L.dq8_qconv2d_workspace_bytes_ex(i64x4(*x.shape), i64x4(*w.shape), i64x4(*out_shape), md) if workspace else 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    args = (_ptr(x), i64x4(*x.shape), _ptr(w), i64x4(*w.shape),
            (C.c_int32 * 4)(*padding), md, _ptr(out),
            i64x4(*out_shape), epilogue, _ptr(bias), bias_kind, _ptr(sx), _ptr(sw),
            sw.numel() if sw is not None else 0, _ptr(so), zo, _ptr(ws), ws_bytes)
    if post is not None:
        if variant != -1:
            raise ValueError("fused operators go with the library's own choice of kernel")
        po, keep = post if isinstance(post, tuple) else (post, None)
        st = L.dq8_qconv2d_fused(*args, C.byref(po), _stream())
    elif variant == -1:
        st = L.dq8_qconv2d_ws(*args, _stream())
    else:       # a forced kernel variant: the tests' entry point, in the test-hooks library
        L = _lib.hooks()
        st = L.dq8_qconv2d_variant(variant, *args, _stream())
    _lib.check(st, "dq8_qconv2d", L)
    return out


def mfma_probe(a32, b32, a16, b16):
    d32 = torch.empty((32, 32), dtype=torch.int32, device=a32.device)
    d16 = torch.empty((16, 16), dtype=torch.int32, device=a32.device)
    st = _lib.hooks().dq8_mfma_probe(_ptr(a32), _ptr(b32), _ptr(d32), _ptr(a16), _ptr(b16),
                                     _ptr(d16), _stream())
    _lib.check(st, "dq8_mfma_probe", _lib.hooks())
    return d32, d16
