"""Loads libdisc_q8_ral.so (the HIP kernels + RAL runtime) through ctypes.

There is no fallback: if the library has not been built, loading raises.
"""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libdisc_q8_ral.so")
# the same library plus the tests' entry points (tests/dq8_test_hooks.h): kernel variant
# selection and the MFMA layout probe, which the product library does not carry
HOOKS_LIB_PATH = os.path.join(_PKG, "libdisc_q8_testhooks.so")

_lib = None
_hooks = None

_I64, _I32, _INT, _VP, _SZ = C.c_int64, C.c_int32, C.c_int, C.c_void_p, C.c_size_t
_F32 = C.c_float

# name -> (restype, argtypes); mirrors include/disc_q8.h
_PROTOS = {
    "dq8_last_error": (C.c_char_p, []),
    "dq8_version": (_INT, []),
    "dq8_device_info": (_INT, [C.POINTER(_INT)] * 3),
    "dq8_quantize": (_INT, [_VP, _VP, _INT, _I64, _I64, _I64, _VP, _VP, _I64, _I32,
                            _I32, _INT, _VP]),
    "dq8_dequantize": (_INT, [_VP, _INT, _VP, _I64, _I64, _I64, _VP, _VP, _I64, _VP]),
    "dq8_quantize_ex": (_INT, [_VP, _INT, _VP, _INT, _I64, _I64, _I64, _VP, _VP, _I64, _I64, _I64,
                               _INT, _VP]),
    "dq8_dequantize_ex": (_INT, [_VP, _INT, _VP, _I64, _I64, _I64, _VP, _VP, _I64, _VP]),
    "dq8_qgemm_workspace_bytes": (_SZ, [_I64, _I64, _I64, _INT, _INT]),
    "dq8_qgemm_workspace_bytes_zp": (_SZ, [_I64, _I64, _I64, _INT, _INT, _I32, _I32]),
    "dq8_qgemm": (_INT, [_VP, _I64, _VP, _I64, _VP, _I64, _I64, _I64, _I64, _INT, _INT,
                         _INT, _VP, _INT, _VP, _I64, _VP, _I64, _VP, _I64, _I32, _I32,
                         _I32, _VP, _SZ, _VP]),
    "dq8_qgemm_variant": (_INT, [_INT, _VP, _I64, _VP, _I64, _VP, _I64, _I64, _I64, _I64,
                                 _INT, _INT, _INT, _VP, _INT, _VP, _I64, _VP, _I64, _VP,
                                 _I64, _I32, _I32, _I32, _VP, _SZ, _VP]),
    "dq8_qgemm_num_variants": (_INT, []),
    "dq8_qgemm_variant_name": (C.c_char_p, [_INT]),
    "dq8_qconv2d": (_INT, [_VP, C.POINTER(_I64), _VP, C.POINTER(_I64), C.POINTER(_I32),
                           C.POINTER(_I32), _VP, C.POINTER(_I64), _INT, _VP, _INT, _VP,
                           _VP, _I64, _VP, _I32, _VP]),
    "dq8_qconv2d_variant": (_INT, [_INT, _VP, C.POINTER(_I64), _VP, C.POINTER(_I64),
                                   C.POINTER(_I32), C.POINTER(_I32), _VP,
                                   C.POINTER(_I64), _INT, _VP, _INT, _VP, _VP, _I64,
                                   _VP, _I32, _VP, _SZ, _VP]),
    "dq8_qconv2d_ws": (_INT, [_VP, C.POINTER(_I64), _VP, C.POINTER(_I64), C.POINTER(_I32),
                              C.POINTER(_I32), _VP, C.POINTER(_I64), _INT, _VP, _INT, _VP,
                              _VP, _I64, _VP, _I32, _VP, _SZ, _VP]),
    "dq8_qconv2d_workspace_bytes": (_SZ, [C.POINTER(_I64), C.POINTER(_I64), C.POINTER(_I32)]),
    "dq8_qconv2d_workspace_bytes_ex": (_SZ, [C.POINTER(_I64), C.POINTER(_I64), C.POINTER(_I64),
                                             C.POINTER(_I32)]),
    "dq8_mfma_probe": (_INT, [_VP] * 7),
    "dq8_lut8": (_INT, [_VP, _VP, _I64, _VP, _VP]),
    "dq8_weight_only_qgemm_workspace_bytes": (C.c_size_t, [_I64, _I64, _INT]),
    "dq8_weight_only_qgemm_workspace_bytes_ex": (C.c_size_t, [_I64, _I64, _I64, _INT, _INT]),
    "dq8_weight_only_qgemm": (_INT, [_VP, _INT, _I64, _VP, _INT, _I64, _INT, _VP, _VP, _VP, _VP,
                                     _I64, _I64, _I64, _I64, _VP, C.c_size_t, _VP]),
    "dq8_qlinear_f32_fused_max_rows": (_I64, [_I64, _I64]),
    "dq8_qlinear_f32": (_INT, [_VP, _I64, _VP, _I64, _VP, _I64, _I64, _I64, _I64, _INT, _VP, _INT,
                               _VP, _VP, _I64, _VP, _I64, _I32, _INT, _VP]),
    "dq8_qgemm_kernel_name": (C.c_char_p, [_I64, _I64, _I64, _INT]),
    "dq8_weight_only_undo_compiler_layout": (_INT, [_VP, _VP, _I64, _I64, _VP]),
    "dq8_fake_quant": (_INT, [_VP, _VP, _I64, _I64, _I64, _VP, _VP, _I64, _I32, _I32, _INT, _VP]),
    "dq8_tf_params_bytes": (_SZ, [_I64]),
    "dq8_tf_quantize_v2": (_INT, [_VP, _VP, _INT, _I64, _I64, _I64, _VP, _VP, _INT, _INT, _F32,
                                  _VP, _VP, _VP, _SZ, _VP]),
    "dq8_tf_dequantize": (_INT, [_VP, _INT, _VP, _I64, _I64, _I64, _VP, _VP, _INT, _VP, _SZ,
                                 _VP]),
    "dq8_qgemm_fused": (_INT, [_VP, _I64, _VP, _I64, _VP, _I64, _I64, _I64, _I64, _INT, _INT,
                               _INT, _VP, _INT, _VP, _I64, _VP, _I64, _VP, _I64, _I32, _I32,
                               _I32, _VP, _SZ, _VP, _VP]),
    "dq8_qconv2d_fused": (_INT, [_VP, C.POINTER(_I64), _VP, C.POINTER(_I64), C.POINTER(_I32),
                                 C.POINTER(_I32), _VP, C.POINTER(_I64), _INT, _VP, _INT, _VP,
                                 _VP, _I64, _VP, _I32, _VP, _SZ, _VP, _VP]),
    "dq8_minmax_workspace_bytes": (_SZ, [_I64, _I64, _I64]),
    "dq8_minmax": (_INT, [_VP, _I64, _I64, _I64, _VP, _VP, _VP, _SZ, _VP]),
    "dq8_minmax_static_max_bytes": (_SZ, []),
    "dq8_minmax_static": (_INT, [_VP, _I64, _I64, _I64, _VP, _VP, _VP]),
    "dq8_fill": (_INT, [_VP, _INT, _SZ, _VP]),
}


class PostOps(C.Structure):
    """dq8_postops_t (include/disc_q8.h)."""
    _fields_ = [("residual", _VP), ("residual_kind", _INT), ("ldr", _I64),
                ("residual_scale", _VP), ("residual_zp", _I32), ("relu", _INT),
                ("out_scale", _VP), ("out_zp", _I32), ("table", _VP)]


_HOOKS = ("dq8_qgemm_variant", "dq8_qgemm_num_variants", "dq8_qgemm_variant_name",
          "dq8_qconv2d_variant", "dq8_mfma_probe")


def _bind(L, skip=()):
    for name, (res, args) in _PROTOS.items():
        if name in skip:
            continue
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    return L


def hooks():
    """libdisc_q8_testhooks.so: every entry of the product library (a second copy of the
    kernels, with its own state and its own dq8_last_error) plus the tests' hooks."""
    global _hooks
    if _hooks is None:
        if not os.path.exists(HOOKS_LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m bladedisc_amd.build` "
                "(there is no CPU fallback)" % HOOKS_LIB_PATH)
        _hooks = _bind(C.CDLL(HOOKS_LIB_PATH))
    return _hooks


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m bladedisc_amd.build` "
                "(there is no CPU fallback)" % LIB_PATH)
        _lib = _bind(C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL), skip=_HOOKS)
    return _lib


def check(status, what, L=None):
    if status != 0:
        msg = (L or lib()).dq8_last_error().decode()
        raise RuntimeError("%s failed: %s" % (what, msg))
