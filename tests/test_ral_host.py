"""Host-side RAL tests (no GPU): symbol mangling, the registry, argument packing,
the custom_attrs reader and the error paths a host can force."""
import ctypes as C
import json

import numpy as np
import pytest

from bladedisc_amd import ral

GOLDEN_NAMES = [
    # reference gpu per-tensor ral_qgemm (stream_executor_based_impl.cc:427-437,1973)
    "ral_qgemm___gpu___pvoid_pvoid_m2di8_m2di8_m0df32_m0di32_m0df32_m0di32_m0df32_m0di32_m2di8_i1_i1_i1___void",
    # per-channel weight scale, as registered for cpu at common_context_impl_quantization.cc:1700
    "ral_qgemm___gpu___pvoid_pvoid_m2di8_m2di8_m0df32_m0di32_m1df32_m1di32_m0df32_m0di32_m2di8_i1_i1_i1___void",
    # stream_executor_based_impl.cc:1831-1841,1999-2000
    "ral_qconv___gpu___pvoid_pvoid_m4di8_m4di8_m1di32_m0df32_m0di32_m1df32_m1di32_m0df32_m0di32_m4di8_m1di32___void",
    # the older symmetric entry (common_context_impl_quantization.cc:38-44, registered for cpu at :1680) mirrored on gpu
    "ral_qconv_s8_s8_s8___gpu___pvoid_pvoid_m4di8_m4di8_m1di32_m0df32_m1df32_m0df32_m4di8_m1di32___void",
    # quantized_gpu_kernel_impl.cc:424-475
    "ral_pdll_qgemm___gpu___pvoid_pvoid_m2di8_m2di8_m1di8_m0df32_m0di32_m0df32_m0di32_m0df32_m0di32_pvoid___m2di8",
    "ral_pdll_qgemm___gpu___pvoid_pvoid_m3di8_m2di8_m1di8_m0df32_m0di32_m0df32_m0di32_m0df32_m0di32_pvoid___m3di8",
    "ral_pdll_qgemm___gpu___pvoid_pvoid_m2di8_m2di8_m1df32_m0df32_m0di32_m0df32_m0di32_m0df32_m0di32_pvoid___m2di8",
    "ral_pdll_qgemm___gpu___pvoid_pvoid_m3di8_m2di8_m1df32_m0df32_m0di32_m0df32_m0di32_m0df32_m0di32_pvoid___m3di8",
    # quantized_gpu_kernel_impl.cc:476-481
    "ral_pdll_qgemm_per_channel___gpu___pvoid_pvoid_m2di8_m2di8_m1di8_m1df32_m1di32_m1df32_m1di32_m1df32_m1di32_pvoid___m2di8",
    "ral_pdll_qgemm_per_channel___gpu___pvoid_pvoid_m3di8_m2di8_m1di8_m1df32_m1di32_m1df32_m1di32_m1df32_m1di32_pvoid___m3di8",
    # CPU-style overloads (common_context_impl_quantization.cc:1701-1718) mirrored on gpu
    "ral_pdll_qgemm___gpu___pvoid_pvoid_m2di8_m2di8_m1df32_m0df32_m0di32_m1df32_m1di32_m0df32_m0di32_pvoid___m2di8",
    "ral_pdll_qgemm___gpu___pvoid_pvoid_m4di8_m2di8_m1di32_m0df32_m0di32_m1df32_m1di32_m0df32_m0di32_pvoid___m4di8",
    "ral_pdll_qgemm___gpu___pvoid_pvoid_m3di8_m2di8_m0df32_m0di32_m1df32_m1di32_m0df32_m0di32_pvoid___m3di8",
    # gpu driver set (gpu_driver.cc:27-41; cuda_context_impl.cc:746-764)
    "alloc___gpu___pvoid_i64___pvoid",
    "dealloc___gpu___pvoid_pvoid___void",
    "ral_kernel_launch___gpu___pvoid_ppvoid_i64_pvoid_i64_i64_i64_i64_i64_i64_i32_pvoid_i32_ppvoid___void",
    "d2h____gpu___pvoid_pvoid_pvoid_pvoid_i64___void",
    "ral_gpu_get_stream___gpu___pvoid_i32___pvoid",
    # the AArch64 build's per-tensor ral_pdll_qgemm signatures (weight scale and zero point
    # of rank 0; common_context_impl_quantization.cc:1689-1695), mirrored for device gpu
    "ral_pdll_qgemm___gpu___pvoid_pvoid_m2di8_m2di8_m0df32_m0di32_m0df32_m0di32_m0df32_m0di32_pvoid___m2di8",
    "ral_pdll_qgemm___gpu___pvoid_pvoid_m4di8_m2di8_m0df32_m0di32_m0df32_m0di32_m0df32_m0di32_pvoid___m4di8",
    "ral_pdll_qgemm___gpu___pvoid_pvoid_m3di8_m2di8_m1di32_m0df32_m0di32_m0df32_m0di32_m0df32_m0di32_pvoid___m3di8",
    # weight_only_qgemm.pdll:2-104 with the operand types of test_quantization.py:550,612 (f32) and of
    # disc-convert-weight-layout-for-weight-only-gemm.mlir:5-10 (f16): input, weight ui8 [K,N], [bias,]
    # scale, zero point i32, custom_attrs
    "ral_pdll_weight_only_qgemm___gpu___pvoid_pvoid_m3df32_m2dui8_m1df32_m1di32_pvoid___m3df32",
    "ral_pdll_weight_only_qgemm___gpu___pvoid_pvoid_m3df32_m2dui8_m1df32_m1df32_m1di32_pvoid___m3df32",
    "ral_pdll_weight_only_qgemm___gpu___pvoid_pvoid_m3df16_m2dui8_m1df16_m1di32_pvoid___m3df16",
    "ral_pdll_weight_only_qgemm___gpu___pvoid_pvoid_m2df16_m2dui8_m1df16_m1df16_m1di32_pvoid___m2df16",
]


def test_golden_mangled_names_are_registered():
    names = set(ral.registered_names())
    for g in GOLDEN_NAMES:
        assert g in names, g
        assert ral.api_exists(g)
    for bare in ("ral_qgemm", "ral_pdll_qgemm", "ral_pdll_qgemm_per_channel", "ral_qconv",
                 "ral_quantize", "ral_dequantize", "h2d_", "d2d_", "sync_on_stream",
                 "ral_gpu_as_cu_stream", "ral_gpu_alloc_persistent", "raw_gpu_alloc"):
        assert bare in names
    assert not ral.api_exists("ral_qgemm___gpu___pvoid___void")


def test_mangle_from_packed_args_matches_golden():
    a = ral.Args().scalar("pvoid", 0).scalar("pvoid", 0)
    a.memref("i8", 0, [4, 8]).memref("i8", 0, [16, 8])
    for _ in range(3):
        a.memref("f32", 0, []).memref("i32", 0, [])
    a.memref("i8", 0, [4, 16]).scalar("i1", False).scalar("i1", True).scalar("i1", True)
    assert ral.mangle("ral_qgemm", "gpu", a.arg_codes, a.ret_codes) == GOLDEN_NAMES[0]
    # slots: 2 scalars + 2*(3+4) + 6*3 + (3+4) + 3
    assert len(a._slots) == 2 + 14 + 18 + 7 + 3


def test_attr_blob_reader_round_trip():
    L = ral.lib()
    L.disc_ral_attr_to_json.restype = C.c_int64
    L.disc_ral_attr_to_json.argtypes = [C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t]
    value = {"transpose_a": False, "transpose_b": True, "weight_is_const": True,
             "bias_is_const": True, "data_format": "NHWC", "strides": [1, 2, 2, 1],
             "dilations": [1, 1, 1, 1], "padding": "SAME", "explicit_paddings": [],
             "alpha": 0.5, "count": 7, "nested": [{"k": 1}, "s"]}
    blob = ral.encode_attr(value)
    buf = C.create_string_buffer(4096)
    n = L.disc_ral_attr_to_json(blob, len(blob), buf, 4096)
    assert n > 0
    assert json.loads(buf.value.decode()) == value
    # truncated blobs are rejected, never read past the end
    for cut in (1, 7, 12, len(blob) // 2, len(blob) - 1):
        assert L.disc_ral_attr_to_json(blob[:cut], cut, buf, 4096) == -1
    assert L.disc_ral_attr_to_json(ral._s(b"bogus"), 13, buf, 4096) == -1


def test_dense_elements_attr_splat_is_expanded():
    import struct
    L = ral.lib()
    L.disc_ral_attr_to_json.restype = C.c_int64
    L.disc_ral_attr_to_json.argtypes = [C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t]
    blob = (ral._s(b"denseElementsAttr") + ral._s(b"int") + struct.pack("<I", 32) +
            struct.pack("<q", 1) + struct.pack("<q", 3) + struct.pack("<?", True) +
            ral._s(struct.pack("<i", 5)))
    buf = C.create_string_buffer(1024)
    assert L.disc_ral_attr_to_json(blob, len(blob), buf, 1024) > 0
    got = json.loads(buf.value.decode())
    assert got["dense"] == "int32" and got["shape"] == [3]
    assert got["bytes"] == [5, 0, 0, 0] * 3


def test_unknown_api_and_error_state():
    ctx = ral.RalContext()
    with ctx.execution() as ex:
        with pytest.raises(ral.RalError, match="not found"):
            ex.call("ral_no_such_kernel", "gpu", ral.Args().ctx(ex.handle))
        # the error was cleared by the wrapper; without clearing, later calls are refused
        a = ral.Args().ctx(ex.handle)
        ex.call("ral_no_such_kernel", "gpu", a, check=False)
        st, msg = ctx.last_error()
        assert st != 0 and "ral_no_such_kernel" in msg
        a = ral.Args().ctx(ex.handle).scalar("i32", 0)
        r = a.result_scalar("pvoid")
        r.value = 1234
        ex.call("ral_gpu_get_stream", "gpu", a, check=False)   # refused: context poisoned
        assert r.value == 1234
        ctx.clear_error()
        ex.call("ral_gpu_get_stream", "gpu", a)
        assert (r.value or 0) == 0
    ctx.close()


def test_driver_stream_rules():
    ctx = ral.RalContext()
    with ctx.execution() as ex:
        a = ral.Args().ctx(ex.handle).scalar("i32", 1)
        a.result_scalar("pvoid")
        with pytest.raises(ral.RalError, match="multi-stream not supported"):
            ex.call("ral_gpu_get_stream", "gpu", a)
        a = ral.Args().ctx(ex.handle).scalar("i32", -1)
        a.result_scalar("pvoid")
        with pytest.raises(ral.RalError, match="not a valid stream_id"):
            ex.call("ral_gpu_get_stream", "gpu", a)
    ctx.close()


def _qgemm_args(ex, m, k, wn, wk, out_m, out_n, tp_a=False, tp_b=True):
    a = ex.new_args()
    a.memref("i8", 0x1000, [m, k]).memref("i8", 0x2000, [wn, wk])
    for _ in range(3):
        a.memref("f32", 0x3000, []).memref("i32", 0x4000, [])
    a.memref("i8", 0x5000, [out_m, out_n])
    a.scalar("i1", tp_a).scalar("i1", tp_b).scalar("i1", False)
    return a


def test_qgemm_argument_errors_without_gpu():
    ctx = ral.RalContext()
    with ctx.execution() as ex:
        with pytest.raises(ral.RalError, match="mismatch contraction dim"):
            ex.call("ral_qgemm", "gpu", _qgemm_args(ex, 4, 8, 16, 9, 4, 16))
        with pytest.raises(ral.RalError, match="result shape"):
            ex.call("ral_qgemm", "gpu", _qgemm_args(ex, 4, 8, 16, 8, 4, 15))
        # empty tensors return early, launching nothing (quantized_gpu_kernel_impl.cc:347-351)
        ex.call("ral_qgemm", "gpu", _qgemm_args(ex, 0, 8, 16, 8, 0, 16))
    ctx.close()


def test_pdll_qgemm_empty_input_returns_null_memref_with_shape():
    ctx = ral.RalContext()
    with ctx.execution() as ex:
        a = ex.new_args()
        a.memref("i8", 0, [2, 0, 8]).memref("i8", 0x2000, [16, 8]).memref("i8", 0x3000, [16])
        zp = np.zeros(1, np.int32)
        for _ in range(3):
            a.memref("f32", 0x4000, []).host_array(zp, rank0=True)
        a.blob(ral.encode_attr({}))
        res = a.result_memref("i8", 3)
        name = ex.call("ral_pdll_qgemm", "gpu", a)
        assert name.endswith("___m3di8")
        assert not res.data and list(res.sizes) == [2, 0, 16]
        # contraction mismatch is reported before anything touches the device
        a = ex.new_args()
        a.memref("i8", 0x1000, [2, 9]).memref("i8", 0x2000, [16, 8]).memref("i8", 0x3000, [16])
        for _ in range(3):
            a.memref("f32", 0x4000, []).host_array(zp, rank0=True)
        a.blob(ral.encode_attr({}))
        a.result_memref("i8", 2)
        with pytest.raises(ral.RalError, match="mismatch contraction dim"):
            ex.call("ral_pdll_qgemm", "gpu", a)
    ctx.close()


def test_size_class_pool_is_exposed_through_raw_alloc_names():
    # the allocator's size classes: at most 25 % slack, monotone
    # (checked through the documented rule; the pool itself needs a GPU)
    def size_class(b):
        if b <= 256:
            return 256
        p = 256
        while p < b:
            p <<= 1
        q, c = p >> 3, p >> 1
        while c < b:
            c += q
        return c
    prev = 0
    for b in [1, 255, 256, 257, 300, 1000, 4096, 5000, 10**6, 3 * 2**20 + 1]:
        c = size_class(b)
        assert c >= b and c <= max(256, b * 1.25 + 1) and c >= prev
        prev = c


def test_conv2d_plan_matches_oracle():
    """The attribute -> padding / metadata / result-shape rules of ral_pdll_qconv2d,
    against the oracle's restatement of the reference helpers
    (common_context_impl_quantization.h:27-206), over the attribute forms the reference
    accepts."""
    import itertools
    import oracle as O
    from bladedisc_amd import ral_ops
    cases = 0
    for fmt, pad, (kh, kw), nstr, stride, dil in itertools.product(
            ("NHWC", "NCHW"), ("SAME", "VALID", "EXPLICIT4", "EXPLICIT8"), ((1, 1), (3, 3), (5, 2)),
            (1, 2, 4), (1, 2, 3), (1, 2)):
        h, w, ci, co = 13, 10, 8, 6
        in_shape = (2, h, w, ci) if fmt == "NHWC" else (2, ci, h, w)
        w_shape = (co, kh, kw, ci)
        sp = (1, 2) if fmt == "NHWC" else (2, 3)
        def attr(v):
            if nstr == 1:
                return [v]
            if nstr == 2:
                return [v, v + 1]
            full = [1, 1, 1, 1]
            full[sp[0]], full[sp[1]] = v, v + 1
            return full
        strides, dilations = attr(stride), attr(dil)
        explicit = []
        padding = pad
        if pad == "EXPLICIT4":
            padding, explicit = "EXPLICIT", [1, 2, 0, 3]
        elif pad == "EXPLICIT8":
            padding = "EXPLICIT"
            explicit = [0] * 8
            explicit[2 * sp[0]:2 * sp[0] + 2] = [2, 1]
            explicit[2 * sp[1]:2 * sp[1] + 2] = [0, 1]
        want = O.conv_attrs(in_shape, w_shape, fmt, strides, dilations, padding,
                            explicit_paddings=explicit, weight_is_const=bool(cases & 1))
        got = ral_ops.conv2d_plan(in_shape, w_shape, fmt, strides, dilations, padding,
                                  explicit_paddings=explicit, weight_is_const=bool(cases & 1))
        assert got == tuple(want) or list(got) == [list(want[0]), list(want[1]), list(want[2])], \
            (fmt, pad, kh, kw, strides, dilations, got, want)
        cases += 1
    assert cases == 2 * 4 * 3 * 3 * 3 * 2
    # the closed forms of the reference's own conv tests: 1x1 SAME keeps the size,
    # 3x3 VALID loses two, stride 2 + dilation 2 on 7 -> 2
    assert ral_ops.conv2d_plan((1, 5, 5, 4), (3, 1, 1, 4), "NHWC", [1], [1], "SAME")[2] == [1, 5, 5, 3]
    assert ral_ops.conv2d_plan((1, 5, 5, 4), (3, 3, 3, 4), "NHWC", [1], [1], "VALID")[2] == [1, 3, 3, 3]
    assert ral_ops.conv2d_plan((1, 7, 7, 4), (3, 3, 3, 4), "NHWC", [2], [2], "VALID")[2] == [1, 2, 2, 3]
    for bad in (dict(data_format="NHW"), dict(data_format="ABCD"), dict(padding="FULL"),
                dict(strides=[1, 1, 1]), dict(strides=[0]), dict(explicit_paddings=[1, 2, 3],
                                                                 padding="EXPLICIT")):
        kw = dict(data_format="NHWC", strides=[1], dilations=[1], padding="SAME",
                  explicit_paddings=[])
        kw.update(bad)
        with pytest.raises(ValueError):
            ral_ops.conv2d_plan((1, 5, 5, 4), (3, 3, 3, 4), **kw)


def test_metadata_file_round_trip(tmp_path):
    """Constant store in the reference's metadata-file layout: written, read back,
    duplicate names refused, a damaged file rejected."""
    import struct
    L = ral.lib()
    path = str(tmp_path / "m.metadata").encode()
    names = [b"w0_i8_2x2", b"h0_f32_", b"w1_f32_3"]
    vals = [b"01ff7f80", b"0000803f", b"00"]
    flags = (C.c_uint8 * 3)(0, 1, 0)
    assert L.disc_ral_metadata_emit(path, 3, flags, (C.c_char_p * 3)(*names),
                                    (C.c_char_p * 3)(*vals)) == 0
    raw = open(path, "rb").read()
    # layout: magic, records {is_host u8, len-prefixed key, len-prefixed value}, count
    assert struct.unpack_from("<Q", raw, 0)[0] == 0x1234567890ABCDEF
    assert struct.unpack_from("<Q", raw, len(raw) - 8)[0] == 3
    assert raw[8] == 0 and struct.unpack_from("<Q", raw, 9)[0] == len(names[0])
    assert raw[17:17 + len(names[0])] == names[0]
    h, d = C.c_int(), C.c_int()
    probes = (C.c_char_p * 4)(*(names + [b"absent_i8_1"]))
    assert L.disc_ral_metadata_count(path, C.byref(h), C.byref(d), probes, 4) == 0
    assert (h.value, d.value) == (1, 2)
    # duplicate device constant
    dup = str(tmp_path / "dup.metadata").encode()
    assert L.disc_ral_metadata_emit(dup, 2, (C.c_uint8 * 2)(0, 0), (C.c_char_p * 2)(b"a_i8_1", b"a_i8_1"),
                                    (C.c_char_p * 2)(b"00", b"01")) != 0
    # truncated and wrong-magic files
    bad = str(tmp_path / "bad.metadata")
    open(bad, "wb").write(raw[:-12])
    assert L.disc_ral_metadata_count(bad.encode(), None, None, probes, 4) != 0
    open(bad, "wb").write(b"\x00" * 8 + raw[8:])
    assert L.disc_ral_metadata_count(bad.encode(), None, None, probes, 4) != 0
    assert L.disc_ral_metadata_count(str(tmp_path / "nope").encode(), None, None, probes, 4) != 0


def test_program_io_bindings_on_host_memory():
    """ral_recv_input / ral_send_output / take_output with plain host buffers: inputs are
    found by index and rank, an output that is an input is forwarded, unknown indices
    are errors."""
    L = ral.lib()
    L.disc_ral_execution_take_output.restype = C.c_void_p
    L.disc_ral_output_data.restype = C.c_void_p
    L.disc_ral_output_dim.restype = C.c_int64
    ctx = ral.RalContext()
    try:
        with ctx.execution() as ex:
            buf = np.arange(12, dtype=np.float32)
            assert L.disc_ral_execution_bind_input(C.c_void_p(ex.handle), 3,
                                                   C.c_void_p(buf.ctypes.data),
                                                   (C.c_int64 * 2)(3, 4), 2) == 0
            a = ral.Args().ctx(ex.handle)
            a.scalar("i64", 3)
            res = a.result_memref("f32", 2)
            ex.call("ral_recv_input", "cpu", a)
            assert res.data == buf.ctypes.data and list(res.sizes) == [3, 4]
            assert list(res.strides) == [4, 1]
            # send it back as output 0
            a = ral.Args().ctx(ex.handle)
            a.scalar("i64", 0)
            a.memref("f32", buf.ctypes.data, [3, 4])
            ex.call("ral_send_output", "cpu", a)
            out = L.disc_ral_execution_take_output(C.c_void_p(ex.handle), 0)
            assert out and L.disc_ral_output_data(C.c_void_p(out)) == buf.ctypes.data
            assert L.disc_ral_output_owned(C.c_void_p(out)) == 0
            assert [L.disc_ral_output_dim(C.c_void_p(out), i) for i in range(2)] == [3, 4]
            L.disc_ral_output_destroy(C.c_void_p(out))
        own = ral.RalContext()
        with own.execution() as ex:
            a = ral.Args().ctx(ex.handle)
            a.scalar("i64", 7)
            a.result_memref("f32", 2)
            with pytest.raises(ral.RalError, match="invalid input index"):
                ex.call("ral_recv_input", "cpu", a)
        own.close()
    finally:
        ctx.close()
