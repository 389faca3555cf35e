"""A whole compiled program on the runtime: a C stand-in for a DISC-generated `main`
(tests/programs/qlinear_program.c) fetches its input, materialises its constants from
a metadata file, runs quantize -> ral_pdll_qgemm -> dequantize and hands back its
output, all through tao_ral_call_impl.  Checked against the CPU oracle."""
import ctypes as C
import os
import shutil
import subprocess

import numpy as np
import pytest

torch = pytest.importorskip("torch")
import oracle as O  # noqa: E402

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def hexstr(a):
    return np.ascontiguousarray(a).tobytes().hex()


@pytest.fixture(scope="module")
def program(tmp_path_factory):
    if shutil.which("gcc") is None:
        pytest.skip("gcc is needed to build the stand-in program")
    from bladedisc_amd import ral
    d = tmp_path_factory.mktemp("program")
    blob = ral.encode_attr({"transpose_a": False, "transpose_b": True, "weight_is_const": True,
                            "bias_is_const": True})
    with open(d / "attrs.c", "w") as f:
        f.write("const unsigned char kQgemmAttrs[] = {%s, 0};\n" % ", ".join(str(b) for b in blob))
    so = str(d / "libqlinear_program.so")
    subprocess.check_call(["gcc", "-O1", "-shared", "-fPIC", "-o", so,
                           os.path.join(HERE, "programs", "qlinear_program.c"), str(d / "attrs.c")])
    return C.CDLL(so), d


def test_compiled_program_runs_on_the_runtime(program):
    lib, d = program
    from bladedisc_amd import baseline_configs as cfg
    from bladedisc_amd import ral
    L = ral.lib()
    c = cfg.config1()
    names = ["w0_i8_768x768", "b0_f32_768", "sw0_f32_768", "sx0_f32_", "so0_f32_", "z0_i32_"]
    values = [hexstr(c["w_q"]), hexstr(c["bias"]), hexstr(c["sw"]),
              hexstr(np.array([c["sx"]], np.float32)), hexstr(np.array([c["so"]], np.float32)),
              hexstr(np.array([0], np.int32))]
    meta = str(d / "program.metadata").encode()
    n = len(names)
    L.disc_ral_metadata_emit.restype = C.c_int
    rc = L.disc_ral_metadata_emit(meta, n, (C.c_uint8 * n)(*([0] * n)),
                                  (C.c_char_p * n)(*[s.encode() for s in names]),
                                  (C.c_char_p * n)(*[v.encode() for v in values]))
    assert rc == 0

    L.disc_ral_context_create_for_program.restype = C.c_void_p
    L.disc_ral_execution_take_output.restype = C.c_void_p
    L.disc_ral_output_data.restype = C.c_void_p
    L.disc_ral_output_dim.restype = C.c_int64
    stream = torch.cuda.current_stream().cuda_stream
    ctx = L.disc_ral_context_create_for_program(C.c_void_p(stream), 0, None, None, None, 1, meta)
    assert ctx
    call_impl = C.cast(L.tao_ral_call_impl, C.c_void_p).value
    try:
        for m in (64, 5):                       # two executions, a dynamic M, cached constants
            x = torch.from_numpy(np.ascontiguousarray(c["x"][:m])).cuda()
            ex = L.disc_ral_execution_context_create(C.c_void_p(ctx))
            assert L.disc_ral_execution_bind_input(C.c_void_p(ex), 0, C.c_void_p(x.data_ptr()),
                                                   (C.c_int64 * 2)(m, 768), 2) == 0
            ctx_struct = (C.c_void_p * 2)(ex, call_impl)
            lib.disc_program_main(ctx_struct)
            msg = C.c_char_p()
            assert L.tao_ral_last_error(C.c_void_p(ctx), C.byref(msg)) == 0, msg.value
            out = L.disc_ral_execution_take_output(C.c_void_p(ex), 0)
            fwd = L.disc_ral_execution_take_output(C.c_void_p(ex), 1)
            assert out and fwd
            assert L.disc_ral_output_rank(C.c_void_p(out)) == 2
            assert [L.disc_ral_output_dim(C.c_void_p(out), i) for i in range(2)] == [m, 768]
            # output 0 was allocated by the program: the handle owns it; output 1 is the
            # input buffer handed back and stays the caller's
            assert L.disc_ral_output_owned(C.c_void_p(out)) == 1
            assert L.disc_ral_output_owned(C.c_void_p(fwd)) == 0
            assert L.disc_ral_output_data(C.c_void_p(fwd)) == x.data_ptr()
            torch.cuda.synchronize()
            y = ral.device_view(L.disc_ral_output_data(C.c_void_p(out)), (m, 768),
                                torch.float32).cpu().numpy()
            # oracle: the same chain on the host
            xq = O.quantize(c["x"][:m], c["sx"], 0)
            acc = O.gemm_s32(xq, c["w_q"], tp_b=True)
            b32 = O.bias_f32_to_s32(c["bias"], float(c["sx"]), c["sw"])
            yq = O.requant_cpu(acc, float(c["sx"]), c["sw"], float(c["so"]), b32=b32)
            np.testing.assert_array_equal(y, O.dequantize(yq, c["so"], 0))
            L.disc_ral_output_destroy(C.c_void_p(out))
            L.disc_ral_output_destroy(C.c_void_p(fwd))
            L.disc_ral_execution_context_destroy(C.c_void_p(ex))
    finally:
        torch.cuda.synchronize()
        L.disc_ral_context_destroy(C.c_void_p(ctx))


def test_compiled_program_captured_into_a_graph(program):
    """A serving loop replays a compiled program from a HIP graph.  After one ordinary
    execution (constants loaded, the context's pool holds buffers of every size the program
    asks for) a second execution of `main` runs under stream capture -- no entry on the way may
    allocate device memory, synchronise or copy through the host -- and the graph is replayed
    three times on new input contents, with eager work and synchronisations in between; every
    replay must give the oracle's bits."""
    lib, d = program
    from bladedisc_amd import baseline_configs as cfg
    from bladedisc_amd import ral
    L = ral.lib()
    c = cfg.config1()
    names = ["w0_i8_768x768", "b0_f32_768", "sw0_f32_768", "sx0_f32_", "so0_f32_", "z0_i32_"]
    values = [hexstr(c["w_q"]), hexstr(c["bias"]), hexstr(c["sw"]),
              hexstr(np.array([c["sx"]], np.float32)), hexstr(np.array([c["so"]], np.float32)),
              hexstr(np.array([0], np.int32))]
    meta = str(d / "captured.metadata").encode()
    n = len(names)
    L.disc_ral_metadata_emit.restype = C.c_int
    assert L.disc_ral_metadata_emit(meta, n, (C.c_uint8 * n)(*([0] * n)),
                                    (C.c_char_p * n)(*[s.encode() for s in names]),
                                    (C.c_char_p * n)(*[v.encode() for v in values])) == 0
    L.disc_ral_context_create_for_program.restype = C.c_void_p
    L.disc_ral_execution_take_output.restype = C.c_void_p
    L.disc_ral_output_data.restype = C.c_void_p
    side = torch.cuda.Stream()
    ctx = L.disc_ral_context_create_for_program(C.c_void_p(side.cuda_stream), 0, None, None, None,
                                                1, meta)
    assert ctx
    call_impl = C.cast(L.tao_ral_call_impl, C.c_void_p).value
    m = 48
    x = torch.zeros((m, 768), device="cuda")

    def run_main():
        ex = L.disc_ral_execution_context_create(C.c_void_p(ctx))
        assert L.disc_ral_execution_bind_input(C.c_void_p(ex), 0, C.c_void_p(x.data_ptr()),
                                               (C.c_int64 * 2)(m, 768), 2) == 0
        lib.disc_program_main((C.c_void_p * 2)(ex, call_impl))
        msg = C.c_char_p()
        assert L.tao_ral_last_error(C.c_void_p(ctx), C.byref(msg)) == 0, msg.value
        out = L.disc_ral_execution_take_output(C.c_void_p(ex), 0)
        fwd = L.disc_ral_execution_take_output(C.c_void_p(ex), 1)
        L.disc_ral_output_destroy(C.c_void_p(fwd))
        L.disc_ral_execution_context_destroy(C.c_void_p(ex))
        return out

    def want(xs):
        xq = O.quantize(xs, c["sx"], 0)
        acc = O.gemm_s32(xq, c["w_q"], tp_b=True)
        b32 = O.bias_f32_to_s32(c["bias"], float(c["sx"]), c["sw"])
        return O.dequantize(O.requant_cpu(acc, float(c["sx"]), c["sw"], float(c["so"]), b32=b32),
                            c["so"], 0)

    try:
        x.copy_(torch.from_numpy(np.ascontiguousarray(c["x"][:m])))
        side.wait_stream(torch.cuda.current_stream())
        warm = run_main()                                   # ordinary execution: warms everything
        side.synchronize()
        L.disc_ral_output_destroy(C.c_void_p(warm))         # its result goes back to the pool
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            g.capture_begin()
            out = run_main()
            g.capture_end()
        y = ral.device_view(L.disc_ral_output_data(C.c_void_p(out)), (m, 768), torch.float32)
        rng = np.random.default_rng(11)
        for rep in range(3):
            xs = (rng.standard_normal((m, 768)) * (rep + 1)).astype(np.float32)
            x.copy_(torch.from_numpy(xs))
            y.zero_()
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            np.testing.assert_array_equal(y.cpu().numpy(), want(xs))
        del g
        L.disc_ral_output_destroy(C.c_void_p(out))
    finally:
        torch.cuda.synchronize()
        L.disc_ral_context_destroy(C.c_void_p(ctx))


def test_process_level_constant_store(program):
    """DISC_USE_GLOBAL_CONST_STORE=1 (common_context_impl.cc:57-64): contexts made from one
    metadata file share one store of constants, which outlives all but the last of them; without
    the switch a second context has to load the file itself.  In child processes: the switch is
    read once per process."""
    import sys
    lib, d = program
    so = str(d / "libqlinear_program.so")
    script = os.path.join(HERE, "programs", "shared_const_store_scenario.py")
    for value, want in (("1", 0), (None, 3)):
        env = dict(os.environ)
        env.pop("DISC_USE_GLOBAL_CONST_STORE", None)
        if value is not None:
            env["DISC_USE_GLOBAL_CONST_STORE"] = value
        r = subprocess.run([sys.executable, script, so, str(d)], env=env, capture_output=True,
                           text=True, timeout=300)
        assert r.returncode == want, (value, r.returncode, r.stdout[-800:], r.stderr[-800:])
    assert "OK" in r.stdout or want == 3


def _decoy_code_objects():
    """Images a multi-target build could carry next to the gfx950 one: PTX text, and the ELF
    header of a code object for another AMD processor (EM_AMDGPU = 224, e_flags mach 0x4c)."""
    import struct
    ptx = b"//\n// Generated by NVIDIA NVVM Compiler\n.version 7.8\n.target sm_80\n" + b" " * 64
    elf = bytearray(64)
    elf[:7] = b"\x7fELF\x02\x01\x01"
    struct.pack_into("<HHI", elf, 16, 1, 224, 1)
    struct.pack_into("<I", elf, 48, 0x54c)
    return ptx, bytes(elf)


@pytest.mark.parametrize("images", ["one", "three", "none_for_this_device"])
def test_program_with_an_embedded_code_object(program, images):
    """The same program with its dequantize replaced by a fused elementwise kernel that
    travels as a gfx950 code object, the way the compiler ships its generated kernels, and
    is launched through ral_kernel_launch: y = relu(dequantize(qgemm(...))) + x.  Two
    executions (the second finds the loaded module cached), checked bit for bit.  With
    several images per kernel (R context/base/cuda/cuda_context_impl.cc:375-392 picks by
    compute capability) the launch takes the one built for this device, and says so when
    there is none."""
    lib, d = program
    hsaco = os.path.join(HERE, "programs", "fused_dequant_relu_residual.hsaco")
    if not os.path.exists(hsaco):        # normally built beforehand by __graft_entry__.build()
        from bladedisc_amd import build as b
        b.build_test_code_objects()
    blob = open(hsaco, "rb").read()
    blob_buf = C.create_string_buffer(blob, len(blob))      # lives as long as the context
    ptx, other_elf = _decoy_code_objects()
    decoys = [C.create_string_buffer(ptx, len(ptx)), C.create_string_buffer(other_elf, len(other_elf))]
    if images == "one":
        lib.disc_program_set_code_object(C.cast(blob_buf, C.c_void_p))
    else:
        bufs = [decoys[0], decoys[1]] + ([blob_buf] if images == "three" else [])
        arr = (C.c_void_p * len(bufs))(*[C.cast(b, C.c_void_p).value for b in bufs])
        lib.disc_program_set_code_objects(arr, len(bufs))
    from bladedisc_amd import baseline_configs as cfg
    from bladedisc_amd import ral
    L = ral.lib()
    c = cfg.config1()
    names = ["w0_i8_768x768", "b0_f32_768", "sw0_f32_768", "sx0_f32_", "so0_f32_", "z0_i32_"]
    values = [hexstr(c["w_q"]), hexstr(c["bias"]), hexstr(c["sw"]),
              hexstr(np.array([c["sx"]], np.float32)), hexstr(np.array([c["so"]], np.float32)),
              hexstr(np.array([0], np.int32))]
    meta = str(d / "fused.metadata").encode()
    n = len(names)
    L.disc_ral_metadata_emit.restype = C.c_int
    assert L.disc_ral_metadata_emit(meta, n, (C.c_uint8 * n)(*([0] * n)),
                                    (C.c_char_p * n)(*[s.encode() for s in names]),
                                    (C.c_char_p * n)(*[v.encode() for v in values])) == 0
    L.disc_ral_context_create_for_program.restype = C.c_void_p
    L.disc_ral_execution_take_output.restype = C.c_void_p
    L.disc_ral_output_data.restype = C.c_void_p
    stream = torch.cuda.current_stream().cuda_stream
    ctx = L.disc_ral_context_create_for_program(C.c_void_p(stream), 0, None, None, None, 1, meta)
    assert ctx
    call_impl = C.cast(L.tao_ral_call_impl, C.c_void_p).value
    try:
        for m in (64, 7):
            x = torch.from_numpy(np.ascontiguousarray(c["x"][:m])).cuda()
            ex = L.disc_ral_execution_context_create(C.c_void_p(ctx))
            assert L.disc_ral_execution_bind_input(C.c_void_p(ex), 0, C.c_void_p(x.data_ptr()),
                                                   (C.c_int64 * 2)(m, 768), 2) == 0
            lib.disc_program_main_fused((C.c_void_p * 2)(ex, call_impl))
            msg = C.c_char_p()
            if images == "none_for_this_device":
                assert L.tao_ral_last_error(C.c_void_p(ctx), C.byref(msg)) != 0
                assert b"is built for gfx950" in msg.value
                L.tao_ral_clear_error(C.c_void_p(ctx))
                L.disc_ral_execution_context_destroy(C.c_void_p(ex))
                break
            assert L.tao_ral_last_error(C.c_void_p(ctx), C.byref(msg)) == 0, msg.value
            out = L.disc_ral_execution_take_output(C.c_void_p(ex), 0)
            assert out
            torch.cuda.synchronize()
            y = ral.device_view(L.disc_ral_output_data(C.c_void_p(out)), (m, 768),
                                torch.float32).cpu().numpy()
            xq = O.quantize(c["x"][:m], c["sx"], 0)
            acc = O.gemm_s32(xq, c["w_q"], tp_b=True)
            b32 = O.bias_f32_to_s32(c["bias"], float(c["sx"]), c["sw"])
            yq = O.requant_cpu(acc, float(c["sx"]), c["sw"], float(c["so"]), b32=b32)
            deq = yq.astype(np.float32) * np.float32(c["so"])
            want = np.maximum(deq, np.float32(0)) + c["x"][:m].astype(np.float32)
            np.testing.assert_array_equal(y, want)
            L.disc_ral_output_destroy(C.c_void_p(out))
            L.disc_ral_execution_context_destroy(C.c_void_p(ex))
        # a kernel name the code object does not hold is an error, not a crash
        ex = L.disc_ral_execution_context_create(C.c_void_p(ctx))
        a = ral.Args().ctx(ex)
        blobs = (C.c_void_p * 1)(C.cast(blob_buf, C.c_void_p).value)
        a.scalar("ppvoid", C.cast(blobs, C.c_void_p).value).scalar("i64", 1)
        a.scalar("pvoid", C.cast(C.c_char_p(b"no_such_kernel"), C.c_void_p).value)
        for v in (1, 1, 1, 64, 1, 1):
            a.scalar("i64", v)
        a.scalar("i32", 0).scalar("pvoid", None).scalar("i32", 0).scalar("ppvoid", None)
        L.tao_ral_call_impl(C.c_void_p(ex), ral.mangle("ral_kernel_launch", "gpu", a.arg_codes).encode(),
                            a.pack())
        msg = C.c_char_p()
        assert L.tao_ral_last_error(C.c_void_p(ctx), C.byref(msg)) != 0
        assert b"GetFunction" in msg.value
        L.disc_ral_execution_context_destroy(C.c_void_p(ex))
    finally:
        torch.cuda.synchronize()
        L.disc_ral_context_destroy(C.c_void_p(ctx))


def test_missing_constant_is_reported(program):
    lib, d = program
    from bladedisc_amd import ral
    L = ral.lib()
    L.disc_ral_context_create_for_program.restype = C.c_void_p
    meta = str(d / "empty.metadata").encode()
    assert L.disc_ral_metadata_emit(meta, 0, None, None, None) == 0
    ctx = L.disc_ral_context_create_for_program(None, 0, None, None, None, 1, meta)
    x = torch.zeros((4, 768), device="cuda")
    ex = L.disc_ral_execution_context_create(C.c_void_p(ctx))
    L.disc_ral_execution_bind_input(C.c_void_p(ex), 0, C.c_void_p(x.data_ptr()), (C.c_int64 * 2)(4, 768), 2)
    call_impl = C.cast(L.tao_ral_call_impl, C.c_void_p).value
    lib.disc_program_main((C.c_void_p * 2)(ex, call_impl))
    msg = C.c_char_p()
    assert L.tao_ral_last_error(C.c_void_p(ctx), C.byref(msg)) != 0
    assert b"not found in metadata file" in msg.value
    L.disc_ral_execution_context_destroy(C.c_void_p(ex))
    torch.cuda.synchronize()
    L.disc_ral_context_destroy(C.c_void_p(ctx))


def test_dispatch_path_cost_per_call(program, capsys):
    """Whole path of one ral_pdll_qgemm call from compiled code (name lookup, argument
    unpacking, cached attributes, pooled allocation, launch): it must stay in the range of
    the kernel it launches, far from the reference's copy-scales-to-host-and-synchronise
    per call."""
    lib, d = program
    from bladedisc_amd import baseline_configs as cfg
    from bladedisc_amd import ral
    L = ral.lib()
    c = cfg.config1()
    names = ["w0_i8_768x768", "b0_f32_768", "sw0_f32_768", "sx0_f32_", "so0_f32_"]
    values = [hexstr(c["w_q"]), hexstr(c["bias"]), hexstr(c["sw"]),
              hexstr(np.array([c["sx"]], np.float32)), hexstr(np.array([c["so"]], np.float32))]
    meta = str(d / "loop.metadata").encode()
    n = len(names)
    assert L.disc_ral_metadata_emit(meta, n, (C.c_uint8 * n)(*([0] * n)),
                                    (C.c_char_p * n)(*[s.encode() for s in names]),
                                    (C.c_char_p * n)(*[v.encode() for v in values])) == 0
    L.disc_ral_context_create_for_program.restype = C.c_void_p
    ctx = L.disc_ral_context_create_for_program(None, 0, None, None, None, 1, meta)
    ex = L.disc_ral_execution_context_create(C.c_void_p(ctx))
    call_impl = C.cast(L.tao_ral_call_impl, C.c_void_p).value
    lib.disc_program_qgemm_loop.restype = C.c_double
    lib.disc_program_qgemm_loop.argtypes = [C.c_void_p, C.c_int64, C.c_int]
    ctx_struct = (C.c_void_p * 2)(ex, call_impl)
    try:
        report = {}
        for m in (1, 16, 256, 4096):
            lib.disc_program_qgemm_loop(ctx_struct, m, 50)            # warm the caches
            report[m] = lib.disc_program_qgemm_loop(ctx_struct, m, 2000)
        msg = C.c_char_p()
        assert L.tao_ral_last_error(C.c_void_p(ctx), C.byref(msg)) == 0, msg.value
        with capsys.disabled():
            print("\nral_pdll_qgemm from compiled code, us per call (768x768 weights):",
                  {m: round(v, 2) for m, v in report.items()})
        assert report[1] < 25 and report[16] < 25
    finally:
        L.disc_ral_execution_context_destroy(C.c_void_p(ex))
        torch.cuda.synchronize()
        L.disc_ral_context_destroy(C.c_void_p(ctx))


class _CountingAllocator:
    """Device memory for a context through the C callbacks of disc_ral_context_create, with
    every request and every return recorded (backed by torch tensors)."""

    def __init__(self):
        self.live, self.allocated, self.freed = {}, [], []
        self._alloc = C.CFUNCTYPE(C.c_void_p, C.c_size_t, C.c_void_p)(self._on_alloc)
        self._dealloc = C.CFUNCTYPE(None, C.c_void_p, C.c_void_p)(self._on_dealloc)

    def _on_alloc(self, nbytes, _user):
        t = torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device="cuda")
        self.live[t.data_ptr()] = t
        self.allocated.append(t.data_ptr())
        return t.data_ptr()

    def _on_dealloc(self, ptr, _user):
        self.freed.append(ptr)
        self.live.pop(ptr, None)


def test_inc_ref_aliases_of_inputs_and_constants_outlive_the_execution(program):
    """A compiled graph usually starts by reshaping an input and a constant (inc_ref), and
    later drops the aliases (dealloc).  Neither the caller's input nor the context's
    constant may ever reach the allocator's dealloc -- not from the program's dealloc and
    not when the execution ends -- and the constant serves the next execution intact."""
    _, d = program
    from bladedisc_amd import ral
    L = ral.lib()
    w = (np.arange(24 * 16, dtype=np.int32) % 251 - 125).astype(np.int8).reshape(24, 16)
    meta = str(d / "alias.metadata").encode()
    assert L.disc_ral_metadata_emit(meta, 1, (C.c_uint8 * 1)(0), (C.c_char_p * 1)(b"w0_i8_24x16"),
                                    (C.c_char_p * 1)(hexstr(w).encode())) == 0
    L.disc_ral_context_create_for_program.restype = C.c_void_p
    alloc = _CountingAllocator()
    stream = torch.cuda.current_stream().cuda_stream
    ctx_h = L.disc_ral_context_create_for_program(C.c_void_p(stream), 0, alloc._alloc, alloc._dealloc,
                                                  None, 1, meta)
    assert ctx_h
    name = C.create_string_buffer(b"w0_i8_24x16")
    x = torch.arange(6 * 8, dtype=torch.float32, device="cuda").reshape(6, 8)
    const_ptrs = []

    class _Ctx:                      # the little of ral.RalContext that RalExecution uses
        handle, _L, _names = ctx_h, L, {}
        _name = ral.RalContext._name
        last_error = ral.RalContext.last_error
        clear_error = ral.RalContext.clear_error

    try:
        for run in range(2):
            ex = ral.RalExecution(_Ctx())
            assert L.disc_ral_execution_bind_input(C.c_void_p(ex.handle), 0, C.c_void_p(x.data_ptr()),
                                                   (C.c_int64 * 2)(6, 8), 2) == 0
            # the constant, as a [24, 16] memref
            a = ex.new_args().scalar("pvoid", C.addressof(name)).scalar("i32", 0)
            cst = a.result_memref("i8", 2)
            ex.call("ral_const", "gpu", a)
            const_ptrs.append(cst.data)
            # reshape it to [384] and the input to [48] (inc_ref with a host shape operand)
            a = ex.new_args().memref("i8", cst.data, [24, 16]).host_array(np.array([384], np.int64))
            flat_w = a.result_memref("i8", 1)
            ex.call("inc_ref", "gpu", a)
            a = ex.new_args().memref("f32", x.data_ptr(), [6, 8]).host_array(np.array([48], np.int64))
            flat_x = a.result_memref("f32", 1)
            ex.call("inc_ref", "gpu", a)
            assert flat_w.data == cst.data and flat_x.data == x.data_ptr()
            assert flat_w.sizes[0] == 384 and flat_x.sizes[0] == 48
            # a buffer of the program's own, never handed back: returns with the execution
            own = ex.alloc(1000)
            if run == 0:
                ex.dealloc(flat_w.data)      # the program drops its aliases ...
                ex.dealloc(flat_x.data)
            ex.sync()                        # ... or (second run) leaves them to the end
            got = ral.device_view(cst.data, (24, 16), torch.int8).cpu().numpy()
            np.testing.assert_array_equal(got, w)
            ex.close()
            assert own in alloc.freed
            assert x.data_ptr() not in alloc.freed
            assert not set(const_ptrs) & set(alloc.freed)
        assert const_ptrs[0] == const_ptrs[1]      # served from the context's store
    finally:
        torch.cuda.synchronize()
        L.disc_ral_context_destroy(C.c_void_p(ctx_h))
    # the context returns its constants when it goes, and only then
    assert const_ptrs[0] in alloc.freed
    assert x.data_ptr() not in alloc.freed


def test_memset_service_inside_a_captured_graph():
    """ral_gpu_memset is a kernel launch, so an execution captured into a HIP graph can
    contain it: every replay clears the buffer again (odd sizes and alignments included),
    with the program's own eager work between replays."""
    from bladedisc_amd import ral
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        ctx = ral.RalContext(stream=side.cuda_stream)
        buf = torch.full((4099,), 7, dtype=torch.uint8, device="cuda")
        graph = torch.cuda.CUDAGraph()
        with ctx.execution() as ex:
            def memset(ptr, value, nbytes):
                a = ex.new_args().scalar("pvoid", ptr).scalar("i32", value).scalar("i64", nbytes)
                ex.call("ral_gpu_memset", "gpu", a)
            memset(buf.data_ptr() + 3, 0x5a, 4090)          # eager, unaligned head and tail
            side.synchronize()
            want = np.full(4099, 7, np.uint8)
            want[3:4093] = 0x5a
            np.testing.assert_array_equal(buf.cpu().numpy(), want)
            with torch.cuda.graph(graph, stream=side):
                memset(buf.data_ptr() + 1, 0, 4097)
                memset(buf.data_ptr() + 64, 0xff, 16)
            want[1:4098] = 0
            want[64:80] = 0xff
            for rep in range(4):
                buf.fill_(9 + rep)                           # eager work between the replays
                want[0] = want[4098] = 9 + rep
                graph.replay()
                side.synchronize()
                np.testing.assert_array_equal(buf.cpu().numpy(), want, err_msg="replay %d" % rep)
        ctx.close()
