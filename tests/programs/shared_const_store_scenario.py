"""Two contexts of one process made from the same metadata file (run as a script by
tests/test_gpu_program.py, because DISC_USE_GLOBAL_CONST_STORE is read once per process).

  context A runs the program (constants materialised), the metadata file is deleted,
  context B is created and runs, A is destroyed, B runs again, B is destroyed.

With the process-level constant store B finds the constants A loaded, and they outlive A.
Without it B has no metadata to load from and its first run reports the missing constant:
exit code 3.  Usage: shared_const_store_scenario.py <libqlinear_program.so> <work dir>"""
import ctypes as C
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle as O  # noqa: E402
from bladedisc_amd import baseline_configs as cfg  # noqa: E402
from bladedisc_amd import ral  # noqa: E402


def main():
    lib = C.CDLL(sys.argv[1])
    work = sys.argv[2]
    L = ral.lib()
    c = cfg.config1()
    hexstr = lambda a: np.ascontiguousarray(a).tobytes().hex()  # noqa: E731
    names = ["w0_i8_768x768", "b0_f32_768", "sw0_f32_768", "sx0_f32_", "so0_f32_", "z0_i32_"]
    values = [hexstr(c["w_q"]), hexstr(c["bias"]), hexstr(c["sw"]),
              hexstr(np.array([c["sx"]], np.float32)), hexstr(np.array([c["so"]], np.float32)),
              hexstr(np.array([0], np.int32))]
    meta = os.path.join(work, "shared.metadata").encode()
    n = len(names)
    L.disc_ral_metadata_emit.restype = C.c_int
    assert L.disc_ral_metadata_emit(meta, n, (C.c_uint8 * n)(*([0] * n)),
                                    (C.c_char_p * n)(*[s.encode() for s in names]),
                                    (C.c_char_p * n)(*[v.encode() for v in values])) == 0
    L.disc_ral_context_create_for_program.restype = C.c_void_p
    L.disc_ral_execution_take_output.restype = C.c_void_p
    L.disc_ral_output_data.restype = C.c_void_p
    stream = torch.cuda.current_stream().cuda_stream
    call_impl = C.cast(L.tao_ral_call_impl, C.c_void_p).value

    def create():
        ctx = L.disc_ral_context_create_for_program(C.c_void_p(stream), 0, None, None, None, 1, meta)
        assert ctx
        return ctx

    def run(ctx, m):
        x = torch.from_numpy(np.ascontiguousarray(c["x"][:m])).cuda()
        ex = L.disc_ral_execution_context_create(C.c_void_p(ctx))
        assert L.disc_ral_execution_bind_input(C.c_void_p(ex), 0, C.c_void_p(x.data_ptr()),
                                               (C.c_int64 * 2)(m, 768), 2) == 0
        lib.disc_program_main((C.c_void_p * 2)(ex, call_impl))
        msg = C.c_char_p()
        if L.tao_ral_last_error(C.c_void_p(ctx), C.byref(msg)) != 0:
            print("runtime error:", msg.value.decode(), flush=True)
            L.disc_ral_execution_context_destroy(C.c_void_p(ex))
            return False
        out = L.disc_ral_execution_take_output(C.c_void_p(ex), 0)
        fwd = L.disc_ral_execution_take_output(C.c_void_p(ex), 1)
        torch.cuda.synchronize()
        y = ral.device_view(L.disc_ral_output_data(C.c_void_p(out)), (m, 768),
                            torch.float32).cpu().numpy()
        xq = O.quantize(c["x"][:m], c["sx"], 0)
        acc = O.gemm_s32(xq, c["w_q"], tp_b=True)
        b32 = O.bias_f32_to_s32(c["bias"], float(c["sx"]), c["sw"])
        yq = O.requant_cpu(acc, float(c["sx"]), c["sw"], float(c["so"]), b32=b32)
        np.testing.assert_array_equal(y, O.dequantize(yq, c["so"], 0))
        L.disc_ral_output_destroy(C.c_void_p(out))
        L.disc_ral_output_destroy(C.c_void_p(fwd))
        L.disc_ral_execution_context_destroy(C.c_void_p(ex))
        return True

    def alias_of_a_constant(ctx_h):
        """inc_ref (a reshape) of a constant, then dealloc of the alias, as compiled graphs do:
        a constant of the process-level store must count as persistent although no context's
        allocator made it."""
        class _Ctx:                      # the little of ral.RalContext that RalExecution uses
            handle, _L, _names = ctx_h, L, {}
            _name = ral.RalContext._name
            last_error = ral.RalContext.last_error
            clear_error = ral.RalContext.clear_error

        ex = ral.RalExecution(_Ctx())
        name = C.create_string_buffer(b"b0_f32_768")
        a = ex.new_args().scalar("pvoid", C.addressof(name)).scalar("i32", 1)
        cst = a.result_memref("f32", 1)
        ex.call("ral_const", "gpu", a)
        a = ex.new_args().memref("f32", cst.data, [768]).host_array(np.array([2, 384], np.int64))
        alias = a.result_memref("f32", 2)
        ex.call("inc_ref", "gpu", a)
        assert alias.data == cst.data and [alias.sizes[0], alias.sizes[1]] == [2, 384]
        ex.dealloc(alias.data)
        ex.sync()
        got = ral.device_view(cst.data, (768,), torch.float32).cpu().numpy()
        np.testing.assert_array_equal(got, c["bias"])
        ex.close()

    a = create()
    assert run(a, 8)
    alias_of_a_constant(a)
    assert run(a, 8)                      # the constant is intact after its alias was dropped
    os.remove(meta)                       # from here on only an already loaded store can serve
    b = L.disc_ral_context_create_for_program(C.c_void_p(stream), 0, None, None, None, 1, meta)
    if not b or not run(b, 5):
        print("context B could not get its constants", flush=True)
        return 3
    torch.cuda.synchronize()
    L.disc_ral_context_destroy(C.c_void_p(a))
    assert run(b, 16)                     # the constants outlive the context that loaded them
    torch.cuda.synchronize()
    L.disc_ral_context_destroy(C.c_void_p(b))
    c2 = None
    try:                                  # the last user released the store: nothing left to serve
        c2 = L.disc_ral_context_create_for_program(C.c_void_p(stream), 0, None, None, None, 1, meta)
        ok = bool(c2) and run(c2, 4)
    finally:
        if c2:
            L.disc_ral_context_destroy(C.c_void_p(c2))
    if ok:
        print("a store outlived its last context", flush=True)
        return 4
    print("OK", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
