"""Host-side mirror of the RAL calling convention, for tests and the benchmark.

It does what code emitted by the DISC compiler does: build the mangled symbol
``name___device___argcodes___retcodes`` (reference: disc/transforms/disc_to_llvm.cc
:117-168), pack every scalar into its own slot of a ``void**`` with each memref
expanded to ``basePtr, data, offset, sizes[N], strides[N]`` and one trailing slot
per result (:302-365), and call ``tao_ral_call_impl(exec_ctx, name, args)``.
"""
import ctypes as C

from . import _lib

_SCALAR_CODES = {
    "i1": C.c_bool, "i8": C.c_int8, "ui8": C.c_uint8, "i32": C.c_int32,
    "i64": C.c_int64, "f32": C.c_float, "f64": C.c_double, "pvoid": C.c_void_p,
    "ppvoid": C.c_void_p,
}

_TORCH_CODES = None
_BLOBS = {}


def _torch_code(dtype):
    global _TORCH_CODES
    if _TORCH_CODES is None:
        import torch
        _TORCH_CODES = {torch.int8: "i8", torch.uint8: "ui8", torch.int32: "i32",
                        torch.int64: "i64", torch.float32: "f32", torch.float64: "f64",
                        torch.bool: "i1", torch.float16: "f16", torch.bfloat16: "bf16",
                        torch.int16: "i16"}
    return _TORCH_CODES[dtype]


def mangle(name, device, arg_codes, ret_codes=()):
    """The symbol the compiler emits for a dispatch op."""
    return "%s___%s___%s___%s" % (name, device, "_".join(arg_codes),
                                  "_".join(ret_codes) if ret_codes else "void")


def memref_struct(rank):
    """ctypes layout of MemRefType<T, rank> (reference: ral/ral_helper.h:46-60)."""
    fields = [("basePtr", C.c_void_p), ("data", C.c_void_p), ("offset", C.c_int64)]
    if rank > 0:
        fields += [("sizes", C.c_int64 * rank), ("strides", C.c_int64 * rank)]
    return type("MemRef%d" % rank, (C.Structure,), {"_fields_": fields})


class Args:
    """Builds the packed ``void**`` of one call and remembers the type codes."""

    def __init__(self):
        self._keep = []      # ctypes objects the slots point at
        self._slots = []     # addresses
        self.arg_codes = []
        self.ret_codes = []
        self._results = []   # (struct instance, code)

    def _slot(self, obj):
        self._keep.append(obj)
        self._slots.append(C.addressof(obj))

    def scalar(self, code, value):
        ctype = _SCALAR_CODES[code]
        self._slot(ctype(value))
        self.arg_codes.append(code)
        return self

    def ctx(self, exec_ctx):
        return self.scalar("pvoid", exec_ctx)

    def memref(self, code, data_ptr, sizes, strides=None):
        """A memref of element code `code` (e.g. "i8") over `data_ptr`."""
        sizes = [int(s) for s in sizes]
        if strides is None:
            strides, acc = [], 1
            for s in reversed(sizes):
                strides.insert(0, acc)
                acc *= s
        self._slot(C.c_void_p(data_ptr))
        self._slot(C.c_void_p(data_ptr))
        self._slot(C.c_int64(0))
        for s in sizes:
            self._slot(C.c_int64(s))
        for s in strides:
            self._slot(C.c_int64(int(s)))
        self.arg_codes.append("m%dd%s" % (len(sizes), code))
        return self

    def tensor(self, t, rank0=False):
        """A torch tensor (device or host) as a memref; rank0=True passes a
        one-element tensor as a rank-0 memref."""
        if rank0:
            return self.memref(_torch_code(t.dtype), t.data_ptr(), [])
        return self.memref(_torch_code(t.dtype), t.data_ptr(), list(t.shape),
                           list(t.stride()))

    def host_array(self, arr, rank0=False):
        """A numpy array kept alive by the pack, passed as a host memref."""
        import numpy as np
        codes = {np.dtype(np.int32): "i32", np.dtype(np.float32): "f32",
                 np.dtype(np.int8): "i8", np.dtype(np.int64): "i64"}
        arr = np.ascontiguousarray(arr)
        self._keep.append(arr)
        return self.memref(codes[arr.dtype], arr.ctypes.data,
                           [] if rank0 else list(arr.shape))

    def blob(self, data):
        """The serialized custom_attrs of a ral_pdll_* call (NUL appended, as the
        compiler does)."""
        # The runtime caches parsed attrs by blob address (blobs are constants of
        # a compiled program), so equal blobs share one never-freed buffer here.
        key = bytes(data)
        buf = _BLOBS.get(key)
        if buf is None:
            buf = _BLOBS[key] = C.create_string_buffer(key + b"\0")
        self._slot(C.c_void_p(C.addressof(buf)))
        self.arg_codes.append("pvoid")
        return self

    def result_memref(self, code, rank):
        st = memref_struct(rank)()
        self._results.append(st)
        self.ret_codes.append("m%dd%s" % (rank, code))
        return st

    def result_scalar(self, code):
        obj = _SCALAR_CODES[code]()
        self._results.append(obj)
        self.ret_codes.append(code)
        return obj

    def pack(self):
        addrs = list(self._slots) + [C.addressof(r) for r in self._results]
        arr = (C.c_void_p * max(len(addrs), 1))(*addrs)
        self._keep.append(arr)
        return arr


def _bind(L):
    if getattr(L, "_ral_bound", False):
        return
    VP = C.c_void_p
    L.tao_ral_call_impl.restype = None
    L.tao_ral_call_impl.argtypes = [VP, C.c_char_p, C.POINTER(VP)]
    L.tao_ral_last_error.restype = C.c_int32
    L.tao_ral_last_error.argtypes = [VP, C.POINTER(C.c_char_p)]
    L.tao_ral_clear_error.restype = None
    L.tao_ral_clear_error.argtypes = [VP]
    L.disc_ral_context_create.restype = VP
    L.disc_ral_context_create.argtypes = [VP, C.c_int, VP, VP, VP, C.c_int]
    L.disc_ral_context_destroy.restype = None
    L.disc_ral_context_destroy.argtypes = [VP]
    L.disc_ral_execution_context_create.restype = VP
    L.disc_ral_execution_context_create.argtypes = [VP]
    L.disc_ral_execution_context_destroy.restype = None
    L.disc_ral_execution_context_destroy.argtypes = [VP]
    L.disc_ral_execution_context_get_context.restype = VP
    L.disc_ral_execution_context_get_context.argtypes = [VP]
    L.disc_ral_api_count.restype = C.c_int
    L.disc_ral_api_name.restype = C.c_char_p
    L.disc_ral_api_name.argtypes = [C.c_int]
    L.disc_ral_api_exists.restype = C.c_int
    L.disc_ral_api_exists.argtypes = [C.c_char_p]
    L._ral_bound = True


def lib():
    L = _lib.lib()
    _bind(L)
    return L


def registered_names():
    L = lib()
    return [L.disc_ral_api_name(i).decode() for i in range(L.disc_ral_api_count())]


def api_exists(name):
    return bool(lib().disc_ral_api_exists(name.encode()))


class RalError(RuntimeError):
    pass


class RalContext:
    """A RAL Context on the current device, bound to one HIP stream."""

    def __init__(self, stream=0, device_ordinal=0, cache_workspace=True):
        self._L = lib()
        self.handle = self._L.disc_ral_context_create(C.c_void_p(stream), device_ordinal,
                                                      None, None, None, int(cache_workspace))
        if not self.handle:
            raise RalError("disc_ral_context_create failed")
        self._names = {}   # keep name buffers alive: lookups are cached by pointer

    def close(self):
        if self.handle:
            self._L.disc_ral_context_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def last_error(self):
        msg = C.c_char_p()
        st = self._L.tao_ral_last_error(self.handle, C.byref(msg))
        return st, (msg.value or b"").decode()

    def clear_error(self):
        self._L.tao_ral_clear_error(self.handle)

    def execution(self):
        return RalExecution(self)

    def _name(self, s):
        buf = self._names.get(s)
        if buf is None:
            buf = C.create_string_buffer(s.encode())
            self._names[s] = buf
        return buf


class RalExecution:
    """One run: owns an ExecutionContext; `call` raises RalError on failure."""

    def __init__(self, ctx):
        self.ctx = ctx
        self._L = ctx._L
        self.handle = self._L.disc_ral_execution_context_create(ctx.handle)
        if not self.handle:
            raise RalError("disc_ral_execution_context_create failed")

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def close(self):
        if self.handle:
            self._L.disc_ral_execution_context_destroy(self.handle)
            self.handle = None

    def new_args(self):
        """Args pre-filled with the two leading operands every kernel entry takes:
        the execution context and stream handle 0."""
        return Args().ctx(self.handle).scalar("pvoid", 0)

    def call(self, name, device, args, check=True):
        full = mangle(name, device, args.arg_codes, args.ret_codes)
        packed = args.pack()
        self._L.tao_ral_call_impl(self.handle, self.ctx._name(full),
                                  C.cast(packed, C.POINTER(C.c_void_p)))
        if check:
            st, msg = self.ctx.last_error()
            if st != 0:
                self.ctx.clear_error()
                raise RalError(msg)
        return full

    # -- driver services, called the way compiled code calls them -----------
    def alloc(self, nbytes):
        a = Args().ctx(self.handle).scalar("i64", nbytes)
        r = a.result_scalar("pvoid")
        self.call("alloc", "gpu", a)
        return r.value

    def dealloc(self, ptr):
        a = Args().ctx(self.handle).scalar("pvoid", ptr)
        self.call("dealloc", "gpu", a)

    def alloc_persistent(self, nbytes):
        """Device memory that outlives executions and goes with the context, as a program's
        constants do."""
        a = Args().ctx(self.handle).scalar("i64", nbytes)
        r = a.result_scalar("pvoid")
        self.call("ral_gpu_alloc_persistent", "gpu", a)
        return r.value

    def sync(self):
        a = Args().ctx(self.handle).scalar("pvoid", 0)
        self.call("sync_on_stream", "gpu", a)


# ---------------------------------------------------------------- custom_attrs
def _s(b):
    return C.c_int64(len(b)).value.to_bytes(8, "little", signed=True) + b


def encode_attr(value):
    """Serialises a Python value the way the compiler serialises custom_attrs
    (reference: disc/transforms/disc_lower_to_library_call.cc:684-848)."""
    import struct
    if isinstance(value, dict):
        out = _s(b"dict") + struct.pack("<q", len(value))
        for k, v in value.items():
            out += _s(k.encode()) + encode_attr(v)
        return out
    if isinstance(value, bool):
        return _s(b"bool") + struct.pack("<?", value)
    if isinstance(value, int):
        return _s(b"int") + struct.pack("<q", value)
    if isinstance(value, float):
        return _s(b"float") + struct.pack("<d", value)
    if isinstance(value, str):
        return _s(b"str") + _s(value.encode())
    if isinstance(value, (list, tuple)):
        if all(isinstance(v, int) and not isinstance(v, bool) for v in value):
            return _s(b"intArray") + struct.pack("<q", len(value)) + b"".join(
                struct.pack("<q", v) for v in value)
        return _s(b"array") + struct.pack("<q", len(value)) + b"".join(
            encode_attr(v) for v in value)
    raise TypeError("cannot serialise %r" % (value,))


def device_view(ptr, shape, dtype, device="cuda"):
    """A torch tensor over `ptr` (device memory owned by someone else), no copy."""
    import torch
    typestr = {torch.int8: "|i1", torch.uint8: "|u1", torch.float32: "<f4", torch.int32: "<i4"}[dtype]

    class _Holder:
        pass

    h = _Holder()
    h.__cuda_array_interface__ = {"shape": tuple(int(s) for s in shape), "typestr": typestr,
                                  "data": (int(ptr), False), "version": 2}
    return torch.as_tensor(h, device=device)


def memref_to_tensor(st, dtype, device="cuda"):
    """Wraps a result memref (callee-allocated device buffer) as a torch tensor
    without copying.  The buffer stays owned by the execution context."""
    import torch
    rank = len(st.sizes) if hasattr(st, "sizes") else 0
    sizes = [st.sizes[i] for i in range(rank)]
    n = 1
    for s in sizes:
        n *= s
    if n == 0 or not st.data:
        return torch.empty(sizes, dtype=dtype, device=device)
    itemsize = torch.empty((), dtype=dtype).element_size()

    class _Holder:
        pass

    h = _Holder()
    h.__cuda_array_interface__ = {
        "shape": tuple(sizes),
        "typestr": "<i4" if dtype == torch.int32 else {1: "|i1", 2: "<f2", 4: "<f4"}[itemsize],
        "data": (int(st.data), False), "version": 2,
    }
    return torch.as_tensor(h, device=device)
