"""A small XLA-FFI host in Python: builds ``XLA_FFI_CallFrame`` structs with ctypes and calls
the library's handlers the way ``CustomCallThunk`` does
(xla/backends/gpu/runtime/custom_call_thunk.cc:110-157,394-422), including the function
table (``XLA_FFI_Api``) a handler calls back into for errors and for the stream.

Struct layouts restate xla/ffi/api/c_api.h (same field order as include/xla_ffi_abi.h).
Device memory and streams come from the caller (torch tensors' ``data_ptr()`` and
``torch.cuda.current_stream().cuda_stream``); nothing here touches the GPU itself.
"""
import ctypes as C
import os

from . import dtypes

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
LIB_PATH = os.path.join(_LIB_DIR, "libxla_amd_quant.so")

HANDLER_SYMBOLS = {
    "xla_amd.dequant_dot": "xla_amd_dequant_dot",
    "xla_amd.fp8_scaled_dot": "xla_amd_fp8_scaled_dot",
    "xla_amd.rowwise_quantize_fp8": "xla_amd_rowwise_quantize_fp8",
}
EXPORTED_SYMBOLS = list(HANDLER_SYMBOLS.values()) + [
    "xla_amd_register_handlers", "xla_amd_launch_dequant_dot", "xla_amd_launch_dequant_dot_static_scratch",
    "xla_amd_launch_fp8_scaled_dot",
    "xla_amd_launch_rowwise_quantize_fp8", "xla_amd_dequant_dot_workspace_bytes", "xla_amd_dequant_dot_workspace_bytes_nk",
    "xla_amd_fp8_scaled_dot_workspace_bytes", "xla_amd_fp8_scaled_dot_workspace_bytes_typed", "xla_amd_last_error",
    "xla_amd_last_kernel",
    "xla_amd_debug_set_option"]
SELFCHECK_SYMBOLS = ["xla_amd_selfcheck_tanh_division_mismatches", "xla_amd_selfcheck_stream",
                     "xla_amd_selfcheck_launch_empty"]

STAGE_INSTANTIATE, STAGE_PREPARE, STAGE_INITIALIZE, STAGE_EXECUTE, STAGE_RECORD = range(5)
ATTR_ARRAY, ATTR_DICTIONARY, ATTR_SCALAR, ATTR_STRING = 1, 2, 3, 4
ERROR_CODES = {0: "OK", 3: "INVALID_ARGUMENT", 9: "FAILED_PRECONDITION", 12: "UNIMPLEMENTED",
               13: "INTERNAL"}
TRAIT_COMMAND_BUFFER_COMPATIBLE = 1


class Extension(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("type", C.c_int), ("next", C.c_void_p)]


class ApiVersion(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p),
                ("major_version", C.c_int), ("minor_version", C.c_int)]


class ErrorCreateArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p),
                ("message", C.c_char_p), ("errc", C.c_int)]


class Buffer(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("dtype", C.c_int),
                ("data", C.c_void_p), ("rank", C.c_int64), ("dims", C.POINTER(C.c_int64))]


class ByteSpan(C.Structure):
    _fields_ = [("ptr", C.c_char_p), ("len", C.c_size_t)]


class Scalar(C.Structure):
    _fields_ = [("dtype", C.c_int), ("value", C.c_void_p)]


class Array(C.Structure):
    _fields_ = [("dtype", C.c_int), ("size", C.c_size_t), ("data", C.c_void_p)]


class Args(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("size", C.c_int64),
                ("types", C.POINTER(C.c_int)), ("args", C.POINTER(C.c_void_p))]


class Attrs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("size", C.c_int64),
                ("types", C.POINTER(C.c_int)), ("names", C.POINTER(C.POINTER(ByteSpan))),
                ("attrs", C.POINTER(C.c_void_p))]


class CallFrame(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("api", C.c_void_p),
                ("ctx", C.c_void_p), ("stage", C.c_int), ("args", Args), ("rets", Args),
                ("attrs", Attrs), ("future", C.c_void_p)]


CALL_FRAME_STRUCT_SIZE = CallFrame.attrs.offset + C.sizeof(Attrs)


class StreamGetArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("ctx", C.c_void_p),
                ("stream", C.c_void_p)]


class RegisterArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("name", ByteSpan),
                ("platform", ByteSpan), ("instantiate", C.c_void_p), ("prepare", C.c_void_p),
                ("initialize", C.c_void_p), ("execute", C.c_void_p), ("record", C.c_void_p),
                ("traits", C.c_uint32)]


class Metadata(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("api_version", ApiVersion), ("traits", C.c_uint32),
                ("state_type_id", C.c_int64)]


class MetadataExtension(C.Structure):
    _fields_ = [("base", Extension), ("metadata", C.POINTER(Metadata))]


_FN = C.CFUNCTYPE(C.c_void_p, C.c_void_p)
_API_SLOTS = ["Error_Create", "Error_GetDetails", "Error_Destroy", "Handler_Register", "Stream_Get",
              "Type_Register", "InvokeContext_Get", "State_Set", "State_Get",
              "DeviceMemory_Allocate", "DeviceMemory_Free", "ThreadPool_Schedule",
              "ThreadPool_NumThreads", "Future_Create", "Future_SetAvailable", "Future_SetError",
              "RunId_Get", "DeviceOrdinal_Get", "InvokeContext_FindExtension"]


class Api(C.Structure):
    _fields_ = ([("struct_size", C.c_size_t), ("extension_start", C.c_void_p),
                 ("api_version", ApiVersion), ("internal_api", C.c_void_p)] +
                [(n, _FN) for n in _API_SLOTS])


class FfiError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("%s: %s" % (ERROR_CODES.get(code, code), message))
        self.code = code
        self.message = message


class Host:
    """Owns the function table; one per process is enough.  ``stream`` is the hipStream_t
    (an int) handed to handlers through XLA_FFI_Stream_Get."""

    def __init__(self, stream=0, fail_stream_get=False):
        self.stream = stream
        self.fail_stream_get = fail_stream_get
        self.errors = {}
        self.registry = {}
        self._next_error = 1
        self._keep = []
        api = Api()
        api.struct_size = Api.InvokeContext_FindExtension.offset + C.sizeof(_FN)
        api.api_version = ApiVersion(C.sizeof(ApiVersion), None, 0, 4)

        def error_create(p):
            a = C.cast(p, C.POINTER(ErrorCreateArgs)).contents
            h = self._next_error
            self._next_error += 1
            self.errors[h] = (a.errc, a.message.decode())
            return h

        def stream_get(p):
            a = C.cast(p, C.POINTER(StreamGetArgs)).contents
            if self.fail_stream_get:
                h = self._next_error
                self._next_error += 1
                self.errors[h] = (3, "XLA FFI GPU context is not available")
                return h
            a.stream = self.stream
            return None

        def handler_register(p):
            a = C.cast(p, C.POINTER(RegisterArgs)).contents
            name = C.string_at(a.name.ptr, a.name.len).decode()
            platform = C.string_at(a.platform.ptr, a.platform.len).decode()
            self.registry[(name, platform.lower())] = (a.execute, a.traits)
            return None

        def unimplemented(p):
            h = self._next_error
            self._next_error += 1
            self.errors[h] = (12, "not implemented by this host")
            return h

        table = {"Error_Create": error_create, "Stream_Get": stream_get,
                 "Handler_Register": handler_register}
        for n in _API_SLOTS:
            cb = _FN(table.get(n, unimplemented))
            self._keep.append(cb)
            setattr(api, n, cb)
        self.api = api

    def take_error(self, handle):
        return self.errors.pop(handle)

    def api_address(self):
        return C.addressof(self.api)

    def ctx(self):
        return 0xC0FFEE


class NativeHost:
    """The same services implemented in C++ (libxla_amd_host.so): no Python runs between a
    handler and its function table, so replays are not slowed down by callbacks."""

    def __init__(self, stream=0):
        L = host_library()
        self._h = L.xla_amd_host_create()
        self.stream = stream

    @property
    def stream(self):
        return self._stream

    @stream.setter
    def stream(self, value):
        self._stream = value
        host_library().xla_amd_host_set_stream(self._h, value)

    def api_address(self):
        return host_library().xla_amd_host_api(self._h)

    def ctx(self):
        return self._h

    def take_error(self, handle):
        buf = C.create_string_buffer(4096)
        code = host_library().xla_amd_host_take_error(handle, buf, len(buf))
        return code, buf.value.decode()

    def register(self, register_symbol="xla_amd_register_handlers"):
        fn = C.cast(getattr(library(), register_symbol), C.c_void_p)
        err = host_library().xla_amd_host_register(self._h, fn)
        if err:
            raise FfiError(*self.take_error(err))

    def set_recording(self, on):
        """While on, frames of this host carry a record extension (what XLA attaches while it records
        a command buffer).  Returns how many times a handler has asked for stream capture so far."""
        return host_library().xla_amd_host_set_recording(self._h, int(bool(on)))

    def find_handler(self, target, platform="rocm"):
        return host_library().xla_amd_host_find_handler(self._h, target.encode(), platform.encode())


class LaunchDequantDot(C.Structure):
    """XlaAmdDequantDot of include/xla_amd_quant.h (the launcher layer below the handlers)."""
    _fields_ = [("lhs", C.c_void_p), ("weights", C.c_void_p), ("scales", C.c_void_p), ("bias", C.c_void_p),
                ("out", C.c_void_p), ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
                ("batch", C.c_int64), ("M", C.c_int64), ("K", C.c_int64), ("N", C.c_int64),
                ("group", C.c_int64), ("scale_batch", C.c_int64), ("weight_dtype", C.c_int32),
                ("scale_dtype", C.c_int32), ("bias_dtype", C.c_int32), ("dequant_type", C.c_int32),
                ("dot_type", C.c_int32), ("epilogue_type", C.c_int32), ("epilogue", C.c_int32),
                ("zero_points", C.c_void_p), ("group_sizes", C.c_void_p), ("group_sizes_dtype", C.c_int32),
                ("rhs_contracting_dim", C.c_int32), ("out_dtype", C.c_int32), ("out_transposed", C.c_int32),
                ("lhs_k_major", C.c_int32), ("d_scale", C.c_void_p), ("d_scale_multiplies", C.c_int32)]


_lib = None


def library():
    """The HIP library, loaded once.  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: run `python -m xla_amd.build` (hipcc, gfx950); "
                               "this package has no CPU fallback" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        for sym in HANDLER_SYMBOLS.values():
            fn = getattr(L, sym)
            fn.restype = C.c_void_p
            fn.argtypes = [C.c_void_p]
        L.xla_amd_register_handlers.restype = C.c_void_p
        L.xla_amd_register_handlers.argtypes = [C.c_void_p]
        L.xla_amd_last_error.restype = C.c_char_p
        L.xla_amd_last_kernel.restype = C.c_char_p
        L.xla_amd_debug_set_option.argtypes = [C.c_char_p, C.c_int]
        L.xla_amd_dequant_dot_workspace_bytes.restype = C.c_size_t
        L.xla_amd_dequant_dot_workspace_bytes.argtypes = [C.c_int64] * 4 + [C.c_int32]
        L.xla_amd_dequant_dot_workspace_bytes_nk.restype = C.c_size_t
        L.xla_amd_dequant_dot_workspace_bytes_nk.argtypes = [C.c_int64] * 4 + [C.c_int32]
        for sym in ("xla_amd_launch_dequant_dot", "xla_amd_launch_dequant_dot_static_scratch"):
            getattr(L, sym).restype = C.c_int
            getattr(L, sym).argtypes = [C.POINTER(LaunchDequantDot), C.c_void_p]
        L.xla_amd_fp8_scaled_dot_workspace_bytes.restype = C.c_size_t
        L.xla_amd_fp8_scaled_dot_workspace_bytes.argtypes = [C.c_int64] * 3 + [C.c_int32]
        L.xla_amd_fp8_scaled_dot_workspace_bytes_typed.restype = C.c_size_t
        L.xla_amd_fp8_scaled_dot_workspace_bytes_typed.argtypes = [C.c_int64] * 3 + [C.c_int32] * 2
        _lib = L
    return _lib


def _buffer(dtype, data_ptr, dims):
    dims = list(dims)
    arr = (C.c_int64 * max(len(dims), 1))(*dims)
    b = Buffer(C.sizeof(Buffer), None, dtype, data_ptr, len(dims), C.cast(arr, C.POINTER(C.c_int64)))
    return b, arr


_SCALAR_CTYPES = {dtypes.PRED: C.c_bool, dtypes.S8: C.c_int8, dtypes.S16: C.c_int16,
                  dtypes.S32: C.c_int32, dtypes.S64: C.c_int64, dtypes.U8: C.c_uint8,
                  dtypes.U32: C.c_uint32, dtypes.U64: C.c_uint64, dtypes.F32: C.c_float,
                  dtypes.F64: C.c_double}


class Attr:
    """Typed attribute value: Attr.i32(3), Attr.i64(0), Attr.f32(1e-6), Attr.pred(True), Attr.str("BIAS")."""

    def __init__(self, kind, dtype, value):
        self.kind, self.dtype, self.value = kind, dtype, value

    i32 = staticmethod(lambda v: Attr(ATTR_SCALAR, dtypes.S32, int(v)))
    i64 = staticmethod(lambda v: Attr(ATTR_SCALAR, dtypes.S64, int(v)))
    f32 = staticmethod(lambda v: Attr(ATTR_SCALAR, dtypes.F32, float(v)))
    f64 = staticmethod(lambda v: Attr(ATTR_SCALAR, dtypes.F64, float(v)))
    pred = staticmethod(lambda v: Attr(ATTR_SCALAR, dtypes.PRED, bool(v)))
    str = staticmethod(lambda v: Attr(ATTR_STRING, 0, v))
    i64_array = staticmethod(lambda v: Attr(ATTR_ARRAY, dtypes.S64, list(v)))


class Frame:
    """One call frame plus everything it points at (kept alive as attributes)."""

    def __init__(self, host, args, rets, attrs=None, stage=STAGE_EXECUTE):
        """args/rets: lists of (dtype, data_ptr, dims); attrs: dict name -> Attr."""
        self.host = host
        keep = self._keep = []
        f = self.frame = CallFrame()
        f.struct_size = CALL_FRAME_STRUCT_SIZE
        f.api = host.api_address()
        f.ctx = host.ctx()
        f.stage = stage

        def fill(side, items):
            n = len(items)
            types = (C.c_int * max(n, 1))(*([1] * n))
            ptrs = (C.c_void_p * max(n, 1))()
            for i, (dt, ptr, dims) in enumerate(items):
                b, arr = _buffer(dt, ptr, dims)
                keep.extend([b, arr])
                ptrs[i] = C.addressof(b)
            side.struct_size = C.sizeof(Args)
            side.size = n
            side.types = C.cast(types, C.POINTER(C.c_int))
            side.args = C.cast(ptrs, C.POINTER(C.c_void_p))
            keep.extend([types, ptrs])

        fill(f.args, args)
        fill(f.rets, rets)
        attrs = attrs or {}
        names = sorted(attrs)                     # XLA passes attributes sorted by name
        n = len(names)
        types = (C.c_int * max(n, 1))()
        nptrs = (C.POINTER(ByteSpan) * max(n, 1))()
        vptrs = (C.c_void_p * max(n, 1))()
        for i, name in enumerate(names):
            a = attrs[name]
            raw = name.encode()
            span = ByteSpan(raw, len(raw))
            keep.extend([raw, span])
            nptrs[i] = C.pointer(span)
            types[i] = a.kind
            if a.kind == ATTR_SCALAR:
                val = _SCALAR_CTYPES[a.dtype](a.value)
                sc = Scalar(a.dtype, C.cast(C.pointer(val), C.c_void_p))
                keep.extend([val, sc])
                vptrs[i] = C.addressof(sc)
            elif a.kind == ATTR_STRING:
                sraw = a.value.encode()
                sspan = ByteSpan(sraw, len(sraw))
                keep.extend([sraw, sspan])
                vptrs[i] = C.addressof(sspan)
            else:
                data = (_SCALAR_CTYPES[a.dtype] * max(len(a.value), 1))(*a.value)
                arr = Array(a.dtype, len(a.value), C.cast(data, C.c_void_p))
                keep.extend([data, arr])
                vptrs[i] = C.addressof(arr)
        f.attrs.struct_size = C.sizeof(Attrs)
        f.attrs.size = n
        f.attrs.types = C.cast(types, C.POINTER(C.c_int))
        f.attrs.names = C.cast(nptrs, C.POINTER(C.POINTER(ByteSpan)))
        f.attrs.attrs = C.cast(vptrs, C.POINTER(C.c_void_p))
        keep.extend([types, nptrs, vptrs])

    def address(self):
        return C.addressof(self.frame)


def invoke(target, frame):
    """Calls the handler registered for ``target``; raises FfiError on a non-null result."""
    fn = getattr(library(), HANDLER_SYMBOLS[target])
    err = fn(frame.address())
    if err:
        code, msg = frame.host.take_error(err)
        raise FfiError(code, msg)


HOST_LIB_PATH = os.path.join(_LIB_DIR, "libxla_amd_host.so")
_host_lib = None


def host_library():
    """The host-only helper library (frame replay, HLO rewrite pass); no GPU code inside."""
    global _host_lib
    if _host_lib is None:
        if not os.path.exists(HOST_LIB_PATH):
            raise RuntimeError("%s is missing: run `python -m xla_amd.build host`" % HOST_LIB_PATH)
        L = C.CDLL(HOST_LIB_PATH)
        L.xla_amd_host_replay.restype = C.c_void_p
        L.xla_amd_host_replay.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64,
                                          C.POINTER(C.c_int64)]
        L.xla_amd_host_create.restype = C.c_void_p
        L.xla_amd_host_destroy.argtypes = [C.c_void_p]
        L.xla_amd_host_api.restype = C.c_void_p
        L.xla_amd_host_api.argtypes = [C.c_void_p]
        L.xla_amd_host_set_stream.argtypes = [C.c_void_p, C.c_void_p]
        L.xla_amd_host_take_error.restype = C.c_int
        L.xla_amd_host_take_error.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t]
        L.xla_amd_host_register.restype = C.c_void_p
        L.xla_amd_host_register.argtypes = [C.c_void_p, C.c_void_p]
        L.xla_amd_host_find_handler.restype = C.c_void_p
        L.xla_amd_host_find_handler.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p]
        L.xla_amd_host_set_recording.restype = C.c_int
        L.xla_amd_host_set_recording.argtypes = [C.c_void_p, C.c_int]
        L.xla_amd_host_handler_traits.restype = C.c_int64
        L.xla_amd_host_handler_traits.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p]
        _host_lib = L
    return _host_lib


class Replay:
    """A fixed sequence of (target, Frame) pairs that is re-invoked from native code, like the
    custom-call thunks of a compiled executable being run step after step."""

    def __init__(self, calls):
        self.calls = list(calls)
        n = len(self.calls)
        lib = library()
        self._handlers = (C.c_void_p * n)(*[C.cast(getattr(lib, HANDLER_SYMBOLS[t]), C.c_void_p).value
                                            for t, _ in self.calls])
        self._frames = (C.c_void_p * n)(*[f.address() for _, f in self.calls])

    def run(self, rounds=1):
        failed = C.c_int64(-1)
        err = host_library().xla_amd_host_replay(self._handlers, self._frames, len(self.calls), rounds,
                                                 C.byref(failed))
        if err:
            code, msg = self.calls[0][1].host.take_error(err)
            raise FfiError(code, "call %d: %s" % (failed.value, msg))


def query_metadata(target, host):
    """The registration-time handshake (xla/ffi/invoke.cc:218-233): returns (major, minor, traits)."""
    md = Metadata()
    md.struct_size = Metadata.traits.offset + C.sizeof(C.c_uint32)
    ext = MetadataExtension()
    ext.base.struct_size = C.sizeof(MetadataExtension)
    ext.base.type = 1
    ext.metadata = C.pointer(md)
    fr = Frame(host, [], [])
    fr.frame.extension_start = C.addressof(ext)
    invoke(target, fr)
    return md.api_version.major_version, md.api_version.minor_version, md.traits


def last_kernel():
    return library().xla_amd_last_kernel().decode()


SELFCHECK_LIB_PATH = os.path.join(_LIB_DIR, "libxla_amd_selfcheck.so")
_selfcheck_lib = None


def selfcheck_library():
    """Test and benchmark aids (exhaustive numerics checks, HBM stream yardstick, empty kernel): a
    library of their own, because unlike the product they allocate and synchronise."""
    global _selfcheck_lib
    if _selfcheck_lib is None:
        if not os.path.exists(SELFCHECK_LIB_PATH):
            raise RuntimeError("%s is missing: run `python -m xla_amd.build selfcheck`" % SELFCHECK_LIB_PATH)
        L = C.CDLL(SELFCHECK_LIB_PATH)
        L.xla_amd_selfcheck_tanh_division_mismatches.restype = C.c_longlong
        L.xla_amd_selfcheck_tanh_division_mismatches.argtypes = []
        L.xla_amd_selfcheck_stream.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        L.xla_amd_selfcheck_launch_empty.argtypes = [C.c_void_p, C.c_int, C.c_int]
        _selfcheck_lib = L
    return _selfcheck_lib


def debug_stream(dst_ptr, src_ptr, nbytes, stream):
    """Plain HBM stream (copy, or read-only with dst None) on `stream`: the benchmark's yardstick."""
    rc = selfcheck_library().xla_amd_selfcheck_stream(dst_ptr or None, src_ptr, nbytes, stream)
    if rc:
        raise RuntimeError("xla_amd_selfcheck_stream failed: %d" % rc)


def launch_empty(stream, count, workgroups=1):
    """`count` launches of a kernel that does nothing, back to back on `stream`."""
    rc = selfcheck_library().xla_amd_selfcheck_launch_empty(stream, count, workgroups)
    if rc:
        raise RuntimeError("xla_amd_selfcheck_launch_empty failed: %d" % rc)


def set_option(key, value):
    rc = library().xla_amd_debug_set_option(key.encode(), int(value))
    if rc != 0:
        raise KeyError(key)
