"""Python view of the HLO side of libxla_amd_host.so: the rewrite pass that turns the
quantized-inference patterns into this library's custom calls, and a JSON dump of a module."""
import ctypes as C
import json

from . import ffi


class _Callbacks(C.Structure):
    _fields_ = [("dequant_workspace_bytes", C.c_void_p), ("fp8_workspace_bytes", C.c_void_p),
                ("dequant_nk_workspace_bytes", C.c_void_p)]


def _lib():
    L = ffi.host_library()
    if not getattr(L, "_hlo_ready", False):
        for name in ("xla_amd_hlo_rewrite", "xla_amd_hlo_print", "xla_amd_hlo_to_json"):
            getattr(L, name).restype = C.c_void_p
        L.xla_amd_hlo_rewrite.argtypes = [C.c_char_p, C.c_void_p, C.POINTER(C.c_void_p), C.POINTER(C.c_int)]
        L.xla_amd_hlo_print.argtypes = [C.c_char_p, C.POINTER(C.c_void_p)]
        L.xla_amd_hlo_to_json.argtypes = [C.c_char_p, C.POINTER(C.c_void_p)]
        L.xla_amd_host_free.argtypes = [C.c_void_p]
        L._hlo_ready = True
    return L


def _take(L, p):
    if not p:
        return None
    s = C.string_at(p).decode()
    L.xla_amd_host_free(p)
    return s


class HloError(ValueError):
    pass


def rewrite(text, with_scratch=True):
    """Runs QuantFusionRewriter.  Returns (new_text, rewrites, refusals).  Scratch results are
    sized by the kernel library's own workspace queries when ``with_scratch``."""
    L = _lib()
    cb = None
    if with_scratch:
        q = ffi.library()
        cb = _Callbacks(C.cast(q.xla_amd_dequant_dot_workspace_bytes, C.c_void_p).value,
                        C.cast(q.xla_amd_fp8_scaled_dot_workspace_bytes_typed, C.c_void_p).value,
                        C.cast(q.xla_amd_dequant_dot_workspace_bytes_nk, C.c_void_p).value)
    log = C.c_void_p()
    n = C.c_int(0)
    out = L.xla_amd_hlo_rewrite(text.encode(), C.byref(cb) if cb else None, C.byref(log), C.byref(n))
    log_text = _take(L, log.value) or ""
    if not out:
        raise HloError(log_text)
    new_text = _take(L, out)
    lines = [l for l in log_text.splitlines() if l]
    return (new_text, [l[len("rewrite: "):] for l in lines if l.startswith("rewrite: ")],
            [l[len("refused: "):] for l in lines if l.startswith("refused: ")])


def print_module(text):
    L = _lib()
    err = C.c_void_p()
    out = L.xla_amd_hlo_print(text.encode(), C.byref(err))
    if not out:
        raise HloError(_take(L, err.value))
    return _take(L, out)


def to_json(text):
    L = _lib()
    err = C.c_void_p()
    out = L.xla_amd_hlo_to_json(text.encode(), C.byref(err))
    if not out:
        raise HloError(_take(L, err.value))
    return json.loads(_take(L, out))
