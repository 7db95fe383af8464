"""The C-ABI boundary checked against the reference's own FFI headers (xla/ffi/api/{c_api,api,ffi}.h,
header-only, compiled here with g++ from where they lie; nothing of them is copied).

* tests/ffi_ref/register_static.cc registers the library's three handlers with the real
  XLA_FFI_REGISTER_HANDLER macro; the native host's registry -- which follows
  xla/ffi/ffi_registry.cc:87-158: metadata query, API version window, traits, duplicate rule -- must
  then hold exactly those symbols.
* tests/ffi_ref/decode_frames.cc holds handlers written with the reference's Ffi::Bind() DSL; they are
  handed the very call frames xla_amd.ops builds for each custom call, so the reference's decoder
  (api.h Handler::Call) is what reads this package's frame producer.

Skipped where the reference tree or a host compiler is missing (the GPU box)."""
import ctypes as C
import os
import shutil
import subprocess

import pytest
import torch

from xla_amd import dtypes, ffi, ops

REFERENCE = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(os.path.dirname(HERE), "xla_amd", "lib")

pytestmark = pytest.mark.skipif(
    not os.path.exists(os.path.join(REFERENCE, "xla/ffi/api/api.h")) or shutil.which("g++") is None,
    reason="needs the reference's FFI headers and g++")


def _compile(tmp, source, extra=()):
    out = os.path.join(str(tmp), os.path.splitext(source)[0] + ".so")
    cmd = ["g++", "-std=c++17", "-O1", "-fPIC", "-shared", "-w", "-I" + REFERENCE,
           os.path.join(HERE, "ffi_ref", source), "-o", out, *extra]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    return out


@pytest.fixture(scope="module")
def registered(tmp_path_factory):
    ffi.library()
    ffi.host_library()          # both loaded before the object that links against them
    path = _compile(tmp_path_factory.mktemp("ffi_ref"), "register_static.cc",
                    ["-L" + LIB_DIR, "-lxla_amd_quant", "-lxla_amd_host", "-Wl,-rpath," + LIB_DIR])
    return C.CDLL(path)         # static initialisers run here


def test_reference_macro_registers_the_exported_handlers(registered):
    host = ffi.NativeHost()
    lib = ffi.library()
    for target, symbol in ffi.HANDLER_SYMBOLS.items():
        want = C.cast(getattr(lib, symbol), C.c_void_p).value
        for platform in ("ROCM", "rocm", "gpu"):      # canonicalised: platform_util.cc:64-91
            assert host.find_handler(target, platform) == want, (target, platform)
        assert host.find_handler(target, "cuda") is None
        traits = ffi.host_library().xla_amd_host_handler_traits(None, target.encode(), b"rocm")
        assert traits & 1, "command-buffer compatible (c_api.h XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE)"
    assert host.find_handler("xla_amd.no_such_call", "rocm") is None


def test_duplicate_registration_rule(registered):
    same, other = C.c_int(-1), C.c_int(-1)
    registered.register_again(C.byref(same), C.byref(other))
    assert same.value == 0                      # the same handler again: accepted
    assert other.value == 3                     # another handler under the name: INVALID_ARGUMENT
    # and the library's own dynamic registration lands on the same entries
    host = ffi.NativeHost()
    host.register()
    want = C.cast(ffi.library().xla_amd_dequant_dot, C.c_void_p).value
    assert host.find_handler("xla_amd.dequant_dot") == want


def test_registry_refuses_what_the_reference_refuses():
    """No execute stage; a handler that reports an API version outside [0.1, 0.4]."""
    host = ffi.NativeHost()
    api = C.cast(host.api_address(), C.POINTER(ffi.Api)).contents

    def register(execute, name=b"test.bad"):
        a = ffi.RegisterArgs()
        a.struct_size = C.sizeof(ffi.RegisterArgs)
        a.name = ffi.ByteSpan(name, len(name))
        a.platform = ffi.ByteSpan(b"ROCM", 4)
        a.execute = execute
        a.traits = 0
        err = api.Handler_Register(C.addressof(a))
        return host.take_error(err) if err else (0, "")

    code, msg = register(None)
    assert code == 3 and "must provide an execute implementation" in msg

    def make(major, minor):
        @ffi._FN
        def handler(p):
            frame = C.cast(p, C.POINTER(ffi.CallFrame)).contents
            ext = C.cast(frame.extension_start, C.POINTER(ffi.MetadataExtension)).contents
            ext.metadata.contents.api_version.major_version = major
            ext.metadata.contents.api_version.minor_version = minor
            return None
        return handler

    too_new, ancient, fine = make(0, 5), make(0, 0), make(0, 2)
    code, msg = register(C.cast(too_new, C.c_void_p), b"test.too_new")
    assert code == 3 and "API version (0.5) is incompatible" in msg and "(0.4)" in msg and "(0.1)" in msg
    code, msg = register(C.cast(ancient, C.c_void_p), b"test.ancient")
    assert code == 3 and "API version (0.0) is incompatible" in msg
    assert register(C.cast(fine, C.c_void_p), b"test.fine") == (0, "")
    assert host.find_handler("test.too_new") is None and host.find_handler("test.fine") is not None


# ---- the frame producer read by the reference's decoder -----------------------------------------

@pytest.fixture(scope="module")
def decoder(tmp_path_factory):
    L = C.CDLL(_compile(tmp_path_factory.mktemp("ffi_ref_decode"), "decode_frames.cc"))
    L.ref_decode_log.restype = C.c_char_p
    for name in ("ref_decode_dequant_dot", "ref_decode_dequant_dot_grouped", "ref_decode_fp8_scaled_dot",
                 "ref_decode_fp8_scaled_dot_f8_result", "ref_decode_rowwise_quantize_fp8"):
        getattr(L, name).restype = C.c_void_p
        getattr(L, name).argtypes = [C.c_void_p]
    return L


@pytest.fixture
def cpu_frames(monkeypatch):
    """xla_amd.ops builds its frames from tensor metadata only; with the device check off it does so
    for host tensors, which is all a decoder needs."""
    monkeypatch.setattr(ops, "_check_cuda", lambda *t: None)


def _buf(what, dtype, tensor_or_ptr, dims):
    ptr = tensor_or_ptr if isinstance(tensor_or_ptr, int) else tensor_or_ptr.data_ptr()
    return "%s dtype=%d dims=[%s] ptr=%d;" % (what, dtype, ",".join(str(int(d)) for d in dims), ptr)


def _decode(decoder, symbol, call):
    decoder.ref_decode_reset()
    err = getattr(decoder, symbol)(call.frame.address())
    if err:
        raise ffi.FfiError(*call.frame.host.take_error(err))
    return decoder.ref_decode_log().decode()


def test_reference_decoder_reads_dequant_dot_frames(decoder, cpu_frames):
    M, K, N, G = 3, 256, 64, 64
    lhs = torch.zeros((M, K), dtype=torch.bfloat16)
    w4 = torch.zeros((K * N // 2,), dtype=torch.uint8)
    sc = torch.zeros((K // G, N), dtype=torch.bfloat16)
    bias = torch.zeros((N,), dtype=torch.bfloat16)
    scratch = torch.zeros((128,), dtype=torch.uint8)
    call = ops.dequant_dot(lhs, w4, sc, bias, weight_dtype="s4", weight_shape=(K, N), epilogue="BIAS_SILU",
                           dequant_type="bf16", scale_group_size=G, scratch=scratch, build_only=True)
    got = _decode(decoder, "ref_decode_dequant_dot_grouped", call)
    want = (_buf("arg", dtypes.BF16, lhs, (M, K)) + _buf("arg", dtypes.S4, w4, (K, N)) +
            _buf("arg", dtypes.BF16, sc, (K // G, N)) + _buf("ret", dtypes.BF16, call.result, (M, N)) +
            _buf("arg", dtypes.BF16, bias, (N,)) + _buf("ret", dtypes.U8, scratch, (128,)) +
            "dequant_type=%d;dot_type=%d;epilogue=BIAS_SILU;epilogue_type=%d;scale_group_size=%d;"
            % (dtypes.BF16, dtypes.F32, dtypes.F32, G))
    assert got == want
    # without the optional attribute and without bias or scratch; batched s8
    lhs3 = torch.zeros((2, M, K), dtype=torch.bfloat16)
    w8 = torch.zeros((2, K, N), dtype=torch.int8)
    scf = torch.zeros((2, N), dtype=torch.float32)
    call = ops.dequant_dot(lhs3, w8, scf, None, weight_dtype="s8", dot_type="bf16", epilogue_type="bf16",
                           scratch=None, build_only=True)
    got = _decode(decoder, "ref_decode_dequant_dot", call)
    want = (_buf("arg", dtypes.BF16, lhs3, (2, M, K)) + _buf("arg", dtypes.S8, w8, (2, K, N)) +
            _buf("arg", dtypes.F32, scf, (2, N)) + _buf("ret", dtypes.BF16, call.result, (2, M, N)) +
            "dequant_type=%d;dot_type=%d;epilogue=DEFAULT;epilogue_type=%d;" % (dtypes.F32, dtypes.BF16, dtypes.BF16))
    assert got == want
    # the reference's decoder counts attributes: the grouped binding refuses a frame without its fifth
    with pytest.raises(ffi.FfiError, match="Wrong number of attributes"):
        _decode(decoder, "ref_decode_dequant_dot_grouped", call)


def test_reference_decoder_reads_fp8_scaled_dot_frames(decoder, cpu_frames):
    M, K, N = 4, 64, 32
    a = torch.zeros((M, K), dtype=torch.uint8)
    b = torch.zeros((K, N), dtype=torch.uint8)
    sa, sb = torch.zeros((), dtype=torch.float32), torch.zeros((N,), dtype=torch.float32)
    bias = torch.zeros((N,), dtype=torch.bfloat16)
    call = ops.fp8_scaled_dot(a, b, sa, sb, bias, epilogue="BIAS_GELU", scratch=None, build_only=True)
    got = _decode(decoder, "ref_decode_fp8_scaled_dot", call)
    want = (_buf("arg", dtypes.F8E4M3FN, a, (M, K)) + _buf("arg", dtypes.F8E4M3FN, b, (K, N)) +
            _buf("arg", dtypes.F32, sa, ()) + _buf("arg", dtypes.F32, sb, (N,)) +
            _buf("ret", dtypes.BF16, call.result, (M, N)) + _buf("arg", dtypes.BF16, bias, (N,)) +
            "dequant_type=%d;dot_type=%d;epilogue=BIAS_GELU;epilogue_type=%d;rhs_contracting_dim=0;"
            % (dtypes.F32, dtypes.F32, dtypes.F32))
    assert got == want
    # f8 result with its scale operand, the amax result and the extra attribute
    z = torch.zeros((), dtype=torch.float32)
    bt = torch.zeros((N, K), dtype=torch.uint8)
    call = ops.fp8_scaled_dot(a, bt, sa, sa, None, rhs_contracting_dim=1, d_scale=z, d_scale_multiplies=True,
                              amax=True, scratch=None, build_only=True)
    got = _decode(decoder, "ref_decode_fp8_scaled_dot_f8_result", call)
    out, amax = call.result
    want = (_buf("arg", dtypes.F8E4M3FN, a, (M, K)) + _buf("arg", dtypes.F8E4M3FN, bt, (N, K)) +
            _buf("arg", dtypes.F32, sa, ()) + _buf("arg", dtypes.F32, sa, ()) +
            _buf("ret", dtypes.F8E4M3FN, out, (M, N)) + _buf("arg", dtypes.F32, z, ()) +
            _buf("ret", dtypes.F32, amax, ()) +
            "dequant_type=%d;dot_type=%d;epilogue=DEFAULT;epilogue_type=%d;rhs_contracting_dim=1;d_scale_multiplies=1;"
            % (dtypes.F32, dtypes.F32, dtypes.F32))
    assert got == want


def test_reference_decoder_reads_rowwise_quantize_frames(decoder, cpu_frames):
    R, Cc = 5, 128
    x = torch.zeros((R, Cc), dtype=torch.bfloat16)
    gamma = torch.zeros((Cc,), dtype=torch.bfloat16)
    call = ops.rowwise_quantize_fp8(x, gamma, eps=0.5, build_only=True)
    q, scales = call.result
    got = _decode(decoder, "ref_decode_rowwise_quantize_fp8", call)
    want = (_buf("arg", dtypes.BF16, x, (R, Cc)) + _buf("ret", dtypes.F8E4M3FN, q, (R, Cc)) +
            _buf("ret", dtypes.F32, scales, (R,)) + _buf("arg", dtypes.BF16, gamma, (Cc,)) + "eps=0.5;rmsnorm=1;")
    assert got == want
    # a wrong attribute type is caught by the reference's decoder with its own diagnostic
    frame = ffi.Frame(ops.host(), [(dtypes.BF16, x.data_ptr(), (R, Cc))],
                      [(dtypes.F8E4M3FN, q.data_ptr(), (R, Cc)), (dtypes.F32, scales.data_ptr(), (R,))],
                      {"rmsnorm": ffi.Attr.i32(1), "eps": ffi.Attr.f32(1e-6)})
    decoder.ref_decode_reset()
    err = decoder.ref_decode_rowwise_quantize_fp8(frame.address())
    assert err
    code, msg = ops.host().take_error(err)
    assert code == 3 and "Wrong scalar data type: expected PRED but got S32" in msg
