"""The drop-in boundary without a GPU: the shared library loads, exports every symbol the
public header declares, speaks the FFI handshake, and rejects malformed call frames with the
reference binding's wording (xla/ffi/api/ffi_test.cc:869-932, api.h:2296-2424).  All of these
paths return before any HIP call, so they run on a CPU-only machine."""
import ctypes as C
import os
import re
import subprocess

import pytest

from xla_amd import dtypes, ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE = 0x1000  # never dereferenced: every test here fails before a launch


def test_library_exports_every_declared_symbol():
    lib = ffi.library()
    header = open(os.path.join(ROOT, "include", "xla_amd_quant.h")).read()
    declared = set(re.findall(r"XLA_AMD_EXPORT[^;(]*?\b(xla_amd_\w+)\s*\(", header))
    assert declared == set(ffi.EXPORTED_SYMBOLS), declared ^ set(ffi.EXPORTED_SYMBOLS)
    for sym in declared:
        assert getattr(lib, sym) is not None
    # the test and benchmark aids live in a library of their own and nowhere in the product
    header = open(os.path.join(ROOT, "include", "xla_amd_selfcheck.h")).read()
    aids = set(re.findall(r"XLA_AMD_SELFCHECK_EXPORT[^;(]*?\b(xla_amd_\w+)\s*\(", header))
    assert aids == set(ffi.SELFCHECK_SYMBOLS), aids ^ set(ffi.SELFCHECK_SYMBOLS)
    for sym in aids:
        assert getattr(ffi.selfcheck_library(), sym) is not None
        assert not hasattr(lib, sym)


def test_metadata_handshake():
    host = ffi.Host()
    for target in ffi.HANDLER_SYMBOLS:
        major, minor, traits = ffi.query_metadata(target, host)
        assert (major, minor) == (0, 4)
        assert traits & ffi.TRAIT_COMMAND_BUFFER_COMPATIBLE


def test_register_handlers_for_rocm():
    host = ffi.Host()
    err = ffi.library().xla_amd_register_handlers(C.addressof(host.api))
    assert not err
    assert set(host.registry) == {(t, "rocm") for t in ffi.HANDLER_SYMBOLS}
    for (target, _), (fn, traits) in host.registry.items():
        sym = getattr(ffi.library(), ffi.HANDLER_SYMBOLS[target])
        assert fn == C.cast(sym, C.c_void_p).value
        assert traits == ffi.TRAIT_COMMAND_BUFFER_COMPATIBLE


def quant_frame(host, x_dims=(4, 64), g_dims=(64,), q_dtype=dtypes.F8E4M3FN, attrs=None, n_rets=2, **kw):
    args = [(dtypes.BF16, FAKE, x_dims), (dtypes.BF16, FAKE, g_dims)]
    rets = [(q_dtype, FAKE, x_dims), (dtypes.F32, FAKE, (x_dims[0],))][:n_rets]
    return ffi.Frame(host, args, rets, attrs or {}, **kw)


def test_wrong_call_frame_struct_size():
    host = ffi.Host()
    fr = quant_frame(host)
    fr.frame.struct_size += 8
    with pytest.raises(ffi.FfiError, match=r"Unexpected XLA_FFI_CallFrame size: expected \d+ got \d+"):
        ffi.invoke("xla_amd.rowwise_quantize_fp8", fr)


def test_wrong_stage():
    host = ffi.Host()
    with pytest.raises(ffi.FfiError, match="Wrong execution stage: expected `execute` but got `prepare`"):
        ffi.invoke("xla_amd.rowwise_quantize_fp8", quant_frame(host, stage=ffi.STAGE_PREPARE))


def test_wrong_number_of_arguments_and_results():
    host = ffi.Host()
    fr = ffi.Frame(host, [], [(dtypes.F8E4M3FN, FAKE, (1, 1)), (dtypes.F32, FAKE, (1,))])
    with pytest.raises(ffi.FfiError, match=r"\[execute\] Wrong number of arguments: expected at least 1 but got 0"):
        ffi.invoke("xla_amd.rowwise_quantize_fp8", fr)
    with pytest.raises(ffi.FfiError, match=r"Wrong number of results: expected 2 but got 1"):
        ffi.invoke("xla_amd.rowwise_quantize_fp8", quant_frame(host, n_rets=1))
    fr = ffi.Frame(host, [(dtypes.BF16, FAKE, (2, 8))] * 2, [(dtypes.BF16, FAKE, (2, 8))])
    with pytest.raises(ffi.FfiError, match=r"Wrong number of arguments: expected at least 3 but got 2"):
        ffi.invoke("xla_amd.dequant_dot", fr)


def test_wrong_buffer_dtype_and_rank_are_diagnosed_by_position():
    host = ffi.Host()
    with pytest.raises(ffi.FfiError) as e:
        ffi.invoke("xla_amd.rowwise_quantize_fp8", quant_frame(host, q_dtype=dtypes.S32))
    assert "Failed to decode all FFI handler operands (bad operands at: 2)" in e.value.message
    assert "Wrong buffer dtype: expected F8E4M3FN but got S32" in e.value.message
    with pytest.raises(ffi.FfiError) as e:
        ffi.invoke("xla_amd.rowwise_quantize_fp8", quant_frame(host, g_dims=(8, 8)))
    assert "bad operands at: 1" in e.value.message
    assert "Wrong buffer rank: expected 1 but got 2" in e.value.message
    assert e.value.code == 3


def test_wrong_attribute_types():
    host = ffi.Host()
    with pytest.raises(ffi.FfiError, match="Wrong scalar data type: expected F32 but got F64"):
        ffi.invoke("xla_amd.rowwise_quantize_fp8", quant_frame(host, attrs={"eps": ffi.Attr.f64(1e-6)}))
    with pytest.raises(ffi.FfiError, match="Wrong attribute type: expected scalar but got string"):
        ffi.invoke("xla_amd.rowwise_quantize_fp8", quant_frame(host, attrs={"rmsnorm": ffi.Attr.str("yes")}))
    args = [(dtypes.BF16, FAKE, (2, 8)), (dtypes.S8, FAKE, (8, 4)), (dtypes.F32, FAKE, (4,))]
    rets = [(dtypes.BF16, FAKE, (2, 4))]
    with pytest.raises(ffi.FfiError, match="Unknown epilogue `TANH`"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, args, rets, {"epilogue": ffi.Attr.str("TANH")}))
    with pytest.raises(ffi.FfiError, match="Wrong attribute type: expected string but got scalar"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, args, rets, {"epilogue": ffi.Attr.i32(1)}))


def test_shape_validation_happens_before_any_launch():
    host = ffi.Host()
    args = [(dtypes.BF16, FAKE, (2, 8)), (dtypes.S4, FAKE, (16, 4)), (dtypes.BF16, FAKE, (4,))]
    with pytest.raises(ffi.FfiError, match="xla_amd.dequant_dot: contracting dimensions differ"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, args, [(dtypes.BF16, FAKE, (2, 4))]))
    a = [(dtypes.F8E4M3FN, FAKE, (4, 8)), (dtypes.F8E4M3FN, FAKE, (8, 4)), (dtypes.F32, FAKE, ()),
         (dtypes.F32, FAKE, ())]
    with pytest.raises(ffi.FfiError, match="xla_amd.fp8_scaled_dot: result shape must be M,N"):
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, a, [(dtypes.BF16, FAKE, (4, 5))]))
    # a scale is one value, or a vector along the operand's free dimension
    with pytest.raises(ffi.FfiError, match="xla_amd.fp8_scaled_dot: a rank-1 a_scale must have M elements"):
        a2 = list(a)
        a2[2] = (dtypes.F32, FAKE, (3,))
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, a2, [(dtypes.BF16, FAKE, (4, 4))]))
    with pytest.raises(ffi.FfiError, match="xla_amd.fp8_scaled_dot: a rank-1 b_scale must have N elements"):
        a2 = list(a)
        a2[3] = (dtypes.F32, FAKE, (8,))
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, a2, [(dtypes.BF16, FAKE, (4, 4))]))
    # an f8e4m3fn result brings its per-tensor scale as the last operand
    with pytest.raises(ffi.FfiError, match="an F8E4M3FN result takes a, b, a_scale, b_scale, \\[bias,\\] d_scale"):
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, a, [(dtypes.F8E4M3FN, FAKE, (4, 4))]))
    with pytest.raises(ffi.FfiError, match="a BF16 result takes a, b, a_scale, b_scale\\[, bias\\]"):
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, a + [(dtypes.BF16, FAKE, (4,)), (dtypes.F32, FAKE, ())],
                                                       [(dtypes.BF16, FAKE, (4, 4))], {"epilogue": ffi.Attr.str("BIAS")}))
    with pytest.raises(ffi.FfiError, match="results are out\\[, amax\\]\\[, scratch\\]"):
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, a + [(dtypes.F32, FAKE, ())],
                                                       [(dtypes.F8E4M3FN, FAKE, (4, 4)), (dtypes.U8, FAKE, (64,)),
                                                        (dtypes.F32, FAKE, ())]))
    with pytest.raises(ffi.FfiError, match="Wrong buffer rank: expected 0 but got 1 \\(d_scale\\)"):
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, a + [(dtypes.F32, FAKE, (4,))],
                                                       [(dtypes.F8E4M3FN, FAKE, (4, 4))]))
    # block scales: f8e8m0fnu [rows, K/32] on both operands, rhs [N,K]
    mx = [(dtypes.F8E4M3FN, FAKE, (4, 64)), (dtypes.F8E4M3FN, FAKE, (8, 64)), (dtypes.F8E8M0FNU, FAKE, (4, 2)),
          (dtypes.F8E8M0FNU, FAKE, (8, 2))]
    with pytest.raises(ffi.FfiError, match="block scales go with a \\[M,K\\] and b \\[N,K\\]"):
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, mx, [(dtypes.BF16, FAKE, (4, 64))]))
    with pytest.raises(ffi.FfiError, match="block scales must be \\[M,K/32\\] and \\[N,K/32\\]"):
        bad = list(mx)
        bad[3] = (dtypes.F8E8M0FNU, FAKE, (8, 3))
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, bad, [(dtypes.BF16, FAKE, (4, 8))],
                                                       {"rhs_contracting_dim": ffi.Attr.i64(1)}))
    with pytest.raises(ffi.FfiError, match="Wrong buffer dtype: expected F8E8M0FNU but got F32 \\(b_scale\\)"):
        bad = list(mx)
        bad[3] = (dtypes.F32, FAKE, (8, 2))
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, bad, [(dtypes.BF16, FAKE, (4, 8))],
                                                       {"rhs_contracting_dim": ffi.Attr.i64(1)}))
    with pytest.raises(ffi.FfiError, match="Wrong buffer rank: expected 0..1 but got 2"):
        a2 = list(a)
        a2[2] = (dtypes.F32, FAKE, (4, 1))
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, a2, [(dtypes.BF16, FAKE, (4, 4))]))


def test_zero_point_operand_is_recognised_by_its_type():
    """lhs, weights, scales[, zero_points][, bias]: a U4 operand after the scales is the zero points."""
    host = ffi.Host()
    lhs, w4 = (dtypes.BF16, FAKE, (2, 64)), (dtypes.U4, FAKE, (64, 8))
    sc, zp, bias = (dtypes.BF16, FAKE, (2, 8)), (dtypes.U4, FAKE, (2, 8)), (dtypes.BF16, FAKE, (8,))
    out = [(dtypes.BF16, FAKE, (2, 8))]
    with pytest.raises(ffi.FfiError, match="zero points go with U4 weights"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, [lhs, (dtypes.S4, FAKE, (64, 8)), sc, zp], out))
    with pytest.raises(ffi.FfiError, match="zero points must have the shape of the scales"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, [lhs, w4, sc, (dtypes.U4, FAKE, (4, 8))], out))
    with pytest.raises(ffi.FfiError, match="a bias operand goes with a BIAS\\* epilogue"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, [lhs, w4, sc, zp, bias], out))
    with pytest.raises(ffi.FfiError, match="five operands are lhs, weights, scales, zero_points \\(U4\\), bias"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, [lhs, w4, sc, bias, bias], out,
                                                    {"epilogue": ffi.Attr.str("BIAS")}))
    with pytest.raises(ffi.FfiError, match="Wrong buffer dtype"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, [lhs, (dtypes.U8, FAKE, (64, 8)), sc], out))


def test_ragged_dot_operands():
    """An integer operand at the end is the group sizes of a ragged dot: lhs [M,K], weights [G,K,N]."""
    host = ffi.Host()
    lhs, w = (dtypes.BF16, FAKE, (6, 64)), (dtypes.S8, FAKE, (3, 64, 8))
    sc, gs = (dtypes.F32, FAKE, (3, 8)), (dtypes.S32, FAKE, (3,))
    out = [(dtypes.BF16, FAKE, (6, 8))]
    with pytest.raises(ffi.FfiError, match="a ragged dot takes lhs \\[M,K\\] and weights \\[groups,K,N\\]"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, [lhs, (dtypes.S8, FAKE, (64, 8)), (dtypes.F32, FAKE, (8,)), gs], out))
    with pytest.raises(ffi.FfiError, match="group_sizes must have one entry per group of weights"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, [lhs, w, sc, (dtypes.S64, FAKE, (4,))], out))
    with pytest.raises(ffi.FfiError, match="result shape must be"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, [lhs, w, sc, gs], [(dtypes.BF16, FAKE, (3, 6, 8))]))
    with pytest.raises(ffi.FfiError, match="lhs and weights must have the same rank"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, [lhs, w, sc], out))      # no group sizes: not ragged


def test_record_stage_asks_for_stream_capture():
    """At the RECORD stage (XLA building a command buffer, custom_call_thunk.cc:577-684) a handler finds
    the record extension on its invoke context and asks for stream capture of its execute stage;
    it decodes nothing and launches nothing (the buffers here are fake)."""
    host = ffi.NativeHost()
    before = host.set_recording(True)
    try:
        ffi.invoke("xla_amd.rowwise_quantize_fp8", quant_frame(host, stage=ffi.STAGE_RECORD))
        args = [(dtypes.BF16, FAKE, (2, 8)), (dtypes.S8, FAKE, (8, 4)), (dtypes.F32, FAKE, (4,))]
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, args, [(dtypes.BF16, FAKE, (2, 4))], stage=ffi.STAGE_RECORD))
        a = [(dtypes.F8E4M3FN, FAKE, (4, 8)), (dtypes.F8E4M3FN, FAKE, (8, 4)), (dtypes.F32, FAKE, ()), (dtypes.F32, FAKE, ())]
        ffi.invoke("xla_amd.fp8_scaled_dot", ffi.Frame(host, a, [(dtypes.BF16, FAKE, (4, 4))], stage=ffi.STAGE_RECORD))
    finally:
        after = host.set_recording(False)
    assert after - before == 3
    # outside a recording there is no extension to answer to
    with pytest.raises(ffi.FfiError, match=r"\[record\] the call carries no usable record extension"):
        ffi.invoke("xla_amd.rowwise_quantize_fp8", quant_frame(host, stage=ffi.STAGE_RECORD))
    assert host.set_recording(False) == after
    # a host whose function table lacks the lookup reports that instead
    with pytest.raises(ffi.FfiError, match="not implemented by this host"):
        ffi.invoke("xla_amd.rowwise_quantize_fp8", quant_frame(ffi.Host(), stage=ffi.STAGE_RECORD))


def test_stream_get_failure_is_propagated():
    host = ffi.Host(fail_stream_get=True)
    with pytest.raises(ffi.FfiError, match="GPU context is not available"):
        ffi.invoke("xla_amd.rowwise_quantize_fp8", quant_frame(host, x_dims=(0, 64)))


ABI_PROBE = r"""
#include <stdio.h>
#include <stddef.h>
#include HEADER
#define S(t) printf(#t " %zu\n", sizeof(t))
#define O(t, f) printf(#t "." #f " %zu\n", offsetof(t, f))
int main() {
  S(XLA_FFI_CallFrame); O(XLA_FFI_CallFrame, api); O(XLA_FFI_CallFrame, ctx); O(XLA_FFI_CallFrame, stage);
  O(XLA_FFI_CallFrame, args); O(XLA_FFI_CallFrame, rets); O(XLA_FFI_CallFrame, attrs); O(XLA_FFI_CallFrame, future);
  S(XLA_FFI_Buffer); O(XLA_FFI_Buffer, dtype); O(XLA_FFI_Buffer, data); O(XLA_FFI_Buffer, rank); O(XLA_FFI_Buffer, dims);
  S(XLA_FFI_Args); O(XLA_FFI_Args, size); O(XLA_FFI_Args, types); O(XLA_FFI_Args, args);
  S(XLA_FFI_Rets); O(XLA_FFI_Rets, rets);
  S(XLA_FFI_Attrs); O(XLA_FFI_Attrs, types); O(XLA_FFI_Attrs, names); O(XLA_FFI_Attrs, attrs);
  S(XLA_FFI_Scalar); O(XLA_FFI_Scalar, value); S(XLA_FFI_Array); O(XLA_FFI_Array, size); O(XLA_FFI_Array, data);
  S(XLA_FFI_ByteSpan); S(XLA_FFI_Error_Create_Args); O(XLA_FFI_Error_Create_Args, message); O(XLA_FFI_Error_Create_Args, errc);
  S(XLA_FFI_Stream_Get_Args); O(XLA_FFI_Stream_Get_Args, ctx); O(XLA_FFI_Stream_Get_Args, stream);
  S(XLA_FFI_Handler_Register_Args); O(XLA_FFI_Handler_Register_Args, name); O(XLA_FFI_Handler_Register_Args, platform);
  O(XLA_FFI_Handler_Register_Args, bundle); O(XLA_FFI_Handler_Register_Args, traits);
  S(XLA_FFI_Handler_Bundle); O(XLA_FFI_Handler_Bundle, execute);
  S(XLA_FFI_Metadata); O(XLA_FFI_Metadata, api_version); O(XLA_FFI_Metadata, traits); O(XLA_FFI_Metadata, state_type_id);
  S(XLA_FFI_Metadata_Extension); O(XLA_FFI_Metadata_Extension, metadata);
  S(XLA_FFI_Api); O(XLA_FFI_Api, api_version); O(XLA_FFI_Api, internal_api); O(XLA_FFI_Api, XLA_FFI_Error_Create);
  O(XLA_FFI_Api, XLA_FFI_Handler_Register); O(XLA_FFI_Api, XLA_FFI_Stream_Get);
  O(XLA_FFI_Api, XLA_FFI_DeviceMemory_Allocate); O(XLA_FFI_Api, XLA_FFI_DeviceOrdinal_Get);
  O(XLA_FFI_Api, XLA_FFI_InvokeContext_FindExtension);
  printf("frame_struct_size %d\n", (int)XLA_FFI_CallFrame_STRUCT_SIZE);
  printf("api_struct_size %d\n", (int)XLA_FFI_Api_STRUCT_SIZE);
  printf("enums %d %d %d %d %d %d %d\n", XLA_FFI_DataType_BF16, XLA_FFI_DataType_F8E4M3FN, XLA_FFI_DataType_S4,
         XLA_FFI_DataType_S8, XLA_FFI_DataType_F32, XLA_FFI_ExecutionStage_EXECUTE, XLA_FFI_AttrType_STRING);
  printf("version %d %d\n", XLA_FFI_API_MAJOR, XLA_FFI_API_MINOR);
  return 0;
}
"""


def _probe(tmp_path, header, name):
    src = tmp_path / (name + ".cc")
    src.write_text(ABI_PROBE.replace("HEADER", '"%s"' % header))
    exe = tmp_path / name
    subprocess.run(["g++", "-std=c++17", "-o", str(exe), str(src)], check=True)
    return subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout


def test_restated_abi_matches_python_layouts(tmp_path):
    out = _probe(tmp_path, os.path.join(ROOT, "include", "xla_ffi_abi.h"), "mine")
    vals = dict(line.rsplit(" ", 1) for line in out.strip().splitlines() if not line.startswith(("enums", "version")))
    assert int(vals["frame_struct_size"]) == ffi.CALL_FRAME_STRUCT_SIZE
    assert int(vals["XLA_FFI_Buffer"]) == C.sizeof(ffi.Buffer)
    assert int(vals["XLA_FFI_Api"]) == C.sizeof(ffi.Api)
    assert int(vals["XLA_FFI_Handler_Register_Args.traits"]) == ffi.RegisterArgs.traits.offset
    assert int(vals["XLA_FFI_CallFrame.attrs"]) == ffi.CallFrame.attrs.offset


@pytest.mark.skipif(not os.path.exists("/root/reference/xla/ffi/api/c_api.h"),
                    reason="no XLA checkout on this machine")
def test_restated_abi_matches_xla_header(tmp_path):
    mine = _probe(tmp_path, os.path.join(ROOT, "include", "xla_ffi_abi.h"), "mine")
    theirs = _probe(tmp_path, "/root/reference/xla/ffi/api/c_api.h", "theirs")
    assert mine == theirs


def test_native_host_registry_and_errors():
    """The C++ function table: registration by (target, platform), lookup, error ownership."""
    host = ffi.NativeHost()
    host.register()
    for target, sym in ffi.HANDLER_SYMBOLS.items():
        fn = host.find_handler(target, "rocm")
        assert fn == C.cast(getattr(ffi.library(), sym), C.c_void_p).value
        assert host.find_handler(target, "cuda") is None
    fr = quant_frame(host, g_dims=(8, 8))
    with pytest.raises(ffi.FfiError, match="Wrong buffer rank: expected 1 but got 2"):
        ffi.invoke("xla_amd.rowwise_quantize_fp8", fr)
    rp = ffi.Replay([("xla_amd.rowwise_quantize_fp8", quant_frame(host, n_rets=1))])
    with pytest.raises(ffi.FfiError, match="call 0: .*Wrong number of results"):
        rp.run(3)


def test_batched_rank2_scales_need_scale_group_size_when_both_readings_fit():
    """[x,N] scales on a batched dequant_dot are per batch or per group; with x == batch and x | K the
    shape alone cannot tell, so the handler asks for the attribute the rewrite pass always emits."""
    host = ffi.Host()
    args = [(dtypes.BF16, FAKE, (4, 2, 64)), (dtypes.S8, FAKE, (4, 64, 8)), (dtypes.F32, FAKE, (4, 8))]
    rets = [(dtypes.BF16, FAKE, (4, 2, 8))]
    with pytest.raises(ffi.FfiError, match=r"can be read per batch or per group of 16 rows: set scale_group_size"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, args, rets))
    # the attribute is validated against the scales' shape before anything is launched
    with pytest.raises(ffi.FfiError, match=r"scales must be \[K/scale_group_size,N\]"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, args, rets, {"scale_group_size": ffi.Attr.i64(32)}))
    with pytest.raises(ffi.FfiError, match="scale_group_size must divide K"):
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, args, rets, {"scale_group_size": ffi.Attr.i64(48)}))
    with pytest.raises(ffi.FfiError, match="rank-1 scales go with scale_group_size = 0"):
        a1 = [(dtypes.BF16, FAKE, (2, 64)), (dtypes.S8, FAKE, (64, 8)), (dtypes.F32, FAKE, (8,))]
        ffi.invoke("xla_amd.dequant_dot", ffi.Frame(host, a1, [(dtypes.BF16, FAKE, (2, 8))],
                                                    {"scale_group_size": ffi.Attr.i64(16)}))


def test_workspace_sizer_covers_token_chunks():
    """More than 64 tokens of 4-bit weights run as 64-token chunks with the chunk index as the batch
    of one launch: the sizer must report what that launch can use (narrow N wants K-slices), not what
    a single 64-token call would."""
    L = ffi.library()
    s4 = 21
    one = L.xla_amd_dequant_dot_workspace_bytes(1, 64, 8192, 1024, s4)
    two = L.xla_amd_dequant_dot_workspace_bytes(2, 64, 8192, 1024, s4)
    chunked = L.xla_amd_dequant_dot_workspace_bytes(1, 128, 8192, 1024, s4)
    assert two > 0 and chunked >= two, (one, two, chunked)
    # the remainder launch is covered as well
    assert L.xla_amd_dequant_dot_workspace_bytes(1, 64 + 8, 8192, 1024, s4) >= L.xla_amd_dequant_dot_workspace_bytes(1, 8, 8192, 1024, s4)
