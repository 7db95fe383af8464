"""QuantFusionRewriter on HLO text, without a device: FileCheck-style checks on the printed
module, in the manner of the reference's pass tests (gemm_rewriter_fp8_test.cc:137-158).
Patterns are the five benchmark modules plus the shapes of the reference's own test HLO
(gemm_rewriter_fp8_test.cc:469-519,1106-1203,1301+; fusion_emitter_int4_device_test.cc:85-449,
698-716)."""
import re

import pytest

from xla_amd import ffi, hlo, hlo_modules as hm


def check(text, *patterns):
    """Each pattern (regex) must match somewhere after the previous one -- FileCheck's CHECK."""
    pos = 0
    for p in patterns:
        m = re.compile(p).search(text, pos)
        assert m, "CHECK failed: %s\n--- module ---\n%s" % (p, text)
        pos = m.end()


def opcodes(text):
    entry = next(c for c in hlo.to_json(text)["computations"] if c["entry"])
    return [i["opcode"] for i in entry["instructions"]]


def test_parser_round_trip_is_stable():
    for text in (hm.c1_s8_channel(4, 32, 16), hm.c2_s4_group(2, 256, 64), hm.c3_fp8(16, 32, 16),
                 hm.c4_quantize(4, 64), hm.c5_s8_batched(2, 8, 32, 16)):
        once = hlo.print_module(text)
        assert hlo.print_module(once) == once
        j = hlo.to_json(text)
        assert sum(c["entry"] for c in j["computations"]) == 1


def test_parser_accepts_xla_printed_form():
    text = """HloModule m, entry_computation_layout={(bf16[4,8]{1,0})->bf16[4,8]{1,0}}

ENTRY %main.3 (p0: bf16[4,8]) -> bf16[4,8] {
  %p0 = bf16[4,8]{1,0} parameter(0), metadata={op_name="x" source_file="a,b.py"}
  %c = bf16[] constant(1) // trailing comment
  %b = bf16[4,8]{1,0} broadcast(bf16[] %c), dimensions={}
  ROOT %add.1 = bf16[4,8]{1,0} add(bf16[4,8]{1,0} %p0, bf16[4,8]{1,0} %b)
}
"""
    j = hlo.to_json(text)
    ins = j["computations"][0]["instructions"]
    assert [i["name"] for i in ins] == ["p0", "c", "b", "add.1"]
    assert ins[3]["operands"] == ["p0", "b"] and ins[3]["root"]
    assert ins[0]["attrs"]["metadata"].startswith("{op_name=")
    assert ins[0]["shape"] == {"dtype": "bf16", "dims": [4, 8], "layout": "1,0"}


@pytest.mark.parametrize("bad,msg", [
    ("HloModule m\nENTRY e {\n  a = f32[2] add(b, b)\n}\n", "not defined before its use"),
    ("HloModule m\nENTRY e {\n  a = f32[2 parameter(0)\n}\n", "line 3"),
    ("HloModule m\nENTRY e {\n  a = f32[2] parameter(0)\n  a = f32[2] parameter(1)\n}\n", "duplicate"),
    ("HloModule m\n", "no computation"),
])
def test_parser_errors(bad, msg):
    with pytest.raises(hlo.HloError, match=msg):
        hlo.rewrite(bad)


def test_c1_per_channel_s8():
    new, rw, rf = hlo.rewrite(hm.c1_s8_channel())
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s8]"] and rf == []
    check(new, r"%lhs = bf16\[16,4096\] parameter\(0\)", r"%w = s8\[4096,4096\] parameter\(1\)",
          r"\(bf16\[16,4096\]\{1,0\}, s8\[\d+\]\{0\}\) custom-call\(%lhs, %w, %scale\), "
          r'custom_call_target="xla_amd.dequant_dot", api_version=API_VERSION_TYPED_FFI',
          r'epilogue = \\"DEFAULT\\", dequant_type = 11 : i32, dot_type = 11 : i32, epilogue_type = 11 : i32',
          r"ROOT %\S+ = bf16\[16,4096\]\{1,0\} get-tuple-element\(%\S+\), index=0")
    assert sorted(set(opcodes(new))) == ["custom-call", "get-tuple-element", "parameter"]


def test_c2_grouped_s4_with_bias_silu():
    # one token: the scratch result covers the partial sums the decode kernels may pass between workgroups
    new, rw, rf = hlo.rewrite(hm.c2_s4_group(M=1))
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4]"] and rf == []
    want_ws = ffi.library().xla_amd_dequant_dot_workspace_bytes(1, 1, 8192, 28672, 21)
    assert want_ws >= 112 * (16 * 256 * 4 + 16)   # a 16-token tile of sums and a flag per 256-channel strip
    check(new, r"custom-call\(%lhs, %w, %scales, %bias\)",
          r'epilogue = \\"BIAS_SILU\\", dequant_type = 16 : i32, dot_type = 11 : i32, epilogue_type = 11 : i32, '
          r'scale_group_size = 128 : i64')
    assert "s8[%d]{0})" % want_ws in new
    assert sorted(set(opcodes(new))) == ["custom-call", "get-tuple-element", "parameter"]
    # eight tokens: two workgroups per 256-channel strip hand over through the scratch
    new, rw, rf = hlo.rewrite(hm.c2_s4_group(M=8))
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4]"] and rf == []
    assert ffi.library().xla_amd_dequant_dot_workspace_bytes(1, 8, 8192, 28672, 21) == 112 * (16 * 256 * 4 + 16)
    check(new, r"\(bf16\[8,28672\]\{1,0\}, s8\[1836800\]\{0\}\) custom-call\(%lhs, %w, %scales, %bias\)")
    # 64 tokens: the 224 strips fill the machine, no split, no scratch, a plain array result
    new, rw, rf = hlo.rewrite(hm.c2_s4_group(M=64))
    assert ffi.library().xla_amd_dequant_dot_workspace_bytes(1, 64, 8192, 28672, 21) == 0
    check(new, r"ROOT %\S+ = bf16\[64,28672\]\{1,0\} custom-call\(%lhs, %w, %scales, %bias\)")
    assert sorted(set(opcodes(new))) == ["custom-call", "parameter"]
    # x * logistic(x) is the same activation before LogisticExpander has run
    text = hm.c2_s4_group(M=8)
    text = re.sub(r"  %neg = .*\n  %exp = .*\n  %one = .*\n  %one_b = .*\n  %den = .*\n  %sig = f32(\[\d+,\d+\]) divide.*\n",
                  r"  %sig = f32\1 logistic(%z)\n", text)
    assert "logistic" in text
    assert hlo.rewrite(text)[1] == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4]"]


@pytest.mark.parametrize("typed,code", [("f32", 11), ("bf16", 16)])
def test_c3_fp8_bias_gelu(typed, code):
    new, rw, rf = hlo.rewrite(hm.c3_fp8(typed=typed))
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU]"] and rf == []
    check(new, r"custom-call\(%a, %b, %a_scale\S*, %b_scale\S*, %bias\), custom_call_target=\"xla_amd.fp8_scaled_dot\"",
          r'epilogue = \\"BIAS_GELU\\", dequant_type = %d : i32, dot_type = %d : i32, epilogue_type = %d : i32, '
          r'rhs_contracting_dim = 0 : i64' % (code, code, code))
    ragged_n = hlo.rewrite(hm.c3_fp8(512, 4096, 1000, typed=typed))[0]
    if typed == "f32":
        assert "s8[" not in new                # N % 16 == 0: the [K,N] rhs goes in as it is, no scratch
        assert "s8[4096000]{0}" in ragged_n    # K*N bytes to re-lay a [K,N] rhs out with K minor when N % 16 != 0
    else:   # a bf16-typed multiply: room for both operands as bf16, (M + N) * K * 2 bytes, behind the copy
        assert "s8[%d]{0}" % (2 * 8192 * 8192 * 2) in new
        assert "s8[%d]{0}" % (4096000 + (512 + 1000) * 4096 * 2) in ragged_n
    if typed == "bf16":                        # bf16 scalars are widened, as GemmRewriter does
        check(new, r"%a_scale.f32 = f32\[\] convert\(%a_scale\)", r"%b_scale.f32 = f32\[\] convert\(%b_scale\)")


def test_c3_fp8_vector_scales():
    """Scales broadcast along the free dimension of each operand (rows of a, channels of b)
    go in as rank-1 operands; along the contracting dimension they do not factor out of the
    sum and the dot is left alone, with the reason logged."""
    text = hm.c3_fp8(64, 128, 32, vector_scales=True)
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU]"] and rf == []
    check(new, r"custom-call\(%a, %b, %a_scale, %b_scale, %bias\), custom_call_target=\"xla_amd.fp8_scaled_dot\"")
    assert "%a_scale = f32[64] parameter(2)" in new and "%b_scale = f32[32] parameter(3)" in new
    bad = text.replace("%a_scale = f32[64] parameter(2)", "%a_scale = f32[128] parameter(2)") \
              .replace("broadcast(%a_scale), dimensions={0}", "broadcast(%a_scale), dimensions={1}")
    new, rw, rf = hlo.rewrite(bad)
    assert rw == [] and "custom-call" not in new
    assert len(rf) == 1 and "lhs scales vary along the contracting dimension" in rf[0]
    bad = text.replace("%b_scale = f32[32] parameter(3)", "%b_scale = f32[128] parameter(3)") \
              .replace("broadcast(%b_scale), dimensions={1}", "broadcast(%b_scale), dimensions={0}")
    new, rw, rf = hlo.rewrite(bad)
    assert rw == [] and len(rf) == 1 and "rhs scales vary along the contracting dimension" in rf[0]


def test_c3_fp8_with_f8_result():
    """divide (or multiply) by a per-tensor scale -> clamp(+-448) -> convert(f8e4m3fn) after the
    epilogue is taken into the call: the scale is the last operand, the result is f8
    (gemm_rewriter_fp8_test.cc:1665-1690; the reference leaves it unfused on ROCm, :1710)."""
    # N = 40 is no multiple of 16: the [K,N] rhs is re-laid out through K*N bytes of scratch
    for mul in (False, True):
        new, rw, rf = hlo.rewrite(hm.c3_fp8_f8_result(64, 128, 40, multiply=mul))
        assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU, f8 result]"] and rf == []
        check(new, r"\(f8e4m3fn\[64,40\]\{1,0\}, s8\[5120\]\{0\}\) custom-call\(%a, %b, %a_scale, %b_scale, %bias, %d_scale\)",
              r"d_scale_multiplies = %s" % ("true" if mul else "false"))
        assert sorted(set(opcodes(new))) == ["custom-call", "get-tuple-element", "parameter"]
    # the result's own amax (reduce-maximum of abs over both dimensions) becomes a second result
    new, rw, rf = hlo.rewrite(hm.c3_fp8_f8_result(64, 128, 40, amax=True))
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU, f8 result, amax]"] and rf == []
    check(new, r"\(f8e4m3fn\[64,40\]\{1,0\}, f32\[\], s8\[5120\]\{0\}\) custom-call\(%a, %b, %a_scale, %b_scale, %bias, %d_scale\)",
          r"ROOT %result = .* tuple\(%out.out, %amax.amax\)")
    assert sorted(set(opcodes(new))) == ["custom-call", "get-tuple-element", "parameter", "tuple"]
    # a clamp to anything but +-448 is not the f8 saturation: left alone, with the reason
    bad = hm.c3_fp8_f8_result(64, 128, 40).replace("constant(448)", "constant(240)")
    new, rw, rf = hlo.rewrite(bad)
    assert rw == [] and any("is f32, the kernels produce bf16" in r for r in rf)


def test_batched_fp8_dot():
    """One leading batch dimension on both operands (gemm_rewriter_fp8_test.cc:941-957): operands
    and result keep their rank, rhs_contracting_dim counts inside the matrix; per-row scales
    on a batched dot are left alone."""
    for nk in (False, True):
        new, rw, rf = hlo.rewrite(hm.fp8_batched(10, 16, 32, 16, rhs_nk=nk))
        assert rw == ["dot -> xla_amd.fp8_scaled_dot [DEFAULT]"] and rf == []
        check(new, r"bf16\[10,16,16\]\{2,1,0\}.* custom-call\(%x, %y, %x_scale, %y_scale\)",
              r"rhs_contracting_dim = %d : i64" % (1 if nk else 0))
    bad = hm.fp8_batched(10, 16, 32, 16).replace("%x_scale = f32[] parameter(2)", "%x_scale = f32[16] parameter(2)") \
            .replace("broadcast(%x_scale), dimensions={}", "broadcast(%x_scale), dimensions={1}")
    new, rw, rf = hlo.rewrite(bad)
    assert rw == [] and "custom-call" not in new


def test_mxfp8_block_scaled_dot():
    """"__op$block_scaled_dot" with f8e4m3fn operands and f8e8m0fnu scales per 32 of K keeps its
    operands and becomes the library's call (block_scaling_rewriter.h:48-69), with a leading batch
    dimension and with what follows an f32-typed call (bias, GELU, convert to bf16) taken along;
    other scale types or an f32 value leaving the pattern stay for BlockScalingRewriter, with the reason."""
    text = hm.mxfp8_block_scaled_dot(64, 256, 32)
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["result -> xla_amd.fp8_scaled_dot [DEFAULT, block scales]"] and rf == []
    check(new, r"bf16\[64,32\]\{1,0\} custom-call\(%lhs, %rhs, %lhs_scale, %rhs_scale\), custom_call_target=\"xla_amd.fp8_scaled_dot\"",
          r"rhs_contracting_dim = 1 : i64")
    # few rows of lhs: the streaming kernel's K-slices get their scratch (f32 sums, per batch)
    for batch in (0, 3):
        new, rw, rf = hlo.rewrite(hm.mxfp8_block_scaled_dot(16, 4096, 512, batch=batch))
        assert len(rw) == 1 and rf == []
        m = re.search(r"\(bf16\[(?:3,)?16,512\]\{[0-9,]+\}, s8\[(\d+)\]\{0\}\) custom-call\(", new)
        assert m and int(m.group(1)) % (16 * 512 * 4 * max(batch, 1)) == 0 and int(m.group(1)) > 0, new
    new, rw, rf = hlo.rewrite(hm.mxfp8_block_scaled_dot(64, 256, 32, batch=3))
    assert rw == ["result -> xla_amd.fp8_scaled_dot [DEFAULT, block scales, batched]"] and rf == []
    check(new, r"bf16\[3,64,32\]\{2,1,0\} custom-call\(%lhs, %rhs, %lhs_scale, %rhs_scale\), custom_call_target=\"xla_amd.fp8_scaled_dot\"")
    new, rw, rf = hlo.rewrite(hm.mxfp8_block_scaled_dot(64, 256, 32, batch=2, bias_gelu=True))
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU, block scales, batched]"] and rf == []
    check(new, r"bf16\[2,64,32\]\{2,1,0\} custom-call\(%lhs, %rhs, %lhs_scale, %rhs_scale, %bias\), custom_call_target=\"xla_amd.fp8_scaled_dot\"",
          r"epilogue = \\\"BIAS_GELU\\\"")
    assert "tanh" not in new and "__op$block_scaled_dot" not in new
    new, rw, rf = hlo.rewrite(text.replace("f8e8m0fnu", "f8e5m2"))
    assert rw == [] and "__op$block_scaled_dot" in new and "f8e8m0fnu scales" in rf[0]
    new, rw, rf = hlo.rewrite(text.replace("%result = bf16[64,32]", "%result = f32[64,32]"))
    assert rw == [] and "the value leaving the dot pattern is f32" in rf[0]
    new, rw, rf = hlo.rewrite(text.replace("%rhs = f8e4m3fn[32,256]", "%rhs = f8e4m3fn[2,32,256]"))
    assert rw == [] and "must all be rank 2, or rank 3" in rf[0]


def test_quantizer_feeding_a_dot_becomes_two_calls():
    """The quantizer's broadcast scales are reused by the dequantising multiply of the next dot:
    both patterns are taken, the dot reads the quantizer's two results, and none of the
    RMSNorm / amax / divide chain survives."""
    new, rw, rf = hlo.rewrite(hm.quantize_then_fp8_dot(64, 256, 32))
    assert rw == ["q -> xla_amd.rowwise_quantize_fp8 [rmsnorm]", "dot -> xla_amd.fp8_scaled_dot [DEFAULT]"] and rf == []
    check(new, r"custom-call\(%x, %gamma\), custom_call_target=\"xla_amd.rowwise_quantize_fp8\"",
          r"custom-call\(%q.codes, %w, %scale.scales, %w_scale\), custom_call_target=\"xla_amd.fp8_scaled_dot\"")
    assert sorted(set(opcodes(new))) == ["custom-call", "get-tuple-element", "parameter"]


def test_c4_quantize_rmsnorm_and_plain():
    new, rw, rf = hlo.rewrite(hm.c4_quantize())
    assert rw == ["q -> xla_amd.rowwise_quantize_fp8 [rmsnorm]"] and rf == []
    check(new, r"\(f8e4m3fn\[16384,8192\]\{1,0\}, f32\[16384\]\{0\}\) custom-call\(%x, %gamma\)",
          r'backend_config="\{rmsnorm = true, eps = 1e-06 : f32\}"',
          r"ROOT %result = .* tuple\(%q.codes, %scale.scales\)")
    assert sorted(set(opcodes(new))) == ["custom-call", "get-tuple-element", "parameter", "tuple"]
    new, rw, rf = hlo.rewrite(hm.c4_quantize(rmsnorm=False))
    assert rw == ["q -> xla_amd.rowwise_quantize_fp8 [plain]"]
    check(new, r"custom-call\(%x\)", r"rmsnorm = false")
    # reduce-max seeded with 0 instead of -inf is the same amax of absolute values
    assert hlo.rewrite(hm.c4_quantize(rmsnorm=False).replace("constant(-inf)", "constant(0)"))[1]
    # the reciprocal root as one rsqrt instruction: the same call, the same attributes (the CPU
    # backend's portable definition of rsqrt is 1 / sqrt, xla/codegen/intrinsic/rsqrt.cc:178-193)
    new_r, rw_r, rf_r = hlo.rewrite(hm.c4_quantize(rsqrt=True))
    assert rw_r == ["q -> xla_amd.rowwise_quantize_fp8 [rmsnorm]"] and rf_r == []
    assert new_r == hlo.rewrite(hm.c4_quantize())[0]
    assert "rsqrt" in hm.c4_quantize(rsqrt=True) and "rsqrt" not in new_r
    # rsqrt of something else is not the pattern
    bad = hm.c4_quantize(8, 64, rsqrt=True).replace("rsqrt(%ms_eps)", "rsqrt(%ms)")
    assert hlo.rewrite(bad)[1] == [] and "not the RMSNorm form" in hlo.rewrite(bad)[2][0]


def test_c5_batched_s8():
    new, rw, rf = hlo.rewrite(hm.c5_s8_batched())
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s8]"] and rf == []
    check(new, r"bf16\[8,512,14336\]\{2,1,0\}", r"custom-call\(%lhs, %w, %scale\)")


def test_rewrite_without_scratch_callbacks_has_single_result():
    new, rw, _ = hlo.rewrite(hm.c1_s8_channel(), with_scratch=False)
    check(new, r"ROOT %\S+ = bf16\[16,4096\]\{1,0\} custom-call\(%lhs, %w, %scale\)")


FP8_HEAD = """HloModule test
ENTRY test {
  x = f8e4m3fn[16,32] parameter(0)
  y = f8e4m3fn[32,16] parameter(1)
  x_scale = f32[] parameter(2)
  y_scale = f32[] parameter(3)
"""


def test_fp8_scaled_ab_relu_bf16_out():
    text = FP8_HEAD + """  x_f32 = f32[16,32] convert(x)
  y_f32 = f32[32,16] convert(y)
  x_scale_bcast = f32[16,32] broadcast(x_scale), dimensions={}
  y_scale_bcast = f32[32,16] broadcast(y_scale), dimensions={}
  x_unscaled = f32[16,32] multiply(x_f32, x_scale_bcast)
  y_unscaled = f32[32,16] multiply(y_f32, y_scale_bcast)
  dot_a = f32[16,16] dot(x_unscaled, y_unscaled), lhs_contracting_dims={1}, rhs_contracting_dims={0}
  c = f32[] constant(0)
  c_bcast = f32[16,16] broadcast(c), dimensions={}
  relu = f32[16,16] maximum(dot_a, c_bcast)
  ROOT out = bf16[16,16] convert(relu)
}
"""
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["dot_a -> xla_amd.fp8_scaled_dot [RELU]"], (rw, rf)
    check(new, r"custom-call\(%x, %y, %x_scale, %y_scale\)", r'epilogue = \\"RELU\\"')


def test_fp8_f32_result_is_refused_with_reason():
    """ScaledABUnscaledDF8 (gemm_rewriter_fp8_test.cc:469-519) leaves an f32 dot; the kernels
    produce bf16, so the pass says so and leaves the module alone."""
    text = FP8_HEAD + """  x_f32 = f32[16,32] convert(x)
  y_f32 = f32[32,16] convert(y)
  x_scale_bcast = f32[16,32] broadcast(x_scale), dimensions={}
  y_scale_bcast = f32[32,16] broadcast(y_scale), dimensions={}
  x_unscaled = f32[16,32] multiply(x_f32, x_scale_bcast)
  y_unscaled = f32[32,16] multiply(y_f32, y_scale_bcast)
  ROOT out = f32[16,16] dot(x_unscaled, y_unscaled), lhs_contracting_dims={1}, rhs_contracting_dims={0}
}
"""
    new, rw, rf = hlo.rewrite(text)
    assert rw == [] and "custom-call" not in new
    assert len(rf) == 1 and "is f32, the kernels produce bf16" in rf[0]


def test_fp8_divide_by_scale_and_rhs_contracting_minor():
    text = FP8_HEAD.replace("y = f8e4m3fn[32,16]", "y = f8e4m3fn[16,32]") + """  x_bf16 = bf16[16,32] convert(x)
  y_bf16 = bf16[16,32] convert(y)
  xs = bf16[] convert(x_scale)
  ys = bf16[] convert(y_scale)
  x_scale_bcast = bf16[16,32] broadcast(xs), dimensions={}
  y_scale_bcast = bf16[16,32] broadcast(ys), dimensions={}
  x_unscaled = bf16[16,32] divide(x_bf16, x_scale_bcast)
  y_unscaled = bf16[16,32] multiply(y_scale_bcast, y_bf16)
  ROOT out = bf16[16,16] dot(x_unscaled, y_unscaled), lhs_contracting_dims={1}, rhs_contracting_dims={1}
}
"""
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["out -> xla_amd.fp8_scaled_dot [DEFAULT]"], (rw, rf)
    check(new, r"%\S+ = f32\[\] divide\(%one\S*, %\S+\)", r"rhs_contracting_dim = 1 : i64")
    assert "s8[2048]{0}" in new                  # K-minor rhs needs no copy; bf16-typed multiply: both operands as bf16


def test_unscaled_fp8_dot_gets_unit_scales():
    text = """HloModule t
ENTRY e {
  x = f8e4m3fn[16,32] parameter(0)
  y = f8e4m3fn[32,16] parameter(1)
  xb = bf16[16,32] convert(x)
  yb = bf16[32,16] convert(y)
  ROOT d = bf16[16,16] dot(xb, yb), lhs_contracting_dims={1}, rhs_contracting_dims={0}
}
"""
    new, rw, _ = hlo.rewrite(text)
    assert rw == ["d -> xla_amd.fp8_scaled_dot [DEFAULT]"]
    check(new, r"%one\S* = f32\[\]\S* constant\(1\)", r"custom-call\(%x, %y, %one\S*, %one\S*\)")


def test_int4_channel_dequant_with_bias_from_reference_shape():
    """Channel dequantisation of fusion_emitter_int4_device_test.cc:217-247, with the weights
    as the dot's rhs [B,K,N]."""
    text = """HloModule FuseChannelDequantization
ENTRY main {
  w.s4 = s4[32,128,256] parameter(0)
  w.s8 = s8[32,128,256] convert(w.s4)
  w.bf16 = bf16[32,128,256] convert(w.s8)
  s = bf16[32,256] parameter(1)
  s.broadcast.2 = bf16[32,128,256] broadcast(s), dimensions={0,2}
  w.scaled = bf16[32,128,256] multiply(w.bf16, s.broadcast.2)
  a = bf16[32,2,128] parameter(2)
  ROOT dot = bf16[32,2,256] dot(a, w.scaled), lhs_batch_dims={0}, lhs_contracting_dims={2}, rhs_batch_dims={0}, rhs_contracting_dims={1}
}
"""
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s4]"], (rw, rf)
    check(new, r"custom-call\(%a, %w.s4, %s\)", r"dequant_type = 16 : i32, dot_type = 16 : i32")


def test_weights_on_the_lhs_are_taken_and_a_minor_batch_dim_is_left_alone():
    # weights as lhs (fusion_emitter_int4_device_test.cc:93-104 orientation), activations [K,M]: one call
    # whose result is [N,M]
    text = """HloModule t
ENTRY main {
  w = s4[128,256] parameter(0)
  w8 = s8[128,256] convert(w)
  wb = bf16[128,256] convert(w8)
  s = bf16[256] parameter(1)
  sb = bf16[128,256] broadcast(s), dimensions={1}
  ws = bf16[128,256] multiply(wb, sb)
  a = bf16[128,4] parameter(2)
  ROOT dot = bf16[256,4] dot(ws, a), lhs_contracting_dims={0}, rhs_contracting_dims={0}
}
"""
    new, rw, _ = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s4, weights as lhs, activations [K,M]]"], rw
    check(new, r"ROOT %\S+ = bf16\[256,4\]\{1,0\} custom-call\(%a, %w, %s\)",
          r"scale_group_size = 0 : i64, lhs_contracting_dim = 0 : i64, result_transposed = true")
    # RejectTritonFusionForWithMinorBatchDim (fusion_emitter_int4_device_test.cc:698-716)
    text = """HloModule t
ENTRY main {
  lhs = s4[32,64,2] parameter(0)
  lhs_converted = bf16[32,64,2] convert(lhs)
  rhs = bf16[2,64,16] parameter(1)
  ROOT dot = bf16[2,32,16] dot(lhs_converted, rhs), lhs_batch_dims={2}, lhs_contracting_dims={1}, rhs_batch_dims={0}, rhs_contracting_dims={1}
}
"""
    assert hlo.rewrite(text)[1] == []
    # weights as rhs contracting their minor dimension ([N,K]): taken, with rhs_contracting_dim = 1
    text = """HloModule t
ENTRY main {
  a = bf16[4,128] parameter(0)
  w = s8[256,128] parameter(1)
  wf = bf16[256,128] convert(w)
  s = bf16[256] parameter(2)
  sb = bf16[256,128] broadcast(s), dimensions={0}
  ws = bf16[256,128] multiply(wf, sb)
  ROOT dot = bf16[4,256] dot(a, ws), lhs_contracting_dims={1}, rhs_contracting_dims={1}
}
"""
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s8, weights [N,K]]"] and rf == []
    check(new, r"dequant_type = 16 : i32", r"dot_type = 16 : i32", r"rhs_contracting_dim = 1 : i64")


def test_dot_with_second_user_keeps_epilogue_outside():
    text = hm.c1_s8_channel(4, 64, 32).replace("ROOT %out = bf16[4,32] convert(%dot)",
                                               "%out = bf16[4,32] convert(%dot)\n  ROOT %t = (bf16[4,32], f32[4,32]) tuple(%out, %dot)")
    new, rw, rf = hlo.rewrite(text)
    # the f32 dot itself is a value the module keeps: the call returns it, the convert stays outside
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s8, f32 result]"] and rf == []
    check(new, r"f32\[4,32\]\{1,0\}(, s8\[\d+\]\{0\}\))? custom-call\(", r"%out = bf16\[4,32\](\{1,0\})? convert\(%dot\S*\)")


def test_quantize_near_misses_are_refused_with_reasons():
    base = hm.c4_quantize(8, 64)
    _, rw, rf = hlo.rewrite(base.replace("constant(448)", "constant(240)"))
    assert rw == [] and rf == []                       # not even the clamp bounds match
    _, rw, rf = hlo.rewrite(base.replace("%scale = f32[8] divide(%amax, %c448_b)", "%scale = f32[8] multiply(%amax, %c448_b)"))
    assert rw == [] and "scale is not amax / 448" in rf[0]
    rs = base.replace("%rt = f32[8] sqrt(%ms_eps)", "%rt = f32[8] rsqrt(%ms_eps)").replace(
        "%rinv = f32[8] divide(%one_b, %rt)", "%rinv = f32[8] multiply(%one_b, %rt)")
    _, rw, rf = hlo.rewrite(rs)
    assert rw == [] and "not the RMSNorm form" in rf[0]


def test_mutated_modules_are_rejected_or_stay_printable():
    """Line deletions, duplications, swaps and token edits of the canonical modules: the parser
    either rejects the text with an error or the pass returns a module that parses again."""
    import random
    rng = random.Random(5)
    tokens = ["(", ")", "{", "}", "[", "]", ",", "=", "%", ":", " ", "0", "f32", "s4", "f8e4m3fn", "broadcast",
              "dot", "-", "448", "dimensions={0}", "ROOT ", "parameter(0)", "tuple", "clamp"]
    base = [hm.c1_s8_channel(16, 512, 256), hm.c2_s4_group(8, 1024, 512), hm.c3_fp8(64, 128, 32, vector_scales=True),
            hm.c3_fp8_f8_result(64, 128, 32), hm.c4_quantize(24, 2048), hm.c5_s8_batched(2, 128, 256, 512),
            hm.quantize_then_fp8_dot(64, 256, 32)]
    accepted = rejected = 0
    for text in base:
        lines = text.split("\n")
        for _ in range(40):
            b = list(lines)
            kind = rng.random()
            if kind < 0.3:
                del b[rng.randrange(len(b))]
            elif kind < 0.5:
                i = rng.randrange(len(b))
                b.insert(i, b[i])
            elif kind < 0.7:
                i, k = rng.randrange(len(b)), rng.randrange(len(b))
                b[i], b[k] = b[k], b[i]
            else:
                i = rng.randrange(len(b))
                if b[i]:
                    p = rng.randrange(len(b[i]))
                    b[i] = b[i][:p] + rng.choice(tokens) + b[i][p + rng.randrange(3):]
            try:
                new, _, _ = hlo.rewrite("\n".join(b))
            except hlo.HloError:
                rejected += 1
                continue
            accepted += 1
            hlo.print_module(new)
            hlo.to_json(new)
    assert accepted > 20 and rejected > 20, (accepted, rejected)
    with pytest.raises(hlo.HloError, match="computation without a name"):
        hlo.rewrite(hm.c1_s8_channel(16, 512, 256).replace("ENTRY %main {", "ENTRY :%main {"))


def test_amax_consumer_ahead_of_the_convert_stays_defined_before_use():
    """XLA prints in post-order, so a user of the amax reduce may sit above the clamp/convert chain
    that ends the pattern; after the rewrite it must still follow the custom call it now reads."""
    text = hm.c3_fp8_f8_result(64, 128, 32, amax=True)
    # move the amax reduce (and a consumer of it) in front of the divide/clamp/convert chain
    lines = text.split("\n")
    take = [i for i, l in enumerate(lines) if l.strip().startswith(("%abs_v", "%ninf", "%amax ="))]
    moved = [lines[i] for i in take]
    for i in reversed(take):
        del lines[i]
    at = next(i for i, l in enumerate(lines) if l.strip().startswith("%d_scale ="))
    extra = ["  %two = f32[] constant(2)", "  %amax2 = f32[] multiply(%amax, %two)"]
    lines[at:at] = moved + extra
    text = "\n".join(lines).replace("tuple(%out, %amax)", "tuple(%out, %amax2)")
    assert text.index("%amax2 =") < text.index("%clamped =")
    hlo.print_module(text)  # the input itself is well formed
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU, f8 result, amax]"] and rf == []
    again = hlo.print_module(new)  # the parser refuses a use before its definition
    assert again == new
    check(new, r"custom-call\(", r"%amax.amax = f32\[\] get-tuple-element", r"%amax2 = f32\[\] multiply\(%amax.amax, %two\)",
          r"ROOT %result = .* tuple\(%out.out, %amax2\)")


def test_rewrite_keeps_side_effects_and_what_was_already_unused():
    text = hm.c3_fp8(16, 32, 16)
    text = text.replace("  %a_t =", "  %tok = token[] after-all()\n"
                        "  %side = token[] custom-call(%tok), custom_call_target=\"my_side_effect\", "
                        "custom_call_has_side_effect=true\n"
                        "  %unused = f32[] constant(7)\n  %a_t =", 1)
    new, rw, rf = hlo.rewrite(text)
    assert len(rw) == 1 and rf == []
    ops = opcodes(new)
    assert "after-all" in ops and ops.count("custom-call") == 2
    assert "%unused = f32[] constant(7)" in new and "my_side_effect" in new
    # nothing of the matched pattern survives
    assert "tanh" not in ops and "dot" not in ops and "convert" not in ops


@pytest.mark.parametrize("c1,ok", [("0.797884583", True), ("0.79788456", True), ("0.8", False), ("0.79", False),
                                   ("0.7979", True), ("0.79795", False)])
def test_gelu_constants_are_held_to_128_epsilon_of_their_type(c1, ok):
    """gemm_rewriter.cc:472-503: |actual - expected| < |actual + expected| * 128 eps(type)."""
    text = hm.c3_fp8(16, 32, 16).replace("constant(0.797884583)", "constant(%s)" % c1)
    _, rw, _ = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [%s]" % ("BIAS_GELU" if ok else "BIAS")] or (not ok and rw == [])
    if not ok:
        assert not any("GELU" in r for r in rw)
    # a bf16 constant is as coarse as its type: 0.796875 is bf16(0.7978...), within 128 * 2^-7
    bf = hm.c3_fp8(16, 32, 16, typed="bf16").replace("constant(0.797884583)", "constant(0.796875)")
    assert hlo.rewrite(bf)[1] == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU]"]


def test_u4_weights_with_zero_points():
    """(convert(u4 w) - convert(u4 zero)) * scale, grouped: one call with the zero points as the
    operand after the scales; near misses keep their reasons."""
    text = hm.u4_zero_point_group(8, 256, 64, 64)
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS, u4 with zero points]"] and rf == []
    check(new, r"custom-call\(%lhs, %w, %scales, %zero, %bias\), custom_call_target=\"xla_amd.dequant_dot\"",
          r"dequant_type = 16 : i32", r"scale_group_size = 64 : i64")
    assert sorted(set(opcodes(new))) == ["custom-call", "parameter"]
    # zero points of another shape than the scales
    bad = text.replace("%zero = u4[4,64] parameter(3)", "%zero4 = u4[4,64] parameter(3)\n  %zero = u4[4,64] add(%zero4, %zero4)")
    assert hlo.rewrite(bad)[1] == rw          # any u4 [G,N] value serves
    # signed weights with zero points are not a pattern the kernels take
    signed = text.replace("u4[256,64] parameter(1)", "s4[256,64] parameter(1)").replace("%w_g = u4[", "%w_g = s4[")
    new2, rw2, rf2 = hlo.rewrite(signed)
    assert rw2 == [] and any("zero points are taken with u4 weights only" in r for r in rf2)
    # u4 without zero points
    plain = hm.c2_s4_group(4, 256, 64, 64).replace("s4[", "u4[").replace("s8[", "u8[")
    new3, rw3, rf3 = hlo.rewrite(plain)
    assert rw3 == ["dot -> xla_amd.dequant_dot [BIAS_SILU, u4]"] and rf3 == []
    check(new3, r"custom-call\(%lhs, %w, %scales, %bias\)")


def test_ragged_dot_over_expert_weights():
    text = hm.ragged_s8_experts(16, 256, 64, 4)
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS, s8, ragged over 4 groups]"] and rf == []
    check(new, r"custom-call\(%lhs, %w, %scale, %bias, %sizes\), custom_call_target=\"xla_amd.dequant_dot\"",
          r"scale_group_size = 0 : i64")
    assert sorted(set(opcodes(new))) == ["custom-call", "parameter"]
    assert hlo.rewrite(hm.ragged_s8_experts(16, 256, 64, 4, sizes_ty="s64"))[1] == rw
    # any number of rows: the kernel walks a group in chunks of 64
    assert hlo.rewrite(hm.ragged_s8_experts(640, 256, 64, 4))[1] == rw
    for bad, reason in ((text.replace("lhs_ragged_dims={0}", "lhs_ragged_dims={1}"), "ragged dimension on the rows of lhs"),
                        (text.replace("%sizes = s32[4]", "%sizes = u32[4]"), "group sizes must be s32 or s64")):
        new2, rw2, rf2 = hlo.rewrite(bad)
        assert rw2 == [] and any(reason in r for r in rf2), (rw2, rf2)


def test_grouped_scales_behind_a_batch_or_expert_dimension():
    """reshape([B,K/g,g,N] product) -> [B,K,N]: grouped scales [B,K/g,N] on batched weights, and on the
    expert weights of a ragged dot; scale_group_size carries g."""
    new, rw, rf = hlo.rewrite(hm.batched_s4_group(2, 8, 256, 64, 64))
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s4]"] and rf == []
    check(new, r"custom-call\(%lhs, %w, %scales\), custom_call_target=\"xla_amd.dequant_dot\"",
          r"scale_group_size = 64 : i64")
    assert sorted(set(opcodes(new))) == ["custom-call", "parameter"]
    text = hm.ragged_s4_group_experts(16, 256, 64, 4, 64)
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS, s4, ragged over 4 groups]"] and rf == []
    check(new, r"custom-call\(%lhs, %w, %scales, %bias, %sizes\), custom_call_target=\"xla_amd.dequant_dot\"",
          r"scale_group_size = 64 : i64")
    assert sorted(set(opcodes(new))) == ["custom-call", "parameter"]
    # scales of another expert count are not this pattern
    bad = text.replace("%scales = bf16[4,4,64] parameter(2)", "%scales = bf16[2,4,64] parameter(2)")
    assert hlo.rewrite(bad)[1] == []


def test_c3_fp8_vector_scales_under_a_bf16_multiply():
    """Per-row / per-channel scales with every op bf16-typed: taken (the rounded operands go to the bf16
    matrix cores); the bf16 vectors are widened to the f32 the handler reads, and the scratch holds both
    operands as bf16."""
    new, rw, rf = hlo.rewrite(hm.c3_fp8(64, 128, 32, typed="bf16", vector_scales=True))
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU]"] and rf == []
    check(new, r"%a_scale.f32 = f32\[64\]\{0\} convert\(%a_scale\)", r"%b_scale.f32 = f32\[32\]\{0\} convert\(%b_scale\)",
          r"s8\[%d\]\{0\}\) custom-call\(%%a, %%b, %%a_scale.f32, %%b_scale.f32, %%bias\)" % ((64 + 32) * 128 * 2),
          r"dequant_type = 16 : i32")


def test_weights_with_the_contracting_dimension_minor():
    """dot(lhs, dequantised [N,K] weights), rhs_contracting_dims = {1} (the spelling of
    fusion_emitter_int4_device_test.cc:867-892): one call with rhs_contracting_dim = 1, the scales
    [N] or [N,K/g] as they are, scratch sized by the [N,K] kernels' own query."""
    new, rw, rf = hlo.rewrite(hm.k_minor_s8_channel(16, 4096, 4096))
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s8, weights [N,K]]"] and rf == []
    ws = ffi.library().xla_amd_dequant_dot_workspace_bytes_nk(1, 16, 4096, 4096, 2)
    check(new, r"%w = s8\[4096,4096\] parameter\(1\)",
          r"\(bf16\[16,4096\]\{1,0\}, s8\[%d\]\{0\}\) custom-call\(%%lhs, %%w, %%scale\)" % ws,
          r"scale_group_size = 0 : i64, rhs_contracting_dim = 1 : i64")
    assert ws > 0
    new, rw, rf = hlo.rewrite(hm.k_minor_s4_group(8, 8192, 28672))
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4, weights [N,K]]"] and rf == []
    check(new, r"%scales = bf16\[28672,64\] parameter\(2\)", r"custom-call\(%lhs, %w, %scales, %bias\)",
          r"dequant_type = 16 : i32", r"scale_group_size = 128 : i64, rhs_contracting_dim = 1 : i64")
    assert sorted(set(opcodes(new))) == ["custom-call", "get-tuple-element", "parameter"]
    new, rw, rf = hlo.rewrite(hm.k_minor_s4_group(8, 2048, 512, 256, typed="f32"))
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4, weights [N,K]]"] and rf == []
    check(new, r"dequant_type = 11 : i32", r"scale_group_size = 256 : i64, rhs_contracting_dim = 1 : i64")
    new, rw, rf = hlo.rewrite(hm.k_minor_u4_zero_point_group(8, 256, 64, 64))
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS, u4 with zero points, weights [N,K]]"] and rf == []
    check(new, r"%zero = u4\[64,4\] parameter\(3\)", r"custom-call\(%lhs, %w, %scales, %zero, %bias\)")
    new, rw, rf = hlo.rewrite(hm.k_minor_s8_batched(3, 20, 1024, 392))
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s8, weights [N,K]]"] and rf == []
    check(new, r"%scale = f32\[3,392\] parameter\(2\)", r"custom-call\(%lhs, %w, %scale\)", r"rhs_contracting_dim = 1 : i64")
    # scales broadcast along the wrong dimension of [N,K] weights are no dequantisation of them
    bad = hm.k_minor_s8_channel(16, 64, 64).replace("broadcast(%scale), dimensions={0}", "broadcast(%scale), dimensions={1}")
    assert hlo.rewrite(bad)[1] == []
    # the [K,N] spelling keeps its attributes (no rhs_contracting_dim)
    assert "rhs_contracting_dim" not in hlo.rewrite(hm.c1_s8_channel())[0]


def test_ragged_dot_over_k_minor_experts():
    """ragged-dot whose experts are stored [G,N,K] (rhs_contracting_dims = {2}): the same call with
    rhs_contracting_dim = 1; scales [G,N] or [G,N,K/g]."""
    new, rw, rf = hlo.rewrite(hm.k_minor_ragged_s8_experts(32, 512, 256, 4))
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS, s8, ragged over 4 groups, weights [G,N,K]]"] and rf == []
    check(new, r"%w = s8\[4,256,512\] parameter\(1\)", r"custom-call\(%lhs, %w, %scale, %bias, %sizes\)",
          r"scale_group_size = 0 : i64, rhs_contracting_dim = 1 : i64")
    new, rw, rf = hlo.rewrite(hm.k_minor_ragged_s4_group_experts(32, 512, 256, 4, 128))
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS, s4, ragged over 4 groups, weights [G,N,K]]"] and rf == []
    check(new, r"%scales = bf16\[4,256,4\] parameter\(2\)", r"custom-call\(%lhs, %w, %scales, %bias, %sizes\)",
          r"scale_group_size = 128 : i64, rhs_contracting_dim = 1 : i64")
    # the group dimension anywhere but in front is left alone, as for [G,K,N]
    bad = hm.k_minor_ragged_s8_experts(32, 512, 256, 4).replace("rhs_group_dims={0}", "rhs_group_dims={1}")
    _, rw, rf = hlo.rewrite(bad)
    assert rw == [] and any("group dimension leading the weights" in r for r in rf)


@pytest.mark.parametrize("case", hm.INT4_DOT_CASES, ids=[c[0] for c in hm.INT4_DOT_CASES])
@pytest.mark.parametrize("weights_on_lhs", [False, True])
def test_reference_int4_shape_table_is_taken(case, weights_on_lhs):
    """Every shape of Int4TestCases (fusion_emitter_int4_device_test.cc:609-645), weights on either
    side: an f32 dot of unscaled converted s4 weights becomes one call with unit scales, the
    contracting dimensions as attributes and -- weights on the lhs -- a transposed result."""
    name, lhs, rhs, lc, rc, out = case
    text = hm.int4_weights_dot(case, weights_on_lhs)
    new, rw, rf = hlo.rewrite(text)
    assert len(rw) == 1 and rf == [], (rw, rf)
    rank = len(lhs)
    w_c, a_c = (lc, rc) if weights_on_lhs else (rc, lc)
    tags = ["DEFAULT", "s4"]
    if w_c == rank - 1:
        tags.append("weights [N,K]")
    if weights_on_lhs:
        tags.append("weights as lhs")
    if a_c == rank - 2:
        tags.append("activations [K,M]")
    tags.append("f32 result")
    assert rw == ["dot -> xla_amd.dequant_dot [%s]" % ", ".join(tags)], rw
    n = (lhs if weights_on_lhs else rhs)[rank - (2 if w_c == rank - 1 else 1)]
    check(new, r"f32\[\] constant\(1\)", r"f32\[%d\]\{0\} broadcast\(%%\S+\), dimensions=\{\}" % n,
          r"f32\[%s\]\{[0-9,]+\}(, s8\[\d+\]\{0\}\))? custom-call\(%%a, %%w, %%\S+unit_scales\)" % ",".join(str(v) for v in out),
          r"dequant_type = 11 : i32, dot_type = 11 : i32")
    assert ("result_transposed = true" in new) == weights_on_lhs
    assert ("lhs_contracting_dim = 0" in new) == (a_c == rank - 2)
    assert ("rhs_contracting_dim = 1" in new) == (w_c == rank - 1)
    assert sorted(set(opcodes(new)) - {"get-tuple-element"}) == ["broadcast", "constant", "custom-call", "parameter"]


def test_dequant_dot_with_f8_result():
    """The D scaling of gemm_rewriter_fp8_test.cc:1665-1690 / :1730-1748 behind a weight-only dot: the
    scale is the call's last operand and the result is f8e4m3fn.  A value that also feeds its own amax
    keeps its f32 result and leaves scaling, clamp, convert and the reduce to the ops after the call."""
    for mul in (False, True):
        new, rw, rf = hlo.rewrite(hm.c2_s4_group_f8_result(8, 256, 64, 64, multiply=mul))
        assert rw == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4, f8 result]"] and rf == [], (rw, rf)
        check(new, r"f8e4m3fn\[8,64\]\{1,0\}(, s8\[\d+\]\{0\}\))? custom-call\(%lhs, %w, %scales, %bias, %d_scale\)",
              r"d_scale_multiplies = %s" % ("true" if mul else "false"))
        assert sorted(set(opcodes(new)) - {"get-tuple-element"}) == ["custom-call", "parameter"]
    text = hm.c2_s4_group_f8_result(8, 256, 64, 64)
    text = text.replace("ENTRY %main {", "%max_f32 {\n  %a = f32[] parameter(0)\n  %b = f32[] parameter(1)\n"
                        "  ROOT %m = f32[] maximum(%a, %b)\n}\n\nENTRY %main {")
    text = text.replace("  ROOT %out = f8e4m3fn[8,64] convert(%clamped)\n", """  %out = f8e4m3fn[8,64] convert(%clamped)
  %abs_v = f32[8,64] abs(%silu)
  %ninf = f32[] constant(-inf)
  %amax = f32[] reduce(%abs_v, %ninf), dimensions={0,1}, to_apply=%max_f32
  ROOT %result = (f8e4m3fn[8,64], f32[]) tuple(%out, %amax)
""")
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4, f32 result]"], (rw, rf)
    assert all("clamp/convert to f8e4m3fn found but not rewritten" in r for r in rf), rf   # the quantizer's matcher looked too
    assert {"clamp", "reduce", "divide", "abs"} <= set(opcodes(new))
    # a clamp to anything but +-448 is not the f8 saturation: the f32 value is the call's result
    bad = hm.c2_s4_group_f8_result(8, 256, 64, 64).replace("constant(448)", "constant(240)")
    new, rw, rf = hlo.rewrite(bad)
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4, f32 result]"] and "clamp" in opcodes(new)


def test_f32_result_with_scales_and_epilogue():
    """The value leaving the pattern may be f32: C2's module without its final convert keeps the f32
    SiLU value as the result (epilogue ops f32-typed, dequantise multiply bf16-typed)."""
    text = hm.c2_s4_group(M=8, K=256, N=64, group=64)
    assert "ROOT %out = bf16[8,64] convert(" in text
    root = re.search(r"ROOT %out = bf16\[8,64\] convert\((%\w+)\)", text).group(1)
    text = re.sub(r"  ROOT %out = bf16\[8,64\] convert\(%\w+\)\n", "", text).replace("  %s = " % root, "  ROOT %s = " % root)
    new, rw, rf = hlo.rewrite(text)
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4, f32 result]"], (rw, rf)
    check(new, r"f32\[8,64\]\{1,0\}")
