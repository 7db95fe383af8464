"""HLO text of the five benchmark configurations, parameterised by shape.

These are the modules a framework would hand to XLA: plain convert / multiply / dot /
reduce ops with no custom calls.  The CPU backend runs them as they are; the rewrite pass
turns each into one custom call of this library.
"""

REDUCERS = """
%add_f32 {
  %a = f32[] parameter(0)
  %b = f32[] parameter(1)
  ROOT %s = f32[] add(%a, %b)
}

%max_f32 {
  %a = f32[] parameter(0)
  %b = f32[] parameter(1)
  ROOT %m = f32[] maximum(%a, %b)
}
"""


def c1_s8_channel(M=16, K=4096, N=4096):
    """bf16 [M,K] . (convert(s8 [K,N]) * f32 scale[N]) -> bf16; f32 multiply, one final rounding."""
    return f"""HloModule c1_s8_channel_dequant_dot

ENTRY %main {{
  %lhs = bf16[{M},{K}] parameter(0)
  %w = s8[{K},{N}] parameter(1)
  %scale = f32[{N}] parameter(2)
  %lhs_f32 = f32[{M},{K}] convert(%lhs)
  %w_f32 = f32[{K},{N}] convert(%w)
  %scale_b = f32[{K},{N}] broadcast(%scale), dimensions={{1}}
  %w_deq = f32[{K},{N}] multiply(%w_f32, %scale_b)
  %dot = f32[{M},{N}] dot(%lhs_f32, %w_deq), lhs_contracting_dims={{1}}, rhs_contracting_dims={{0}}
  ROOT %out = bf16[{M},{N}] convert(%dot)
}}
"""


def c2_s4_group(M=1, K=8192, N=28672, group=128):
    """bf16 [M,K] . bf16(convert(s4 [K,N]) * bf16 scale[K/g,N]) + bias, SiLU in f32 -> bf16.
    The dequantise multiply is bf16-typed, as in XLA's int4 tests."""
    G = K // group
    return f"""HloModule c2_s4_group_dequant_dot

ENTRY %main {{
  %lhs = bf16[{M},{K}] parameter(0)
  %w = s4[{K},{N}] parameter(1)
  %scales = bf16[{G},{N}] parameter(2)
  %bias = bf16[{N}] parameter(3)
  %w_s8 = s8[{K},{N}] convert(%w)
  %w_g = s8[{G},{group},{N}] reshape(%w_s8)
  %w_bf16 = bf16[{G},{group},{N}] convert(%w_g)
  %scales_b = bf16[{G},{group},{N}] broadcast(%scales), dimensions={{0,2}}
  %w_deq_g = bf16[{G},{group},{N}] multiply(%w_bf16, %scales_b)
  %w_deq = bf16[{K},{N}] reshape(%w_deq_g)
  %dot = f32[{M},{N}] dot(%lhs, %w_deq), lhs_contracting_dims={{1}}, rhs_contracting_dims={{0}}
  %bias_f32 = f32[{N}] convert(%bias)
  %bias_b = f32[{M},{N}] broadcast(%bias_f32), dimensions={{1}}
  %z = f32[{M},{N}] add(%dot, %bias_b)
  %neg = f32[{M},{N}] negate(%z)
  %exp = f32[{M},{N}] exponential(%neg)
  %one = f32[] constant(1)
  %one_b = f32[{M},{N}] broadcast(%one), dimensions={{}}
  %den = f32[{M},{N}] add(%one_b, %exp)
  %sig = f32[{M},{N}] divide(%one_b, %den)
  %silu = f32[{M},{N}] multiply(%z, %sig)
  ROOT %out = bf16[{M},{N}] convert(%silu)
}}
"""


def c2_s4_group_f8_result(M=8, K=8192, N=28672, group=128, multiply=False):
    """c2_s4_group whose SiLU value leaves as f8e4m3fn: divided (or multiplied) by a per-tensor scale,
    clamped to +-448 and converted -- the D scaling of gemm_rewriter_fp8_test.cc:1665-1690 / :1730-1748
    behind a weight-only dot, i.e. the activations of the next fp8 dot made in this dot's store."""
    text = c2_s4_group(M, K, N, group)
    head, _ = text.split(f"  ROOT %out = bf16[{M},{N}] convert(%silu)")
    op = "multiply" if multiply else "divide"
    return head + f"""  %d_scale = f32[] parameter(4)
  %d_scale_b = f32[{M},{N}] broadcast(%d_scale), dimensions={{}}
  %scaled = f32[{M},{N}] {op}(%silu, %d_scale_b)
  %lo = f32[] constant(-448)
  %lo_b = f32[{M},{N}] broadcast(%lo), dimensions={{}}
  %hi = f32[] constant(448)
  %hi_b = f32[{M},{N}] broadcast(%hi), dimensions={{}}
  %clamped = f32[{M},{N}] clamp(%lo_b, %scaled, %hi_b)
  ROOT %out = f8e4m3fn[{M},{N}] convert(%clamped)
}}
"""


def u4_zero_point_group(M=8, K=4096, N=4096, group=128, typed="bf16"):
    """bf16 [M,K] . ((convert(u4 [K,N]) - convert(u4 zero[K/g,N])) * scale[K/g,N]) + bias -> bf16: the
    asymmetric 4-bit weight-only form (one zero point and one scale per group and channel).
    typed="bf16": convert, subtract and multiply are bf16-typed, one rounding per dequantised weight
    (the difference of two integers below 16 is exact); typed="f32" is not taken by the kernels for
    grouped scales and shows a refusal."""
    G, t = K // group, typed
    return f"""HloModule u4_zero_point_group_dequant_dot

ENTRY %main {{
  %lhs = bf16[{M},{K}] parameter(0)
  %w = u4[{K},{N}] parameter(1)
  %scales = {t}[{G},{N}] parameter(2)
  %zero = u4[{G},{N}] parameter(3)
  %bias = bf16[{N}] parameter(4)
  %w_g = u4[{G},{group},{N}] reshape(%w)
  %w_t = {t}[{G},{group},{N}] convert(%w_g)
  %zero_t = {t}[{G},{N}] convert(%zero)
  %zero_b = {t}[{G},{group},{N}] broadcast(%zero_t), dimensions={{0,2}}
  %w_centered = {t}[{G},{group},{N}] subtract(%w_t, %zero_b)
  %scales_b = {t}[{G},{group},{N}] broadcast(%scales), dimensions={{0,2}}
  %w_deq_g = {t}[{G},{group},{N}] multiply(%w_centered, %scales_b)
  %w_deq = {t}[{K},{N}] reshape(%w_deq_g)
  %dot = f32[{M},{N}] dot(%lhs, %w_deq), lhs_contracting_dims={{1}}, rhs_contracting_dims={{0}}
  %bias_f32 = f32[{N}] convert(%bias)
  %bias_b = f32[{M},{N}] broadcast(%bias_f32), dimensions={{1}}
  %z = f32[{M},{N}] add(%dot, %bias_b)
  ROOT %out = bf16[{M},{N}] convert(%z)
}}
"""


def ragged_s8_experts(M=32, K=4096, N=4096, groups=8, sizes_ty="s32"):
    """ragged-dot(bf16 [M,K], convert(s8 [G,K,N]) * f32 scale[G,N], group sizes [G]) + bias -> bf16:
    a decode step of a mixture of experts whose tokens are sorted by expert (the shape of
    ragged_dot_rewriter_test.cc:78-82 with quantised weights)."""
    G = groups
    return f"""HloModule ragged_s8_experts_dequant_dot

ENTRY %main {{
  %lhs = bf16[{M},{K}] parameter(0)
  %w = s8[{G},{K},{N}] parameter(1)
  %scale = f32[{G},{N}] parameter(2)
  %bias = bf16[{N}] parameter(3)
  %sizes = {sizes_ty}[{G}] parameter(4)
  %lhs_f32 = f32[{M},{K}] convert(%lhs)
  %w_f32 = f32[{G},{K},{N}] convert(%w)
  %scale_b = f32[{G},{K},{N}] broadcast(%scale), dimensions={{0,2}}
  %w_deq = f32[{G},{K},{N}] multiply(%w_f32, %scale_b)
  %dot = f32[{M},{N}] ragged-dot(%lhs_f32, %w_deq, %sizes), lhs_contracting_dims={{1}}, rhs_contracting_dims={{1}}, lhs_ragged_dims={{0}}, rhs_group_dims={{0}}
  %bias_f32 = f32[{N}] convert(%bias)
  %bias_b = f32[{M},{N}] broadcast(%bias_f32), dimensions={{1}}
  %z = f32[{M},{N}] add(%dot, %bias_b)
  ROOT %out = bf16[{M},{N}] convert(%z)
}}
"""


def ragged_s4_group_experts(M=32, K=4096, N=4096, groups=8, group=128):
    """ragged-dot(bf16 [M,K], bf16(convert(s4 [G,K,N]) * bf16 scale[G,K/g,N]), group sizes [G]) + bias
    -> bf16: 4-bit experts with one scale per `group` rows of K and channel, the dequantise multiply
    bf16-typed (one rounding per weight) as in c2_s4_group."""
    G, Kg = groups, K // group
    return f"""HloModule ragged_s4_group_experts_dequant_dot

ENTRY %main {{
  %lhs = bf16[{M},{K}] parameter(0)
  %w = s4[{G},{K},{N}] parameter(1)
  %scales = bf16[{G},{Kg},{N}] parameter(2)
  %bias = bf16[{N}] parameter(3)
  %sizes = s32[{G}] parameter(4)
  %w_s8 = s8[{G},{K},{N}] convert(%w)
  %w_g = s8[{G},{Kg},{group},{N}] reshape(%w_s8)
  %w_bf16 = bf16[{G},{Kg},{group},{N}] convert(%w_g)
  %scales_b = bf16[{G},{Kg},{group},{N}] broadcast(%scales), dimensions={{0,1,3}}
  %w_deq_g = bf16[{G},{Kg},{group},{N}] multiply(%w_bf16, %scales_b)
  %w_deq = bf16[{G},{K},{N}] reshape(%w_deq_g)
  %dot = f32[{M},{N}] ragged-dot(%lhs, %w_deq, %sizes), lhs_contracting_dims={{1}}, rhs_contracting_dims={{1}}, lhs_ragged_dims={{0}}, rhs_group_dims={{0}}
  %bias_f32 = f32[{N}] convert(%bias)
  %bias_b = f32[{M},{N}] broadcast(%bias_f32), dimensions={{1}}
  %z = f32[{M},{N}] add(%dot, %bias_b)
  ROOT %out = bf16[{M},{N}] convert(%z)
}}
"""


def batched_s4_group(B=4, M=8, K=1024, N=512, group=128):
    """bf16 [B,M,K] . bf16(convert(s4 [B,K,N]) * bf16 scale[B,K/g,N]), batch dimension 0 -> bf16
    [B,M,N]: equally sized experts with 4-bit weights and grouped scales."""
    Kg = K // group
    return f"""HloModule batched_s4_group_dequant_dot

ENTRY %main {{
  %lhs = bf16[{B},{M},{K}] parameter(0)
  %w = s4[{B},{K},{N}] parameter(1)
  %scales = bf16[{B},{Kg},{N}] parameter(2)
  %w_s8 = s8[{B},{K},{N}] convert(%w)
  %w_g = s8[{B},{Kg},{group},{N}] reshape(%w_s8)
  %w_bf16 = bf16[{B},{Kg},{group},{N}] convert(%w_g)
  %scales_b = bf16[{B},{Kg},{group},{N}] broadcast(%scales), dimensions={{0,1,3}}
  %w_deq_g = bf16[{B},{Kg},{group},{N}] multiply(%w_bf16, %scales_b)
  %w_deq = bf16[{B},{K},{N}] reshape(%w_deq_g)
  %dot = f32[{B},{M},{N}] dot(%lhs, %w_deq), lhs_batch_dims={{0}}, rhs_batch_dims={{0}}, lhs_contracting_dims={{2}}, rhs_contracting_dims={{1}}
  ROOT %out = bf16[{B},{M},{N}] convert(%dot)
}}
"""


def c3_fp8(M=8192, K=8192, N=8192, typed="f32", vector_scales=False):
    """f8 [M,K] . f8 [K,N] with per-tensor scales, + bias, GELU(tanh) -> bf16.  typed="f32":
    f32 ops and one final rounding; typed="bf16": every op bf16-typed (the shape of
    gemm_rewriter_fp8_test.cc:1110-1141).  vector_scales: a_scale is f32[M], one per row of a
    (what a row-wise quantizer hands on), and b_scale f32[N], one per output channel."""
    t = typed
    scale_decl = (f"  %a_scale = {t}[] parameter(2)\n  %b_scale = {t}[] parameter(3)\n")
    a_dims, b_dims = "", ""
    if vector_scales:
        scale_decl = (f"  %a_scale = {t}[{M}] parameter(2)\n  %b_scale = {t}[{N}] parameter(3)\n")
        a_dims, b_dims = "0", "1"
    tail = (f"  ROOT %out = bf16[{M},{N}] convert(%gelu)\n" if t == "f32" else "")
    root = "" if t == "f32" else "ROOT "
    bias_line = (f"  %bias_t = f32[{N}] convert(%bias)\n" if t == "f32" else "")
    bias_name = "%bias_t" if t == "f32" else "%bias"
    return f"""HloModule c3_fp8_scaled_dot

ENTRY %main {{
  %a = f8e4m3fn[{M},{K}] parameter(0)
  %b = f8e4m3fn[{K},{N}] parameter(1)
{scale_decl}  %bias = bf16[{N}] parameter(4)
  %a_t = {t}[{M},{K}] convert(%a)
  %b_t = {t}[{K},{N}] convert(%b)
  %a_scale_b = {t}[{M},{K}] broadcast(%a_scale), dimensions={{{a_dims}}}
  %b_scale_b = {t}[{K},{N}] broadcast(%b_scale), dimensions={{{b_dims}}}
  %a_deq = {t}[{M},{K}] multiply(%a_t, %a_scale_b)
  %b_deq = {t}[{K},{N}] multiply(%b_t, %b_scale_b)
  %dot = {t}[{M},{N}] dot(%a_deq, %b_deq), lhs_contracting_dims={{1}}, rhs_contracting_dims={{0}}
{bias_line}  %bias_b = {t}[{M},{N}] broadcast({bias_name}), dimensions={{1}}
  %z = {t}[{M},{N}] add(%dot, %bias_b)
  %z2 = {t}[{M},{N}] multiply(%z, %z)
  %z3 = {t}[{M},{N}] multiply(%z, %z2)
  %c0 = {t}[] constant(0.044715)
  %c0_b = {t}[{M},{N}] broadcast(%c0), dimensions={{}}
  %z3c = {t}[{M},{N}] multiply(%z3, %c0_b)
  %inner = {t}[{M},{N}] add(%z, %z3c)
  %c1 = {t}[] constant(0.797884583)
  %c1_b = {t}[{M},{N}] broadcast(%c1), dimensions={{}}
  %arg = {t}[{M},{N}] multiply(%inner, %c1_b)
  %tanh = {t}[{M},{N}] tanh(%arg)
  %one = {t}[] constant(1)
  %one_b = {t}[{M},{N}] broadcast(%one), dimensions={{}}
  %onep = {t}[{M},{N}] add(%tanh, %one_b)
  %half = {t}[] constant(0.5)
  %half_b = {t}[{M},{N}] broadcast(%half), dimensions={{}}
  %cdf = {t}[{M},{N}] multiply(%onep, %half_b)
  {root}%gelu = {t}[{M},{N}] multiply(%z, %cdf)
{tail}}}
"""


def fp8_batched(B=10, M=16, K=32, N=16, rhs_nk=False):
    """Batched f8 dot with per-tensor scales -> bf16 (the shape of gemm_rewriter_fp8_test.cc:941-957,
    with the result converted to bf16)."""
    bshape = f"{B},{N},{K}" if rhs_nk else f"{B},{K},{N}"
    rcd = 2 if rhs_nk else 1
    return f"""HloModule fp8_batched_scaled_dot

ENTRY %main {{
  %x = f8e4m3fn[{B},{M},{K}] parameter(0)
  %y = f8e4m3fn[{bshape}] parameter(1)
  %x_scale = f32[] parameter(2)
  %y_scale = f32[] parameter(3)
  %x_f32 = f32[{B},{M},{K}] convert(%x)
  %y_f32 = f32[{bshape}] convert(%y)
  %x_scale_b = f32[{B},{M},{K}] broadcast(%x_scale), dimensions={{}}
  %y_scale_b = f32[{bshape}] broadcast(%y_scale), dimensions={{}}
  %x_unscaled = f32[{B},{M},{K}] multiply(%x_f32, %x_scale_b)
  %y_unscaled = f32[{bshape}] multiply(%y_f32, %y_scale_b)
  %dot = f32[{B},{M},{N}] dot(%x_unscaled, %y_unscaled), lhs_contracting_dims={{2}}, rhs_contracting_dims={{{rcd}}}, lhs_batch_dims={{0}}, rhs_batch_dims={{0}}
  ROOT %out = bf16[{B},{M},{N}] convert(%dot)
}}
"""


def mxfp8_block_scaled_dot(M=8192, K=8192, N=8192, batch=0, bias_gelu=False):
    """MXFP8: f8e4m3fn operands [M,K] and [N,K] with one f8e8m0fnu scale per 32 elements of K, as
    the "__op$block_scaled_dot" custom call of block_scaling_rewriter.h:48-69 -> bf16 [M,N].
    batch: a leading batch dimension on every operand and the result (the header's second example).
    bias_gelu: the custom call yields f32 and a bias add and GELU(tanh) follow before the convert
    to bf16, as behind the dot of c3_fp8."""
    lead = f"{batch}," if batch else ""
    o = f"{lead}{M},{N}"
    head = f"""HloModule mxfp8_block_scaled_dot

ENTRY %main {{
  %lhs = f8e4m3fn[{lead}{M},{K}] parameter(0)
  %rhs = f8e4m3fn[{lead}{N},{K}] parameter(1)
  %lhs_scale = f8e8m0fnu[{lead}{M},{K // 32}] parameter(2)
  %rhs_scale = f8e8m0fnu[{lead}{N},{K // 32}] parameter(3)
"""
    if not bias_gelu:
        return head + f"""  ROOT %result = bf16[{o}] custom-call(%lhs, %rhs, %lhs_scale, %rhs_scale), custom_call_target="__op$block_scaled_dot"
}}
"""
    return head + f"""  %bias = bf16[{N}] parameter(4)
  %dot = f32[{o}] custom-call(%lhs, %rhs, %lhs_scale, %rhs_scale), custom_call_target="__op$block_scaled_dot"
  %bias_t = f32[{N}] convert(%bias)
  %bias_b = f32[{o}] broadcast(%bias_t), dimensions={{{2 if batch else 1}}}
  %z = f32[{o}] add(%dot, %bias_b)
  %z2 = f32[{o}] multiply(%z, %z)
  %z3 = f32[{o}] multiply(%z, %z2)
  %c0 = f32[] constant(0.044715)
  %c0_b = f32[{o}] broadcast(%c0), dimensions={{}}
  %z3c = f32[{o}] multiply(%z3, %c0_b)
  %inner = f32[{o}] add(%z, %z3c)
  %c1 = f32[] constant(0.797884583)
  %c1_b = f32[{o}] broadcast(%c1), dimensions={{}}
  %arg = f32[{o}] multiply(%inner, %c1_b)
  %tanh = f32[{o}] tanh(%arg)
  %one = f32[] constant(1)
  %one_b = f32[{o}] broadcast(%one), dimensions={{}}
  %onep = f32[{o}] add(%tanh, %one_b)
  %half = f32[] constant(0.5)
  %half_b = f32[{o}] broadcast(%half), dimensions={{}}
  %cdf = f32[{o}] multiply(%onep, %half_b)
  %gelu = f32[{o}] multiply(%z, %cdf)
  ROOT %out = bf16[{o}] convert(%gelu)
}}
"""


def c3_fp8_f8_result(M=8192, K=8192, N=8192, multiply=False, vector_scales=False, amax=False):
    """The f32-typed C3 module with an f8e4m3fn result: the GELU value is divided (or multiplied)
    by a per-tensor scale, clamped to +-448 and converted -- the D scaling of
    gemm_rewriter_fp8_test.cc:1665-1690 (divide) / :1730-1748 (multiply)."""
    text = c3_fp8(M, K, N, typed="f32", vector_scales=vector_scales)
    head, _ = text.split(f"  ROOT %out = bf16[{M},{N}] convert(%gelu)")
    op = "multiply" if multiply else "divide"
    if amax:  # the result's own amax beside it (gemm_rewriter_fp8_test.cc:2559-2600)
        head = head.replace("ENTRY %main {", "%max_f32 {\n  %a = f32[] parameter(0)\n  %b = f32[] parameter(1)\n"
                            "  ROOT %m = f32[] maximum(%a, %b)\n}\n\nENTRY %main {")
        root, tail = "", f"""  %abs_v = f32[{M},{N}] abs(%gelu)
  %ninf = f32[] constant(-inf)
  %amax = f32[] reduce(%abs_v, %ninf), dimensions={{0,1}}, to_apply=%max_f32
  ROOT %result = (f8e4m3fn[{M},{N}], f32[]) tuple(%out, %amax)
"""
    else:
        root, tail = "ROOT ", ""
    return head + f"""  %d_scale = f32[] parameter(5)
  %d_scale_b = f32[{M},{N}] broadcast(%d_scale), dimensions={{}}
  %scaled = f32[{M},{N}] {op}(%gelu, %d_scale_b)
  %lo = f32[] constant(-448)
  %lo_b = f32[{M},{N}] broadcast(%lo), dimensions={{}}
  %hi = f32[] constant(448)
  %hi_b = f32[{M},{N}] broadcast(%hi), dimensions={{}}
  %clamped = f32[{M},{N}] clamp(%lo_b, %scaled, %hi_b)
  {root}%out = f8e4m3fn[{M},{N}] convert(%clamped)
{tail}}}
"""


def c4_quantize(rows=16384, cols=8192, rmsnorm=True, eps=1e-6, rsqrt=False):
    """RMSNorm (f32 math, bf16 result) -> per-row amax -> scale = amax/448 -> clamp -> f8e4m3fn.
    rsqrt: the reciprocal root spelled as one rsqrt instruction instead of 1 / sqrt."""
    R, C = rows, cols
    root = (f"  %rinv = f32[{R}] rsqrt(%ms_eps)\n" if rsqrt else
            f"  %rt = f32[{R}] sqrt(%ms_eps)\n  %one = f32[] constant(1)\n"
            f"  %one_b = f32[{R}] broadcast(%one), dimensions={{}}\n  %rinv = f32[{R}] divide(%one_b, %rt)\n")
    if rmsnorm:
        norm = f"""  %gamma = bf16[{C}] parameter(1)
  %x_f32 = f32[{R},{C}] convert(%x)
  %sq = f32[{R},{C}] multiply(%x_f32, %x_f32)
  %zero = f32[] constant(0)
  %ssum = f32[{R}] reduce(%sq, %zero), dimensions={{1}}, to_apply=%add_f32
  %count = f32[] constant({C})
  %count_b = f32[{R}] broadcast(%count), dimensions={{}}
  %ms = f32[{R}] divide(%ssum, %count_b)
  %eps = f32[] constant({eps!r})
  %eps_b = f32[{R}] broadcast(%eps), dimensions={{}}
  %ms_eps = f32[{R}] add(%ms, %eps_b)
{root}  %rinv_b = f32[{R},{C}] broadcast(%rinv), dimensions={{0}}
  %xn = f32[{R},{C}] multiply(%x_f32, %rinv_b)
  %gamma_f32 = f32[{C}] convert(%gamma)
  %gamma_b = f32[{R},{C}] broadcast(%gamma_f32), dimensions={{1}}
  %y_f32 = f32[{R},{C}] multiply(%xn, %gamma_b)
  %y = bf16[{R},{C}] convert(%y_f32)
"""
        ysrc = "%y"
    else:
        norm = ""
        ysrc = "%x"
    return f"""HloModule c4_rowwise_quantize_fp8
{REDUCERS}
ENTRY %main {{
  %x = bf16[{R},{C}] parameter(0)
{norm}  %yf = f32[{R},{C}] convert({ysrc})
  %absy = f32[{R},{C}] abs(%yf)
  %ninf = f32[] constant(-inf)
  %amax = f32[{R}] reduce(%absy, %ninf), dimensions={{1}}, to_apply=%max_f32
  %c448 = f32[] constant(448)
  %c448_b = f32[{R}] broadcast(%c448), dimensions={{}}
  %scale = f32[{R}] divide(%amax, %c448_b)
  %scale_b = f32[{R},{C}] broadcast(%scale), dimensions={{0}}
  %scaled = f32[{R},{C}] divide(%yf, %scale_b)
  %lo = f32[] constant(-448)
  %lo_b = f32[{R},{C}] broadcast(%lo), dimensions={{}}
  %hi = f32[] constant(448)
  %hi_b = f32[{R},{C}] broadcast(%hi), dimensions={{}}
  %clamped = f32[{R},{C}] clamp(%lo_b, %scaled, %hi_b)
  %q = f8e4m3fn[{R},{C}] convert(%clamped)
  ROOT %result = (f8e4m3fn[{R},{C}], f32[{R}]) tuple(%q, %scale)
}}
"""


def quantize_then_fp8_dot(rows=16384, cols=8192, N=8192, eps=1e-6):
    """One layer boundary: RMSNorm + row-wise f8e4m3fn quantisation of x[rows,cols] (the C4
    pattern), whose codes and per-row scales are dequantised straight into a dot with f8
    weights [cols,N] under a per-tensor scale -> bf16 [rows,N]."""
    R, C = rows, cols
    text = c4_quantize(rows, cols, rmsnorm=True, eps=eps).replace("HloModule c4_rowwise_quantize_fp8",
                                                                  "HloModule quantize_then_fp8_dot")
    head, _ = text.split("  ROOT %result")
    return head + f"""  %w = f8e4m3fn[{C},{N}] parameter(2)
  %w_scale = f32[] parameter(3)
  %q_f32 = f32[{R},{C}] convert(%q)
  %a_deq = f32[{R},{C}] multiply(%q_f32, %scale_b)
  %w_f32 = f32[{C},{N}] convert(%w)
  %w_scale_b = f32[{C},{N}] broadcast(%w_scale), dimensions={{}}
  %w_deq = f32[{C},{N}] multiply(%w_f32, %w_scale_b)
  %dot = f32[{R},{N}] dot(%a_deq, %w_deq), lhs_contracting_dims={{1}}, rhs_contracting_dims={{0}}
  ROOT %out = bf16[{R},{N}] convert(%dot)
}}
"""


def c5_s8_batched(B=8, M=512, K=4096, N=14336):
    """bf16 [B,M,K] . (convert(s8 [B,K,N]) * f32 scale[B,N]), batch dimension 0 -> bf16 [B,M,N]."""
    return f"""HloModule c5_s8_batched_dequant_dot

ENTRY %main {{
  %lhs = bf16[{B},{M},{K}] parameter(0)
  %w = s8[{B},{K},{N}] parameter(1)
  %scale = f32[{B},{N}] parameter(2)
  %lhs_f32 = f32[{B},{M},{K}] convert(%lhs)
  %w_f32 = f32[{B},{K},{N}] convert(%w)
  %scale_b = f32[{B},{K},{N}] broadcast(%scale), dimensions={{0,2}}
  %w_deq = f32[{B},{K},{N}] multiply(%w_f32, %scale_b)
  %dot = f32[{B},{M},{N}] dot(%lhs_f32, %w_deq), lhs_batch_dims={{0}}, lhs_contracting_dims={{2}}, rhs_batch_dims={{0}}, rhs_contracting_dims={{1}}
  ROOT %out = bf16[{B},{M},{N}] convert(%dot)
}}
"""


# ---- weights stored [N,K]: the dot contracts the minor dimension of its rhs, the layout of a
# checkpoint written for y = x W^T (fusion_emitter_int4_device_test.cc:867-892)

def k_minor_s8_channel(M=16, K=4096, N=4096):
    """bf16 [M,K] . (convert(s8 [N,K]) * f32 scale[N])^T -> bf16; f32 multiply."""
    return f"""HloModule k_minor_s8_channel_dequant_dot

ENTRY %main {{
  %lhs = bf16[{M},{K}] parameter(0)
  %w = s8[{N},{K}] parameter(1)
  %scale = f32[{N}] parameter(2)
  %lhs_f32 = f32[{M},{K}] convert(%lhs)
  %w_f32 = f32[{N},{K}] convert(%w)
  %scale_b = f32[{N},{K}] broadcast(%scale), dimensions={{0}}
  %w_deq = f32[{N},{K}] multiply(%w_f32, %scale_b)
  %dot = f32[{M},{N}] dot(%lhs_f32, %w_deq), lhs_contracting_dims={{1}}, rhs_contracting_dims={{1}}
  ROOT %out = bf16[{M},{N}] convert(%dot)
}}
"""


def k_minor_s4_group(M=1, K=8192, N=28672, group=128, typed="bf16"):
    """bf16 [M,K] . typed(convert(s4 [N,K]) * scale[N,K/g])^T + bias, SiLU in f32 -> bf16."""
    G, t = K // group, typed
    return f"""HloModule k_minor_s4_group_dequant_dot

ENTRY %main {{
  %lhs = bf16[{M},{K}] parameter(0)
  %w = s4[{N},{K}] parameter(1)
  %scales = {t}[{N},{G}] parameter(2)
  %bias = bf16[{N}] parameter(3)
  %w_s8 = s8[{N},{K}] convert(%w)
  %w_g = s8[{N},{G},{group}] reshape(%w_s8)
  %w_t = {t}[{N},{G},{group}] convert(%w_g)
  %scales_b = {t}[{N},{G},{group}] broadcast(%scales), dimensions={{0,1}}
  %w_deq_g = {t}[{N},{G},{group}] multiply(%w_t, %scales_b)
  %w_deq = {t}[{N},{K}] reshape(%w_deq_g)
  %dot = f32[{M},{N}] dot(%lhs, %w_deq), lhs_contracting_dims={{1}}, rhs_contracting_dims={{1}}
  %bias_f32 = f32[{N}] convert(%bias)
  %bias_b = f32[{M},{N}] broadcast(%bias_f32), dimensions={{1}}
  %z = f32[{M},{N}] add(%dot, %bias_b)
  %neg = f32[{M},{N}] negate(%z)
  %exp = f32[{M},{N}] exponential(%neg)
  %one = f32[] constant(1)
  %one_b = f32[{M},{N}] broadcast(%one), dimensions={{}}
  %den = f32[{M},{N}] add(%one_b, %exp)
  %sig = f32[{M},{N}] divide(%one_b, %den)
  %silu = f32[{M},{N}] multiply(%z, %sig)
  ROOT %out = bf16[{M},{N}] convert(%silu)
}}
"""


def k_minor_u4_zero_point_group(M=8, K=4096, N=4096, group=128):
    """bf16 [M,K] . bf16((convert(u4 [N,K]) - convert(u4 zero[N,K/g])) * bf16 scale[N,K/g])^T + bias -> bf16."""
    G = K // group
    return f"""HloModule k_minor_u4_zero_point_group_dequant_dot

ENTRY %main {{
  %lhs = bf16[{M},{K}] parameter(0)
  %w = u4[{N},{K}] parameter(1)
  %scales = bf16[{N},{G}] parameter(2)
  %zero = u4[{N},{G}] parameter(3)
  %bias = bf16[{N}] parameter(4)
  %w_g = u4[{N},{G},{group}] reshape(%w)
  %w_t = bf16[{N},{G},{group}] convert(%w_g)
  %zero_t = bf16[{N},{G}] convert(%zero)
  %zero_b = bf16[{N},{G},{group}] broadcast(%zero_t), dimensions={{0,1}}
  %w_centered = bf16[{N},{G},{group}] subtract(%w_t, %zero_b)
  %scales_b = bf16[{N},{G},{group}] broadcast(%scales), dimensions={{0,1}}
  %w_deq_g = bf16[{N},{G},{group}] multiply(%w_centered, %scales_b)
  %w_deq = bf16[{N},{K}] reshape(%w_deq_g)
  %dot = f32[{M},{N}] dot(%lhs, %w_deq), lhs_contracting_dims={{1}}, rhs_contracting_dims={{1}}
  %bias_f32 = f32[{N}] convert(%bias)
  %bias_b = f32[{M},{N}] broadcast(%bias_f32), dimensions={{1}}
  %z = f32[{M},{N}] add(%dot, %bias_b)
  ROOT %out = bf16[{M},{N}] convert(%z)
}}
"""


def k_minor_s8_batched(B=8, M=512, K=4096, N=14336):
    """bf16 [B,M,K] . (convert(s8 [B,N,K]) * f32 scale[B,N])^T, batch dimension 0 -> bf16 [B,M,N]."""
    return f"""HloModule k_minor_s8_batched_dequant_dot

ENTRY %main {{
  %lhs = bf16[{B},{M},{K}] parameter(0)
  %w = s8[{B},{N},{K}] parameter(1)
  %scale = f32[{B},{N}] parameter(2)
  %lhs_f32 = f32[{B},{M},{K}] convert(%lhs)
  %w_f32 = f32[{B},{N},{K}] convert(%w)
  %scale_b = f32[{B},{N},{K}] broadcast(%scale), dimensions={{0,1}}
  %w_deq = f32[{B},{N},{K}] multiply(%w_f32, %scale_b)
  %dot = f32[{B},{M},{N}] dot(%lhs_f32, %w_deq), lhs_batch_dims={{0}}, lhs_contracting_dims={{2}}, rhs_batch_dims={{0}}, rhs_contracting_dims={{2}}
  ROOT %out = bf16[{B},{M},{N}] convert(%dot)
}}
"""


def k_minor_ragged_s8_experts(M=32, K=4096, N=4096, groups=8, sizes_ty="s32"):
    """ragged-dot(bf16 [M,K], convert(s8 [G,N,K]) * f32 scale[G,N], group sizes [G]) + bias -> bf16:
    experts stored with the contracting dimension minor."""
    G = groups
    return f"""HloModule k_minor_ragged_s8_experts_dequant_dot

ENTRY %main {{
  %lhs = bf16[{M},{K}] parameter(0)
  %w = s8[{G},{N},{K}] parameter(1)
  %scale = f32[{G},{N}] parameter(2)
  %bias = bf16[{N}] parameter(3)
  %sizes = {sizes_ty}[{G}] parameter(4)
  %lhs_f32 = f32[{M},{K}] convert(%lhs)
  %w_f32 = f32[{G},{N},{K}] convert(%w)
  %scale_b = f32[{G},{N},{K}] broadcast(%scale), dimensions={{0,1}}
  %w_deq = f32[{G},{N},{K}] multiply(%w_f32, %scale_b)
  %dot = f32[{M},{N}] ragged-dot(%lhs_f32, %w_deq, %sizes), lhs_contracting_dims={{1}}, rhs_contracting_dims={{2}}, lhs_ragged_dims={{0}}, rhs_group_dims={{0}}
  %bias_f32 = f32[{N}] convert(%bias)
  %bias_b = f32[{M},{N}] broadcast(%bias_f32), dimensions={{1}}
  %z = f32[{M},{N}] add(%dot, %bias_b)
  ROOT %out = bf16[{M},{N}] convert(%z)
}}
"""


def k_minor_ragged_s4_group_experts(M=32, K=4096, N=4096, groups=8, group=128):
    """ragged-dot(bf16 [M,K], bf16(convert(s4 [G,N,K]) * bf16 scale[G,N,K/g]), group sizes [G]) + bias -> bf16."""
    G, Kg = groups, K // group
    return f"""HloModule k_minor_ragged_s4_group_experts_dequant_dot

ENTRY %main {{
  %lhs = bf16[{M},{K}] parameter(0)
  %w = s4[{G},{N},{K}] parameter(1)
  %scales = bf16[{G},{N},{Kg}] parameter(2)
  %bias = bf16[{N}] parameter(3)
  %sizes = s32[{G}] parameter(4)
  %w_s8 = s8[{G},{N},{K}] convert(%w)
  %w_g = s8[{G},{N},{Kg},{group}] reshape(%w_s8)
  %w_bf16 = bf16[{G},{N},{Kg},{group}] convert(%w_g)
  %scales_b = bf16[{G},{N},{Kg},{group}] broadcast(%scales), dimensions={{0,1,2}}
  %w_deq_g = bf16[{G},{N},{Kg},{group}] multiply(%w_bf16, %scales_b)
  %w_deq = bf16[{G},{N},{K}] reshape(%w_deq_g)
  %dot = f32[{M},{N}] ragged-dot(%lhs, %w_deq, %sizes), lhs_contracting_dims={{1}}, rhs_contracting_dims={{2}}, lhs_ragged_dims={{0}}, rhs_group_dims={{0}}
  %bias_f32 = f32[{N}] convert(%bias)
  %bias_b = f32[{M},{N}] broadcast(%bias_f32), dimensions={{1}}
  %z = f32[{M},{N}] add(%dot, %bias_b)
  ROOT %out = bf16[{M},{N}] convert(%z)
}}
"""


# The shape table of the reference's parametrised int4 tests (Int4TestCases,
# fusion_emitter_int4_device_test.cc:609-645): name, lhs dims, rhs dims, lhs and rhs contracting
# dimension, result dims.  The 3-d cases carry a batch dimension 0 on both operands.
INT4_DOT_CASES = [
    ("int4_dot_128_16_x_128_256", (128, 16), (128, 256), 0, 0, (16, 256)),
    ("int4_dot_128_16_x_256_128", (128, 16), (256, 128), 0, 1, (16, 256)),
    ("int4_dot_16_128_x_256_128", (16, 128), (256, 128), 1, 1, (16, 256)),
    ("int4_dot_16_128_x_128_256", (16, 128), (128, 256), 1, 0, (16, 256)),
    ("int4_dot_1_128_x_256_128", (1, 128), (256, 128), 1, 1, (1, 256)),
    ("int4_dot_128_1_x_256_128", (128, 1), (256, 128), 0, 1, (1, 256)),
    ("int4_dot_16_128_x_128_1", (16, 128), (128, 1), 1, 0, (16, 1)),
    ("int4_dot_16_128_x_1_128", (16, 128), (1, 128), 1, 1, (16, 1)),
    ("dot_8_128_16_x_8_128_256", (8, 128, 16), (8, 128, 256), 1, 1, (8, 16, 256)),
    ("dot_8_128_16_x_8_256_128", (8, 128, 16), (8, 256, 128), 1, 2, (8, 16, 256)),
    ("dot_8_16_128_x_8_256_128", (8, 16, 128), (8, 256, 128), 2, 2, (8, 16, 256)),
    ("dot_8_16_128_x_8_128_256", (8, 16, 128), (8, 128, 256), 2, 1, (8, 16, 256)),
    ("dot_8_1_128_x_8_256_128", (8, 1, 128), (8, 256, 128), 2, 2, (8, 1, 256)),
    ("dot_8_128_1_x_8_256_128", (8, 128, 1), (8, 256, 128), 1, 2, (8, 1, 256)),
    ("dot_8_16_128_x_8_128_1", (8, 16, 128), (8, 128, 1), 2, 1, (8, 16, 1)),
    ("dot_8_16_128_x_8_1_128", (8, 16, 128), (8, 1, 128), 2, 2, (8, 16, 1)),
]


def int4_weights_dot(case, weights_on_lhs):
    """The dot of Int4WeightsOnTheLhs[WithBatchDim] / Int4WeightsOnTheRhs
    (fusion_emitter_int4_device_test.cc:495-606) as the module reads before GemmFusion wraps it into a
    fusion: convert(s4 -> s8 -> bf16) of one operand straight into an f32 dot, no scale."""
    name, lhs, rhs, lc, rc, out = case
    d = lambda t: ",".join(str(v) for v in t)
    batch = "lhs_batch_dims={0}, rhs_batch_dims={0}, " if len(lhs) == 3 else ""
    if weights_on_lhs:
        return f"""HloModule lhs_{name}

ENTRY %entry_computation {{
  %w = s4[{d(lhs)}] parameter(0)
  %w.s8 = s8[{d(lhs)}] convert(%w)
  %w.b16 = bf16[{d(lhs)}] convert(%w.s8)
  %a = bf16[{d(rhs)}] parameter(1)
  ROOT %dot = f32[{d(out)}] dot(%w.b16, %a), {batch}lhs_contracting_dims={{{lc}}}, rhs_contracting_dims={{{rc}}}
}}
"""
    return f"""HloModule rhs_{name}

ENTRY %entry_computation {{
  %a = bf16[{d(lhs)}] parameter(0)
  %w = s4[{d(rhs)}] parameter(1)
  %w.s8 = s8[{d(rhs)}] convert(%w)
  %w.b16 = bf16[{d(rhs)}] convert(%w.s8)
  ROOT %dot = f32[{d(out)}] dot(%a, %w.b16), {batch}lhs_contracting_dims={{{lc}}}, rhs_contracting_dims={{{rc}}}
}}
"""
