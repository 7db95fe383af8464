"""Writes the hlo-opt lit tests of the in-tree pass (xla/backends/gpu/transforms/tests/*.hlo).

Each file is one module of xla_amd.hlo_modules at a small shape with a RUN line for hlo-opt and
CHECK lines taken from what the offline matcher (the same rules on HLO text) produces for it: the
custom call line with its operands, target and attributes, or the refusal.  tests/
test_intree_pass_in_step.py runs every committed file through the offline matcher again, so the
expectations cannot drift.

    python xla_amd/intree/make_lit_tests.py        # regenerates the files
"""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
OUT = os.path.join(HERE, "xla", "backends", "gpu", "transforms", "tests")


def cases():
    from xla_amd import hlo_modules as hm
    gelu_far = hm.c3_fp8(64, 128, 32).replace("constant(0.044715)", "constant(0.05)")
    return [
        ("quant_fusion_rewriter_s8_per_channel", hm.c1_s8_channel(16, 256, 128)),
        ("quant_fusion_rewriter_s4_grouped_silu", hm.c2_s4_group(8, 256, 64, 64)),
        ("quant_fusion_rewriter_s4_grouped_silu_f8_result", hm.c2_s4_group_f8_result(8, 256, 64, 64)),
        ("quant_fusion_rewriter_u4_zero_points", hm.u4_zero_point_group(8, 256, 64, 64)),
        ("quant_fusion_rewriter_s8_batched", hm.c5_s8_batched(2, 8, 32, 16)),
        ("quant_fusion_rewriter_s8_ragged_experts", hm.ragged_s8_experts(16, 256, 64, 4)),
        ("quant_fusion_rewriter_s8_ragged_experts_prefill", hm.ragged_s8_experts(640, 256, 64, 4)),
        ("quant_fusion_rewriter_s4_ragged_experts_group_scales", hm.ragged_s4_group_experts(16, 256, 64, 4, 64)),
        ("quant_fusion_rewriter_s4_batched_group_scales", hm.batched_s4_group(2, 8, 256, 64, 64)),
        ("quant_fusion_rewriter_fp8_bias_gelu", hm.c3_fp8(64, 128, 32)),
        ("quant_fusion_rewriter_fp8_bf16_typed", hm.c3_fp8(64, 128, 32, typed="bf16")),
        ("quant_fusion_rewriter_k_minor_s8_channel", hm.k_minor_s8_channel(16, 4096, 4096)),
        ("quant_fusion_rewriter_k_minor_s4_group", hm.k_minor_s4_group(8, 8192, 28672)),
        ("quant_fusion_rewriter_k_minor_ragged_s8_experts", hm.k_minor_ragged_s8_experts(32, 512, 256, 4)),
        ("quant_fusion_rewriter_k_minor_u4_zero_points", hm.k_minor_u4_zero_point_group(8, 256, 64, 64)),
        ("quant_fusion_rewriter_fp8_vector_scales", hm.c3_fp8(64, 128, 32, vector_scales=True)),
        ("quant_fusion_rewriter_fp8_bf16_typed_vector_scales", hm.c3_fp8(64, 128, 32, typed="bf16", vector_scales=True)),
        ("quant_fusion_rewriter_fp8_f8_result_amax", hm.c3_fp8_f8_result(64, 128, 32, amax=True)),
        ("quant_fusion_rewriter_rowwise_quantize_rmsnorm", hm.c4_quantize(8, 64)),
        ("quant_fusion_rewriter_rowwise_quantize_rsqrt", hm.c4_quantize(8, 64, rsqrt=True)),
        ("quant_fusion_rewriter_rowwise_quantize_plain", hm.c4_quantize(8, 64, rmsnorm=False)),
        ("quant_fusion_rewriter_quantize_then_dot", hm.quantize_then_fp8_dot(8, 64, 32)),
        ("quant_fusion_rewriter_int4_weights_on_the_rhs_f32", hm.int4_weights_dot(hm.INT4_DOT_CASES[1], False)),
        ("quant_fusion_rewriter_int4_weights_on_the_lhs_f32", hm.int4_weights_dot(hm.INT4_DOT_CASES[3], True)),
        ("quant_fusion_rewriter_int4_weights_on_the_lhs_batched", hm.int4_weights_dot(hm.INT4_DOT_CASES[9], True)),
        ("quant_fusion_rewriter_mxfp8_block_scaled_dot", hm.mxfp8_block_scaled_dot(64, 256, 32)),
        ("quant_fusion_rewriter_mxfp8_batched_bias_gelu", hm.mxfp8_block_scaled_dot(64, 256, 32, batch=2, bias_gelu=True)),
        ("quant_fusion_rewriter_refuses_far_gelu_constant", gelu_far),
    ]


def expectations(text):
    """CHECK lines for one module: its custom calls (operands, target, attributes) or, when nothing
    was rewritten, CHECK-NOT of the targets."""
    from xla_amd import hlo
    new, rewrites, refusals = hlo.rewrite(text)
    lines = []
    for line in new.splitlines():
        m = re.search(r"custom-call\((.*?)\), custom_call_target=\"(xla_amd\.[a-z0-9_]+)\".*backend_config=\"\{(.*)\}\"", line)
        if not m:
            continue
        operands, target, cfg = m.group(1), m.group(2), m.group(3).replace('\\"', '"')
        # operand names change under hlo-opt's renumbering: their count is what is checked
        lines.append("// CHECK: custom-call(%s), custom_call_target=\"%s\"" % (
            ", ".join("%{{.*}}" for _ in operands.split(",")), target))
        lines.append("// CHECK-SAME: api_version=API_VERSION_TYPED_FFI")
        for attr in cfg.split(", "):
            key = attr.split(" = ")[0]
            if key in ("epilogue", "rmsnorm", "scale_group_size", "rhs_contracting_dim", "lhs_contracting_dim", "result_transposed", "d_scale_multiplies",
                       "dequant_type", "dot_type", "epilogue_type"):
                lines.append("// CHECK-SAME: %s" % attr.replace("\\", ""))
    if not lines:
        lines.append("// CHECK-NOT: xla_amd.")
    return lines, rewrites, refusals


def render(name, text):
    lines, rewrites, refusals = expectations(text)
    head = ["// RUN: hlo-opt %s --platform=gpu --passes=quant-fusion-rewriter | FileCheck %s",
            "//",
            "// The offline matcher says: " + ("; ".join(rewrites) if rewrites else "nothing rewritten")]
    head += ["//   refused: " + r for r in refusals]
    return "\n".join(head) + "\n\n" + "\n".join(lines) + "\n\n" + text.strip() + "\n"


def main():
    os.makedirs(OUT, exist_ok=True)
    for name, text in cases():
        with open(os.path.join(OUT, name + ".hlo"), "w") as f:
            f.write(render(name, text))
    print("wrote %d files to %s" % (len(cases()), OUT))


if __name__ == "__main__":
    main()
