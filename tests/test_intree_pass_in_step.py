"""The in-tree form of the rewrite pass (xla_amd/intree/..., written against XLA's HloInstruction
API and not buildable here) is kept in step with the offline matcher that the other tests exercise:
both files must give the same refusal reasons, word for word, and the committed hlo-opt lit tests
must say what the offline matcher does on their modules."""
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INTREE = os.path.join(ROOT, "xla_amd", "intree")
OFFLINE_CC = os.path.join(ROOT, "xla_amd", "csrc", "host", "quant_fusion_rewriter.cc")
INTREE_CC = os.path.join(INTREE, "xla", "backends", "gpu", "transforms", "quant_fusion_rewriter.cc")


def _reasons(path):
    """String literals handed to refuse(...) or assigned to *why, adjacent literals joined."""
    text = open(path).read()
    out = set()
    for m in re.finditer(r'(?:refuse\(|\*why\s*=\s*)((?:\s*(?:lead \?)?\s*"(?:[^"\\]|\\.)*"\s*(?:\+[^";]*?\+?)?\s*(?::)?)+)', text):
        lits = re.findall(r'"((?:[^"\\]|\\.)*)"', m.group(1))
        if lits:
            out.add("".join(lits))
    return out


def test_refusal_reasons_are_the_same_in_both_files():
    offline, intree = _reasons(OFFLINE_CC), _reasons(INTREE_CC)
    assert len(offline) >= 30, sorted(offline)
    assert offline == intree, (sorted(offline - intree), sorted(intree - offline))
    # and the prefixes under which they are logged
    for prefix in ("f8 operands found but not rewritten", "block-scaled dot found but not rewritten",
                   "quantized weights found but not rewritten", "clamp/convert to f8e4m3fn found but not rewritten"):
        assert prefix in open(OFFLINE_CC).read() and prefix in open(INTREE_CC).read(), prefix


def test_custom_call_targets_and_attributes_are_the_same():
    a, b = open(OFFLINE_CC).read(), open(INTREE_CC).read()
    for needle in ('"xla_amd.fp8_scaled_dot"', '"xla_amd.dequant_dot"', '"xla_amd.rowwise_quantize_fp8"',
                   "scale_group_size = ", "rhs_contracting_dim = ", "lhs_contracting_dim = 0", "result_transposed = true",
                   "d_scale_multiplies = ", "rmsnorm = ",
                   "dequant_type = ", "dot_type = ", "epilogue_type = ", "0.7978845608028654", "0.044715",
                   "-448.0", "448.0", "__op$block_scaled_dot"):
        assert needle in a and needle in b, needle


def test_lit_tests_say_what_the_offline_matcher_does():
    sys.path.insert(0, INTREE)
    try:
        import make_lit_tests as gen
    finally:
        sys.path.pop(0)
    cases = gen.cases()
    assert len(cases) >= 12
    for name, text in cases:
        path = os.path.join(gen.OUT, name + ".hlo")
        assert os.path.exists(path), "run python xla_amd/intree/make_lit_tests.py: %s is missing" % path
        assert open(path).read() == gen.render(name, text), "%s is stale: regenerate the lit tests" % name
    # a refusal case really is one, and a rewrite case names its call
    lines, rewrites, refusals = gen.expectations(dict(cases)["quant_fusion_rewriter_refuses_far_gelu_constant"])
    assert rewrites == [] and refusals and lines == ["// CHECK-NOT: xla_amd."]   # 0.05 is not GELU's 0.044715
    lines, rewrites, refusals = gen.expectations(dict(cases)["quant_fusion_rewriter_u4_zero_points"])
    assert rewrites == ["dot -> xla_amd.dequant_dot [BIAS, u4 with zero points]"]
    assert any('custom_call_target="xla_amd.dequant_dot"' in l for l in lines)
