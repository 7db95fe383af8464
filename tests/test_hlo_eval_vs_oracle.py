"""The fused C oracle functions against an op-by-op evaluation of the benchmark HLO modules
(oracle/hlo_eval.py: one numpy op per HLO instruction, re-rounded to the instruction's type).
Both add in the same order, so the comparison is bit for bit: it shows the fused restatement
computes exactly what the un-fused module means under the CPU backend's rounding rules."""
import numpy as np
import pytest

from oracle import hlo_eval
from xla_amd import dtypes, hlo, hlo_modules as hm, workloads


def run_module(text, args):
    return hlo_eval.evaluate(hlo.to_json(text), args)


def test_c1(oracle):
    w = workloads.c1_s8_channel(M=5, K=96, N=40)
    got = run_module(hm.c1_s8_channel(5, 96, 40), [w["lhs"], w["weights"], w["scales"]])
    ref = oracle.dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32")
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("M", [1, 3])
def test_c2(oracle, M):
    w = workloads.c2_s4_group(M=M, K=256, N=48, group=64)
    got = run_module(hm.c2_s4_group(M, 256, 48, 64), [w["lhs"], w["weights"], w["scales"], w["bias"]])
    ref = oracle.dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", bias=w["bias"],
                             group=64, epilogue="silu")
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("typed", ["f32", "bf16"])
def test_c3(oracle, typed):
    w = workloads.c3_fp8(12, 64, 20)
    sa = np.float32(1 / 64)
    scal = dtypes.f32_to_bf16(np.array([sa])) if typed == "bf16" else np.array([sa], np.float32)
    got = run_module(hm.c3_fp8(12, 64, 20, typed=typed), [w["a"], w["b"], scal[0:1].reshape(()), scal[0:1].reshape(()), w["bias"]])
    ref = oracle.fp8_scaled_dot(w["a"], w["b"], sa, sa, mul_ty=typed, bias=w["bias"], dot_ty=typed, ep_ty=typed,
                                epilogue="gelu_tanh")
    assert np.array_equal(got, ref)


def test_c3_vector_scales(oracle):
    """a_scale per row of a, b_scale per output channel: the broadcasts run along dimension 0
    of a and dimension 1 of b."""
    M, K, N = 12, 64, 20
    w = workloads.c3_fp8(M, K, N)
    rng = np.random.default_rng(4)
    sa = rng.uniform(0.005, 0.05, M).astype(np.float32)
    sb = rng.uniform(0.005, 0.05, N).astype(np.float32)
    got = run_module(hm.c3_fp8(M, K, N, vector_scales=True), [w["a"], w["b"], sa, sb, w["bias"]])
    ref = oracle.fp8_scaled_dot(w["a"], w["b"], sa, sb, bias=w["bias"], epilogue="gelu_tanh")
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("multiply", [False, True])
def test_c3_f8_result(oracle, multiply):
    M, K, N = 12, 64, 20
    w = workloads.c3_fp8(M, K, N)
    s, z = np.array(1 / 64, np.float32), np.array(0.0213 if not multiply else 37.5, np.float32)
    got = run_module(hm.c3_fp8_f8_result(M, K, N, multiply=multiply), [w["a"], w["b"], s, s, w["bias"], z])
    ref, _ = oracle.fp8_scaled_dot(w["a"], w["b"], s, s, bias=w["bias"], epilogue="gelu_tanh", d_scale=z,
                                   d_scale_divides=not multiply)
    assert np.array_equal(got, ref)


def test_c3_f8_result_with_amax(oracle):
    M, K, N = 12, 64, 20
    w = workloads.c3_fp8(M, K, N)
    s, z = np.array(1 / 64, np.float32), np.array(0.0213, np.float32)
    codes, amax = run_module(hm.c3_fp8_f8_result(M, K, N, amax=True), [w["a"], w["b"], s, s, w["bias"], z])
    ref, val = oracle.fp8_scaled_dot(w["a"], w["b"], s, s, bias=w["bias"], epilogue="gelu_tanh", d_scale=z)
    assert np.array_equal(codes, ref)
    assert np.float32(amax) == np.max(np.abs(val)) and amax > 0


@pytest.mark.parametrize("nk", [False, True])
def test_batched_fp8_dot(oracle, nk):
    B, M, K, N = 3, 5, 48, 7
    rng = np.random.default_rng(8)
    a = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((B, M, K)) * 32, -448, 448).astype(np.float32))
    b = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((B, K, N)) * 32, -448, 448).astype(np.float32))
    sa, sb = np.array(0.03, np.float32), np.array(0.011, np.float32)
    bb = np.ascontiguousarray(b.transpose(0, 2, 1)) if nk else b
    got = run_module(hm.fp8_batched(B, M, K, N, rhs_nk=nk), [a, bb, sa, sb])
    for i in range(B):
        assert np.array_equal(got[i], oracle.fp8_scaled_dot(a[i], b[i], sa, sb))


def test_mxfp8_block_scaled_dot(oracle):
    M, K, N = 7, 96, 5
    rng = np.random.default_rng(10)
    a8 = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((M, K)) * 8, -448, 448).astype(np.float32))
    b8 = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((N, K)) * 8, -448, 448).astype(np.float32))
    sa = rng.integers(120, 134, (M, K // 32)).astype(np.uint8)
    sb = rng.integers(120, 134, (N, K // 32)).astype(np.uint8)
    got = run_module(hm.mxfp8_block_scaled_dot(M, K, N), [a8, b8, sa, sb])
    assert np.array_equal(got, oracle.block_scaled_dot(a8, b8, sa, sb))


def test_quantize_then_fp8_dot(oracle):
    R, C, N = 6, 96, 10
    x = workloads.c4_quantize(R, C)
    w = workloads.c3_fp8(R, C, N)
    sw = np.array(1 / 32, np.float32)
    got = run_module(hm.quantize_then_fp8_dot(R, C, N), [x["x"], x["gamma"], w["b"], sw])
    q, s = oracle.rmsnorm_quantize_fp8(x["x"], x["gamma"], eps=1e-6)
    assert np.array_equal(got, oracle.fp8_scaled_dot(q, w["b"], s, sw))


@pytest.mark.parametrize("rows,cols", [(4, 256), (3, 1000), (2, 33)])
def test_c4(oracle, rows, cols):
    w = workloads.c4_quantize(rows, cols)
    q, s = run_module(hm.c4_quantize(rows, cols), [w["x"], w["gamma"]])
    q_ref, s_ref = oracle.rmsnorm_quantize_fp8(w["x"], w["gamma"], eps=1e-6)
    assert np.array_equal(s.view(np.uint32), s_ref.view(np.uint32))
    assert np.array_equal(q, q_ref)
    # the rsqrt spelling under its portable definition 1 / sqrt: the same bits
    q2, s2 = run_module(hm.c4_quantize(rows, cols, rsqrt=True), [w["x"], w["gamma"]])
    assert np.array_equal(q2, q_ref) and np.array_equal(s2.view(np.uint32), s_ref.view(np.uint32))


def test_c5(oracle):
    w = workloads.c5_s8_batched(B=2, M=4, K=64, N=24)
    got = run_module(hm.c5_s8_batched(2, 4, 64, 24), [w["lhs"], w["weights"], w["scales"]])
    ref = oracle.dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32")
    assert np.array_equal(got, ref)


def test_u4_zero_points(oracle):
    """The asymmetric 4-bit module op by op (convert, subtract, multiply, each bf16-typed) against
    the fused oracle function: bit for bit."""
    w = workloads.u4_zero_point_group(M=3, K=128, N=24, group=32)
    got = run_module(hm.u4_zero_point_group(3, 128, 24, 32),
                     [w["lhs"], w["weights"], w["scales"], w["zero_points"].astype(np.int8), w["bias"]])
    ref = oracle.dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", bias=w["bias"],
                             group=32, unsigned=True, zero_points=w["zero_points_packed"])
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("sizes", [[3, 3, 3, 3], [5, 0, 2, 1], [0, 0, 12, 0]])
def test_ragged_dot(oracle, sizes):
    """The ragged-dot module op by op (the evaluator's own ragged-dot: one masked dense dot per group)
    against the oracle's composition of per-group calls: bit for bit."""
    w = workloads.ragged_s8_experts(M=12, K=64, N=24, groups=4, sizes=sizes)
    got = run_module(hm.ragged_s8_experts(12, 64, 24, 4),
                     [w["lhs"], w["weights"], w["scales"], w["bias"], w["group_sizes"]])
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("sizes", [[3, 3, 3, 3], [5, 0, 6, 1]])
def test_ragged_dot_s4_group_scales(oracle, sizes):
    """4-bit experts with one bf16 scale per 32 rows of K and channel, bf16-typed multiply: the module
    op by op against the oracle's per-group composition, bit for bit."""
    w = workloads.ragged_s4_group_experts(M=12, K=128, N=24, groups=4, group=32, sizes=sizes)
    got = run_module(hm.ragged_s4_group_experts(12, 128, 24, 4, 32),
                     [w["lhs"], w["weights"], w["scales"], w["bias"], w["group_sizes"]])
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", w["group_sizes"],
                                    bias=w["bias"], group=32)
    assert np.array_equal(got, ref)


def test_batched_s4_group_scales(oracle):
    w = workloads.batched_s4_group(B=3, M=4, K=128, N=24, group=32)
    got = run_module(hm.batched_s4_group(3, 4, 128, 24, 32), [w["lhs"], w["weights"], w["scales"]])
    ref = np.stack([oracle.dequant_dot(w["lhs"][b], dtypes.pack_s4(w["weights"][b]), 4, w["scales"][b], "bf16", "bf16",
                                       group=32) for b in range(3)])
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("kind", ["s8", "s4", "s4_f32", "u4", "batched"])
def test_weights_with_the_contracting_dimension_minor(oracle, kind):
    """Weights stored [N,K] (rhs_contracting_dims = {1}): the module, op by op, on the re-laid-out
    arrays gives the bits of the fused oracle function on the [K,N] arrays it was made from."""
    if kind == "s8":
        w = workloads.c1_s8_channel(M=5, K=96, N=40)
        v = workloads.k_minor(w)
        got = run_module(hm.k_minor_s8_channel(5, 96, 40), [v["lhs"], v["weights"], v["scales"]])
        ref = oracle.dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32")
    elif kind in ("s4", "s4_f32"):
        w = workloads.c2_s4_group(M=3, K=256, N=48, group=64)
        ty = "bf16" if kind == "s4" else "f32"
        if ty == "f32":
            w["scales"] = dtypes.bf16_to_f32(w["scales"])
        v = workloads.k_minor(w)
        got = run_module(hm.k_minor_s4_group(3, 256, 48, 64, typed=ty), [v["lhs"], v["weights"], v["scales"], v["bias"]])
        ref = oracle.dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], ty, ty, bias=w["bias"],
                                 group=64, epilogue="silu")
    elif kind == "u4":
        w = workloads.u4_zero_point_group(M=3, K=128, N=24, group=32)
        v = workloads.k_minor(w)
        got = run_module(hm.k_minor_u4_zero_point_group(3, 128, 24, 32),
                         [v["lhs"], v["weights"], v["scales"], v["zero_points"].astype(np.int8), v["bias"]])
        ref = oracle.dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", bias=w["bias"],
                                 group=32, unsigned=True, zero_points=w["zero_points_packed"])
    else:
        w = workloads.c5_s8_batched(B=2, M=4, K=64, N=24)
        v = workloads.k_minor(w)
        got = run_module(hm.k_minor_s8_batched(2, 4, 64, 24), [v["lhs"], v["weights"], v["scales"]])
        ref = oracle.dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32")
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("kind", ["s8", "s4"])
def test_ragged_dot_over_k_minor_experts(oracle, kind):
    """Experts stored [G,N,K] (rhs_contracting_dims = {2}): the module op by op on the re-laid-out arrays
    gives the bits of the oracle's composition of per-group calls on the [G,K,N] arrays."""
    sizes = [5, 0, 6, 1]
    if kind == "s8":
        w = workloads.ragged_s8_experts(M=12, K=64, N=24, groups=4, sizes=sizes)
        v = workloads.k_minor(w)
        got = run_module(hm.k_minor_ragged_s8_experts(12, 64, 24, 4),
                         [v["lhs"], v["weights"], v["scales"], v["bias"], v["group_sizes"]])
        ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
    else:
        w = workloads.ragged_s4_group_experts(M=12, K=64, N=24, groups=4, group=32, sizes=sizes)
        v = workloads.k_minor(w)
        got = run_module(hm.k_minor_ragged_s4_group_experts(12, 64, 24, 4, 32),
                         [v["lhs"], v["weights"], v["scales"], v["bias"], v["group_sizes"]])
        ref = oracle.ragged_dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", w["group_sizes"],
                                        bias=w["bias"], group=32)
    assert np.array_equal(got, ref)
