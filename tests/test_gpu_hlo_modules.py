"""End to end on the GPU: the benchmark HLO modules go through the rewrite pass, the rewritten
module runs through the FFI registry (xla_amd/hlo_runner.py), and the result is compared with
the op-by-op CPU evaluation of the *original* module -- what run_hlo_module does with
--reference_platform (xla/tools/run_hlo_module.cc:211-390)."""
import sys

import numpy as np
import pytest
import torch

from oracle import hlo_eval
from tests.gpu_util import check_dot, check_f8_result, dev_bf16, dev_f32, dev_s8, dev_u8, dot_floor, host_bf16
from xla_amd import dtypes, ffi, hlo, hlo_modules as hm, hlo_runner, workloads

pytestmark = pytest.mark.gpu


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def reference(text, args):
    return hlo_eval.evaluate(hlo.to_json(text), args)


def test_c1_module():
    say("module C1")
    M, K, N = 16, 512, 256
    w = workloads.c1_s8_channel(M, K, N)
    text = hm.c1_s8_channel(M, K, N)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_bf16(w["lhs"]), dev_s8(w["weights"]), dev_f32(w["scales"])])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s8]"]
    ref = reference(text, [w["lhs"], w["weights"], w["scales"]])
    fl = dot_floor(np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64)),
                   np.abs(w["weights"].astype(np.float64)) * w["scales"].astype(np.float64)[None, :], K)
    check_dot(host_bf16(out), ref, fl, "C1 module")


@pytest.mark.parametrize("M", [8, 130])
def test_c2_module(M):
    """M = 130: a prefill-sized token count on the s4 weights (one decode launch per 64 tokens)."""
    say("module C2 M=%d" % M)
    K, N = 1024, 512
    w = workloads.c2_s4_group(M, K, N)
    text = hm.c2_s4_group(M, K, N)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_bf16(w["lhs"]), dev_u8(w["weights_packed"]),
                                                   dev_bf16(w["scales"]), dev_bf16(w["bias"])])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4]"]
    ref = reference(text, [w["lhs"], w["weights"], w["scales"], w["bias"]])
    wd = np.abs(w["weights"].astype(np.float64)) * np.repeat(dtypes.bf16_to_f32(w["scales"]).astype(np.float64), 128, axis=0)
    fl = dot_floor(np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64)), wd, K)
    check_dot(host_bf16(out), ref, fl, "C2 module")


@pytest.mark.parametrize("multiply", [False, True])
def test_c2_module_f8_result(oracle, multiply):
    say("module C2 with an f8 result, multiply=%s" % multiply)
    M, K, N = 8, 1024, 512
    w = workloads.c2_s4_group(M, K, N)
    text = hm.c2_s4_group_f8_result(M, K, N, multiply=multiply)
    z = np.array(1 / 0.37 if multiply else 0.37, np.float32)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_bf16(w["lhs"]), dev_u8(w["weights_packed"]),
                                                   dev_bf16(w["scales"]), dev_bf16(w["bias"]), dev_f32(z)])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS_SILU, s4, f8 result]"]
    ref = reference(text, [w["lhs"], w["weights"], w["scales"], w["bias"], z])
    val = oracle.dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", bias=w["bias"], bias_ty="bf16",
                             group=128, epilogue="silu", f32_result=True)
    wd = np.abs(w["weights"].astype(np.float64)) * np.repeat(dtypes.bf16_to_f32(w["scales"]).astype(np.float64), 128, axis=0)
    fl = dot_floor(np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64)), wd, K)
    got = out.cpu().numpy().view(np.uint8)
    assert list(got.shape) == [M, N]
    assert check_f8_result(got, ref, val, z, not multiply, fl, "C2 f8 result") <= got.size // 8


def test_c3_module():
    say("module C3")
    M, K, N = 128, 256, 128
    w = workloads.c3_fp8(M, K, N)
    text = hm.c3_fp8(M, K, N)
    s = np.array(1 / 64, np.float32)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_u8(w["a"]), dev_u8(w["b"]), dev_f32(s), dev_f32(s), dev_bf16(w["bias"])])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU]"]
    ref = reference(text, [w["a"], w["b"], s, s, w["bias"]])
    fa = np.abs(dtypes.f8e4m3fn_to_f32(w["a"]).astype(np.float64)) / 64
    fb = np.abs(dtypes.f8e4m3fn_to_f32(w["b"]).astype(np.float64)) / 64
    check_dot(host_bf16(out), ref, dot_floor(fa, fb, K) + 1.2 * 2.0 ** -12 * np.sqrt((fa * fa) @ (fb * fb)), "C3 module")


def test_c3_module_vector_scales():
    say("module C3 with per-row / per-channel scales")
    M, K, N = 128, 256, 144
    w = workloads.c3_fp8(M, K, N)
    text = hm.c3_fp8(M, K, N, vector_scales=True)
    rng = np.random.default_rng(8)
    sa = rng.uniform(0.004, 0.04, M).astype(np.float32)
    sb = rng.uniform(0.004, 0.04, N).astype(np.float32)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_u8(w["a"]), dev_u8(w["b"]), dev_f32(sa), dev_f32(sb), dev_bf16(w["bias"])])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU]"]
    ref = reference(text, [w["a"], w["b"], sa, sb, w["bias"]])
    fa = np.abs(dtypes.f8e4m3fn_to_f32(w["a"]).astype(np.float64)) * sa[:, None]
    fb = np.abs(dtypes.f8e4m3fn_to_f32(w["b"]).astype(np.float64)) * sb[None, :]
    check_dot(host_bf16(out), ref, dot_floor(fa, fb, K) + 1.2 * 2.0 ** -12 * np.sqrt((fa * fa) @ (fb * fb)), "C3 vector scales")


def test_c3_module_vector_scales_under_a_bf16_multiply():
    say("module C3, every op bf16-typed, per-row / per-channel scales")
    M, K, N = 128, 256, 144
    w = workloads.c3_fp8(M, K, N)
    text = hm.c3_fp8(M, K, N, typed="bf16", vector_scales=True)
    rng = np.random.default_rng(9)
    sa = dtypes.f32_to_bf16(rng.uniform(0.004, 0.04, M).astype(np.float32))
    sb = dtypes.f32_to_bf16(rng.uniform(0.004, 0.04, N).astype(np.float32))
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_u8(w["a"]), dev_u8(w["b"]), dev_bf16(sa), dev_bf16(sb), dev_bf16(w["bias"])])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU]"]
    ref = reference(text, [w["a"], w["b"], sa, sb, w["bias"]])
    fa = np.abs(dtypes.f8e4m3fn_to_f32(w["a"]).astype(np.float64)) * dtypes.bf16_to_f32(sa).astype(np.float64)[:, None]
    fb = np.abs(dtypes.f8e4m3fn_to_f32(w["b"]).astype(np.float64)) * dtypes.bf16_to_f32(sb).astype(np.float64)[None, :]
    check_dot(host_bf16(out), ref, dot_floor(fa, fb, K), "C3 bf16-typed vector scales")


def test_c3_module_f8_result(oracle):
    say("module C3 with an f8 result")
    M, K, N = 128, 256, 144
    w = workloads.c3_fp8(M, K, N)
    s, z = np.array(1 / 64, np.float32), np.array(0.0171, np.float32)
    text = hm.c3_fp8_f8_result(M, K, N)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_u8(w["a"]), dev_u8(w["b"]), dev_f32(s), dev_f32(s),
                                                   dev_bf16(w["bias"]), dev_f32(z)])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU, f8 result]"]
    ref = reference(text, [w["a"], w["b"], s, s, w["bias"], z])
    _, val = oracle.fp8_scaled_dot(w["a"], w["b"], s, s, bias=w["bias"], epilogue="gelu_tanh", d_scale=z)
    fa = np.abs(dtypes.f8e4m3fn_to_f32(w["a"]).astype(np.float64)) / 64
    fb = np.abs(dtypes.f8e4m3fn_to_f32(w["b"]).astype(np.float64)) / 64
    floor = dot_floor(fa, fb, K) + 1.2 * 2.0 ** -12 * np.sqrt((fa * fa) @ (fb * fb))
    got = out.cpu().numpy().view(np.uint8)
    assert check_f8_result(got, ref, val, z, True, floor, "C3 f8 result") <= got.size // 50


def test_c3_module_f8_result_with_amax(oracle):
    say("module C3 with an f8 result and its amax")
    M, K, N = 128, 256, 144
    w = workloads.c3_fp8(M, K, N)
    s, z = np.array(1 / 64, np.float32), np.array(0.0171, np.float32)
    text = hm.c3_fp8_f8_result(M, K, N, amax=True)
    (out, amax), rw, _ = hlo_runner.compile_and_run(text, [dev_u8(w["a"]), dev_u8(w["b"]), dev_f32(s), dev_f32(s),
                                                           dev_bf16(w["bias"]), dev_f32(z)])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU, f8 result, amax]"]
    ref_codes, ref_amax = reference(text, [w["a"], w["b"], s, s, w["bias"], z])
    ref_amax = float(np.asarray(ref_amax).reshape(-1)[0])
    assert abs(float(amax) - ref_amax) <= ref_amax * 2.0 ** -7
    assert (out.cpu().numpy().view(np.uint8) != ref_codes).sum() <= out.numel() // 50


def test_batched_fp8_module(oracle):
    say("module batched fp8 dot")
    B, M, K, N = 4, 64, 128, 48
    rng = np.random.default_rng(12)
    a = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((B, M, K)) * 32, -448, 448).astype(np.float32))
    b = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((B, K, N)) * 32, -448, 448).astype(np.float32))
    sa, sb = np.array(0.03, np.float32), np.array(0.011, np.float32)
    text = hm.fp8_batched(B, M, K, N)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_u8(a), dev_u8(b), dev_f32(sa), dev_f32(sb)])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [DEFAULT]"]
    ref = reference(text, [a, b, sa, sb])
    got = host_bf16(out)
    for i in range(B):
        fa = np.abs(dtypes.f8e4m3fn_to_f32(a[i]).astype(np.float64)) * 0.03
        fb = np.abs(dtypes.f8e4m3fn_to_f32(b[i]).astype(np.float64)) * 0.011
        check_dot(got[i], ref[i], dot_floor(fa, fb, K) + 1.2 * 2.0 ** -12 * np.sqrt((fa * fa) @ (fb * fb)), "batch %d" % i)


def test_mxfp8_module(oracle):
    say("module MXFP8 block-scaled dot")
    M, K, N = 128, 256, 96
    rng = np.random.default_rng(6)
    a = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((M, K)) * 8, -448, 448).astype(np.float32))
    b = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((N, K)) * 8, -448, 448).astype(np.float32))
    sa = rng.integers(118, 134, (M, K // 32)).astype(np.uint8)
    sb = rng.integers(118, 134, (N, K // 32)).astype(np.uint8)
    text = hm.mxfp8_block_scaled_dot(M, K, N)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_u8(a), dev_u8(b), dev_u8(sa), dev_u8(sb)])
    torch.cuda.synchronize()
    assert rw == ["result -> xla_amd.fp8_scaled_dot [DEFAULT, block scales]"]
    ref = reference(text, [a, b, sa, sb])
    ad = np.abs(dtypes.f8e4m3fn_to_f32(a).astype(np.float64)) * np.repeat(2.0 ** (sa.astype(np.float64) - 127), 32, axis=1)
    bd = np.abs(dtypes.f8e4m3fn_to_f32(b).astype(np.float64)) * np.repeat(2.0 ** (sb.astype(np.float64) - 127), 32, axis=1)
    check_dot(host_bf16(out), ref, dot_floor(ad, bd.T, K) + 1.2 * 2.0 ** -12 * np.sqrt((ad * ad) @ (bd * bd).T), "MXFP8 module")


@pytest.mark.parametrize("M,K", [(128, 256), (16, 8192)])
@pytest.mark.parametrize("batch", [0, 3])
def test_mxfp8_module_with_bias_gelu(oracle, batch, M, K):
    """The block-scaled custom call yielding f32, a bias add, GELU and the convert to bf16 behind it,
    with and without a leading batch dimension: one call after the pass, against the op-by-op
    evaluation of the original module.  16 rows take the streaming kernel, K split over workgroups
    through the scratch the pass asked for."""
    say("module MXFP8 block-scaled dot + bias + GELU, batch=%d M=%d K=%d" % (batch, M, K))
    N = 96
    rng = np.random.default_rng(16)
    lead = (batch,) if batch else ()
    a = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal(lead + (M, K)) * 4, -448, 448).astype(np.float32))
    b = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal(lead + (N, K)) * 4, -448, 448).astype(np.float32))
    sa = rng.integers(120, 128, lead + (M, K // 32)).astype(np.uint8)
    sb = rng.integers(120, 128, lead + (N, K // 32)).astype(np.uint8)
    bias = dtypes.f32_to_bf16(rng.standard_normal(N).astype(np.float32))
    text = hm.mxfp8_block_scaled_dot(M, K, N, batch=batch, bias_gelu=True)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_u8(a), dev_u8(b), dev_u8(sa), dev_u8(sb), dev_bf16(bias)])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.fp8_scaled_dot [BIAS_GELU, block scales%s]" % (", batched" if batch else "")]
    assert ffi.last_kernel() == ("fp8_scaled_dot_tiled_mx" if M > 32 else "fp8_dot_decode_mx_m16")
    if M <= 32:
        assert ffi.library().xla_amd_fp8_scaled_dot_workspace_bytes(M, K, N, 1) > 0 and "s8[" in hlo.rewrite(text)[0]
    ref = reference(text, [a, b, sa, sb, bias])
    got = host_bf16(out)
    for i in range(max(batch, 1)):
        ai, bi, sai, sbi = (v[i] if batch else v for v in (a, b, sa, sb))
        ad = np.abs(dtypes.f8e4m3fn_to_f32(ai).astype(np.float64)) * np.repeat(2.0 ** (sai.astype(np.float64) - 127), 32, axis=1)
        bd = np.abs(dtypes.f8e4m3fn_to_f32(bi).astype(np.float64)) * np.repeat(2.0 ** (sbi.astype(np.float64) - 127), 32, axis=1)
        floor = 1.2 * (dot_floor(ad, bd.T, K) + 1.2 * 2.0 ** -12 * np.sqrt((ad * ad) @ (bd * bd).T))
        check_dot(got[i] if batch else got, ref[i] if batch else ref, floor, "MXFP8 module + bias + GELU, batch %d" % i)


def test_quantize_then_fp8_dot_module(oracle):
    """RMSNorm + quantize feeding an f8 dot: two custom calls after the pass, against the op-by-op
    evaluation of the original module."""
    say("module quantize -> fp8 dot")
    R, C, N = 96, 512, 128
    x = workloads.c4_quantize(R, C)
    w = workloads.c3_fp8(R, C, N)
    sw = np.array(1 / 64, np.float32)
    text = hm.quantize_then_fp8_dot(R, C, N)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_bf16(x["x"]), dev_bf16(x["gamma"]), dev_u8(w["b"]), dev_f32(sw)])
    torch.cuda.synchronize()
    assert rw == ["q -> xla_amd.rowwise_quantize_fp8 [rmsnorm]", "dot -> xla_amd.fp8_scaled_dot [DEFAULT]"]
    ref = reference(text, [x["x"], x["gamma"], w["b"], sw])
    q, s = oracle.rmsnorm_quantize_fp8(x["x"], x["gamma"], eps=1e-6)
    fa = np.abs(dtypes.f8e4m3fn_to_f32(q).astype(np.float64)) * s[:, None]
    fb = np.abs(dtypes.f8e4m3fn_to_f32(w["b"]).astype(np.float64)) / 64
    check_dot(host_bf16(out), ref, dot_floor(fa, fb, C) + 1.2 * 2.0 ** -12 * np.sqrt((fa * fa) @ (fb * fb)), "quantize -> dot")


@pytest.mark.parametrize("rmsnorm,rsqrt", [(True, False), (False, False), (True, True)])
def test_c4_module_bit_exact(rmsnorm, rsqrt):
    """rsqrt: the reciprocal root written as one `rsqrt` op (evaluated as 1 / sqrt by the reference
    evaluator, rsqrt.cc:178-193) rewrites to the same call and the same bits."""
    say("module C4 rmsnorm=%s rsqrt=%s" % (rmsnorm, rsqrt))
    rows, cols = 24, 2048
    w = workloads.c4_quantize(rows, cols)
    text = hm.c4_quantize(rows, cols, rmsnorm=rmsnorm, rsqrt=rsqrt)
    args_dev = [dev_bf16(w["x"])] + ([dev_bf16(w["gamma"])] if rmsnorm else [])
    (q, s), rw, _ = hlo_runner.compile_and_run(text, args_dev)
    torch.cuda.synchronize()
    assert len(rw) == 1 and "rowwise_quantize_fp8" in rw[0]
    q_ref, s_ref = reference(text, [w["x"]] + ([w["gamma"]] if rmsnorm else []))
    assert np.array_equal(s.cpu().numpy().view(np.uint32), s_ref.view(np.uint32))
    assert np.array_equal(q.cpu().numpy(), q_ref)


def test_c5_module():
    say("module C5")
    B, M, K, N = 2, 128, 256, 256
    w = workloads.c5_s8_batched(B, M, K, N)
    text = hm.c5_s8_batched(B, M, K, N)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_bf16(w["lhs"]), dev_s8(w["weights"]), dev_f32(w["scales"])])
    torch.cuda.synchronize()
    ref = reference(text, [w["lhs"], w["weights"], w["scales"]])
    wd = np.abs(w["weights"].astype(np.float64)) * w["scales"].astype(np.float64)[:, None, :]
    check_dot(host_bf16(out), ref, dot_floor(np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64)), wd, K), "C5 module")


@pytest.mark.parametrize("M", [24, 150])
def test_ragged_experts_modules(M):
    """ragged-dot modules (s8 experts with a scale per expert and channel; s4 experts with scales per
    128 rows of K as well) through the pass and the registry; the group sizes are a device operand."""
    say("module ragged experts M=%d" % M)
    K, N, G = 512, 256, 4
    for kind in ("s8", "s4"):
        if kind == "s8":
            w, text = workloads.ragged_s8_experts(M, K, N, G), hm.ragged_s8_experts(M, K, N, G)
            ops_in = [dev_bf16(w["lhs"]), dev_s8(w["weights"]), dev_f32(w["scales"]), dev_bf16(w["bias"])]
            ref_in = [w["lhs"], w["weights"], w["scales"], w["bias"], w["group_sizes"]]
            wd = np.max(np.abs(w["weights"].astype(np.float64)) * w["scales"].astype(np.float64)[:, None, :], axis=0)
        else:
            w, text = workloads.ragged_s4_group_experts(M, K, N, G, 128), hm.ragged_s4_group_experts(M, K, N, G, 128)
            ops_in = [dev_bf16(w["lhs"]), dev_u8(w["weights_packed"]), dev_bf16(w["scales"]), dev_bf16(w["bias"])]
            ref_in = [w["lhs"], w["weights"], w["scales"], w["bias"], w["group_sizes"]]
            wd = np.max(np.abs(w["weights"].astype(np.float64)) *
                        np.repeat(dtypes.bf16_to_f32(w["scales"]).astype(np.float64), 128, axis=1), axis=0)
        sizes = torch.from_numpy(w["group_sizes"].astype(np.int32)).cuda()
        out, rw, _ = hlo_runner.compile_and_run(text, ops_in + [sizes])
        torch.cuda.synchronize()
        assert rw == ["dot -> xla_amd.dequant_dot [BIAS, %s, ragged over 4 groups]" % kind], rw
        ref = reference(text, ref_in)
        fl = dot_floor(np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64)), wd, K)
        check_dot(host_bf16(out), ref, fl, "ragged %s module M=%d" % (kind, M))


@pytest.mark.parametrize("kind", ["s8", "s4"])
def test_k_minor_ragged_experts_modules(kind):
    """ragged-dot modules over experts stored [G,N,K] through the pass and the registry."""
    say("module ragged experts stored [G,N,K]: %s" % kind)
    M, K, N, G = 40, 512, 264, 4
    if kind == "s8":
        v = workloads.k_minor(workloads.ragged_s8_experts(M, K, N, G))
        text = hm.k_minor_ragged_s8_experts(M, K, N, G)
        ops_in = [dev_bf16(v["lhs"]), dev_s8(v["weights"]), dev_f32(v["scales"]), dev_bf16(v["bias"])]
        wd = np.max(np.abs(v["weights"].astype(np.float64)) * v["scales"].astype(np.float64)[:, :, None], axis=0)
    else:
        v = workloads.k_minor(workloads.ragged_s4_group_experts(M, K, N, G, 128))
        text = hm.k_minor_ragged_s4_group_experts(M, K, N, G, 128)
        ops_in = [dev_bf16(v["lhs"]), dev_u8(v["weights_packed"]), dev_bf16(v["scales"]), dev_bf16(v["bias"])]
        wd = np.max(np.abs(v["weights"].astype(np.float64)) *
                    np.repeat(dtypes.bf16_to_f32(v["scales"]).astype(np.float64), 128, axis=2), axis=0)
    sizes = torch.from_numpy(v["group_sizes"].astype(np.int32)).cuda()
    out, rw, _ = hlo_runner.compile_and_run(text, ops_in + [sizes])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.dequant_dot [BIAS, %s, ragged over 4 groups, weights [G,N,K]]" % kind], rw
    assert ffi.last_kernel().startswith("dequant_dot_nk_"), ffi.last_kernel()
    ref = reference(text, [v["lhs"], v["weights"], v["scales"], v["bias"], v["group_sizes"]])
    fl = dot_floor(np.abs(dtypes.bf16_to_f32(v["lhs"]).astype(np.float64)), wd.T, K)
    check_dot(host_bf16(out), ref, fl, "ragged [G,N,K] %s module" % kind)


def test_batched_s4_group_module():
    say("module batched s4 group scales")
    B, M, K, N = 3, 8, 512, 256
    w = workloads.batched_s4_group(B, M, K, N, 128)
    text = hm.batched_s4_group(B, M, K, N, 128)
    out, rw, _ = hlo_runner.compile_and_run(text, [dev_bf16(w["lhs"]), dev_u8(w["weights_packed"]), dev_bf16(w["scales"])])
    torch.cuda.synchronize()
    assert rw == ["dot -> xla_amd.dequant_dot [DEFAULT, s4]"], rw
    ref = reference(text, [w["lhs"], w["weights"], w["scales"]])
    wd = np.abs(w["weights"].astype(np.float64)) * np.repeat(dtypes.bf16_to_f32(w["scales"]).astype(np.float64), 128, axis=1)
    fl = dot_floor(np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64)), wd, K)
    check_dot(host_bf16(out), ref, fl, "batched s4 group module")


@pytest.mark.parametrize("kind", ["s8", "s4", "s4_f32", "u4", "batched"])
def test_k_minor_weight_modules(kind):
    """Weights stored [N,K] (rhs_contracting_dims = {1}): module -> pass -> handler, against the
    op-by-op evaluation of the same module."""
    say("module with [N,K] weights: %s" % kind)
    if kind == "s8":
        M, K, N = 16, 1024, 520
        v = workloads.k_minor(workloads.c1_s8_channel(M=M, K=K, N=N))
        text = hm.k_minor_s8_channel(M, K, N)
        host_args = [v["lhs"], v["weights"], v["scales"]]
        dev_args = [dev_bf16(v["lhs"]), dev_s8(v["weights"]), dev_f32(v["scales"])]
        want = "dot -> xla_amd.dequant_dot [DEFAULT, s8, weights [N,K]]"
        sv = np.repeat(v["scales"].astype(np.float64)[:, None], K, axis=1)
    elif kind in ("s4", "s4_f32"):
        M, K, N, g = 24, 1024, 520, 128
        w = workloads.c2_s4_group(M=M, K=K, N=N, group=g)
        ty = "bf16" if kind == "s4" else "f32"
        if ty == "f32":
            w["scales"] = dtypes.bf16_to_f32(w["scales"])
        v = workloads.k_minor(w)
        text = hm.k_minor_s4_group(M, K, N, g, typed=ty)
        host_args = [v["lhs"], v["weights"], v["scales"], v["bias"]]
        dev_args = [dev_bf16(v["lhs"]), dev_u8(v["weights_packed"]),
                    dev_bf16(v["scales"]) if ty == "bf16" else dev_f32(v["scales"]), dev_bf16(v["bias"])]
        want = "dot -> xla_amd.dequant_dot [BIAS_SILU, s4, weights [N,K]]"
        sc = dtypes.bf16_to_f32(v["scales"]) if ty == "bf16" else v["scales"]
        sv = np.repeat(sc.astype(np.float64), g, axis=1)
    elif kind == "u4":
        M, K, N, g = 8, 512, 264, 64
        v = workloads.k_minor(workloads.u4_zero_point_group(M=M, K=K, N=N, group=g))
        text = hm.k_minor_u4_zero_point_group(M, K, N, g)
        host_args = [v["lhs"], v["weights"], v["scales"], v["zero_points"].astype(np.int8), v["bias"]]
        dev_args = [dev_bf16(v["lhs"]), dev_u8(v["weights_packed"]), dev_bf16(v["scales"]),
                    dev_u8(v["zero_points_packed"]), dev_bf16(v["bias"])]
        want = "dot -> xla_amd.dequant_dot [BIAS, u4 with zero points, weights [N,K]]"
        sv = np.repeat(dtypes.bf16_to_f32(v["scales"]).astype(np.float64), g, axis=1) * 2.0   # |w - z| <= 15
    else:
        B, M, K, N = 3, 20, 1024, 392
        v = workloads.k_minor(workloads.c5_s8_batched(B=B, M=M, K=K, N=N))
        text = hm.k_minor_s8_batched(B, M, K, N)
        host_args = [v["lhs"], v["weights"], v["scales"]]
        dev_args = [dev_bf16(v["lhs"]), dev_s8(v["weights"]), dev_f32(v["scales"])]
        want = "dot -> xla_amd.dequant_dot [DEFAULT, s8, weights [N,K]]"
        sv = np.repeat(v["scales"].astype(np.float64)[:, :, None], K, axis=2)
    out, rw, _ = hlo_runner.compile_and_run(text, dev_args)
    torch.cuda.synchronize()
    assert rw == [want]
    assert ffi.last_kernel().startswith("dequant_dot_nk_"), ffi.last_kernel()
    ref = reference(text, host_args)
    wd = np.abs(v["weights"].astype(np.float64)) * sv          # [.., N, K]
    fl = dot_floor(np.abs(dtypes.bf16_to_f32(v["lhs"]).astype(np.float64)), np.swapaxes(wd, -1, -2), K)
    check_dot(host_bf16(out), ref, fl, "[N,K] %s module" % kind)


def test_unrewritten_module_does_not_run():
    say("module with nothing to rewrite")
    text = "HloModule m\nENTRY e {\n  a = f32[4] parameter(0)\n  ROOT b = f32[4] add(a, a)\n}\n"
    with pytest.raises(NotImplementedError, match="was not rewritten into a custom call"):
        hlo_runner.compile_and_run(text, [torch.zeros(4, device="cuda")])


@pytest.mark.parametrize("case", hm.INT4_DOT_CASES, ids=[c[0] for c in hm.INT4_DOT_CASES])
@pytest.mark.parametrize("weights_on_lhs", [False, True])
def test_reference_int4_shape_table(case, weights_on_lhs):
    """The modules of Int4WeightsOnTheLhs[WithBatchDim] / Int4WeightsOnTheRhs over Int4TestCases
    (fusion_emitter_int4_device_test.cc:495-645): f32 dot of unscaled s4 weights on either side, both
    contracting dimensions on both operands, with and without a batch dimension.  Integer weights
    and bf16 activations: compared with the op-by-op evaluation of the unrewritten module (the
    reference compares at 1e-5 .. 1e-2, :603-604, :557-558)."""
    from tests.gpu_util import check_dot_f32
    name, lhs, rhs, lc, rc, out_dims = case
    say("module %s %s" % ("lhs" if weights_on_lhs else "rhs", name))
    import zlib
    rng = np.random.default_rng(zlib.crc32(name.encode()) + int(weights_on_lhs))
    w_dims, a_dims = (lhs, rhs) if weights_on_lhs else (rhs, lhs)
    w = rng.integers(-8, 8, size=w_dims).astype(np.int8)
    a = dtypes.f32_to_bf16(rng.standard_normal(a_dims).astype(np.float32))
    text = hm.int4_weights_dot(case, weights_on_lhs)
    wd, ad = dev_u8(dtypes.pack_s4(w)), dev_bf16(a)
    out, rw, rf = hlo_runner.compile_and_run(text, [wd, ad] if weights_on_lhs else [ad, wd])
    torch.cuda.synchronize()
    assert len(rw) == 1 and "f32 result" in rw[0] and rf == [], (rw, rf)
    assert list(out.shape) == list(out_dims) and out.dtype == torch.float32
    ref = reference(text, [w, a] if weights_on_lhs else [a, w])
    # floor from sum |a| |w| over k, laid out like the result
    rank = len(lhs)
    w_c, a_c = (lc, rc) if weights_on_lhs else (rc, lc)
    wa = np.abs(w.astype(np.float64))
    aa = np.abs(dtypes.bf16_to_f32(a).astype(np.float64))
    wkn = wa if w_c == rank - 2 else np.swapaxes(wa, -1, -2)        # [..,K,N]
    amk = aa if a_c == rank - 1 else np.swapaxes(aa, -1, -2)        # [..,M,K]
    s = amk @ wkn                                                   # [..,M,N]
    if weights_on_lhs:
        s = np.swapaxes(s, -1, -2)
    check_dot_f32(out.cpu().numpy(), ref, 8 * 2.0 ** -24 * s, "int4 table %s %s" % (name, ffi.last_kernel()))
