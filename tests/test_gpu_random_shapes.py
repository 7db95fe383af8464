"""Seeded random shapes through every handler against the oracle: ragged M, K, N and group sizes,
every epilogue, both typings -- whatever kernel the launcher picks for them."""
import sys

import numpy as np
import pytest
import torch

from tests.gpu_util import dev_bf16
from tests.test_gpu_dequant_dot import compare, ragged_floor, run_dot, run_ragged
from tests.gpu_util import dot_floor
from tests.test_gpu_fp8_dot import EPI, floor_for, reference, run
from tests.gpu_util import check_dot
from xla_amd import dtypes, ffi, ops, workloads

pytestmark = pytest.mark.gpu

EPILOGUES = ["DEFAULT", "BIAS", "RELU", "BIAS_RELU", "GELU", "BIAS_GELU", "SILU", "BIAS_SILU"]


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def test_dequant_dot_random_shapes(oracle):
    rng = np.random.default_rng(2024)
    kernels = set()
    for case in range(36):
        bits = int(rng.choice([4, 8]))
        M = int(rng.choice([1, 2, 5, 8, 13, 16, 17, 31, 32, 40, 64, 65, 100, 200]))
        group = int(rng.choice([8, 16, 32, 64, 128]))
        K = group * int(rng.integers(1, 40))
        N = int(rng.choice([8, 24, 64, 100, 128, 136, 256, 520, 1000]))
        per_channel = bool(rng.integers(0, 2))
        if per_channel:
            group = K
        if bits == 4 and (K * N) % 2:
            N += 1
        epilogue = EPILOGUES[int(rng.integers(0, 8))]
        typed = "bf16" if rng.integers(0, 2) else "f32"
        # (grouped scales under an f32 multiply: group-factored sums when the group is whole 32-row steps
        # and the shape fits, the one-thread-per-output kernel otherwise)
        say("dequant_dot #%d s%d M=%d K=%d N=%d group=%d %s %s" % (case, bits, M, K, N, group, epilogue, typed))
        lhs = dtypes.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
        wq = rng.integers(-8 if bits == 4 else -127, 8 if bits == 4 else 128, size=(K, N)).astype(np.int8)
        sc = rng.uniform(1e-3, 2e-2, size=(K // group, N)).astype(np.float32)
        if per_channel:
            sc = sc.reshape(N)
        w = dict(lhs=lhs, weights=wq, scales=dtypes.f32_to_bf16(sc) if typed == "bf16" else sc,
                 bias=dtypes.f32_to_bf16(rng.standard_normal(N).astype(np.float32)) if "BIAS" in epilogue else None,
                 weight_dtype="s%d" % bits, weight_shape=(K, N), group=group, dequant_type=typed, epilogue=epilogue)
        got, kern = run_dot(w)
        kernels.add(kern.split("_v")[0])
        compare(oracle, w, got, "#%d %s" % (case, kern))
    assert len(kernels) >= 3, kernels    # decode, tiled and generic all took part


def test_dequant_dot_k_minor_random_shapes(oracle):
    """The same draw with the weights stored [N,K] (rhs_contracting_dim = 1)."""
    from tests.test_gpu_dequant_dot_nk import run_nk
    rng = np.random.default_rng(4048)
    kernels = set()
    for case in range(30):
        bits = int(rng.choice([4, 8]))
        M = int(rng.choice([1, 2, 5, 8, 13, 16, 17, 31, 32, 40, 64, 65, 100, 200]))
        group = int(rng.choice([8, 16, 32, 64, 128, 256]))
        K = group * int(rng.integers(1, 24))
        N = int(rng.choice([8, 24, 64, 100, 128, 136, 256, 520, 1000]))
        per_channel = bool(rng.integers(0, 2))
        if per_channel:
            group = K
        if bits == 4 and K % 2:
            K += 1; group = K; per_channel = True
        epilogue = EPILOGUES[int(rng.integers(0, 8))]
        typed = "bf16" if rng.integers(0, 2) else "f32"
        say("dequant_dot [N,K] #%d s%d M=%d K=%d N=%d group=%d %s %s" % (case, bits, M, K, N, group, epilogue, typed))
        lhs = dtypes.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
        wq = rng.integers(-8 if bits == 4 else -127, 8 if bits == 4 else 128, size=(K, N)).astype(np.int8)
        sc = rng.uniform(1e-3, 2e-2, size=(K // group, N)).astype(np.float32)
        if per_channel:
            sc = sc.reshape(N)
        w = dict(lhs=lhs, weights=wq, scales=dtypes.f32_to_bf16(sc) if typed == "bf16" else sc,
                 bias=dtypes.f32_to_bf16(rng.standard_normal(N).astype(np.float32)) if "BIAS" in epilogue else None,
                 weight_dtype="s%d" % bits, weight_shape=(K, N), group=group, dequant_type=typed, epilogue=epilogue)
        if bits == 4:
            w["weights_packed"] = dtypes.pack_s4(wq)
        got, kern = run_nk(w)
        kernels.add("generic" if kern.endswith("generic") else kern.rsplit("_", 1)[-1])
        compare(oracle, w, got, "[N,K] #%d %s" % (case, kern))
    assert len(kernels) >= 3, kernels    # rounded, factored (or group-factored) and generic all took part


def test_fp8_dot_random_shapes(oracle):
    rng = np.random.default_rng(77)
    for case in range(16):
        M = int(rng.choice([1, 7, 16, 100, 256, 300]))
        K = 16 * int(rng.integers(1, 40)) if rng.integers(0, 4) else int(rng.integers(1, 300))
        N = int(rng.choice([16, 40, 64, 200, 256, 272]))
        nk = bool(rng.integers(0, 2))
        w = workloads.c3_fp8(M, K, N)
        w["epilogue"] = EPILOGUES[int(rng.integers(0, 8))]
        if "BIAS" not in w["epilogue"]:
            w["bias"] = None
        vec = int(rng.integers(0, 4))
        if vec & 1:
            w["a_scale"] = rng.uniform(0.004, 0.04, M).astype(np.float32)
        if vec & 2:
            w["b_scale"] = rng.uniform(0.004, 0.04, N).astype(np.float32)
        say("fp8_scaled_dot #%d M=%d K=%d N=%d nk=%s %s scales=%d" % (case, M, K, N, nk, w["epilogue"], vec))
        got, kern = run(w, nk=nk)
        n_floor = check_dot(got, reference(oracle, w), floor_for(w, exact_kernel="exact" in kern), "#%d %s" % (case, kern))
        assert n_floor <= max(8, got.size // 20)


def test_fp8_dot_bf16_typed_random_shapes(oracle):
    """A bf16-typed dequantise multiply over row counts on both sides of what one streaming launch takes,
    K long enough for passes to be chosen, scales that are powers of two, that are not, and vectors: whichever
    of the f8 kernels, their rounding form, the bf16-operand kernels and the exact kernel the launcher picks."""
    rng = np.random.default_rng(78)
    kernels = set()
    for case in range(18):
        M = int(rng.choice([1, 20, 48, 49, 64, 65, 96, 130]))
        K = 16 * int(rng.choice([8, 33, 64, 128, 200]))
        N = int(rng.choice([40, 64, 200, 264]))
        nk = bool(rng.integers(0, 2))
        w = workloads.c3_fp8(M, K, N)
        w["epilogue"] = EPILOGUES[int(rng.integers(0, 8))]
        if "BIAS" not in w["epilogue"]:
            w["bias"] = None
        kind = int(rng.integers(0, 4))   # 0: powers of two, 1: any scalar, 2: per-row a, 3: both vectors
        if kind == 0:
            w["a_scale"], w["b_scale"] = np.float32(1 / 32), np.float32(1 / 128)
        elif kind == 1:
            w["a_scale"], w["b_scale"] = np.float32(0.0234375), np.float32(0.01171875)   # 3/128, 3/256
        else:
            w["a_scale"] = rng.uniform(0.004, 0.04, M).astype(np.float32)
            if kind == 3:
                w["b_scale"] = rng.uniform(0.004, 0.04, N).astype(np.float32)
        say("fp8_scaled_dot bf16-typed #%d M=%d K=%d N=%d nk=%s %s scales=%d" % (case, M, K, N, nk, w["epilogue"], kind))
        got, kern = run(w, nk=nk, dequant_type="bf16")
        kernels.add("rounded" if "rounded" in kern else "bf16_operands" if "bf16_operands" in kern else kern.split("_m")[0])
        ref = reference(oracle, w, dequant_type="bf16")
        n_floor = check_dot(got, ref, floor_for(w, exact_kernel=kind != 0), "#%d %s" % (case, kern))
        assert n_floor <= max(8, got.size // 20)
    assert {"rounded", "bf16_operands"} <= kernels, kernels


def test_rowwise_quantize_random_shapes(oracle):
    rng = np.random.default_rng(5)
    for case in range(12):
        R = int(rng.integers(1, 40))
        C = int(rng.choice([8, 33, 256, 1000, 1024, 4096, 5000, 8192, 16384, 20000, 33001]))
        rms = bool(rng.integers(0, 2))
        say("rowwise_quantize_fp8 #%d R=%d C=%d rmsnorm=%s" % (case, R, C, rms))
        x = dtypes.f32_to_bf16((rng.standard_normal((R, C)) * rng.choice([1e-3, 1.0, 300.0])).astype(np.float32))
        g = dtypes.f32_to_bf16(rng.uniform(0.5, 1.5, C).astype(np.float32))
        q, s = ops.rowwise_quantize_fp8(dev_bf16(x), dev_bf16(g) if rms else None, eps=1e-6)
        torch.cuda.synchronize()
        if rms:
            q_ref, s_ref = oracle.rmsnorm_quantize_fp8(x, g, eps=1e-6)
        else:  # without RMSNorm the pattern is amax / 448, divide, clamp, convert: plain numpy
            xf = dtypes.bf16_to_f32(x)
            s_ref = (np.abs(xf).max(axis=1) / np.float32(448)).astype(np.float32)
            q_ref = oracle.f32_to_f8e4m3fn(np.clip((xf / s_ref[:, None]).astype(np.float32), -448, 448))
        assert np.array_equal(s.cpu().numpy().view(np.uint32), s_ref.view(np.uint32)), case
        assert np.array_equal(q.cpu().numpy().view(np.uint8), q_ref), case


def test_ragged_dot_random_shapes(oracle):
    """Random row counts, expert counts and splits (empty groups, sizes that overrun M, rows nobody
    owns), s8 experts with a scale per channel and s4 experts with group scales: whichever of the
    decode chunks and the grouped GEMM the launcher picks."""
    rng = np.random.default_rng(31)
    kernels = set()
    for case in range(14):
        s4 = bool(rng.integers(0, 2))
        G = int(rng.integers(1, 7))
        M = int(rng.choice([1, 7, 40, 64, 65, 130, 300, 520, 700]))
        K = 128 * int(rng.integers(1, 9))
        N = int(rng.choice([64, 128, 264, 512]))
        sizes = rng.multinomial(int(M * rng.choice([0.6, 1.0, 1.3])), np.ones(G) / G)
        if rng.integers(0, 3) == 0:
            sizes[int(rng.integers(0, G))] = 0
        say("ragged #%d %s M=%d K=%d N=%d G=%d sizes=%s" % (case, "s4" if s4 else "s8", M, K, N, G, list(sizes)))
        if s4:
            w = workloads.ragged_s4_group_experts(M=M, K=K, N=N, groups=G, group=128, sizes=sizes)
            ref = oracle.ragged_dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", w["group_sizes"],
                                            bias=w["bias"], group=128)
            wd = np.max(np.abs(w["weights"].astype(np.float64)) *
                        np.repeat(dtypes.bf16_to_f32(w["scales"]).astype(np.float64), 128, axis=1), axis=0)
            floor = dot_floor(np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64)), wd, K)
        else:
            w = workloads.ragged_s8_experts(M=M, K=K, N=N, groups=G, sizes=sizes)
            ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
            floor = ragged_floor(w)
        # matrices this small are always cheaper in the decode kernel's chunks: every other case asks for the tiles
        force = 3 if case % 2 else 0
        try:
            got, kern = run_ragged(w, force_kernel=force)
        except ffi.FfiError as e:   # the tiles take more than 64 rows and 16-byte rows of weights
            assert force == 3 and "does not cover this shape" in str(e), e
            got, kern = run_ragged(w)
        kernels.add("tiled" if "tiled" in kern else "decode")
        check_dot(got, ref, floor, "ragged #%d %s" % (case, kern))
    assert kernels == {"tiled", "decode"}, kernels
