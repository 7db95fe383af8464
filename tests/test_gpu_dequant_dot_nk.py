"""GPU parity of xla_amd.dequant_dot over weights stored [N,K] (rhs_contracting_dim = 1, the
spelling of fusion_emitter_int4_device_test.cc:867-892).  The values of such a dot are those of
the [K,N] call on the transposed arrays, so the reference is the oracle on the [K,N] workload the
case was made from; the dequantised weights themselves are read back bit-exactly with one-hot
activations."""
import sys

import numpy as np
import pytest
import torch

from tests.gpu_util import dev_bf16, dev_f32, dev_s8, dev_u8, host_bf16
from tests.test_gpu_dequant_dot import compare
from xla_amd import dtypes, ffi, ops, workloads

pytestmark = pytest.mark.gpu


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def run_nk(w, force_kernel=0, slices=0, ct=0, scratch="auto"):
    """w: a [K,N] workload; runs it with the weights re-laid out [N,K]."""
    v = workloads.k_minor(w)
    lhs = dev_bf16(v["lhs"])
    wt = dev_u8(v["weights_packed"]) if v["weight_dtype"] in ("s4", "u4") else dev_s8(v["weights"])
    zp = dev_u8(v["zero_points_packed"]) if v.get("zero_points_packed") is not None else None
    sc = dev_bf16(v["scales"]) if v["scales"].dtype == np.uint16 else dev_f32(v["scales"])
    bias = None
    if v.get("bias") is not None:
        bias = dev_bf16(v["bias"]) if v["bias"].dtype == np.uint16 else dev_f32(v["bias"])
    ffi.set_option("dequant_dot_kernel", force_kernel)
    ffi.set_option("dequant_dot_slices", slices)
    ffi.set_option("dequant_dot_nk_ct", ct)
    try:
        out = ops.dequant_dot(lhs, wt, sc, bias, weight_dtype=v["weight_dtype"], weight_shape=v["weight_shape"],
                              epilogue=v["epilogue"], dequant_type=v["dequant_type"], dot_type=v.get("dot_type", "f32"),
                              epilogue_type=v.get("epilogue_type", "f32"), zero_points=zp,
                              scale_group_size=0 if v["group"] == v["lhs"].shape[-1] else v["group"],
                              rhs_contracting_dim=1, scratch=scratch)
        torch.cuda.synchronize()
    finally:
        for k in ("dequant_dot_kernel", "dequant_dot_slices", "dequant_dot_nk_ct"):
            ffi.set_option(k, 0)
    return host_bf16(out), ffi.last_kernel()


@pytest.mark.parametrize("M", [1, 8, 16, 17, 32, 40, 64])
def test_s4_group_scales_bf16_multiply(oracle, M):
    say("dequant_dot [N,K] s4 group 128 bf16 multiply M=%d" % M)
    w = workloads.c2_s4_group(M=M, K=4096, N=1024)
    got, kern = run_nk(w)
    assert kern == "dequant_dot_nk_s4_m%d_rounded" % (16 if M <= 16 else 32 if M <= 32 else 64), kern
    compare(oracle, w, got, "[N,K] s4 M=%d %s" % (M, kern))


@pytest.mark.parametrize("M", [3, 16, 24, 33, 64])
def test_s8_per_channel_f32_multiply(oracle, M):
    say("dequant_dot [N,K] s8 per channel M=%d" % M)
    w = workloads.c1_s8_channel(M=M, K=2048, N=1000)
    got, kern = run_nk(w)
    assert kern == "dequant_dot_nk_s8_m%d_factored" % (16 if M <= 16 else 32 if M <= 32 else 64), kern
    compare(oracle, w, got, "[N,K] s8 M=%d %s" % (M, kern))


@pytest.mark.parametrize("ct", [1, 2, 4])
@pytest.mark.parametrize("slices", [1, 2, 4])
def test_channel_tiles_and_k_slices(oracle, ct, slices):
    say("dequant_dot [N,K] s4 ct=%d slices=%d" % (ct, slices))
    w = workloads.c2_s4_group(M=5, K=2048, N=328, group=64)
    got, kern = run_nk(w, ct=ct, slices=slices)
    assert kern.startswith("dequant_dot_nk_s4_m16") and kern.endswith("_rounded"), kern
    compare(oracle, w, got, "[N,K] s4 %s slices=%d" % (kern, slices))
    w = workloads.c1_s8_channel(M=9, K=1024, N=200)
    got, kern = run_nk(w, ct=ct, slices=slices)
    assert kern.startswith("dequant_dot_nk_s8_m16") and kern.endswith("_factored"), kern
    compare(oracle, w, got, "[N,K] s8 %s slices=%d" % (kern, slices))


def test_k_slices_without_scratch_run_as_one(oracle):
    say("dequant_dot [N,K] s8 few channels, no scratch")
    w = workloads.c1_s8_channel(M=4, K=4096, N=256)
    got, kern = run_nk(w)
    got2, kern2 = run_nk(w, scratch=None)
    assert kern == kern2 == "dequant_dot_nk_s8_m16_factored"
    compare(oracle, w, got, "[N,K] sliced")
    compare(oracle, w, got2, "[N,K] unsliced")


@pytest.mark.parametrize("kind,M", [("s8", 8), ("s8", 48), ("s4", 8), ("s4", 32), ("u4", 16)])
def test_group_scales_f32_multiply(oracle, kind, M):
    """f32-typed multiply with group scales: per-group integer sums folded with the scale."""
    say("dequant_dot [N,K] %s group scales f32 multiply M=%d" % (kind, M))
    if kind == "s8":
        w = workloads.c1_s8_channel(M=M, K=2048, N=520)
        w["scales"] = np.random.default_rng(5).uniform(1e-3, 1e-2, (2048 // 128, 520)).astype(np.float32)
        w["group"] = 128
    elif kind == "s4":
        w = workloads.c2_s4_group(M=M, K=2048, N=520, group=256)
        w["dequant_type"] = "f32"
    else:
        w = workloads.u4_zero_point_group(M=M, K=2048, N=520, group=128)
        w["dequant_type"] = "f32"
    got, kern = run_nk(w)
    assert kern.endswith("_group_factored_zp" if kind == "u4" else "_group_factored"), kern
    compare(oracle, w, got, "[N,K] %s %s" % (kind, kern))


@pytest.mark.parametrize("M", [2, 16, 30])
def test_u4_zero_points(oracle, M):
    say("dequant_dot [N,K] u4 + zero points M=%d" % M)
    w = workloads.u4_zero_point_group(M=M, K=2048, N=776, group=64)
    got, kern = run_nk(w)
    assert kern.startswith("dequant_dot_nk_s4_m") and kern.endswith("_rounded_zp"), kern
    compare(oracle, w, got, "[N,K] u4 zp M=%d" % M)


@pytest.mark.parametrize("kind", ["s8", "s4", "u4"])
def test_one_hot_reads_back_the_dequantised_weights(oracle, kind):
    """Activation row m is the unit vector of k = (m * 37 + 5) % K: output [m, n] is weight (n, k)
    dequantised, with no sum to hide behind."""
    say("dequant_dot [N,K] one-hot %s" % kind)
    K, N, M = 512, 264, 64
    if kind == "s8":
        w = workloads.c1_s8_channel(M=M, K=K, N=N)
    elif kind == "s4":
        w = workloads.c2_s4_group(M=M, K=K, N=N, group=32)
        w["epilogue"], w["bias"] = "DEFAULT", None
    else:
        w = workloads.u4_zero_point_group(M=M, K=K, N=N, group=32)
        w["epilogue"], w["bias"] = "DEFAULT", None
    a = np.zeros((M, K), np.float32)
    ks = (np.arange(M) * 37 + 5) % K
    a[np.arange(M), ks] = 1.0
    w["lhs"] = dtypes.f32_to_bf16(a)
    got, kern = run_nk(w)
    assert kern.startswith("dequant_dot_nk_"), kern
    from tests.test_gpu_dequant_dot import oracle_dot
    assert np.array_equal(got, oracle_dot(oracle, w)), kern


def test_batched_with_per_batch_scales(oracle):
    say("dequant_dot [B,N,K] s8 per batch scales, s4 group scales")
    w = workloads.c5_s8_batched(B=3, M=20, K=1024, N=392)
    got, kern = run_nk(w)
    assert kern == "dequant_dot_nk_s8_m32_factored", kern
    compare(oracle, w, got, "[B,N,K] s8")
    w = workloads.batched_s4_group(B=3, M=8, K=1024, N=264, group=128)
    got, kern = run_nk(w)
    assert kern == "dequant_dot_nk_s4_m16_rounded", kern
    compare(oracle, w, got, "[B,N,K] s4")


@pytest.mark.parametrize("kind", ["s8", "s4"])
def test_more_than_64_tokens_run_in_token_chunks(oracle, kind):
    say("dequant_dot [N,K] %s 200 tokens" % kind)
    w = (workloads.c1_s8_channel(M=200, K=1024, N=392) if kind == "s8"
         else workloads.c2_s4_group(M=200, K=1024, N=392, group=128))
    got, kern = run_nk(w)
    assert kern.startswith("dequant_dot_nk_" + kind), kern
    compare(oracle, w, got, "[N,K] %s 200 tokens" % kind)


@pytest.mark.parametrize("K,N,group", [(1000, 36, 1000), (1096, 50, 8), (72, 7, 24)])
def test_unaligned_shapes_take_the_generic_kernel(oracle, K, N, group):
    say("dequant_dot [N,K] generic K=%d N=%d group=%d" % (K, N, group))
    w = workloads.c1_s8_channel(M=5, K=K, N=N)
    if group != K:
        w["scales"] = np.random.default_rng(6).uniform(1e-3, 1e-2, (K // group, N)).astype(np.float32)
        w["group"] = group
    got, kern = run_nk(w)
    assert kern == "dequant_dot_nk_generic", kern
    compare(oracle, w, got, "[N,K] generic s8")
    w = workloads.c2_s4_group(M=5, K=K, N=N + (N & 1), group=group)
    got, kern = run_nk(w)
    assert kern == "dequant_dot_nk_generic", kern
    compare(oracle, w, got, "[N,K] generic s4")


def test_forced_generic_equals_streaming_kernel_within_tolerance(oracle):
    say("dequant_dot [N,K] forced generic")
    w = workloads.c2_s4_group(M=12, K=1024, N=136, group=128)
    got, kern = run_nk(w, force_kernel=1)
    assert kern == "dequant_dot_nk_generic", kern
    compare(oracle, w, got, "[N,K] forced generic")


def test_bad_arguments():
    say("dequant_dot [N,K] error paths")
    lhs = torch.zeros((4, 64), dtype=torch.bfloat16, device="cuda")
    wt = torch.zeros((32, 64), dtype=torch.int8, device="cuda")
    sc = torch.ones((32,), dtype=torch.float32, device="cuda")
    with pytest.raises(ffi.FfiError, match="come with scale_group_size"):
        ops.dequant_dot(lhs, wt, sc, rhs_contracting_dim=1)
    with pytest.raises(ffi.FfiError, match="rhs_contracting_dim must be 0 or 1"):
        ops.dequant_dot(lhs, wt, sc, rhs_contracting_dim=2, scale_group_size=0)
    sc2 = torch.ones((2, 32), dtype=torch.float32, device="cuda")
    with pytest.raises(ffi.FfiError, match=r"must be \[batch,\]N,K/scale_group_size"):
        ops.dequant_dot(lhs, wt, sc2, rhs_contracting_dim=1, scale_group_size=32)


# ---- more than 64 tokens: the tiled kernel with the [N,K] loaders ----------------------------

@pytest.mark.parametrize("kind,M,K,N,group", [("s8", 300, 1024, 520, 0), ("s8", 65, 4096, 264, 0), ("s4", 300, 1024, 520, 128),
                                              ("s4", 129, 2048, 1000, 32), ("s4", 256, 1024, 256, 1024)])
def test_tiled_kernel_takes_k_minor_weights(oracle, kind, M, K, N, group):
    say("dequant_dot [N,K] tiled %s M=%d K=%d N=%d group=%d" % (kind, M, K, N, group))
    w = (workloads.c1_s8_channel(M=M, K=K, N=N) if kind == "s8" else workloads.c2_s4_group(M=M, K=K, N=N, group=group))
    got, kern = run_nk(w, force_kernel=3)
    assert kern.startswith("dequant_dot_tiled_nk_%s_" % kind), kern
    compare(oracle, w, got, "[N,K] tiled %s" % kern)


@pytest.mark.parametrize("K", [32, 64, 96, 128, 160, 192, 256, 288])
def test_tiled_k_minor_with_few_stages(oracle, K):
    """One to five stages of 64 k through the [N,K] loaders of the tiled kernel."""
    say("dequant_dot [N,K] tiled, K=%d" % K)
    M, N = 130, 264
    w = workloads.c1_s8_channel(M=M, K=K, N=N)
    got, kern = run_nk(w, force_kernel=3)
    assert kern.startswith("dequant_dot_tiled_nk_s8_"), kern
    compare(oracle, w, got, "[N,K] s8 tiled K=%d" % K)
    w = workloads.c2_s4_group(M=M, K=K, N=N, group=32)
    got, kern = run_nk(w, force_kernel=3)
    assert kern.startswith("dequant_dot_tiled_nk_s4_"), kern
    compare(oracle, w, got, "[N,K] s4 tiled K=%d" % K)


def test_tiled_k_minor_batched_and_split_last_round(oracle):
    say("dequant_dot [B,N,K] tiled s8, tiles split along K")
    w = workloads.c5_s8_batched(B=2, M=300, K=2048, N=520)
    got, kern = run_nk(w, force_kernel=3)
    assert kern == "dequant_dot_tiled_nk_s8_factored:tail2", kern   # 2 x 2 x 3 tiles: all of them as pairs
    compare(oracle, w, got, "[B,N,K] tiled s8 split")
    got2, kern2 = run_nk(w, force_kernel=3, scratch=None)
    assert kern2 == "dequant_dot_tiled_nk_s8_factored", kern2
    compare(oracle, w, got2, "[B,N,K] tiled s8 whole")


@pytest.mark.parametrize("kind", ["s8", "s4"])
def test_tiled_k_minor_one_hot(oracle, kind):
    say("dequant_dot [N,K] tiled one-hot %s" % kind)
    K, N, M = 512, 264, 192
    w = workloads.c1_s8_channel(M=M, K=K, N=N) if kind == "s8" else workloads.c2_s4_group(M=M, K=K, N=N, group=32)
    w["epilogue"], w["bias"] = "DEFAULT", None
    a = np.zeros((M, K), np.float32)
    a[np.arange(M), (np.arange(M) * 37 + 5) % K] = 1.0
    w["lhs"] = dtypes.f32_to_bf16(a)
    got, kern = run_nk(w, force_kernel=3)
    assert kern.startswith("dequant_dot_tiled_nk_"), kern
    from tests.test_gpu_dequant_dot import oracle_dot
    assert np.array_equal(got, oracle_dot(oracle, w)), kern


def test_large_prefill_picks_the_tiled_kernel_by_itself(oracle):
    say("dequant_dot [N,K] s8 2048 tokens: routing")
    w = workloads.c1_s8_channel(M=2048, K=2048, N=8192)   # a full round of tiles (fewer tokens on a matrix this small stream)
    got, kern = run_nk(w)
    assert kern.startswith("dequant_dot_tiled_nk_s8_factored"), kern
    # the oracle on a block of rows and channels
    rows, cols = slice(512, 560), slice(1000, 1256)
    blk = dict(w, lhs=w["lhs"][rows], weights=w["weights"][:, cols], scales=w["scales"][cols], weight_shape=(2048, 256))
    compare(oracle, blk, got[rows, cols], "[N,K] tiled s8 block")


# ---- ragged dot over experts stored [G,N,K] ------------------------------------------------------

def run_ragged_nk(w, sizes_dtype=torch.int32, force_kernel=0):
    v = workloads.k_minor(w)
    lhs = dev_bf16(v["lhs"])
    wt = dev_u8(v["weights_packed"]) if v["weight_dtype"] in ("s4", "u4") else dev_s8(v["weights"])
    sc = dev_bf16(v["scales"]) if v["scales"].dtype == np.uint16 else dev_f32(v["scales"])
    bias = dev_bf16(v["bias"]) if v.get("bias") is not None else None
    gs = torch.from_numpy(np.asarray(v["group_sizes"], np.int64)).to(sizes_dtype).cuda()
    ffi.set_option("dequant_dot_kernel", force_kernel)
    try:
        out = ops.dequant_dot(lhs, wt, sc, bias, weight_dtype=v["weight_dtype"], weight_shape=v["weight_shape"],
                              epilogue=v["epilogue"], dequant_type=v["dequant_type"],
                              scale_group_size=0 if v["group"] == v["lhs"].shape[-1] else v["group"], group_sizes=gs,
                              rhs_contracting_dim=1)
        torch.cuda.synchronize()
    finally:
        ffi.set_option("dequant_dot_kernel", 0)
    return host_bf16(out), ffi.last_kernel()


@pytest.mark.parametrize("M,K,N,G,sizes,sizes_dtype", [
    (32, 1024, 512, 8, None, torch.int32), (64, 512, 384, 4, [10, 0, 50, 4], torch.int64),
    (12, 256, 136, 3, [5, 0, 2], torch.int32), (7, 512, 128, 2, [9, 9], torch.int32),
    (40, 512, 256, 5, [0, 0, 0, 0, 0], torch.int64), (200, 512, 264, 3, [150, 0, 30], torch.int32)])
def test_ragged_dot_over_k_minor_experts(oracle, M, K, N, G, sizes, sizes_dtype):
    """Rows sorted by expert, experts stored [G,N,K]: random splits with empty groups, rows that no
    group owns (epilogue(0) = the bias), sizes that overrun M, a call whose groups are all empty, a
    group of more rows than a token chunk."""
    from tests.test_gpu_dequant_dot import ragged_floor
    from tests.gpu_util import check_dot
    say("dequant_dot ragged [G,N,K] M=%d K=%d N=%d G=%d sizes=%s" % (M, K, N, G, sizes))
    w = workloads.ragged_s8_experts(M=M, K=K, N=N, groups=G, sizes=sizes)
    got, kern = run_ragged_nk(w, sizes_dtype)
    assert kern.startswith("dequant_dot_nk_s8_"), kern
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
    check_dot(got, ref, ragged_floor(w), "ragged [G,N,K] %s" % kern)
    got_g, kern_g = run_ragged_nk(w, sizes_dtype, force_kernel=1)
    assert kern_g == "dequant_dot_nk_generic", kern_g
    check_dot(got_g, ref, ragged_floor(w), "ragged [G,N,K] generic")


@pytest.mark.parametrize("G,M", [(70, 90), (130, 300)])
def test_ragged_dot_k_minor_over_many_groups(oracle, G, M):
    """More groups than a wave has lanes (the item search scans the sizes 64 at a time), experts [G,N,K]."""
    from tests.test_gpu_dequant_dot import ragged_floor
    from tests.gpu_util import check_dot
    say("dequant_dot ragged [G,N,K] over %d groups, %d rows" % (G, M))
    rng = np.random.default_rng(G * 1000 + M)
    sizes = rng.multinomial(int(M * 0.9), np.ones(G) / G)
    sizes[rng.integers(0, G, 5)] = 0
    sizes[int(rng.integers(0, G))] += 20
    w = workloads.ragged_s8_experts(M=M, K=256, N=136, groups=G, sizes=sizes)
    got, kern = run_ragged_nk(w, torch.int32)
    assert kern.startswith("dequant_dot_nk_s8_"), kern
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
    check_dot(got, ref, ragged_floor(w), "ragged [G,N,K] over %d groups, %s" % (G, kern))


def test_ragged_dot_k_minor_many_groups_sizes_overrun(oracle):
    """Sizes that add up to one and a half times the rows over 130 groups, experts [G,N,K]: the rows run
    out inside the second block of 64 groups of the item search."""
    from tests.test_gpu_dequant_dot import ragged_floor
    from tests.gpu_util import check_dot
    G, M = 130, 200
    say("dequant_dot ragged [G,N,K], sizes overrun the rows, %d groups, %d rows" % (G, M))
    sizes = np.random.default_rng(77).multinomial(int(M * 1.5), np.ones(G) / G)
    assert int(sizes[:64].sum()) < M < int(sizes[:128].sum())
    w = workloads.ragged_s8_experts(M=M, K=256, N=136, groups=G, sizes=sizes)
    got, kern = run_ragged_nk(w, torch.int64)
    assert kern.startswith("dequant_dot_nk_s8_"), kern
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
    check_dot(got, ref, ragged_floor(w), "ragged [G,N,K], sizes overrun, %s" % kern)


def test_ragged_dot_k_minor_s4_group_scales(oracle):
    from tests.gpu_util import check_dot, dot_floor
    say("dequant_dot ragged [G,N,K] s4 group scales")
    w = workloads.ragged_s4_group_experts(M=48, K=1024, N=264, groups=4, group=128, sizes=[20, 0, 17, 5])
    got, kern = run_ragged_nk(w)
    assert kern.startswith("dequant_dot_nk_s4_"), kern
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", w["group_sizes"],
                                    bias=w.get("bias"), group=128)
    a = np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64))
    wd = np.max(np.abs(w["weights"].astype(np.float64)) *
                np.repeat(dtypes.bf16_to_f32(w["scales"]).astype(np.float64), 128, axis=1), axis=0)
    check_dot(got, ref, dot_floor(a, wd, 1024), "ragged [G,N,K] s4 %s" % kern)


@pytest.mark.parametrize("kind", ["s8", "s4"])
def test_ragged_dot_k_minor_grouped_gemm(oracle, kind):
    """Groups of hundreds of rows: the tiled kernel as a grouped GEMM over [G,N,K] experts."""
    from tests.gpu_util import check_dot, dot_floor
    say("dequant_dot ragged [G,N,K] tiled %s" % kind)
    sizes = [300, 0, 257, 100]
    if kind == "s8":
        w = workloads.ragged_s8_experts(M=700, K=512, N=264, groups=4, sizes=sizes)
        ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
        wd = np.max(np.abs(w["weights"].astype(np.float64)) * w["scales"].astype(np.float64)[:, None, :], axis=0)
    else:
        w = workloads.ragged_s4_group_experts(M=700, K=512, N=264, groups=4, group=128, sizes=sizes)
        ref = oracle.ragged_dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", w["group_sizes"],
                                        bias=w.get("bias"), group=128)
        wd = np.max(np.abs(w["weights"].astype(np.float64)) *
                    np.repeat(dtypes.bf16_to_f32(w["scales"]).astype(np.float64), 128, axis=1), axis=0)
    got, kern = run_ragged_nk(w)
    assert kern.startswith("dequant_dot_tiled_nk_%s_" % kind) and kern.endswith(":ragged"), kern
    a = np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64))
    check_dot(got, ref, dot_floor(a, wd, 512), "ragged [G,N,K] tiled %s" % kind)
