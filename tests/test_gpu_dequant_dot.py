"""GPU parity of xla_amd.dequant_dot against the CPU oracle, through the FFI handler symbol.
Dots accumulate in f32 in a different order than the oracle, so outputs are compared within
2 bf16 ulp (with a cancellation floor derived from sum|a*w|); integer unpacking and the
dequantised weights themselves are checked bit-exactly with one-hot activations."""
import sys

import numpy as np
import pytest
import torch

from tests.gpu_util import check_dot, dev_bf16, dev_f32, dev_s8, dev_u8, dot_floor, host_bf16
from xla_amd import dtypes, ffi, ops, workloads

pytestmark = pytest.mark.gpu


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def run_dot(w, force_kernel=0, slices=0, vec=0, x=None, pair=0, depth=0, steps=0, tail=0, strip=0):
    """x: 1 keeps s4 weights off the kernels that dequantise through the 4x4x4 matrix instruction
    (default: off whenever a strip width `vec` of the other kernels is asked for); pair: 1 takes the
    two-workgroups-per-strip form of those kernels wherever the shape allows, 2 never; tail: 1 keeps
    the tiled kernel from splitting the tiles of its last round along K; strip: 64 or 128 channels per
    strip of the single-launch s8 kernel (0: its own choice)."""
    lhs = dev_bf16(w["lhs"])
    if w["weight_dtype"] in ("s4", "u4"):
        wt = dev_u8(w["weights_packed"] if "weights_packed" in w else dtypes.pack_s4(w["weights"]))
    else:
        wt = dev_s8(w["weights"])
    zp = dev_u8(w["zero_points_packed"]) if w.get("zero_points_packed") is not None else None
    sc = dev_bf16(w["scales"]) if w["scales"].dtype == np.uint16 else dev_f32(w["scales"])
    bias = None
    if w.get("bias") is not None:
        bias = dev_bf16(w["bias"]) if w["bias"].dtype == np.uint16 else dev_f32(w["bias"])
    ffi.set_option("dequant_dot_kernel", force_kernel)
    ffi.set_option("dequant_dot_slices", slices)
    ffi.set_option("dequant_dot_vec", vec)
    ffi.set_option("dequant_dot_x", (1 if vec else 0) if x is None else x)
    ffi.set_option("dequant_dot_pair", pair)
    ffi.set_option("dequant_dot_depth", depth)
    ffi.set_option("dequant_dot_steps", steps)
    ffi.set_option("dequant_dot_strip", strip)
    ffi.set_option("tiled_tail", tail)
    try:
        out = ops.dequant_dot(lhs, wt, sc, bias, weight_dtype=w["weight_dtype"],
                              weight_shape=w["weight_shape"], epilogue=w["epilogue"],
                              dequant_type=w["dequant_type"], dot_type=w.get("dot_type", "f32"),
                              epilogue_type=w.get("epilogue_type", "f32"), zero_points=zp,
                              scale_group_size=0 if w["group"] == w["lhs"].shape[-1] else w["group"])
        torch.cuda.synchronize()
    finally:
        for k in ("dequant_dot_kernel", "dequant_dot_slices", "dequant_dot_vec", "dequant_dot_x", "dequant_dot_pair",
                  "dequant_dot_depth", "dequant_dot_steps", "dequant_dot_strip", "tiled_tail"):
            ffi.set_option(k, 0)
    return host_bf16(out), ffi.last_kernel()


def oracle_dot(oracle, w):
    scale_ty = "bf16" if w["scales"].dtype == np.uint16 else "f32"
    wt = w["weights"]
    bits = 8
    if w["weight_dtype"] in ("s4", "u4"):
        wt, bits = (w["weights_packed"] if "weights_packed" in w else dtypes.pack_s4(w["weights"])), 4
    epi = {"DEFAULT": "none", "BIAS": "none", "RELU": "relu", "BIAS_RELU": "relu", "GELU": "gelu_tanh",
           "BIAS_GELU": "gelu_tanh", "SILU": "silu", "BIAS_SILU": "silu"}[w["epilogue"]]
    bias = w.get("bias")
    return oracle.dequant_dot(w["lhs"], wt, bits, w["scales"],
                              scale_ty, w["dequant_type"], bias=bias,
                              bias_ty="bf16" if (bias is not None and bias.dtype == np.uint16) else "f32",
                              group=w["group"], dot_ty=w.get("dot_type", "f32"),
                              ep_ty=w.get("epilogue_type", "f32"), epilogue=epi,
                              unsigned=w["weight_dtype"] == "u4", zero_points=w.get("zero_points_packed"))


def floor_for(w):
    a = np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64))
    s = w["scales"]
    sv = (dtypes.bf16_to_f32(s) if s.dtype == np.uint16 else s).astype(np.float64)
    wi = np.abs(w["weights"].astype(np.float64))
    if w.get("zero_points") is not None:   # the weights' magnitude is that of w - z
        z = w["zero_points"].astype(np.float64)
        wi = np.abs(w["weights"].astype(np.float64) - np.repeat(z.reshape(-1, z.shape[-1]), w["group"], axis=0).reshape(wi.shape))
    K = w["lhs"].shape[-1]
    if w["lhs"].ndim == 3:
        sv = sv.reshape(w["lhs"].shape[0], -1, sv.shape[-1])
        wd = wi * np.repeat(sv, w["group"], axis=1)
    else:
        sv = sv.reshape(-1, sv.shape[-1])
        wd = wi * np.repeat(sv, w["group"], axis=0)
    return dot_floor(a, wd, K)


def compare(oracle, w, got, what):
    ref = oracle_dot(oracle, w)
    n_floor = check_dot(got, ref, floor_for(w), what)
    # near-zero outputs (cancellation, or the flat tail of GELU/SiLU) are judged by the floor
    assert n_floor <= max(4, got.size // 50), "%s: %d outputs only passed through the floor" % (what, n_floor)


# ---- decode kernels (M <= 64) --------------------------------------------------------------

@pytest.mark.parametrize("M", [1, 8, 32, 40, 48, 64])
def test_c2_shape_reduced_n(oracle, M):
    """Configuration 2 with full K and group 128, N cut to 1024 so the oracle stays fast."""
    say("dequant_dot C2 s4 M=%d K=8192 N=1024" % M)
    w = workloads.c2_s4_group(M=M, K=8192, N=1024)
    got, kern = run_dot(w)
    assert kern.startswith("dequant_dot_decode_s4"), kern
    compare(oracle, w, got, "C2 M=%d %s" % (M, kern))


@pytest.mark.parametrize("M,vec,slices", [(3, 4, 1), (3, 8, 2), (16, 16, 4), (16, 8, 1), (20, 4, 2),
                                          (20, 8, 1), (64, 4, 2)])
def test_s4_decode_variants(oracle, M, vec, slices):
    say("dequant_dot s4 variants M=%d vec=%d slices=%d" % (M, vec, slices))
    w = workloads.c2_s4_group(M=M, K=2048, N=768, group=64)
    got, kern = run_dot(w, force_kernel=2, slices=slices, vec=vec)
    assert "_v%d_" % vec in kern, kern
    compare(oracle, w, got, "s4 %s slices=%d" % (kern, slices))


@pytest.mark.parametrize("M,pair,depth,slices,K,N,group", [
    (1, 2, 4, 1, 2048, 768, 128), (3, 2, 2, 2, 2048, 768, 64), (8, 1, 2, 0, 2048 + 256, 800, 128),
    (8, 2, 2, 1, 1024, 1024, 128), (16, 2, 4, 1, 2048, 768, 128), (16, 1, 2, 0, 4096, 256, 64),
    (20, 2, 2, 2, 2048 + 128, 736, 64), (33, 2, 4, 1, 1536, 512, 128), (48, 2, 2, 1, 1024, 640, 64),
    (64, 2, 2, 2, 2048, 768, 128), (5, 1, 2, 0, 1024 + 64, 1120, 64), (13, 1, 2, 0, 8192, 512, 128)])
def test_s4x_variants(oracle, M, pair, depth, slices, K, N, group):
    """The kernels that scale and transpose through the 4x4x4 matrix instruction: one workgroup per
    128-channel strip or two per 256-channel strip handing over inside the kernel, prefetch depth,
    K-slices, a ragged last strip and a K that is no whole number of waves' shares."""
    say("dequant_dot s4x M=%d pair=%d depth=%d slices=%d K=%d N=%d group=%d" % (M, pair, depth, slices, K, N, group))
    w = workloads.c2_s4_group(M=M, K=K, N=N, group=group)
    got, kern = run_dot(w, force_kernel=2, slices=slices, pair=pair, depth=depth)
    assert kern.startswith("dequant_dot_decode_s4x_") and kern.endswith("_pair") == (pair == 1), kern
    compare(oracle, w, got, "%s slices=%d" % (kern, slices))


@pytest.mark.parametrize("pair", [2, 1])
def test_s4x_unpack_and_dequant_bit_exact(oracle, pair):
    """One-hot activations through the matrix-instruction dequantisation: every output is one
    dequantised weight -- nibble order, sign, the f16 scale operand and the bf16 rounding, exactly;
    scales across the whole f16 window and both signs."""
    say("dequant_dot s4x one-hot pair=%d" % pair)
    K, N, group = 512, 512, 64
    rng = np.random.default_rng(5)
    wv = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
    wv[:16, :16] = np.arange(-8, 8, dtype=np.int8)[:, None]
    mant = rng.integers(128, 256, size=(K // group, N)).astype(np.float32) / 128.0
    expo = rng.integers(-22, 3, size=(K // group, N)).astype(np.float32)
    sign = rng.choice([-1.0, 1.0], size=(K // group, N)).astype(np.float32)
    sc = dtypes.f32_to_bf16(sign * mant * np.exp2(expo))
    for m0 in range(0, K, 16):
        a = np.zeros((16, K), np.float32)
        a[np.arange(16), m0 + np.arange(16)] = 1.0
        w = dict(lhs=dtypes.f32_to_bf16(a), weights=wv, weights_packed=dtypes.pack_s4(wv), scales=sc,
                 bias=None, weight_dtype="s4", weight_shape=(K, N), group=group, dequant_type="bf16",
                 epilogue="DEFAULT")
        got, kern = run_dot(w, force_kernel=2, pair=pair)
        assert kern.startswith("dequant_dot_decode_s4x_") and kern.endswith("_pair") == (pair == 1), kern
        prod = wv[m0:m0 + 16].astype(np.float32) * np.repeat(dtypes.bf16_to_f32(sc), group, axis=0)[m0:m0 + 16]
        want = dtypes.f32_to_bf16(prod)
        assert np.array_equal(dtypes.bf16_to_f32(got), dtypes.bf16_to_f32(want)), kern


@pytest.mark.parametrize("M,pair", [(4, 1), (4, 2), (24, 2)])
def test_s4x_scales_outside_the_f16_window(oracle, M, pair):
    """Zero scales stay on the fast path; huge, tiny, subnormal, infinite and NaN scales flag their
    channel, which the kernel then recomputes with ordinary arithmetic: every channel must still
    match the oracle -- also when the flagged rows lie in only one of the two workgroups of a strip."""
    say("dequant_dot s4x odd scales M=%d pair=%d" % (M, pair))
    K, N, group = 1024, 512, 128
    w = workloads.c2_s4_group(M=M, K=K, N=N, group=group)
    sc = dtypes.bf16_to_f32(w["scales"]).copy()
    sc[0, 3] = 0.0
    sc[:, 7] = 0.0
    sc[1, 40] = 16.0
    sc[2, 41] = 2.0 ** -30
    sc[3, 100] = 1e-39          # subnormal in bf16
    sc[5, 129] = np.inf
    sc[6, 200] = np.nan
    sc[7, 255] = -3.0e4
    sc[0, 300] = 64.0
    sc[7, 301] = 2.0 ** -25
    w["scales"] = dtypes.f32_to_bf16(sc)
    got, kern = run_dot(w, force_kernel=2, pair=pair)
    assert kern.startswith("dequant_dot_decode_s4x_") and kern.endswith("_pair") == (pair == 1), kern
    ref = oracle_dot(oracle, w)
    ok_cols = np.ones(N, bool)
    ok_cols[[129, 200]] = False
    a = np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64))
    wd = np.abs(w["weights"].astype(np.float64)) * np.abs(np.repeat(np.nan_to_num(sc.astype(np.float64), nan=0.0, posinf=0.0), group, axis=0))
    check_dot(got[:, ok_cols], ref[:, ok_cols], dot_floor(a, wd, K)[:, ok_cols], kern)
    # an infinite or NaN scale makes the whole channel non-finite, on both sides
    g, r = dtypes.bf16_to_f32(got), dtypes.bf16_to_f32(ref)
    assert not np.isfinite(r[:, [129, 200]]).any() and not np.isfinite(g[:, [129, 200]]).any()
    assert np.array_equal(np.isnan(g[:, [129, 200]]), np.isnan(r[:, [129, 200]]))


def test_s4x_pair_same_call_frame_replayed(oracle):
    """The hand-over flag is lowered by the finisher, so the very same call frame (same workspace,
    same flag value) can run again and again -- what a captured graph does -- with new activations
    each time; the workspace starts out holding arbitrary bytes."""
    say("dequant_dot s4x pair replay")
    M, K, N = 8, 2048, 1024
    w = workloads.c2_s4_group(M=M, K=K, N=N)
    lhs = dev_bf16(w["lhs"])
    wt, sc, bias = dev_u8(w["weights_packed"]), dev_bf16(w["scales"]), dev_bf16(w["bias"])
    nbytes = ffi.library().xla_amd_dequant_dot_workspace_bytes(1, M, K, N, dtypes.S4)
    ffi.set_option("dequant_dot_pair", 1)
    try:
        nbytes = max(nbytes, ffi.library().xla_amd_dequant_dot_workspace_bytes(1, M, K, N, dtypes.S4))
        scratch = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device="cuda")
        call = ops.dequant_dot(lhs, wt, sc, bias, weight_dtype="s4", weight_shape=(K, N), epilogue="BIAS_SILU",
                               dequant_type="bf16", scratch=scratch, build_only=True)
        rng = np.random.default_rng(9)
        for it in range(4):
            a = dtypes.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
            lhs.copy_(dev_bf16(a))
            out = call.run()
            torch.cuda.synchronize()
            assert ffi.last_kernel() == "dequant_dot_decode_s4x_m16_pair", ffi.last_kernel()
            compare(oracle, dict(w, lhs=a), host_bf16(out), "pair replay %d" % it)
    finally:
        ffi.set_option("dequant_dot_pair", 0)


def s8x_name(steps, strip):
    return "dequant_dot_decode_s8x_m16_%ss%d" % ("n64_" if strip == 64 else "", steps)


@pytest.mark.parametrize("strip", [128, 64])
@pytest.mark.parametrize("M,steps,K,N,epilogue,bf16_vectors", [
    (16, 0, 4096, 4096, "DEFAULT", False), (1, 1, 1024, 640, "BIAS_GELU", False), (5, 2, 1024, 648, "BIAS_SILU", True),
    (16, 4, 4096, 200, "RELU", True), (8, 1, 4096, 384, "BIAS", False), (3, 4, 1024, 128, "DEFAULT", False),
    (12, 2, 512, 1000, "BIAS_RELU", False), (16, 1, 256, 136, "SILU", True)])
def test_s8x_variants(oracle, M, steps, K, N, epilogue, bf16_vectors, strip):
    """The single-launch s8 kernel for small matrices: 1 to 16 K-slices per strip adding up inside the
    kernel, strips of 128 and of 64 channels, a ragged last strip, every epilogue, f32 and bf16 scale
    and bias vectors."""
    say("dequant_dot s8x M=%d steps=%d K=%d N=%d %s bf16_vectors=%s strip=%d" % (M, steps, K, N, epilogue, bf16_vectors, strip))
    w = workloads.c1_s8_channel(M=M, K=K, N=N)
    w["epilogue"] = epilogue
    rng = np.random.default_rng(11)
    if "BIAS" in epilogue:
        w["bias"] = rng.standard_normal(N).astype(np.float32)
        if bf16_vectors:
            w["bias"] = dtypes.f32_to_bf16(w["bias"])
    if bf16_vectors:
        w["scales"] = dtypes.f32_to_bf16(w["scales"])
    got, kern = run_dot(w, force_kernel=2, steps=steps, strip=strip)
    assert kern == s8x_name(steps or 4, strip), kern
    compare(oracle, w, got, kern)


def test_s8x_one_hot_integer_exact_and_batched(oracle):
    """One-hot activations: every output is one weight times its channel's scale, exactly -- byte
    order inside the 8-byte pieces, row order inside a step, the slices' and waves' shares of K.
    Then two batches with their own weights and scales against the oracle."""
    say("dequant_dot s8x one-hot, batched")
    K, N = 512, 256
    rng = np.random.default_rng(12)
    wv = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
    sc = np.exp2(rng.integers(-6, 3, size=N)).astype(np.float32)
    for m0 in range(0, K, 16):
        a = np.zeros((16, K), np.float32)
        a[np.arange(16), m0 + np.arange(16)] = 1.0
        w = dict(lhs=dtypes.f32_to_bf16(a), weights=wv, scales=sc, bias=None, weight_dtype="s8",
                 weight_shape=(K, N), group=K, dequant_type="f32", epilogue="DEFAULT")
        for strip in (128, 64):
            got, kern = run_dot(w, force_kernel=2, steps=1, strip=strip)
            assert kern == s8x_name(1, strip), kern
            want = dtypes.f32_to_bf16(wv[m0:m0 + 16].astype(np.float32) * sc[None, :])
            assert np.array_equal(got, want), (kern, m0)
    w = workloads.c5_s8_batched(B=2, M=7, K=1024, N=392)
    for strip in (128, 64):
        got, kern = run_dot(w, force_kernel=2, steps=2, strip=strip)
        assert kern == s8x_name(2, strip), kern
        compare(oracle, w, got, kern)


def test_s8x_same_call_frame_replayed(oracle):
    """The producers' flags are lowered by the strip's last workgroup, so the very same call frame
    (same workspace, same flag value) can run again and again -- what a captured graph does -- with
    new activations each time; the workspace starts out holding arbitrary bytes."""
    say("dequant_dot s8x replay")
    M, K, N = 16, 4096, 1024
    w = workloads.c1_s8_channel(M=M, K=K, N=N)
    lhs, wt, sc = dev_bf16(w["lhs"]), dev_s8(w["weights"]), dev_f32(w["scales"])
    nbytes = ffi.library().xla_amd_dequant_dot_workspace_bytes(1, M, K, N, dtypes.S8)
    assert nbytes > 0
    scratch = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device="cuda")
    call = ops.dequant_dot(lhs, wt, sc, None, weight_dtype="s8", weight_shape=(K, N), epilogue="DEFAULT",
                           dequant_type="f32", scratch=scratch, build_only=True)
    rng = np.random.default_rng(9)
    for it in range(4):
        a = dtypes.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
        lhs.copy_(dev_bf16(a))
        out = call.run()
        torch.cuda.synchronize()
        assert ffi.last_kernel().startswith("dequant_dot_decode_s8x_m16_"), ffi.last_kernel()
        compare(oracle, dict(w, lhs=a), host_bf16(out), "s8x replay %d" % it)


@pytest.mark.parametrize("which", ["s4", "s8"])
def test_sixteen_wave_workgroups(oracle, which):
    """The whole-CU workgroup (16 waves splitting K, picked by itself only for wide N): ragged K
    per wave, a ragged last strip and fewer tokens than a tile."""
    say("dequant_dot 16-wave workgroups " + which)
    if which == "s4":
        w = workloads.c2_s4_group(M=5, K=4096 + 160, N=1000, group=32)
    else:
        w = workloads.c1_s8_channel(M=13, K=2048 + 72, N=520)
    ffi.set_option("dequant_dot_waves", 16)
    try:
        got, kern = run_dot(w, force_kernel=2, x=1)
    finally:
        ffi.set_option("dequant_dot_waves", 0)
    assert "_w16_" in kern, kern
    compare(oracle, w, got, kern)


def test_s4_unpack_and_dequant_bit_exact(oracle):
    """One-hot activations: every output is one dequantised weight, so nibble order, sign
    extension, the scale lookup and the bf16 rounding are checked exactly."""
    say("dequant_dot s4 one-hot")
    K, N, group = 256, 512, 32
    rng = np.random.default_rng(3)
    wv = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
    wv[:16, :16] = np.arange(-8, 8, dtype=np.int8)[:, None]
    sc = dtypes.f32_to_bf16(rng.uniform(1e-3, 2e-2, size=(K // group, N)).astype(np.float32))
    for m0 in range(0, K, 64):
        a = np.zeros((64, K), np.float32)
        a[np.arange(64), m0 + np.arange(64)] = 1.0
        w = dict(lhs=dtypes.f32_to_bf16(a), weights=wv, weights_packed=dtypes.pack_s4(wv), scales=sc,
                 bias=None, weight_dtype="s4", weight_shape=(K, N), group=group, dequant_type="bf16",
                 epilogue="DEFAULT")
        got, kern = run_dot(w, force_kernel=2)
        prod = wv[m0:m0 + 64].astype(np.float32) * np.repeat(dtypes.bf16_to_f32(sc), group, axis=0)[m0:m0 + 64]
        want = dtypes.f32_to_bf16(prod)
        assert np.array_equal(dtypes.bf16_to_f32(got), dtypes.bf16_to_f32(want)), kern


def test_c1_full_size(oracle):
    say("dequant_dot C1 s8 per-channel full size")
    w = workloads.c1_s8_channel()
    got, kern = run_dot(w)
    assert kern.startswith("dequant_dot_decode_s8"), kern
    compare(oracle, w, got, "C1 " + kern)


@pytest.mark.parametrize("M,vec,slices,deq", [(5, 16, 2, "f32"), (16, 8, 1, "f32"), (24, 8, 2, "f32"),
                                              (64, 4, 1, "f32"), (7, 16, 1, "bf16"), (40, 4, 2, "bf16"),
                                              (48, 8, 1, "f32"), (64, 8, 2, "f32"), (40, 0, 0, "f32"), (64, 0, 0, "f32")])
def test_s8_decode_variants(oracle, M, vec, slices, deq):
    say("dequant_dot s8 variants M=%d vec=%d slices=%d deq=%s" % (M, vec, slices, deq))
    w = workloads.c1_s8_channel(M=M, K=1024, N=640)
    if deq == "bf16":
        w["scales"] = dtypes.f32_to_bf16(w["scales"])
        w["dequant_type"] = "bf16"
    w["bias"] = dtypes.f32_to_bf16(np.random.default_rng(9).standard_normal(640).astype(np.float32))
    w["epilogue"] = "BIAS_GELU"
    got, kern = run_dot(w, force_kernel=2, slices=slices, vec=vec)
    compare(oracle, w, got, "s8 %s" % kern)


def test_s8_one_hot_integer_exact(oracle):
    say("dequant_dot s8 one-hot")
    K, N = 256, 384
    wv = np.random.default_rng(4).integers(-128, 128, size=(K, N)).astype(np.int8)
    sc = np.full((N,), 0.5, np.float32)
    a = np.zeros((64, K), np.float32)
    a[np.arange(64), np.arange(64) * 4] = 1.0
    w = dict(lhs=dtypes.f32_to_bf16(a), weights=wv, scales=sc, bias=None, weight_dtype="s8",
             weight_shape=(K, N), group=K, dequant_type="f32", epilogue="DEFAULT")
    got, kern = run_dot(w, force_kernel=2)
    want = dtypes.f32_to_bf16(wv[np.arange(64) * 4].astype(np.float32) * 0.5)
    assert np.array_equal(dtypes.bf16_to_f32(got), dtypes.bf16_to_f32(want)), kern


@pytest.mark.parametrize("epilogue,ep_ty,dot_ty", [("BIAS_SILU", "f32", "f32"), ("BIAS_GELU", "bf16", "bf16"),
                                                   ("RELU", "bf16", "f32"), ("BIAS", "f32", "bf16"),
                                                   ("GELU", "f32", "f32"), ("SILU", "bf16", "bf16")])
def test_epilogues_and_rounding_points(oracle, epilogue, ep_ty, dot_ty):
    say("dequant_dot epilogue %s ops=%s dot=%s" % (epilogue, ep_ty, dot_ty))
    w = workloads.c2_s4_group(M=8, K=512, N=512)
    w["epilogue"] = epilogue
    if "BIAS" not in epilogue:
        w["bias"] = None
    w["epilogue_type"] = ep_ty
    w["dot_type"] = dot_ty
    got, kern = run_dot(w)
    ref = oracle_dot(oracle, w)
    # per-op bf16 rounding amplifies a last-bit difference of the accumulator into up to one ulp per
    # rounded op downstream; allow the floor of the plain dot times the op count
    fl = floor_for(w) * (12 if ep_ty == "bf16" else 1.2)
    tol_ulp_fail = check_dot(got, ref, fl + (np.abs(dtypes.bf16_to_f32(ref)) * 2.0 ** -6 if ep_ty == "bf16" or dot_ty == "bf16" else 0), kern)
    assert tol_ulp_fail <= got.size // 20


# ---- generic fallback ----------------------------------------------------------------------

@pytest.mark.parametrize("M,K,N,group,bits", [(3, 40, 37, 8, 8), (2, 96, 50, 32, 4), (5, 33, 7, 33, 8),
                                              (70, 128, 130, 128, 4)])
def test_generic_kernel_odd_shapes(oracle, M, K, N, group, bits):
    say("dequant_dot generic M=%d K=%d N=%d group=%d bits=%d" % (M, K, N, group, bits))
    rng = np.random.default_rng(M * 7 + N)
    lo, hi = (-8, 8) if bits == 4 else (-127, 128)
    wv = rng.integers(lo, hi, size=(K, N)).astype(np.int8)
    w = dict(lhs=dtypes.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32)), weights=wv,
             scales=rng.uniform(1e-3, 1e-2, size=(K // group, N)).astype(np.float32),
             bias=rng.standard_normal(N).astype(np.float32), weight_dtype="s4" if bits == 4 else "s8",
             weight_shape=(K, N), group=group, dequant_type="f32", epilogue="BIAS_RELU")
    if bits == 4:
        w["weights_packed"] = dtypes.pack_s4(wv)
    got, kern = run_dot(w)
    assert kern == "dequant_dot_generic", kern
    compare(oracle, w, got, "generic")


# ---- tiled MFMA kernel (M > 64) and batches -------------------------------------------------

@pytest.mark.parametrize("B,M,K,N", [(2, 256, 512, 512), (1, 200, 264, 388), (3, 128, 128, 1024)])
def test_c5_shape_reduced(oracle, B, M, K, N):
    say("dequant_dot C5 batched s8 B=%d M=%d K=%d N=%d" % (B, M, K, N))
    w = workloads.c5_s8_batched(B=B, M=M, K=K, N=N)
    got, kern = run_dot(w, force_kernel=3)   # at these sizes the cost model would pick the decode passes
    assert kern == "dequant_dot_tiled_s8_factored", kern
    compare(oracle, w, got, "C5 reduced")


def test_batched_decode(oracle):
    say("dequant_dot batched decode B=4 M=8")
    w = workloads.c5_s8_batched(B=4, M=8, K=512, N=512)
    got, kern = run_dot(w)
    assert kern.startswith("dequant_dot_decode_s8"), kern
    compare(oracle, w, got, "batched decode")


@pytest.mark.parametrize("K", [8, 40, 64, 72, 128, 136, 192, 200, 256, 320])
def test_tiled_kernels_with_few_stages(oracle, K):
    """One to five stages of 64 rows, whole and ragged: the prologue that loads three stages of weights
    ahead, the loop that runs stages in pairs, a lone stage after the pairs and the last stage."""
    say("dequant_dot tiled kernels, K=%d" % K)
    M, N = 130, 264
    w = workloads.c1_s8_channel(M=M, K=K, N=N)
    got, kern = run_dot(w, force_kernel=3)
    assert kern == "dequant_dot_tiled_s8_factored", kern
    compare(oracle, w, got, "s8 tiled K=%d" % K)
    w = workloads.c2_s4_group(M=M, K=K, N=N, group=8)
    got, kern = run_dot(w, force_kernel=3)
    assert kern == "dequant_dot_tiled_s4_rounded", kern
    compare(oracle, w, got, "s4 tiled K=%d" % K)
    w = workloads.u4_zero_point_group(M=M, K=K, N=N, group=8)
    got, kern = run_dot(w, force_kernel=3)
    assert kern == "dequant_dot_tiled_u4_rounded", kern
    compare(oracle, w, got, "u4 tiled K=%d" % K)


@pytest.mark.parametrize("M,K,N,group", [(200, 1024, 512, 128), (65, 264, 264, 8), (300, 2048, 1000, 64),
                                         (512, 512, 256, 512), (130, 1000, 72, 8)])
def test_s4_group_scales_tiled(oracle, M, K, N, group):
    """Prefill-sized M on s4 weights with bf16 scales per power-of-two group: the tiled MFMA kernel,
    weights dequantised (one rounding each) on the way into LDS."""
    say("dequant_dot s4 tiled M=%d K=%d N=%d group=%d" % (M, K, N, group))
    w = workloads.c2_s4_group(M=M, K=K, N=N, group=group)
    got, kern = run_dot(w, force_kernel=3)   # at these sizes the cost model would pick the decode passes
    assert kern == ("dequant_dot_tiled_s4_rounded:tail2" if K >= 2048 else "dequant_dot_tiled_s4_rounded"), kern
    compare(oracle, w, got, "s4 tiled M=%d" % M)


@pytest.mark.parametrize("zero_points", [True, False])
@pytest.mark.parametrize("M,K,N,group", [(200, 1024, 512, 128), (65, 264, 264, 8), (300, 2048, 1000, 64), (130, 1000, 72, 8)])
def test_u4_group_scales_tiled(oracle, M, K, N, group, zero_points):
    """Prefill-sized M on u4 weights: the tiled MFMA kernel with the zero point folded into the
    constant of the dequantising fma, with zero points and without."""
    say("dequant_dot u4 tiled M=%d K=%d N=%d group=%d zero_points=%s" % (M, K, N, group, zero_points))
    w = workloads.u4_zero_point_group(M=M, K=K, N=N, group=group)
    if not zero_points:
        w["zero_points"] = w["zero_points_packed"] = None
    got, kern = run_dot(w, force_kernel=3)
    assert kern == ("dequant_dot_tiled_u4_rounded:tail2" if K >= 2048 else "dequant_dot_tiled_u4_rounded"), kern
    compare(oracle, w, got, "u4 tiled M=%d" % M)


def test_u4_tiled_dequantised_weights_bit_exact(oracle):
    """One-hot activations pick single dequantised weights out of the tiled kernel: bf16((u - z) * s)
    exactly, every (u, z) pair among them."""
    say("dequant_dot u4 tiled one-hot")
    M, K, N, g = 128, 128, 256, 32
    w = workloads.u4_zero_point_group(M=M, K=K, N=N, group=g)
    w["weights"][:16, :16] = np.arange(16, dtype=np.int8)[:, None]
    w["zero_points"][0, :16] = np.arange(16, dtype=np.uint8)
    pack = lambda v: (v.reshape(-1)[0::2] | (v.reshape(-1)[1::2] << 4)).astype(np.uint8)
    w["weights_packed"] = pack(w["weights"].astype(np.uint8))
    w["zero_points_packed"] = pack(w["zero_points"])
    lhs = np.zeros((M, K), np.float32)
    lhs[np.arange(M), np.arange(M) % K] = 1.0
    w = dict(w, lhs=dtypes.f32_to_bf16(lhs), bias=None, epilogue="DEFAULT")
    got, kern = run_dot(w, force_kernel=3)
    assert kern == "dequant_dot_tiled_u4_rounded", kern
    diff = w["weights"].astype(np.float32) - np.repeat(w["zero_points"], g, axis=0).astype(np.float32)
    want = dtypes.f32_to_bf16(diff * np.repeat(dtypes.bf16_to_f32(w["scales"]), g, axis=0))[np.arange(M) % K]
    assert np.array_equal(got, want)


def test_s4_more_than_64_tokens_picks_the_cheaper_kernel():
    """8192 x 28672 s4 weights: decode passes up to a few hundred tokens, the tiled kernel beyond."""
    say("dequant_dot s4 kernel choice at the C2 weight shape")
    K, N = 8192, 28672
    dev = torch.device("cuda:0")
    wt = torch.zeros(K * N // 2, dtype=torch.uint8, device=dev)
    sc = torch.ones((K // 128, N), dtype=torch.bfloat16, device=dev)
    for M, want in ((128, "dequant_dot_decode_s4x_m64_d2:x64"), (1024, "dequant_dot_tiled_s4_rounded")):
        lhs = torch.zeros((M, K), dtype=torch.bfloat16, device=dev)
        out = ops.dequant_dot(lhs, wt, sc, None, weight_dtype="s4", weight_shape=(K, N), epilogue="DEFAULT",
                              dequant_type="bf16")
        torch.cuda.synchronize()
        assert ffi.last_kernel() == want, (M, ffi.last_kernel())
        assert not bool(out.any())


def test_s4_tiled_dequantised_weights_bit_exact(oracle):
    """One-hot activations pick single dequantised weights out of the tiled kernel: bf16(w * s) exactly."""
    say("dequant_dot s4 tiled one-hot")
    M, K, N, g = 128, 128, 256, 32
    w = workloads.c2_s4_group(M=M, K=K, N=N, group=g)
    lhs = np.zeros((M, K), np.float32)
    lhs[np.arange(M), np.arange(M) % K] = 1.0
    w = dict(w, lhs=dtypes.f32_to_bf16(lhs), bias=None, epilogue="DEFAULT")
    got, kern = run_dot(w, force_kernel=3)
    assert kern == "dequant_dot_tiled_s4_rounded", kern
    sc = np.repeat(dtypes.bf16_to_f32(w["scales"]), g, axis=0)
    want = dtypes.f32_to_bf16((w["weights"].astype(np.float32) * sc).astype(np.float32))[np.arange(M) % K]
    assert np.array_equal(got, want)


@pytest.mark.parametrize("M,K,N,group", [(200, 768, 512, 96), (65, 480, 264, 24)])
def test_s4_group_scales_more_than_64_tokens(oracle, M, K, N, group):
    """Prefill-sized M on s4 weights the tiled kernel does not take (groups that are no power of
    two): the decode kernel once per 64 tokens, and the result equals, bit for bit, separate calls
    on the same token rows."""
    say("dequant_dot s4 group chunked M=%d K=%d N=%d" % (M, K, N))
    w = workloads.c2_s4_group(M=M, K=K, N=N, group=group)
    got, kern = run_dot(w)
    assert kern.startswith("dequant_dot_decode_s4") and kern.endswith(":x64"), kern
    compare(oracle, w, got, "s4 chunked M=%d" % M)
    for m0 in range(0, M, 64):
        part = dict(w, lhs=np.ascontiguousarray(w["lhs"][m0:m0 + 64]))
        alone, _ = run_dot(part)
        assert np.array_equal(alone, got[m0:m0 + 64]), "rows %d.. differ from a call of their own" % m0


def test_batched_grouped_s8_more_than_64_tokens(oracle):
    """Batched s8 weights with per-group scales (not the tiled kernel's per-channel case), 70 tokens."""
    say("dequant_dot batched grouped s8 chunked")
    rng = np.random.default_rng(77)
    B, M, K, N, g = 2, 70, 256, 128, 64
    w = dict(lhs=dtypes.f32_to_bf16(rng.standard_normal((B, M, K)).astype(np.float32)),
             weights=rng.integers(-127, 128, size=(B, K, N)).astype(np.int8),
             scales=dtypes.f32_to_bf16(rng.uniform(1e-3, 1e-2, size=(B, K // g, N)).astype(np.float32)),
             bias=None, weight_dtype="s8", weight_shape=(B, K, N), group=g, dequant_type="bf16",
             epilogue="DEFAULT")
    got, kern = run_dot(w)
    assert kern.startswith("dequant_dot_decode_s8") and kern.endswith(":x64"), kern
    compare(oracle, w, got, "batched grouped s8 chunked")


def test_c5_full_size_sampled_blocks(oracle):
    """Configuration 5 at full size; the oracle evaluates random (expert, row block, column block)
    sub-problems of the same inputs."""
    say("dequant_dot C5 full size")
    w = workloads.c5_s8_batched()
    got, kern = run_dot(w)
    # 896 tiles: three rounds of 256 whole tiles, then the 128 tiles of expert 6's end and expert 7
    # as two workgroups each
    assert kern == "dequant_dot_tiled_s8_factored:tail2", kern
    rng = np.random.default_rng(0)
    for i in range(8):
        b = int(rng.integers(0, 8)); m0 = int(rng.integers(0, 512 - 32)); n0 = int(rng.integers(0, 14336 - 64))
        if i >= 6:
            b = 7   # split tiles for certain
        sub = dict(w, lhs=np.ascontiguousarray(w["lhs"][b, m0:m0 + 32]),
                   weights=np.ascontiguousarray(w["weights"][b][:, n0:n0 + 64]),
                   scales=np.ascontiguousarray(w["scales"][b, n0:n0 + 64]), weight_shape=(4096, 64))
        compare(oracle, sub, got[b, m0:m0 + 32, n0:n0 + 64], "C5 block b=%d m0=%d n0=%d" % (b, m0, n0))


@pytest.mark.parametrize("which,B,M,K,N", [("s8", 1, 300, 2048, 700), ("s8", 2, 257, 2304, 520),
                                           ("s4", 1, 300, 4096, 520)])
def test_tiled_last_round_split_along_k(oracle, which, B, M, K, N):
    """Few tiles (a last round at most half full): every tile runs as two workgroups, the second half
    of K handing its f32 sums to the first through the scratch.  Checked against the oracle, and
    against the same call with the split switched off (sums in another order: a bf16 ulp apart at most)."""
    say("dequant_dot tiled, tail split, %s B=%d M=%d K=%d N=%d" % (which, B, M, K, N))
    if which == "s8":
        w = workloads.c5_s8_batched(B=B, M=M, K=K, N=N)
    else:
        w = workloads.c2_s4_group(M=M, K=K, N=N, group=128)
    base = "dequant_dot_tiled_s8_factored" if which == "s8" else "dequant_dot_tiled_s4_rounded"
    got, kern = run_dot(w, force_kernel=3)
    assert kern == base + ":tail2", kern
    compare(oracle, w, got, "tail split " + which)
    whole, kern = run_dot(w, force_kernel=3, tail=1)
    assert kern == base, kern
    d = np.abs(dtypes.bf16_to_f32(got).astype(np.float64) - dtypes.bf16_to_f32(whole).astype(np.float64))
    mag = np.maximum(np.abs(dtypes.bf16_to_f32(whole).astype(np.float64)), floor_for(w))
    assert np.all(d <= mag * 2.0 ** -7), "split and whole tiles differ by more than a bf16 ulp"


def test_tiled_last_round_split_after_full_rounds(oracle):
    """264 tiles: one round of 256 whole tiles, then 8 tiles as 16 workgroups; the same call frame
    runs three times with new activations (every run moves the slots on to their next generation), on a
    scratch that starts out holding arbitrary bytes."""
    say("dequant_dot tiled, 256 + 8 tiles, replayed")
    B, M, K, N = 3, 1024, 2048, 5632
    w = workloads.c5_s8_batched(B=B, M=M, K=K, N=N)
    lhs, wt, sc = dev_bf16(w["lhs"]), dev_s8(w["weights"]), dev_f32(w["scales"])
    nbytes = ffi.library().xla_amd_dequant_dot_workspace_bytes(B, M, K, N, dtypes.S8)
    assert nbytes == 8 * (256 * 256 * 4 + 16), nbytes   # sums, flag and generation per split tile
    scratch = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device="cuda")
    call = ops.dequant_dot(lhs, wt, sc, None, weight_dtype="s8", weight_shape=(B, K, N), epilogue="DEFAULT",
                           dequant_type="f32", scratch=scratch, build_only=True)
    rng = np.random.default_rng(11)
    for it in range(3):
        a = dtypes.f32_to_bf16(rng.standard_normal((B, M, K)).astype(np.float32))
        lhs.copy_(dev_bf16(a))
        out = call.run()
        torch.cuda.synchronize()
        assert ffi.last_kernel() == "dequant_dot_tiled_s8_factored:tail2", ffi.last_kernel()
        got = host_bf16(out)
        for i in range(8):
            # the split tiles are the last 8 of expert 2 in launch order; sample there and elsewhere
            b = 2 if i < 5 else int(rng.integers(0, B))
            m0 = int(rng.integers(0, M - 32)); n0 = int(rng.integers(0, N - 64))
            sub = dict(w, lhs=np.ascontiguousarray(a[b, m0:m0 + 32]),
                       weights=np.ascontiguousarray(w["weights"][b][:, n0:n0 + 64]),
                       scales=np.ascontiguousarray(w["scales"][b, n0:n0 + 64]), weight_shape=(K, 64))
            compare(oracle, sub, got[b, m0:m0 + 32, n0:n0 + 64], "replay %d block b=%d m0=%d n0=%d" % (it, b, m0, n0))
        # every output once against the unsplit kernel
        if it == 0:
            ffi.set_option("tiled_tail", 1)
            try:
                whole = host_bf16(ops.dequant_dot(lhs, wt, sc, None, weight_dtype="s8", weight_shape=(B, K, N),
                                                  epilogue="DEFAULT", dequant_type="f32"))
                torch.cuda.synchronize()
                assert ffi.last_kernel() == "dequant_dot_tiled_s8_factored", ffi.last_kernel()
            finally:
                ffi.set_option("tiled_tail", 0)
            g, h = dtypes.bf16_to_f32(got).astype(np.float64), dtypes.bf16_to_f32(whole).astype(np.float64)
            differ = g != h
            assert np.all(np.abs(g - h)[differ] <= np.maximum(np.abs(h[differ]) * 2.0 ** -7, 1e-2))
            assert not differ[:2].any(), "whole tiles must not depend on the split"


@pytest.mark.parametrize("M", [1, 8, 32, 64])
def test_c2_full_size_sampled_columns(oracle, M):
    """Configuration 2 at full size; the oracle evaluates column blocks of the same inputs."""
    say("dequant_dot C2 full size M=%d" % M)
    w = workloads.c2_s4_group(M=M)
    got, kern = run_dot(w)
    assert kern.startswith("dequant_dot_decode_s4"), kern
    rng = np.random.default_rng(M)
    for n0 in [0, 28672 - 256] + [int(v) * 2 for v in rng.integers(0, (28672 - 256) // 2, size=3)]:
        wv = np.ascontiguousarray(w["weights"][:, n0:n0 + 256])
        sub = dict(w, weights=wv, weights_packed=dtypes.pack_s4(wv),
                   scales=np.ascontiguousarray(w["scales"][:, n0:n0 + 256]),
                   bias=np.ascontiguousarray(w["bias"][n0:n0 + 256]), weight_shape=(8192, 256))
        compare(oracle, sub, got[:, n0:n0 + 256], "C2 full M=%d n0=%d" % (M, n0))


# ---- errors ---------------------------------------------------------------------------------

def test_dequant_dot_error_paths():
    say("dequant_dot error paths")
    lhs = torch.zeros((4, 64), dtype=torch.bfloat16, device="cuda")
    wt = torch.zeros((64, 32), dtype=torch.int8, device="cuda")
    sc = torch.ones((32,), dtype=torch.float32, device="cuda")
    with pytest.raises(ffi.FfiError, match="contracting dimensions differ"):
        ops.dequant_dot(lhs, torch.zeros((48, 32), dtype=torch.int8, device="cuda"), sc)
    with pytest.raises(ffi.FfiError, match="BIAS"):
        ops.dequant_dot(lhs, wt, sc, epilogue="BIAS")
    with pytest.raises(ffi.FfiError, match="bf16-typed dequantise multiply needs bf16 scales"):
        ops.dequant_dot(lhs, wt, sc, dequant_type="bf16")
    with pytest.raises(ffi.FfiError, match="number of scale groups must divide K"):
        ops.dequant_dot(lhs, wt, torch.ones((5, 32), dtype=torch.float32, device="cuda"))
    out = ops.dequant_dot(torch.zeros((0, 64), dtype=torch.bfloat16, device="cuda"), wt, sc)
    assert out.shape == (0, 32)


# ---- u4 weights with zero points -----------------------------------------------------------

@pytest.mark.parametrize("M,K,N,group,vec,slices", [
    (1, 4096, 1024, 128, 0, 0), (8, 2048, 768, 64, 4, 2), (16, 2048, 512, 32, 8, 1), (20, 1024, 640, 128, 4, 1),
    (33, 1024, 512, 64, 0, 0), (64, 2048, 256, 128, 4, 2), (70, 1024, 512, 128, 0, 0), (5, 100, 42, 50, 0, 0)])
def test_u4_zero_point_decode(oracle, M, K, N, group, vec, slices):
    """Unsigned 4-bit weights with one zero point and one scale per group and channel, bf16-typed
    convert / subtract / multiply: every decode strip width, K-slices, more than 64 tokens as
    chunks, and a shape only the one-thread-per-output kernel takes."""
    say("dequant_dot u4+zp M=%d K=%d N=%d group=%d vec=%d slices=%d" % (M, K, N, group, vec, slices))
    w = workloads.u4_zero_point_group(M=M, K=K, N=N, group=group)
    got, kern = run_dot(w, slices=slices, vec=vec)
    if (K, N) == (100, 42):
        assert kern == "dequant_dot_generic", kern
    else:
        # a forced strip width keeps the call on the first-generation kernels
        family = "dequant_dot_decode_s4_" if vec or group % 64 else "dequant_dot_decode_u4x_"
        assert kern.startswith(family) and (M <= 64 or kern.endswith(":x64")), kern
    compare(oracle, w, got, "u4+zp %s" % kern)


@pytest.mark.parametrize("zero_points", [True, False])
@pytest.mark.parametrize("M,pair,slices,K,N,group", [
    (1, 2, 1, 2048, 768, 128), (8, 1, 0, 2048 + 256, 800, 128), (16, 1, 0, 4096, 256, 64), (3, 2, 2, 2048, 768, 64),
    (20, 2, 2, 2048 + 128, 736, 64), (33, 2, 1, 1536, 512, 128), (64, 2, 1, 2048, 768, 128), (5, 1, 0, 1024 + 64, 1120, 64)])
def test_u4x_variants(oracle, M, pair, slices, K, N, group, zero_points):
    """Unsigned nibbles through the matrix-instruction dequantisation, the zero point riding in the
    scaling MFMA's operand C: one or two workgroups per strip, K-slices, every token-tile count, a
    ragged last strip, with zero points and without (then the nibble itself is the weight)."""
    say("dequant_dot u4x M=%d pair=%d slices=%d K=%d N=%d group=%d zero_points=%s" % (M, pair, slices, K, N, group, zero_points))
    w = workloads.u4_zero_point_group(M=M, K=K, N=N, group=group)
    if not zero_points:
        w["zero_points"] = w["zero_points_packed"] = None
    got, kern = run_dot(w, force_kernel=2, slices=slices, pair=pair)
    assert kern.startswith("dequant_dot_decode_u4x_") and kern.endswith("_pair") == (pair == 1), kern
    compare(oracle, w, got, "%s slices=%d" % (kern, slices))


@pytest.mark.parametrize("pair", [2, 1])
def test_u4x_unpack_and_zero_points_bit_exact(oracle, pair):
    """One-hot activations: every output is one dequantised weight bf16((u - z) * s), exactly -- the
    nibble order of weights and zero points, every (u, z) pair, scales across the f16 window."""
    say("dequant_dot u4x one-hot pair=%d" % pair)
    K, N, group = 512, 512, 64
    rng = np.random.default_rng(15)
    wu = rng.integers(0, 16, size=(K, N)).astype(np.uint8)
    zero = rng.integers(0, 16, size=(K // group, N)).astype(np.uint8)
    wu[:16, :16] = np.arange(16, dtype=np.uint8)[:, None]
    zero[0, :16] = np.arange(16, dtype=np.uint8)
    mant = rng.integers(128, 256, size=(K // group, N)).astype(np.float32) / 128.0
    expo = rng.integers(-22, 3, size=(K // group, N)).astype(np.float32)
    sign = rng.choice([-1.0, 1.0], size=(K // group, N)).astype(np.float32)
    sc = dtypes.f32_to_bf16(sign * mant * np.exp2(expo))
    pack = lambda v: (v.reshape(-1)[0::2] | (v.reshape(-1)[1::2] << 4)).astype(np.uint8)
    diff = wu.astype(np.float32) - np.repeat(zero, group, axis=0).astype(np.float32)
    want_all = dtypes.f32_to_bf16(diff * np.repeat(dtypes.bf16_to_f32(sc), group, axis=0))
    for m0 in range(0, K, 16):
        a = np.zeros((16, K), np.float32)
        a[np.arange(16), m0 + np.arange(16)] = 1.0
        w = dict(lhs=dtypes.f32_to_bf16(a), weights=wu.astype(np.int8), weights_packed=pack(wu), scales=sc,
                 zero_points=zero, zero_points_packed=pack(zero), bias=None, weight_dtype="u4",
                 weight_shape=(K, N), group=group, dequant_type="bf16", epilogue="DEFAULT")
        got, kern = run_dot(w, force_kernel=2, pair=pair)
        assert kern.startswith("dequant_dot_decode_u4x_") and kern.endswith("_pair") == (pair == 1), kern
        assert np.array_equal(dtypes.bf16_to_f32(got), dtypes.bf16_to_f32(want_all[m0:m0 + 16])), (kern, m0)


@pytest.mark.parametrize("M,pair", [(4, 1), (24, 2)])
def test_u4x_scales_outside_the_f16_window(oracle, M, pair):
    """Channels whose scale cannot be an f16 operand are recomputed by the plain loop, which must
    subtract the zero points as well."""
    say("dequant_dot u4x odd scales M=%d pair=%d" % (M, pair))
    K, N, group = 1024, 512, 128
    w = workloads.u4_zero_point_group(M=M, K=K, N=N, group=group)
    sc = dtypes.bf16_to_f32(w["scales"]).copy()
    sc[0, 3] = 0.0
    sc[1, 40] = 16.0
    sc[2, 41] = 2.0 ** -30
    sc[7, 255] = -3.0e4
    sc[0, 300] = 64.0
    sc[7, 301] = 2.0 ** -25
    w["scales"] = dtypes.f32_to_bf16(sc)
    got, kern = run_dot(w, force_kernel=2, pair=pair)
    assert kern.startswith("dequant_dot_decode_u4x_") and kern.endswith("_pair") == (pair == 1), kern
    compare(oracle, w, got, kern)


def test_u4_zero_point_one_hot_bit_exact(oracle):
    """One-hot activations: every output is one dequantised weight bf16((w - z) * s), exactly --
    the nibble order of weights and zero points, unsignedness, the group of each row."""
    say("dequant_dot u4+zp one-hot")
    K, N, group = 256, 256, 64
    w = workloads.u4_zero_point_group(M=16, K=K, N=N, group=group)
    w["weights"][:16, :16] = np.arange(16, dtype=np.int8)[:, None]
    wu = w["weights"].astype(np.uint8)
    w["weights_packed"] = (wu.reshape(-1)[0::2] | (wu.reshape(-1)[1::2] << 4)).astype(np.uint8)
    w["bias"], w["epilogue"] = None, "DEFAULT"
    diff = w["weights"].astype(np.float32) - np.repeat(w["zero_points"], group, axis=0).astype(np.float32)
    want_all = dtypes.f32_to_bf16((diff * np.repeat(dtypes.bf16_to_f32(w["scales"]), group, axis=0)).astype(np.float32))
    for m0 in range(0, K, 16):
        a = np.zeros((16, K), np.float32)
        a[np.arange(16), m0 + np.arange(16)] = 1.0
        got, kern = run_dot(dict(w, lhs=dtypes.f32_to_bf16(a)), force_kernel=2)
        assert np.array_equal(dtypes.bf16_to_f32(got), dtypes.bf16_to_f32(want_all[m0:m0 + 16])), (kern, m0)


@pytest.mark.parametrize("with_zero_points", [False, True])
def test_u4_per_channel_f32_multiply(oracle, with_zero_points):
    """u4 with one scale (and zero point) per output channel under an f32-typed multiply: the integers
    (w - z) go through the matrix cores exactly and the scale multiplies the sum once."""
    say("dequant_dot u4 per-channel f32 zero_points=%s" % with_zero_points)
    M, K, N = 12, 1024, 384
    w = workloads.u4_zero_point_group(M=M, K=K, N=N, group=K)
    w["scales"] = dtypes.bf16_to_f32(w["scales"]).reshape(N)
    w["dequant_type"] = "f32"
    if not with_zero_points:
        w["zero_points"] = w["zero_points_packed"] = None
    else:
        w["zero_points"] = w["zero_points"].reshape(1, N)
    got, kern = run_dot(w, force_kernel=2)
    assert kern.endswith("_factored"), kern
    compare(oracle, w, got, "u4 per-channel %s" % kern)


# ---- ragged dot (tokens sorted by expert, group sizes on the device) -----------------------------

def run_ragged(w, sizes_dtype=torch.int32, force_kernel=0):
    lhs = dev_bf16(w["lhs"])
    wt = dev_u8(w["weights_packed"]) if w["weight_dtype"] == "s4" else dev_s8(w["weights"])
    sc = dev_bf16(w["scales"]) if w["scales"].dtype == np.uint16 else dev_f32(w["scales"])
    bias = dev_bf16(w["bias"]) if w.get("bias") is not None else None
    gs = torch.from_numpy(np.asarray(w["group_sizes"], np.int64)).to(sizes_dtype).cuda()
    ffi.set_option("dequant_dot_kernel", force_kernel)
    try:
        out = ops.dequant_dot(lhs, wt, sc, bias, weight_dtype=w["weight_dtype"], weight_shape=w["weight_shape"],
                              epilogue=w["epilogue"], dequant_type=w["dequant_type"],
                              scale_group_size=0 if w["group"] == w["lhs"].shape[-1] else w["group"], group_sizes=gs)
        torch.cuda.synchronize()
    finally:
        ffi.set_option("dequant_dot_kernel", 0)
    return host_bf16(out), ffi.last_kernel()


def ragged_floor(w):
    a = np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64))
    wd = np.max(np.abs(w["weights"].astype(np.float64)) * w["scales"].astype(np.float64)[:, None, :], axis=0)
    return dot_floor(a, wd, w["lhs"].shape[-1])


@pytest.mark.parametrize("M,K,N,G,sizes,sizes_dtype", [
    (32, 1024, 512, 8, None, torch.int32), (64, 512, 384, 4, [10, 0, 50, 4], torch.int64),
    (16, 2048, 256, 16, None, torch.int32), (12, 256, 136, 3, [5, 0, 2], torch.int32),
    (7, 512, 128, 2, [9, 9], torch.int32), (40, 512, 256, 5, [0, 0, 0, 0, 0], torch.int64)])
def test_ragged_dot_decode(oracle, M, K, N, G, sizes, sizes_dtype):
    """Rows sorted by expert, each group through its own weights: random splits with empty groups,
    s32 and s64 sizes, rows that no group owns (epilogue(0) = the bias), sizes that overrun M (cut
    at M) and a call whose groups are all empty."""
    say("dequant_dot ragged M=%d K=%d N=%d G=%d sizes=%s" % (M, K, N, G, sizes))
    w = workloads.ragged_s8_experts(M=M, K=K, N=N, groups=G, sizes=sizes)
    got, kern = run_ragged(w, sizes_dtype)
    assert kern.startswith("dequant_dot_decode_s8_"), kern
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
    check_dot(got, ref, ragged_floor(w), "ragged %s" % kern)


@pytest.mark.parametrize("G,M", [(70, 90), (130, 300), (64, 64), (65, 16)])
@pytest.mark.parametrize("force", [0, 3])
def test_ragged_dot_over_many_groups(oracle, G, M, force):
    """More groups than a wave has lanes: the search for a workgroup's item (its group and chunk of rows)
    scans the sizes 64 at a time and carries the rows and chunks seen so far into the next block.  Random
    sizes with empty groups, groups of more rows than a chunk, and rows nobody owns; through the decode
    kernel's work items and (forced) through the grouped GEMM's tile slots."""
    if force == 3 and M <= 64:
        pytest.skip("the grouped GEMM takes more than 64 rows")
    say("dequant_dot ragged over %d groups, %d rows, force=%d" % (G, M, force))
    rng = np.random.default_rng(G * 1000 + M)
    sizes = rng.multinomial(int(M * 0.9), np.ones(G) / G)
    sizes[rng.integers(0, G, 5)] = 0
    sizes[int(rng.integers(0, G))] += 20          # one group of more than 16 rows
    K, N = 256, 136
    w = workloads.ragged_s8_experts(M=M, K=K, N=N, groups=G, sizes=sizes)
    got, kern = run_ragged(w, torch.int32, force_kernel=force)
    assert kern == ("dequant_dot_tiled_s8_factored:ragged" if force == 3 else kern) and ("ragged" in kern or "decode" in kern), kern
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
    check_dot(got, ref, ragged_floor(w), "ragged over %d groups, %s" % (G, kern))


@pytest.mark.parametrize("force", [0, 3])
@pytest.mark.parametrize("sizes_dtype", [torch.int32, torch.int64])
def test_ragged_dot_many_groups_sizes_overrun(oracle, force, sizes_dtype):
    """Sizes that add up to one and a half times the rows, over 130 groups: the rows run out inside the
    second block of 64 groups that the item search scans, the group they run out in is cut at M and every
    later group owns nothing."""
    G, M = 130, 200
    say("dequant_dot ragged, sizes overrun the rows, %d groups, %d rows, force=%d" % (G, M, force))
    rng = np.random.default_rng(77)
    sizes = rng.multinomial(int(M * 1.5), np.ones(G) / G)
    assert int(sizes[:64].sum()) < M < int(sizes[:128].sum())
    w = workloads.ragged_s8_experts(M=M, K=256, N=136, groups=G, sizes=sizes)
    got, kern = run_ragged(w, sizes_dtype, force_kernel=force)
    assert kern == "dequant_dot_tiled_s8_factored:ragged" if force == 3 else kern.startswith("dequant_dot_decode_s8_"), kern
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
    check_dot(got, ref, ragged_floor(w), "ragged, sizes overrun, %s" % kern)


def test_ragged_dot_equals_per_group_calls_and_generic_kernel(oracle):
    """Every row of the ragged result is bit-identical to an ordinary call on its group's rows with
    that group's weights (the same kernel does both); the one-thread-per-output kernel, which finds
    each row's group by itself, agrees with the oracle too."""
    say("dequant_dot ragged vs per-group calls, generic kernel")
    w = workloads.ragged_s8_experts(M=24, K=1024, N=256, groups=4, sizes=[7, 1, 0, 11])
    got, kern = run_ragged(w)
    start = 0
    for g, n in enumerate(w["group_sizes"]):
        if n:
            sub = dict(w, lhs=w["lhs"][start:start + n], weights=w["weights"][g], scales=w["scales"][g],
                       weight_shape=w["weights"][g].shape)
            one, k1 = run_dot(sub, force_kernel=2, x=1)
            assert np.array_equal(got[start:start + n], one), (g, kern, k1)
        start += n
    assert np.array_equal(got[start:], np.broadcast_to(w["bias"], (24 - start, 256)))
    got_generic, kern = run_ragged(w, force_kernel=1)
    assert kern == "dequant_dot_generic", kern
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
    check_dot(got_generic, ref, ragged_floor(w), "ragged generic")


@pytest.mark.parametrize("nk", [False, True])
def test_ragged_dot_without_any_group(nk):
    """A ragged dot over zero groups (weights [0,K,N], group_sizes [0]): no row has a group, so every
    row is epilogue(0 + bias) -- the result must be written, not left as it was."""
    say("dequant_dot ragged, zero groups, nk=%s" % nk)
    M, K, N = 9, 256, 136
    lhs = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    wt = torch.zeros((0, N, K) if nk else (0, K, N), dtype=torch.int8, device="cuda")
    sc = torch.zeros((0, N), dtype=torch.float32, device="cuda")
    bias_h = dtypes.f32_to_bf16(np.linspace(-3.0, 3.0, N).astype(np.float32))
    gs = torch.zeros((0,), dtype=torch.int32, device="cuda")
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    ops.dequant_dot(lhs, wt, sc, dev_bf16(bias_h), weight_dtype="s8", epilogue="BIAS_RELU", dequant_type="f32", scale_group_size=0,
                    group_sizes=gs, rhs_contracting_dim=1 if nk else 0, out=out)
    torch.cuda.synchronize()
    assert ffi.last_kernel() == "dequant_dot:ragged_no_groups"
    want = np.where(dtypes.bf16_to_f32(bias_h) > 0, bias_h, 0).astype(np.uint16)
    assert np.array_equal(host_bf16(out), np.broadcast_to(want, (M, N)))


@pytest.mark.parametrize("M,K,N,G,sizes", [
    (200, 512, 256, 4, [70, 0, 129, 1]), (640, 1024, 512, 8, None), (130, 512, 128, 2, [130, 0]),
    (100, 256, 128, 3, [10, 20, 30]), (300, 512, 256, 4, [0, 400, 7, 0])])
def test_ragged_dot_more_than_64_rows(oracle, M, K, N, G, sizes):
    """A ragged dot over any number of rows: every group is walked in chunks of 64 rows (a group of
    130 rows as 64 + 64 + 2, one group that owns all rows, sizes that overrun M, 40 rows that no
    group owns); rows of one group are bit-identical to an ordinary call on them."""
    say("dequant_dot ragged prefill M=%d K=%d N=%d G=%d sizes=%s" % (M, K, N, G, sizes))
    w = workloads.ragged_s8_experts(M=M, K=K, N=N, groups=G, sizes=sizes)
    got, kern = run_ragged(w)
    assert kern == "dequant_dot_decode_s8_v4_m64_factored", kern   # few strips: the narrow ones
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
    check_dot(got, ref, ragged_floor(w), "ragged prefill %s" % kern)
    start = 0
    for g, n in enumerate(w["group_sizes"]):
        n = int(min(n, M - start))
        if n > 0:
            rows = slice(start, start + min(n, 64))   # the first chunk of the group, as a call of its own
            sub = dict(w, lhs=np.ascontiguousarray(w["lhs"][rows]), weights=w["weights"][g], scales=w["scales"][g],
                       weight_shape=w["weights"][g].shape)
            one, k1 = run_dot(sub, force_kernel=2, x=1)
            if k1 == kern:   # same kernel (64 rows): same bits
                assert np.array_equal(got[rows], one), (g, kern, k1)
        start += n
    assert np.array_equal(got[start:], np.broadcast_to(w["bias"], (M - start, N)))


@pytest.mark.parametrize("M,K,N,G,group,sizes", [
    (32, 1024, 512, 4, 128, None), (16, 512, 256, 3, 64, [9, 0, 5]), (200, 512, 256, 4, 128, [70, 0, 129, 1])])
def test_ragged_dot_s4_group_scales(oracle, M, K, N, G, group, sizes):
    """4-bit experts with bf16 scales per group of rows and channel under a bf16-typed multiply (one
    rounding per weight), at decode and prefill row counts."""
    say("dequant_dot ragged s4 M=%d K=%d N=%d G=%d group=%d sizes=%s" % (M, K, N, G, group, sizes))
    w = workloads.ragged_s4_group_experts(M=M, K=K, N=N, groups=G, group=group, sizes=sizes)
    got, kern = run_ragged(w)
    assert kern.startswith("dequant_dot_decode_s4_") and kern.endswith("_rounded"), kern
    ref = oracle.ragged_dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", w["group_sizes"],
                                    bias=w["bias"], group=group)
    a = np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64))
    wd = np.max(np.abs(w["weights"].astype(np.float64)) *
                np.repeat(dtypes.bf16_to_f32(w["scales"]).astype(np.float64), group, axis=1), axis=0)
    check_dot(got, ref, dot_floor(a, wd, K), "ragged s4 %s" % kern)


@pytest.mark.parametrize("kind,G,K,N,rows,tiled", [
    ("s8", 8, 4096, 2048, 512, True), ("s8", 2, 14336, 4096, 96, False), ("s8", 32, 2048, 1536, 96, False),
    ("s8", 128, 2048, 1536, 96, True), ("s4", 4, 4096, 14336, 96, False), ("s4", 4, 4096, 14336, 192, True),
    ("s8", 4, 1024, 512, 160, False)])
def test_ragged_dot_choice_of_kernel(oracle, kind, G, K, N, rows, tiled):
    """Chunks of the decode kernel or tiles of the grouped GEMM, priced on the average group: few experts
    of large matrices stay with the chunks well past 96 rows each (fewer than 256 tiles leave the chip
    partly idle for a whole round), many small experts move to tiles at 96.  Either way the oracle's rows."""
    say("dequant_dot ragged choice %s G=%d K=%d N=%d rows/expert=%d" % (kind, G, K, N, rows))
    sizes = [rows] * G
    if kind == "s8":
        w = workloads.ragged_s8_experts(M=G * rows, K=K, N=N, groups=G, sizes=sizes)
    else:
        w = workloads.ragged_s4_group_experts(M=G * rows, K=K, N=N, groups=G, group=128, sizes=sizes)
    got, kern = run_ragged(w)
    assert kern.endswith(":ragged") == tiled and (tiled or kern.startswith("dequant_dot_decode_")), kern
    other, kern2 = run_ragged(w, force_kernel=2 if tiled else 3)
    assert kern2.endswith(":ragged") != tiled, kern2
    if kind == "s8":
        ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
        floor = ragged_floor(w)
    else:
        ref = oracle.ragged_dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", w["group_sizes"],
                                        bias=w["bias"], group=128)
        wd = np.max(np.abs(w["weights"].astype(np.float64)) *
                    np.repeat(dtypes.bf16_to_f32(w["scales"]).astype(np.float64), 128, axis=1), axis=0)
        floor = dot_floor(np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64)), wd, K)
    check_dot(got, ref, floor, "ragged choice %s" % kern)
    check_dot(other, ref, floor, "ragged choice, the other kernel %s" % kern2)


@pytest.mark.parametrize("kind,M,K,N,G,sizes", [
    ("s8", 640, 1024, 512, 4, None), ("s8", 700, 512, 300, 3, [256, 1, 300]), ("s8", 512, 512, 256, 2, [0, 512]),
    ("s8", 400, 512, 256, 4, [500, 3, 3, 3]), ("s4", 600, 1024, 512, 3, None), ("s4", 300, 2048, 256, 2, [10, 200])])
def test_ragged_dot_grouped_gemm(oracle, kind, M, K, N, G, sizes):
    """The tiled kernel as a grouped GEMM (taken by itself where its tiles are priced below the decode
    kernel's chunks, see test_ragged_dot_choice_of_kernel) -- 256-row tiles per
    group, found on the device from the group sizes (a group of 257 rows is two tiles, the second with
    one live row; empty groups, one group owning everything, sizes that overrun M, rows nobody owns)."""
    say("dequant_dot ragged grouped GEMM %s M=%d K=%d N=%d G=%d sizes=%s" % (kind, M, K, N, G, sizes))
    if kind == "s8":
        w = workloads.ragged_s8_experts(M=M, K=K, N=N, groups=G, sizes=sizes)
        ref = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"], bias=w["bias"])
        floor = ragged_floor(w)
        want = "dequant_dot_tiled_s8_factored:ragged"
    else:
        w = workloads.ragged_s4_group_experts(M=M, K=K, N=N, groups=G, group=128, sizes=sizes)
        ref = oracle.ragged_dequant_dot(w["lhs"], w["weights_packed"], 4, w["scales"], "bf16", "bf16", w["group_sizes"],
                                        bias=w["bias"], group=128)
        wd = np.max(np.abs(w["weights"].astype(np.float64)) *
                    np.repeat(dtypes.bf16_to_f32(w["scales"]).astype(np.float64), 128, axis=1), axis=0)
        floor = dot_floor(np.abs(dtypes.bf16_to_f32(w["lhs"]).astype(np.float64)), wd, K)
        want = "dequant_dot_tiled_s4_rounded:ragged"
    got, kern = run_ragged(w, force_kernel=3)   # matrices this small are cheaper in chunks: the tiles are asked for
    assert kern == want, kern
    check_dot(got, ref, floor, "ragged grouped GEMM %s" % kind)
    # the decode kernel in 64-row chunks computes the same module
    chunks, kern2 = run_ragged(w, force_kernel=2)
    assert kern2.startswith("dequant_dot_decode_"), kern2
    check_dot(chunks, ref, floor, "ragged chunks %s" % kind)
    owned = int(min(M, np.sum(np.clip(w["group_sizes"], 0, None))))
    assert np.array_equal(got[owned:], np.broadcast_to(w["bias"], (M - owned, N)))


@pytest.mark.parametrize("bits,M,K,N,group,scale_ty,epilogue", [
    (8, 5, 1024, 256, 128, "f32", "BIAS_GELU"), (8, 24, 512, 128, 32, "bf16", "DEFAULT"), (8, 40, 2048, 512, 64, "f32", "BIAS"),
    (8, 64, 1024, 256, 256, "f32", "SILU"), (4, 8, 2048, 512, 128, "f32", "BIAS_SILU"), (4, 30, 1024, 256, 64, "bf16", "RELU"),
    (8, 200, 512, 128, 64, "f32", "DEFAULT"), (4, 50, 1024, 256, 128, "f32", "BIAS"), (4, 100, 512, 128, 64, "bf16", "DEFAULT")])
def test_group_scales_under_f32_multiply(oracle, bits, M, K, N, group, scale_ty, epilogue):
    """convert(w) * scale[K/g,N] f32-typed: every product is an f32 in the reference; the kernel adds a
    group's integers exactly and multiplies the group's sum by its scale (2^-24 per term apart, inside
    the floor that summation order already needs).  s8 and s4, f32 and bf16 scales, up to 64 tokens
    per launch (200 tokens: 64-token chunks)."""
    say("dequant_dot group scales, f32 multiply: s%d M=%d K=%d N=%d group=%d %s %s" % (bits, M, K, N, group, scale_ty, epilogue))
    rng = np.random.default_rng(100 + M)
    sc = rng.uniform(1e-3, 2e-2, size=(K // group, N)).astype(np.float32)
    w = dict(lhs=dtypes.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32)),
             weights=rng.integers(-8 if bits == 4 else -127, 8 if bits == 4 else 128, size=(K, N)).astype(np.int8),
             scales=dtypes.f32_to_bf16(sc) if scale_ty == "bf16" else sc,
             bias=dtypes.f32_to_bf16(rng.standard_normal(N).astype(np.float32)) if "BIAS" in epilogue else None,
             weight_dtype="s%d" % bits, weight_shape=(K, N), group=group, dequant_type="f32", epilogue=epilogue)
    got, kern = run_dot(w)
    assert "_group_factored" in kern, kern
    if bits == 4 and M > 32:   # two sets of accumulators per tile: 4-bit weights go 32 tokens at a time
        assert kern.endswith(":x32"), kern
    compare(oracle, w, got, "group-factored %s" % kern)
    generic, kern2 = run_dot(w, force_kernel=1)   # one thread per output, every product rounded to f32
    assert kern2 == "dequant_dot_generic", kern2
    compare(oracle, w, generic, "generic")


def test_u4_zero_points_group_scales_under_f32_multiply(oracle):
    say("dequant_dot u4 + zero points, group scales, f32 multiply")
    w = workloads.u4_zero_point_group(M=12, K=1024, N=256, group=128)
    w = dict(w, dequant_type="f32")
    got, kern = run_dot(w)
    assert kern == "dequant_dot_decode_s4_v4_m16_group_factored", kern
    compare(oracle, w, got, "u4 group-factored")
