"""GPU parity of xla_amd.fp8_scaled_dot against the CPU oracle, through the FFI handler symbol."""
import sys

import numpy as np
import pytest
import torch

from tests.gpu_util import check_dot, check_f8_result, dev_bf16, dev_f32, dev_u8, dot_floor, host_bf16
from xla_amd import dtypes, ffi, ops, workloads

pytestmark = pytest.mark.gpu


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


EPI = {"DEFAULT": "none", "BIAS": "none", "RELU": "relu", "BIAS_RELU": "relu", "GELU": "gelu_tanh",
       "BIAS_GELU": "gelu_tanh", "SILU": "silu", "BIAS_SILU": "silu"}


def run(w, nk=False, force=0, scratch="auto", **types):
    a = dev_u8(w["a"])
    b = dev_u8(np.ascontiguousarray(w["b"].T) if nk else w["b"])
    sa = dev_f32(np.array(w["a_scale"], np.float32))
    sb = dev_f32(np.array(w["b_scale"], np.float32))
    bias = dev_bf16(w["bias"]) if w.get("bias") is not None else None
    ffi.set_option("fp8_dot_kernel", force)
    try:
        out = ops.fp8_scaled_dot(a, b, sa, sb, bias, rhs_contracting_dim=1 if nk else 0,
                                 epilogue=w["epilogue"], scratch=scratch, **types)
        torch.cuda.synchronize()
    finally:
        ffi.set_option("fp8_dot_kernel", 0)
    return host_bf16(out), ffi.last_kernel()


def reference(oracle, w, **types):
    return oracle.fp8_scaled_dot(w["a"], w["b"], w["a_scale"], w["b_scale"], b_is_nk=False,
                                 mul_ty=types.get("dequant_type", "f32"), bias=w.get("bias"),
                                 dot_ty=types.get("dot_type", "f32"), ep_ty=types.get("epilogue_type", "f32"),
                                 epilogue=EPI[w["epilogue"]])


def floor_for(w, exact_kernel=False):
    """Absolute floor under the 2-ulp rule.  The exact kernel adds in f32, so only summation order
    differs from the oracle.  v_mfma_f32_16x16x128_f8f6f4 does not: inside one instruction the
    products of a group of 8 consecutive k are aligned to the group's largest exponent and bits
    more than ~13 below it are dropped (measured: 2 products of 448*448 swallow their 6
    neighbours of 4.0, but not of 16.0).  Each product therefore carries an error of up to
    2^-13 of its group's maximum; summed as a random walk that is 2^-13 * sqrt(sum (a*b)^2),
    taken with a factor 2 of slack and 1.2 for the slope of GELU/SiLU."""
    sa, sb = np.asarray(w["a_scale"], np.float64), np.asarray(w["b_scale"], np.float64)
    a = np.abs(dtypes.f8e4m3fn_to_f32(w["a"]).astype(np.float64)) * (sa[:, None] if sa.ndim else sa)
    b = np.abs(dtypes.f8e4m3fn_to_f32(w["b"]).astype(np.float64)) * (sb[None, :] if sb.ndim else sb)
    f32_order = dot_floor(a, b, w["a"].shape[1])
    if exact_kernel:
        return f32_order
    return f32_order + 1.2 * 2.0 ** -12 * np.sqrt((a * a) @ (b * b))


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("M,K,N", [(256, 512, 384), (128, 1024, 128), (130, 272, 200), (16, 32, 16)])
def test_c3_shape_reduced(oracle, M, K, N, nk):
    say("fp8_scaled_dot M=%d K=%d N=%d nk=%s" % (M, K, N, nk))
    w = workloads.c3_fp8(M, K, N)
    got, kern = run(w, nk=nk, force=2 if M > 64 else 0)   # (few tiles: the launcher itself would stream them in passes)
    assert kern.startswith("fp8_dot_decode" if M <= 48 else "fp8_scaled_dot_tiled"), kern
    n_floor = check_dot(got, reference(oracle, w), floor_for(w), kern)
    assert n_floor <= got.size // 100


def test_rhs_layouts_take_their_own_paths(oracle):
    """[N,K] streams as it is, [K,N] with whole 16-channel chunks is transposed on the way out of
    LDS, any other [K,N] (or a forced one) through a pre-pass; all three must agree with the oracle."""
    say("fp8_scaled_dot rhs layouts")
    w = workloads.c3_fp8(192, 640, 272)
    ref = reference(oracle, w)
    seen = set()
    for nk, layout in [(True, 0), (False, 0), (False, 1)]:
        ffi.set_option("fp8_dot_layout", layout)
        try:
            got, kern = run(w, nk=nk, force=2)
        finally:
            ffi.set_option("fp8_dot_layout", 0)
        seen.add(kern)
        n_floor = check_dot(got, ref, floor_for(w), kern)
        assert n_floor <= got.size // 100
    assert seen == {"fp8_scaled_dot_tiled", "fp8_scaled_dot_tiled_kn", "fp8_scaled_dot_tiled+transpose"}, seen
    w2 = workloads.c3_fp8(80, 128, 200)  # 200 % 16 != 0: no direct [K,N] path
    got, kern = run(w2, nk=False, force=2)
    assert kern == "fp8_scaled_dot_tiled+transpose", kern
    # K = 128: many outputs sit on the flat tail of GELU, where only the floor clause is meaningful
    assert check_dot(got, reference(oracle, w2), floor_for(w2), kern) <= got.size // 25


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("which", ["a", "b", "ab"])
def test_vector_scales(oracle, which, nk):
    """a_scale per row of a and/or b_scale per output channel, on ragged tiles."""
    say("fp8_scaled_dot vector scales %s nk=%s" % (which, nk))
    M, K, N = 300, 512, 272
    w = workloads.c3_fp8(M, K, N)
    rng = np.random.default_rng(17)
    if "a" in which:
        w["a_scale"] = rng.uniform(0.004, 0.04, M).astype(np.float32)
    if "b" in which:
        w["b_scale"] = rng.uniform(0.004, 0.04, N).astype(np.float32)
    got, kern = run(w, nk=nk)
    assert kern.startswith("fp8_scaled_dot_tiled"), kern
    n_floor = check_dot(got, reference(oracle, w), floor_for(w), kern)
    assert n_floor <= got.size // 100
    # the slow kernel takes the same vectors
    got, kern = run(w, nk=nk, force=1)
    assert kern == "fp8_scaled_dot_exact", kern
    check_dot(got, reference(oracle, w), floor_for(w, exact_kernel=True), kern)
    # a bf16-typed multiply rounds every scaled operand: the bf16-operand kernel (the exact one without scratch)
    got, kern = run(w, nk=nk, dequant_type="bf16")
    assert kern == "fp8_scaled_dot_bf16_operands", kern
    check_dot(got, reference(oracle, w, dequant_type="bf16"), floor_for(w, exact_kernel=True), kern)
    got, kern = run(w, nk=nk, dequant_type="bf16", scratch=None)
    assert kern == "fp8_scaled_dot_exact", kern
    check_dot(got, reference(oracle, w, dequant_type="bf16"), floor_for(w, exact_kernel=True), kern)


def test_quantized_rows_feed_the_dot(oracle):
    """rowwise_quantize_fp8 -> fp8_scaled_dot: the quantizer's codes and per-row scales go
    straight in as a and a_scale.  Codes and scales are bit-exact against the oracle, so the
    dot is compared on the oracle's own chain."""
    say("rowwise_quantize_fp8 feeding fp8_scaled_dot")
    R, C, N = 200, 1024, 256
    x = workloads.c4_quantize(R, C)
    q, s = ops.rowwise_quantize_fp8(dev_bf16(x["x"]), dev_bf16(x["gamma"]), eps=1e-6)
    w = workloads.c3_fp8(R, C, N)
    b, sb = dev_u8(w["b"]), dev_f32(np.array(w["b_scale"], np.float32))
    out = ops.fp8_scaled_dot(q, b, s, sb, dev_bf16(w["bias"]), epilogue="BIAS_GELU")
    torch.cuda.synchronize()
    kern = ffi.last_kernel()
    assert kern.startswith("fp8_scaled_dot_tiled"), kern
    q_ref, s_ref = oracle.rmsnorm_quantize_fp8(x["x"], x["gamma"], eps=1e-6)
    assert np.array_equal(q.cpu().numpy().view(np.uint8), q_ref) and np.array_equal(s.cpu().numpy(), s_ref)
    w.update(a=q_ref, a_scale=s_ref)
    n_floor = check_dot(host_bf16(out), reference(oracle, w), floor_for(w), kern)
    assert n_floor <= out.numel() // 100


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("mode", ["divide", "multiply", "divide_by_odd_scale", "exact_kernel"])
def test_f8_result(oracle, mode, nk):
    """f8e4m3fn result = convert(clamp(v / d_scale)): codes inside the window the dot's own
    tolerance allows, and nearly all of them equal to the oracle's."""
    say("fp8_scaled_dot f8 result %s nk=%s" % (mode, nk))
    M, K, N = 300, 512, 272
    w = workloads.c3_fp8(M, K, N)
    divides = mode != "multiply"
    # all-ones significand: the reciprocal shortcut must step aside for the IEEE divide
    z = {"divide": np.float32(0.0117), "multiply": np.float32(85.0),
         "divide_by_odd_scale": np.frombuffer(np.uint32(0x3c7fffff).tobytes(), np.float32)[0],
         "exact_kernel": np.float32(0.0117)}[mode]
    a, b = dev_u8(w["a"]), dev_u8(np.ascontiguousarray(w["b"].T) if nk else w["b"])
    s64 = dev_f32(np.array(1 / 64, np.float32))
    ffi.set_option("fp8_dot_kernel", 1 if mode == "exact_kernel" else 0)
    try:
        out = ops.fp8_scaled_dot(a, b, s64, s64, dev_bf16(w["bias"]), rhs_contracting_dim=1 if nk else 0,
                                 epilogue="BIAS_GELU", d_scale=dev_f32(np.array(z, np.float32)),
                                 d_scale_multiplies=not divides)
        torch.cuda.synchronize()
    finally:
        ffi.set_option("fp8_dot_kernel", 0)
    kern = ffi.last_kernel()
    assert out.dtype == torch.uint8
    assert ("exact" in kern) == (mode == "exact_kernel") and (mode == "exact_kernel" or kern.endswith("_f8")), kern
    ref, val = oracle.fp8_scaled_dot(w["a"], w["b"], 1 / 64, 1 / 64, bias=w["bias"], epilogue="gelu_tanh",
                                     d_scale=z, d_scale_divides=divides)
    differ = check_f8_result(out.cpu().numpy(), ref, val, z, divides, floor_for(w, exact_kernel=mode == "exact_kernel"), kern)
    assert differ <= out.numel() // 50, differ


@pytest.mark.parametrize("force", [0, 1])
def test_f8_result_amax(oracle, force):
    """amax next to the f8 result: max |v| over the ragged result, from atomics into a result the
    call itself zeroes -- so two calls in a row, the second on smaller values, must not see the first."""
    say("fp8_scaled_dot f8 result with amax, kernel option %d" % force)
    M, K, N = 300, 512, 272
    w = workloads.c3_fp8(M, K, N)
    z = np.float32(0.0117)
    a, b, bias = dev_u8(w["a"]), dev_u8(w["b"]), dev_bf16(w["bias"])
    ffi.set_option("fp8_dot_kernel", force)
    try:
        for scale in (1 / 64, 1 / 512):
            s = dev_f32(np.array(scale, np.float32))
            out, amax = ops.fp8_scaled_dot(a, b, s, s, bias, epilogue="BIAS_GELU", amax=True,
                                           d_scale=dev_f32(np.array(z, np.float32)))
            torch.cuda.synchronize()
            _, val = oracle.fp8_scaled_dot(w["a"], w["b"], scale, scale, bias=w["bias"], epilogue="gelu_tanh", d_scale=z)
            want = float(np.max(np.abs(val)))
            assert abs(float(amax) - want) <= want * 2.0 ** -7, (float(amax), want)
    finally:
        ffi.set_option("fp8_dot_kernel", 0)
    # a NaN anywhere makes the maximum NaN
    bn = w["b"].copy()
    bn[7, 5] = 0x7F
    s = dev_f32(np.array(1 / 64, np.float32))
    _, amax = ops.fp8_scaled_dot(a, dev_u8(bn), s, s, bias, epilogue="BIAS_GELU", amax=True,
                                 d_scale=dev_f32(np.array(z, np.float32)))
    torch.cuda.synchronize()
    assert np.isnan(float(amax))


@pytest.mark.parametrize("nk,N", [(True, 272), (False, 272), (False, 200)])
def test_batched(oracle, nk, N):
    """One leading batch dimension: every batch against the oracle, bf16 and f8 results (with the
    amax over all batches); a [K,N] rhs whose N has no whole 16-channel chunks takes the exact kernel."""
    say("fp8_scaled_dot batched nk=%s N=%d" % (nk, N))
    B, M, K = 3, 150, 256
    ws = [workloads.c3_fp8(M, K, N) for _ in range(B)]
    rng = np.random.default_rng(3)
    for i, w in enumerate(ws):   # different data per batch
        w["a"] = np.roll(w["a"], 17 * i, axis=0)
        w["b"] = np.roll(w["b"], 5 * i, axis=1)
    a = dev_u8(np.stack([w["a"] for w in ws]))
    b = dev_u8(np.stack([np.ascontiguousarray(w["b"].T) if nk else w["b"] for w in ws]))
    s64, bias = dev_f32(np.array(1 / 64, np.float32)), dev_bf16(ws[0]["bias"])
    out = ops.fp8_scaled_dot(a, b, s64, s64, bias, rhs_contracting_dim=1 if nk else 0, epilogue="BIAS_GELU")
    torch.cuda.synchronize()
    kern = ffi.last_kernel()
    assert ("exact" in kern) == (N % 16 != 0), kern
    got = host_bf16(out)
    for i, w in enumerate(ws):
        check_dot(got[i], reference(oracle, w), floor_for(w, exact_kernel="exact" in kern), "batch %d %s" % (i, kern))
    z = np.float32(0.0117)
    out8, amax = ops.fp8_scaled_dot(a, b, s64, s64, bias, rhs_contracting_dim=1 if nk else 0, epilogue="BIAS_GELU",
                                    d_scale=dev_f32(np.array(z, np.float32)), amax=True)
    torch.cuda.synchronize()
    want_amax = 0.0
    for i, w in enumerate(ws):
        ref, val = oracle.fp8_scaled_dot(w["a"], w["b"], 1 / 64, 1 / 64, bias=w["bias"], epilogue="gelu_tanh", d_scale=z)
        check_f8_result(out8[i].cpu().numpy(), ref, val, z, True, floor_for(w, exact_kernel="exact" in kern), "f8 batch %d" % i)
        want_amax = max(want_amax, float(np.max(np.abs(val))))
    assert abs(float(amax) - want_amax) <= want_amax * 2.0 ** -7


def mx_case(M, K, N, seed):
    rng = np.random.default_rng(seed)
    a = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((M, K)) * 8, -448, 448).astype(np.float32))
    b = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((N, K)) * 8, -448, 448).astype(np.float32))
    sa = rng.integers(118, 134, (M, K // 32)).astype(np.uint8)
    sb = rng.integers(118, 134, (N, K // 32)).astype(np.uint8)
    return a, b, sa, sb


def mx_floor(a, b, sa, sb, exact_kernel):
    ad = np.abs(dtypes.f8e4m3fn_to_f32(a).astype(np.float64)) * np.repeat(2.0 ** (sa.astype(np.float64) - 127), 32, axis=1)
    bd = np.abs(dtypes.f8e4m3fn_to_f32(b).astype(np.float64)) * np.repeat(2.0 ** (sb.astype(np.float64) - 127), 32, axis=1)
    fl = dot_floor(ad, bd.T, a.shape[1])
    return fl if exact_kernel else fl + 1.2 * 2.0 ** -12 * np.sqrt((ad * ad) @ (bd * bd).T)


@pytest.mark.parametrize("M,K,N", [(64, 128, 64), (300, 512, 272), (256, 1024, 256), (100, 96, 40)])
def test_mxfp8_block_scales(oracle, M, K, N):
    """f8e8m0fnu scales per 32 elements of K on both operands, multiplied in by the matrix cores;
    K that is not a multiple of 128 (and the forced slow kernel) take the exact kernel, which
    must match the oracle bit for bit: every product and partial sum is the same f32 operation."""
    say("fp8_scaled_dot MXFP8 M=%d K=%d N=%d" % (M, K, N))
    a, b, sa, sb = mx_case(M, K, N, 7)
    ref = oracle.block_scaled_dot(a, b, sa, sb)
    da, db, dsa, dsb = dev_u8(a), dev_u8(b), dev_u8(sa), dev_u8(sb)
    ffi.set_option("fp8_dot_kernel", 2 if K % 128 == 0 else 0)   # (64 rows would go through the streaming kernel twice)
    try:
        out = ops.fp8_scaled_dot(da, db, dsa, dsb, rhs_contracting_dim=1)
        torch.cuda.synchronize()
    finally:
        ffi.set_option("fp8_dot_kernel", 0)
    kern = ffi.last_kernel()
    assert kern == ("fp8_scaled_dot_tiled_mx" if K % 128 == 0 else "fp8_scaled_dot_exact"), kern
    n_floor = check_dot(host_bf16(out), ref, mx_floor(a, b, sa, sb, "exact" in kern), kern)
    assert n_floor <= out.numel() // 50
    ffi.set_option("fp8_dot_kernel", 1)
    try:
        out = ops.fp8_scaled_dot(da, db, dsa, dsb, rhs_contracting_dim=1)
        torch.cuda.synchronize()
    finally:
        ffi.set_option("fp8_dot_kernel", 0)
    assert ffi.last_kernel() == "fp8_scaled_dot_exact"
    assert np.array_equal(host_bf16(out), ref)


@pytest.mark.parametrize("epilogue,dot_ty,ep_ty", [("BIAS_GELU", "f32", "f32"), ("BIAS_SILU", "bf16", "bf16"), ("RELU", "f32", "f32"),
                                                  ("BIAS", "f32", "f32")])
def test_mxfp8_with_an_epilogue(oracle, epilogue, dot_ty, ep_ty):
    """Block scales with a bias and an activation behind the dot, on the tiled and on the exact kernel."""
    say("fp8_scaled_dot MXFP8 %s dot %s epilogue %s" % (epilogue, dot_ty, ep_ty))
    names = {"BIAS_GELU": "gelu_tanh", "BIAS_SILU": "silu", "RELU": "relu", "BIAS": "none"}
    for (M, K, N) in ((300, 512, 272), (70, 96, 40)):
        a, b, sa, sb = mx_case(M, K, N, 11)
        rng = np.random.default_rng(3)
        bias = dtypes.f32_to_bf16(rng.standard_normal(N).astype(np.float32)) if "BIAS" in epilogue else None
        ref = oracle.block_scaled_dot(a, b, sa, sb, bias=bias, dot_ty=dot_ty, ep_ty=ep_ty, epilogue=names[epilogue])
        out = ops.fp8_scaled_dot(dev_u8(a), dev_u8(b), dev_u8(sa), dev_u8(sb), dev_bf16(bias) if bias is not None else None,
                                 rhs_contracting_dim=1, epilogue=epilogue, dot_type=dot_ty, epilogue_type=ep_ty)
        torch.cuda.synchronize()
        kern = ffi.last_kernel()
        assert kern == ("fp8_scaled_dot_tiled_mx" if K % 128 == 0 else "fp8_scaled_dot_exact"), kern
        if "exact" in kern:
            assert np.array_equal(host_bf16(out), ref)
        else:
            # the floor is that of the value entering the activation; both activations have slope <= 1.13
            check_dot(host_bf16(out), ref, 1.2 * mx_floor(a, b, sa, sb, False), kern + " " + epilogue)


def test_mxfp8_batched(oracle):
    """One leading batch dimension on the operands, their block scales and the result."""
    say("fp8_scaled_dot MXFP8 batched")
    for (B, M, K, N) in ((3, 130, 256, 264), (2, 40, 64, 72)):
        cases = [mx_case(M, K, N, 20 + i) for i in range(B)]
        a, b, sa, sb = (np.stack([c[j] for c in cases]) for j in range(4))
        out = ops.fp8_scaled_dot(dev_u8(a), dev_u8(b), dev_u8(sa), dev_u8(sb), rhs_contracting_dim=1)
        torch.cuda.synchronize()
        kern = ffi.last_kernel()
        assert kern == ("fp8_scaled_dot_tiled_mx" if K % 128 == 0 else "fp8_scaled_dot_exact"), kern
        got = host_bf16(out)
        for i in range(B):
            ref = oracle.block_scaled_dot(a[i], b[i], sa[i], sb[i])
            if "exact" in kern:
                assert np.array_equal(got[i], ref), i
            else:
                check_dot(got[i], ref, mx_floor(a[i], b[i], sa[i], sb[i], False), "%s batch %d" % (kern, i))


def test_mxfp8_one_block_at_a_time(oracle):
    """Data in a single 32-element block of K, a different scale on every block: each block must
    come out multiplied by its own two scales exactly (products of small integers, exact sums)."""
    say("fp8_scaled_dot MXFP8 block by block")
    M, K, N = 64, 256, 64
    rng = np.random.default_rng(2)
    ai = rng.integers(-3, 4, (M, K)).astype(np.float32)
    bi = rng.integers(-3, 4, (N, K)).astype(np.float32)
    sa = np.repeat((121 + np.arange(K // 32)).astype(np.uint8)[None, :], M, axis=0)
    sb = np.repeat((134 - 2 * np.arange(K // 32)).astype(np.uint8)[None, :], N, axis=0)   # sa + sb differs from block to block
    sb[:, :] += (np.arange(N) % 3).astype(np.uint8)[:, None]
    for j in range(K // 32):
        a1 = np.zeros_like(ai)
        a1[:, 32 * j:32 * j + 32] = ai[:, 32 * j:32 * j + 32]
        a8, b8 = dtypes.f32_to_f8e4m3fn(a1), dtypes.f32_to_f8e4m3fn(bi)
        ffi.set_option("fp8_dot_kernel", 2)
        try:
            out = ops.fp8_scaled_dot(dev_u8(a8), dev_u8(b8), dev_u8(sa), dev_u8(sb), rhs_contracting_dim=1)
            torch.cuda.synchronize()
        finally:
            ffi.set_option("fp8_dot_kernel", 0)
        assert ffi.last_kernel() == "fp8_scaled_dot_tiled_mx"
        assert np.array_equal(host_bf16(out), oracle.block_scaled_dot(a8, b8, sa, sb)), j


def test_f8_result_special_values(oracle):
    """NaN operands give NaN codes, a huge value over a tiny scale saturates at +-448, -0 stays -0;
    a zero scale follows IEEE (x/0 = +-inf -> +-448, 0/0 = NaN)."""
    say("fp8_scaled_dot f8 result special values")
    M, K, N = 64, 64, 64
    a = np.zeros((M, K), np.float32)
    a[np.arange(M), np.arange(M) % K] = 1.0           # selector rows: out[m, n] = b[m % K, n]
    bvals = np.zeros((K, N), np.float32)
    bvals[0, :] = 448.0
    bvals[1, :] = -448.0
    bvals[2, :] = 2.0 ** -9
    bvals[3, :] = -0.0
    b8 = dtypes.f32_to_f8e4m3fn(bvals)
    b8[4, N - 1] = 0x7F                                # NaN: the whole last column (0 * NaN = NaN)
    a8 = dtypes.f32_to_f8e4m3fn(a)
    one = dev_f32(np.array(1.0, np.float32))
    for z in (np.float32(1e-30), np.float32(0.0), np.float32(3.0)):
        out = ops.fp8_scaled_dot(dev_u8(a8), dev_u8(b8), one, one, d_scale=dev_f32(np.array(z, np.float32)))
        torch.cuda.synchronize()
        ref, _ = oracle.fp8_scaled_dot(a8, b8, 1.0, 1.0, d_scale=z)
        got = out.cpu().numpy()
        nan = (ref & 0x7F) == 0x7F
        assert np.array_equal(nan, (got & 0x7F) == 0x7F), z
        assert np.array_equal(got[~nan], ref[~nan]), z


@pytest.mark.parametrize("epilogue", ["BIAS_GELU", "SILU"])
def test_closed_form_activations_opt_in(oracle, epilogue):
    """Option "tiled_epilogue" = 1: x * sigmoid(.) with the hardware exponential.  Same values as the
    op-by-op default to 2 bf16 ulp wherever the result is not negligible; in the far negative tail
    (results below 2e-5 in magnitude) the reference's own cancellation is the larger error, so
    there only an absolute bound holds."""
    say("fp8_scaled_dot closed-form " + epilogue)
    w = workloads.c3_fp8(256, 512, 384)
    w["epilogue"] = epilogue
    if "BIAS" not in epilogue:
        w["bias"] = None
    strict, _ = run(w)
    ffi.set_option("tiled_epilogue", 1)
    try:
        got, kern = run(w)
    finally:
        ffi.set_option("tiled_epilogue", 0)
    assert kern.startswith("fp8_scaled_dot_tiled")
    assert not np.array_equal(got, strict)                      # it did take the other path
    n_floor = check_dot(got, reference(oracle, w), floor_for(w) + 2e-5,
                        "OPT-IN closed-form %s (floor + 2e-5), not the default path: %s" % (epilogue, kern))
    big = np.abs(dtypes.bf16_to_f32(strict)) > 1e-3
    from tests.gpu_util import bf16_ordinal
    assert np.all(np.abs(bf16_ordinal(got[big]) - bf16_ordinal(strict[big])) <= 2)


def test_fp8_one_hot_exact(oracle):
    """A = selector rows of 1.0: outputs are single B values times the scales, exactly."""
    say("fp8_scaled_dot one-hot")
    K, N = 256, 256
    a = np.zeros((128, K), np.float32)
    a[np.arange(128), np.arange(128) * 2] = 1.0
    b8 = np.tile(np.arange(256, dtype=np.uint8), (K, 1))
    b8 = np.roll(b8, 3, axis=1)
    b8[(b8 & 0x7F) == 0x7F] = 0x3A
    w = dict(a=dtypes.f32_to_f8e4m3fn(a), b=b8, a_scale=np.float32(0.5), b_scale=np.float32(0.25),
             bias=None, epilogue="DEFAULT")
    for nk in (False, True):
        got, kern = run(w, nk=nk)
        want = dtypes.f32_to_bf16(dtypes.f8e4m3fn_to_f32(b8[np.arange(128) * 2]) * np.float32(0.125))
        assert np.array_equal(dtypes.bf16_to_f32(got), dtypes.bf16_to_f32(want)), kern


def test_reference_pattern_bf16_typed_ops(oracle):
    """The reference's own test pattern (gemm_rewriter_fp8_test.cc:1110-1141): every op bf16-typed."""
    say("fp8_scaled_dot bf16-typed pattern")
    w = workloads.c3_fp8(128, 256, 128)
    types = dict(dequant_type="bf16", dot_type="bf16", epilogue_type="bf16")
    got, kern = run(w, **types)
    ref = reference(oracle, w, **types)
    # the dot itself is rounded to bf16 here, so an accumulator difference far below one ulp can
    # flip that rounding; the flip then passes through bias add and nine more bf16-rounded ops.
    # Allow 6 ulp of the result (the reference's own ErrorSpec for this pattern is 1e-2,
    # gemm_rewriter_fp8_test.cc:110).
    fl = floor_for(w) * 12 + np.abs(dtypes.bf16_to_f32(ref)) * 6 * 2.0 ** -8
    check_dot(got, ref, fl, kern)


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("M,K,N", [(64, 128, 64), (300, 520, 272), (130, 264, 200)])
def test_bf16_typed_multiply_with_any_scale(oracle, M, K, N, nk):
    """bf16-typed dequantise multiply with scales that are no powers of two: every a * a_scale and
    b * b_scale is rounded to bf16, so the f8 kernel (which scales the sum) does not serve the call;
    a pre-pass writes the rounded operands as bf16 and the bf16 matrix cores multiply them.  bf16
    products are exact in f32: only the order of the sum differs from the oracle (the strict floor).
    With power-of-two scales the same launches leave the f8 kernel's result untouched."""
    say("fp8_scaled_dot bf16-typed multiply, scales 0.3 / 0.013, M=%d K=%d N=%d nk=%s" % (M, K, N, nk))
    w = workloads.c3_fp8(M, K, N)
    w["a_scale"] = np.float32(0.3)
    w["b_scale"] = np.float32(0.013)
    types = dict(dequant_type="bf16")
    got, kern = run(w, nk=nk, **types)
    # K % 16 != 0 keeps the f8 kernel out altogether; otherwise both are enqueued and the scales decide
    # (64 rows of a [K,N] rhs: the streaming kernels' own rounding form, "|rounded")
    assert kern == ("fp8_scaled_dot_bf16_operands" if K % 16 else kern) and kern.endswith(("bf16_operands", "|rounded")), kern
    n_floor = check_dot(got, reference(oracle, w, **types), floor_for(w, exact_kernel=True), kern)
    assert n_floor <= max(8, got.size // 50)
    exact, kern2 = run(w, nk=nk, force=1, **types)
    assert kern2 == "fp8_scaled_dot_exact", kern2
    check_dot(exact, reference(oracle, w, **types), floor_for(w, exact_kernel=True), kern2)
    w2 = dict(w, a_scale=np.float32(1 / 64), b_scale=np.float32(1 / 32))
    got2, kern3 = run(w2, nk=nk, **types)
    assert kern3.endswith(("bf16_operands", "|rounded")), kern3
    if K % 16 == 0:
        plain, _ = run(w2, nk=nk)   # f32-typed: the f8 kernel alone; identical values for power-of-two scales
        assert np.array_equal(got2, plain)
    else:
        check_dot(got2, reference(oracle, w2, **types), floor_for(w2, exact_kernel=True), kern3)


@pytest.mark.parametrize("which", ["a", "b", "ab"])
def test_bf16_typed_multiply_with_vector_scales(oracle, which):
    say("fp8_scaled_dot bf16-typed multiply, vector scales on %s" % which)
    M, K, N = 200, 256, 136
    w = workloads.c3_fp8(M, K, N)
    rng = np.random.default_rng(8)
    if "a" in which:
        w["a_scale"] = rng.uniform(0.004, 0.04, M).astype(np.float32)
    if "b" in which:
        w["b_scale"] = rng.uniform(0.004, 0.04, N).astype(np.float32)
    types = dict(dequant_type="bf16")
    got, kern = run(w, **types)
    assert kern == "fp8_scaled_dot_bf16_operands", kern
    n_floor = check_dot(got, reference(oracle, w, **types), floor_for(w, exact_kernel=True), kern)
    assert n_floor <= got.size // 50


def test_bf16_typed_multiply_without_scratch_takes_exact_kernel(oracle):
    say("fp8_scaled_dot bf16-typed multiply with scale 0.3, no scratch")
    w = workloads.c3_fp8(64, 128, 64)
    w["a_scale"] = np.float32(0.3)
    types = dict(dequant_type="bf16")
    got, kern = run(w, scratch=None, **types)
    assert kern == "fp8_dot_decode_kn_m64|rounded", kern   # the form that rounds the scaled operands runs for this scale
    n_floor = check_dot(got, reference(oracle, w, **types), floor_for(w, exact_kernel=True), kern)
    assert n_floor <= got.size // 100


def test_exact_kernel_and_missing_scratch(oracle):
    say("fp8_scaled_dot exact kernel / no scratch")
    w = workloads.c3_fp8(80, 80, 44)   # (N % 8 != 0: not for the streaming kernels)
    got, kern = run(w, scratch=None)
    assert kern == "fp8_scaled_dot_exact", kern
    check_dot(got, reference(oracle, w), floor_for(w, exact_kernel=True), kern)
    with pytest.raises(ffi.FfiError, match="tiled kernel needs"):
        run(w, force=2, scratch=None)


def test_c3_full_size_sampled_blocks(oracle):
    """Configuration 3 at full size; the oracle evaluates random row/column blocks of the same
    inputs."""
    say("fp8_scaled_dot C3 full size")
    w = workloads.c3_fp8()
    got, kern = run(w)
    assert kern.startswith("fp8_scaled_dot_tiled"), kern
    rng = np.random.default_rng(1)
    for _ in range(6):
        m0 = int(rng.integers(0, 8192 - 32)); n0 = int(rng.integers(0, 8192 - 64))
        sub = dict(w, a=np.ascontiguousarray(w["a"][m0:m0 + 32]), b=np.ascontiguousarray(w["b"][:, n0:n0 + 64]),
                   bias=np.ascontiguousarray(w["bias"][n0:n0 + 64]))
        n_floor = check_dot(got[m0:m0 + 32, n0:n0 + 64], reference(oracle, sub), floor_for(sub),
                            "C3 block m0=%d n0=%d" % (m0, n0))
        assert n_floor <= 32


def test_fp8_error_paths():
    say("fp8_scaled_dot error paths")
    a = torch.zeros((16, 32), dtype=torch.uint8, device="cuda")
    b = torch.zeros((48, 16), dtype=torch.uint8, device="cuda")
    one = torch.ones((), dtype=torch.float32, device="cuda")
    with pytest.raises(ffi.FfiError, match="contracting dimensions differ"):
        ops.fp8_scaled_dot(a, b, one, one)
    with pytest.raises(ffi.FfiError, match="rhs_contracting_dim"):
        ops.fp8_scaled_dot(a, torch.zeros((32, 16), dtype=torch.uint8, device="cuda"), one, one,
                           rhs_contracting_dim=2)


# ---- tiles of a last round that is at most a quarter full run as two workgroups along K ------------------

def _split_case(mode):
    M, K, N = 300, 2304, 272        # 2 x 2 tiles, 18 stages of 128: halves of 9 stages each
    if mode == "mx":
        return mx_case(M, K, N, 17)
    w = workloads.c3_fp8(M, K, N)
    if mode == "vector_scales":
        rng = np.random.default_rng(8)
        w["a_scale"] = rng.uniform(0.004, 0.04, M).astype(np.float32)
        w["b_scale"] = rng.uniform(0.004, 0.04, N).astype(np.float32)
    return w


@pytest.mark.parametrize("mode", ["kn", "nk", "vector_scales", "mx", "f8_result"])
@pytest.mark.parametrize("drop_flags", [False, True])
def test_last_round_split_along_k(oracle, mode, drop_flags):
    """Few tiles and a long K: every tile is two workgroups, the one on the second half of K hands its sums
    over.  drop_flags: that workgroup never raises its flag, the other gives up after a few polls and does
    the second half itself (every kernel exits normally); the next ordinary call on the same scratch
    must give the ordinary result bit for bit.  Unsplit tiles (option "tiled_tail" = 1) sum K in the order
    the give-up path uses."""
    say("fp8_scaled_dot split last round, %s, drop_flags=%s" % (mode, drop_flags))
    scratch = torch.empty(4 << 20, dtype=torch.uint8, device="cuda")
    case = _split_case(mode)

    def once(drop=False, whole=False):
        ffi.set_option("handover_test", 1 if drop else 0)
        ffi.set_option("tiled_tail", 1 if whole else 0)
        try:
            if mode == "mx":
                a, b, sa, sb = case
                out = ops.fp8_scaled_dot(dev_u8(a), dev_u8(b), dev_u8(sa), dev_u8(sb), rhs_contracting_dim=1, scratch=scratch)
            elif mode == "f8_result":
                out, amax = ops.fp8_scaled_dot(dev_u8(case["a"]), dev_u8(case["b"]), s64, s64, dev_bf16(case["bias"]),
                                               epilogue="BIAS_GELU", d_scale=dev_f32(np.array(z, np.float32)), amax=True,
                                               scratch=scratch)
                torch.cuda.synchronize()
                return (out.cpu().numpy(), float(amax)), ffi.last_kernel()
            else:
                nk = mode == "nk"
                out = ops.fp8_scaled_dot(dev_u8(case["a"]), dev_u8(np.ascontiguousarray(case["b"].T) if nk else case["b"]),
                                         dev_f32(np.array(case["a_scale"], np.float32)), dev_f32(np.array(case["b_scale"], np.float32)),
                                         dev_bf16(case["bias"]), rhs_contracting_dim=1 if nk else 0, epilogue="BIAS_GELU",
                                         scratch=scratch)
            torch.cuda.synchronize()
            return host_bf16(out), ffi.last_kernel()
        finally:
            ffi.set_option("handover_test", 0)
            ffi.set_option("tiled_tail", 0)

    s64, z = dev_f32(np.array(1 / 64, np.float32)), np.float32(0.0117)
    normal, kern = once()
    assert kern.endswith(":tail2"), kern
    got, kern = once(drop=drop_flags)
    assert kern.endswith(":tail2"), kern
    if mode == "mx":
        a, b, sa, sb = case
        check_dot(got, oracle.block_scaled_dot(a, b, sa, sb), mx_floor(a, b, sa, sb, False), kern)
    elif mode == "f8_result":
        ref, val = oracle.fp8_scaled_dot(case["a"], case["b"], 1 / 64, 1 / 64, bias=case["bias"], epilogue="gelu_tanh", d_scale=z)
        check_f8_result(got[0], ref, val, z, True, floor_for(case), kern)
        want = float(np.max(np.abs(val)))
        assert abs(got[1] - want) <= want * 2.0 ** -7
    else:
        check_dot(got, reference(oracle, case), floor_for(case), kern)
    if drop_flags:
        whole, kern = once(whole=True)
        assert not kern.endswith(":tail2"), kern
        if mode == "f8_result":
            assert np.array_equal(got[0], whole[0]) and got[1] == whole[1]
        else:
            assert np.array_equal(got, whole)
    again, _ = once()
    if mode == "f8_result":
        assert np.array_equal(again[0], normal[0]) and again[1] == normal[1]
    else:
        assert np.array_equal(again, normal)
