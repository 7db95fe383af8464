"""Result and operand layouts of xla_amd.dequant_dot beyond bf16 [M,N] = lhs [M,K] . W: an f32 result
(the dot's own value, fusion_emitter_int4_device_test.cc:101,205,320,508), the dequantised weights as
the lhs of the dot (result [N,M], :495-523), activations stored [K,M] (the dot contracts their major dimension, the shape
table :609-645) and an f8e4m3fn result (the D scaling of gemm_rewriter_fp8_test.cc:1665-1690, :1730-1748
on the dot's f32 value) -- against the CPU oracle, through the FFI handler."""
import numpy as np
import pytest
import torch

from tests.gpu_util import check_dot, check_dot_f32, check_f8_result, dev_bf16, dev_f32, dev_s8, dev_u8, host_bf16
from tests.test_gpu_dequant_dot import floor_for, oracle_dot, say
from xla_amd import dtypes, ffi, ops, workloads

pytestmark = pytest.mark.gpu


def run(w, nk=False, out_dtype="bf16", transposed=False, lhs_k_major=False, force_kernel=0, d_scale=None,
        d_scale_multiplies=False):
    v = workloads.k_minor(w) if nk else w
    lhs_h = v["lhs"]
    if lhs_k_major:
        lhs_h = np.ascontiguousarray(np.swapaxes(lhs_h, -1, -2))
    lhs = dev_bf16(lhs_h)
    if v["weight_dtype"] in ("s4", "u4"):
        wt = dev_u8(v["weights_packed"])
    else:
        wt = dev_s8(v["weights"])
    sc = dev_bf16(v["scales"]) if v["scales"].dtype == np.uint16 else dev_f32(v["scales"])
    bias = None
    if v.get("bias") is not None and "BIAS" in v["epilogue"]:
        bias = dev_bf16(v["bias"]) if v["bias"].dtype == np.uint16 else dev_f32(v["bias"])
    K = w["lhs"].shape[-1]
    ffi.set_option("dequant_dot_kernel", force_kernel)
    try:
        out = ops.dequant_dot(lhs, wt, sc, bias, weight_dtype=v["weight_dtype"], weight_shape=v["weight_shape"],
                              epilogue=v["epilogue"], dequant_type=v["dequant_type"],
                              scale_group_size=0 if w["group"] == K else w["group"],
                              rhs_contracting_dim=1 if nk else 0, out_dtype=out_dtype, result_transposed=transposed,
                              lhs_contracting_dim=0 if lhs_k_major else 1,
                              d_scale=None if d_scale is None else dev_f32(np.array(d_scale, np.float32)),
                              d_scale_multiplies=d_scale_multiplies)
        torch.cuda.synchronize()
    finally:
        ffi.set_option("dequant_dot_kernel", 0)
    got = out.cpu().numpy() if (out_dtype == "f32" or d_scale is not None) else host_bf16(out)
    if transposed:
        got = np.swapaxes(got, -1, -2)
    return got, ffi.last_kernel()


def reference(oracle, w, f32):
    if not f32:
        return oracle_dot(oracle, w)
    scale_ty = "bf16" if w["scales"].dtype == np.uint16 else "f32"
    wt, bits = (w["weights_packed"], 4) if w["weight_dtype"] in ("s4", "u4") else (w["weights"], 8)
    epi = {"DEFAULT": "none", "BIAS": "none", "BIAS_SILU": "silu", "BIAS_GELU": "gelu_tanh"}[w["epilogue"]]
    bias = w.get("bias") if "BIAS" in w["epilogue"] else None
    return oracle.dequant_dot(w["lhs"], wt, bits, w["scales"], scale_ty, w["dequant_type"], bias=bias,
                              bias_ty="bf16" if (bias is not None and bias.dtype == np.uint16) else "f32",
                              group=w["group"], epilogue=epi, f32_result=True)


CASES = [
    # (workload, kwargs): s4 grouped under a bf16 multiply; s8 per channel under an f32 multiply
    ("s4", dict(M=8, K=512, N=256, group=128)),
    ("s4", dict(M=40, K=1024, N=136, group=64)),
    ("s4", dict(M=100, K=512, N=128, group=128)),        # more than 64 tokens: token chunks
    ("s8", dict(M=16, K=1024, N=256)),
    ("s8", dict(M=3, K=264, N=40)),                      # unaligned: one thread per output
    ("s8", dict(M=130, K=256, N=64)),
]


def make(kind, kw):
    return workloads.c2_s4_group(**kw) if kind == "s4" else workloads.c1_s8_channel(**kw)


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("kind,kw", CASES)
def test_f32_result(oracle, kind, kw, nk):
    say("dequant_dot f32 result %s %s nk=%s" % (kind, kw, nk))
    w = make(kind, kw)
    got, kern = run(w, nk=nk, out_dtype="f32")
    assert got.dtype == np.float32
    check_dot_f32(got, reference(oracle, w, True), floor_for(w), "f32 result %s" % kern)
    # the same call with a bf16 result is this value rounded, up to the summation order
    got16, _ = run(w, nk=nk)
    check_dot(got16, dtypes.f32_to_bf16(got), floor_for(w), "f32 result rounded vs bf16 result")


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("lhs_k_major", [False, True])
@pytest.mark.parametrize("kind,kw", [CASES[0], CASES[1], CASES[3], CASES[4], CASES[5]])
def test_weights_as_the_lhs_of_the_dot(oracle, kind, kw, nk, lhs_k_major):
    """dot(dequantised weights, activations): the result is [N,M]; activations [M,K] or [K,M]; f32 and
    bf16 results.  DEFAULT epilogue (a bias along N would broadcast along the other dimension)."""
    say("dequant_dot weights as lhs %s %s nk=%s lhs_k_major=%s" % (kind, kw, nk, lhs_k_major))
    w = dict(make(kind, kw), epilogue="DEFAULT", bias=None)
    for out_dtype in ("f32", "bf16"):
        got, kern = run(w, nk=nk, out_dtype=out_dtype, transposed=True, lhs_k_major=lhs_k_major)
        ref = reference(oracle, w, out_dtype == "f32")
        if out_dtype == "f32":
            check_dot_f32(got, ref, floor_for(w), "weights as lhs, f32, %s" % kern)
        else:
            check_dot(got, ref, floor_for(w), "weights as lhs, bf16, %s" % kern)


def test_one_hot_activations_read_single_weights_back_in_every_layout(oracle):
    """One-hot activations select single dequantised weights: bit-exact in f32, whichever side the
    weights are on and however the activations are stored (a swapped index shows as a wrong weight)."""
    say("dequant_dot layouts, one-hot")
    M, K, N, g = 6, 256, 64, 64
    w = workloads.c2_s4_group(M=M, K=K, N=N, group=g)
    hot = np.zeros((M, K), np.float32)
    ks = [0, 1, 63, 64, 129, 255]
    hot[np.arange(M), ks] = 1.0
    w = dict(w, lhs=dtypes.f32_to_bf16(hot), epilogue="DEFAULT", bias=None)
    s32 = dtypes.bf16_to_f32(w["scales"])
    want = np.stack([dtypes.bf16_to_f32(dtypes.f32_to_bf16(w["weights"][k].astype(np.float32) * s32[k // g])) for k in ks])
    for nk in (False, True):
        for transposed in (False, True):
            for lhs_k_major in (False, True):
                got, kern = run(w, nk=nk, out_dtype="f32", transposed=transposed, lhs_k_major=lhs_k_major)
                assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32)), (nk, transposed, lhs_k_major, kern)


def f8_codes(v, z, divides):
    """convert(clamp(-448, v / z | v * z, 448)) op by op on f32, as the HLO evaluates it."""
    v = np.asarray(v, np.float32)
    t = (v / np.float32(z) if divides else v * np.float32(z)).astype(np.float32)
    return dtypes.f32_to_f8e4m3fn(np.clip(t, -448, 448))


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("divides", [True, False])
@pytest.mark.parametrize("kind,kw", CASES)
def test_f8_result(oracle, kind, kw, nk, divides):
    """An f8e4m3fn result: the codes of the oracle's f32 value scaled, clamped and cast, up to the window
    the dot itself is matched to (the rule of the fp8 dot's f8 result)."""
    say("dequant_dot f8 result %s %s nk=%s divides=%s" % (kind, kw, nk, divides))
    w = make(kind, kw)
    val = reference(oracle, w, True)
    amax = float(np.nanmax(np.abs(val)))
    # the largest value lands at 600: some codes saturate at 448, most use the format's whole range
    z = np.float32(amax / 600.0) if divides else np.float32(600.0 / amax)
    got, kern = run(w, nk=nk, d_scale=z, d_scale_multiplies=not divides)
    assert got.dtype == np.uint8 and got.shape == val.shape
    ref = f8_codes(val, z, divides)
    assert (np.abs(dtypes.f8e4m3fn_to_f32(ref)) == 448).any()
    differ = check_f8_result(got, ref, val, z, divides, floor_for(w), "f8 result %s" % kern)
    assert differ <= max(8, got.size // 8), (differ, got.size)


@pytest.mark.parametrize("divides", [True, False])
def test_f8_result_of_single_weights_bit_exact(oracle, divides):
    """One-hot activations make the dot's value a single dequantised weight, exact in f32: the codes
    must then be exactly convert(clamp(v / z)) with an IEEE quotient (z is chosen so that v * (1/z)
    rounds differently for many v), in every layout, saturating beyond +-448."""
    say("dequant_dot f8 result, one-hot, divides=%s" % divides)
    M, K, N, g = 6, 256, 64, 64
    w = workloads.c2_s4_group(M=M, K=K, N=N, group=g)
    hot = np.zeros((M, K), np.float32)
    ks = [0, 1, 63, 64, 129, 255]
    hot[np.arange(M), ks] = 1.0
    w = dict(w, lhs=dtypes.f32_to_bf16(hot), epilogue="DEFAULT", bias=None)
    s32 = dtypes.bf16_to_f32(w["scales"])
    v = np.stack([dtypes.bf16_to_f32(dtypes.f32_to_bf16(w["weights"][k].astype(np.float32) * s32[k // g])) for k in ks])
    amax = float(np.abs(v).max())
    odd = np.frombuffer(np.uint32(0x3c7fffff).tobytes(), np.float32)[0]   # 0.0156249991: not a power of two
    z = np.float32(odd * amax / 8.0) if divides else np.float32(500.0 / amax)
    want = f8_codes(v, z, divides)
    assert (np.abs(dtypes.f8e4m3fn_to_f32(want)) == 448).any()
    for nk in (False, True):
        for transposed in (False, True):
            for lhs_k_major in (False, True):
                got, kern = run(w, nk=nk, transposed=transposed, lhs_k_major=lhs_k_major, d_scale=z,
                                d_scale_multiplies=not divides)
                assert np.array_equal(got, want), (nk, transposed, lhs_k_major, kern, int((got != want).sum()))


def test_f8_result_special_values(oracle):
    """A NaN stays one through the clamp and +-inf saturates at +-448: a NaN scale in one channel, and
    single products that overflow f32 (one-hot activations of +-3e38 on weights of magnitude >= 1)."""
    say("dequant_dot f8 result, special values")
    M, K, N = 4, 64, 32
    w = workloads.c1_s8_channel(M=M, K=K, N=N)
    hot = np.zeros((M, K), np.float32)
    hot[np.arange(M), [0, 5, 17, 63]] = [1.0, 3e38, -3e38, 1.0]
    sc = np.full(N, 4.0, np.float32)
    sc[5] = np.nan
    wt = w["weights"].copy()
    wt[wt == 0] = 1
    w = dict(w, lhs=dtypes.f32_to_bf16(hot), scales=sc, weights=wt, epilogue="DEFAULT", bias=None)
    v = reference(oracle, w, True)
    assert np.isinf(v[1:3, :5]).all() and np.isnan(v[:, 5]).all()
    z = np.float32(0.25)
    want = f8_codes(v, z, True)
    got, kern = run(w, d_scale=z)
    assert np.array_equal(got, want), (kern, int((got != want).sum()))
    assert (want[:, 5] & 0x7f == 0x7f).all() and (want[1:3, :5] & 0x7f == 0x7e).all()


def test_refusals():
    t = torch.zeros((8, 64), dtype=torch.bfloat16, device="cuda")
    wt = torch.zeros((64, 32), dtype=torch.int8, device="cuda")
    sc = torch.ones((32,), dtype=torch.float32, device="cuda")
    b = torch.zeros((32,), dtype=torch.float32, device="cuda")
    with pytest.raises(Exception, match="DEFAULT epilogue only"):
        ops.dequant_dot(t, wt, sc, b, epilogue="BIAS", result_transposed=True)
    with pytest.raises(Exception, match="lhs_contracting_dim must be 0"):
        ops.dequant_dot(t, wt, sc, lhs_contracting_dim=2)
