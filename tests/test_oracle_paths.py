"""Pins the fused functions of the CPU oracle with what the mathematics fixes:
library routines, one-hot / power-of-two special cases with exact answers, brute
force in float64 on tiny shapes, and order probes.  None of these re-types the
oracle's own formulas.
"""
import numpy as np
import pytest

from xla_amd import dtypes


def bf16(x):
    return dtypes.f32_to_bf16(np.asarray(x, np.float32))


def as_f32(h):
    return dtypes.bf16_to_f32(h)


# ---- tanh / exp against libm --------------------------------------------------

def test_tanh_matches_libm(oracle):
    x = np.concatenate([np.linspace(-25, 25, 200001), np.array([0.0, 1e-5, -3e-4, 4e-4, 7.99, 8.5, 19.9, 20.0, -20.0, 1e30])]).astype(np.float32)
    got = oracle.tanh_f32(x).astype(np.float64)
    want = np.tanh(x.astype(np.float64))
    assert np.max(np.abs(got - want)) < 5e-7       # ~4 f32 ulp; a wrong coefficient is off by >1e-4
    assert np.all(np.abs(got) <= 1.0)
    assert np.array_equal(oracle.tanh_f32(-x), -oracle.tanh_f32(x))   # odd function, exactly
    small = np.array([1e-5, -3.9e-4], np.float32)
    assert np.array_equal(oracle.tanh_f32(small), small)             # |x| < 4e-4 -> x


def test_exp_matches_libm(oracle):
    x = np.linspace(-87, 88, 300001).astype(np.float32)
    got = oracle.exp_f32(x).astype(np.float64)
    want = np.exp(x.astype(np.float64))
    assert np.max(np.abs(got / want - 1.0)) < 2.0 ** -21.5
    assert oracle.exp_f32(np.array([0.0], np.float32))[0] == 1.0
    assert oracle.exp_f32(np.array([-200.0], np.float32))[0] == 0.0   # clamps, then 2^-127 -> 0
    assert np.isinf(oracle.exp_f32(np.array([89.0], np.float32))[0]) or \
        oracle.exp_f32(np.array([89.0], np.float32))[0] > 3e38


def test_fused_and_separate_roundings_are_both_the_reference(oracle):
    """The CPU backend may fuse a multiply into the add it feeds (cpu_aot_loader.cc:49-55), so the
    oracle carries both spellings.  They are different functions (some inputs differ) and both stay
    within a few f32 ulp of each other and of libm; an fma is never less accurate than the pair."""
    x = np.linspace(-9, 9, 400001).astype(np.float32)
    fused_t, fused_e = oracle.tanh_f32(x), oracle.exp_f32(x)
    with oracle.fp_contract(False):
        sep_t, sep_e = oracle.tanh_f32(x), oracle.exp_f32(x)
    assert oracle.lib().xo_get_fp_contract() == 1
    assert np.any(fused_t != sep_t) and np.any(fused_e != sep_e)
    assert np.max(np.abs(fused_t.astype(np.float64) - sep_t)) <= 4 * 2.0 ** -23
    assert np.max(np.abs(fused_e.astype(np.float64) / sep_e - 1)) <= 4 * 2.0 ** -23
    want_t, want_e = np.tanh(x.astype(np.float64)), np.exp(x.astype(np.float64))
    assert np.mean(np.abs(fused_t - want_t)) <= np.mean(np.abs(sep_t - want_t)) * 1.02
    assert np.mean(np.abs(fused_e / want_e - 1)) <= np.mean(np.abs(sep_e / want_e - 1)) * 1.02
    # tanh.cc:51-59 picks the clamp "in a way that the tanh approximation on that input is exactly
    # 1.0" for the with_fma constant it passes for f32 (tanh.cc:187): true of the fused spelling
    # only -- the separate roundings land 3 ulp short, which is what pins mul_add's operand order
    clamp = np.array([7.99881172180175781, 8.5, 12.0, -7.99881172180175781, -19.0], np.float32)
    assert np.array_equal(oracle.tanh_f32(clamp), np.sign(clamp))
    with oracle.fp_contract(False):
        assert np.all(np.abs(oracle.tanh_f32(clamp)) < 1.0)


# ---- epilogue -----------------------------------------------------------------

def _gelu64(x):
    return 0.5 * x * (1 + np.tanh(np.sqrt(2 / np.pi) * (x + 0.044715 * x ** 3)))


def _silu64(x):
    return x / (1 + np.exp(-x))


@pytest.mark.parametrize("epi,fn", [("gelu_tanh", _gelu64), ("silu", _silu64),
                                    ("relu", lambda v: np.maximum(v, 0)), ("none", lambda v: v)])
def test_epilogue_f32_close_to_float64(oracle, epi, fn):
    L = oracle.lib()
    xs = np.linspace(-12, 12, 4001).astype(np.float32)
    bias = np.float32(0.375)
    for has_bias in (0, 1):
        got = np.array([L.xo_epilogue_one(float(v), 0, 0, has_bias, float(bias), oracle.EPILOGUES[epi])
                        for v in xs], np.uint16)
        want = fn(xs.astype(np.float64) + (float(bias) if has_bias else 0.0))
        # single final rounding: within one bf16 step of the float64 value, plus the f32
        # cancellation noise of x*(1+tanh) / x*sigmoid in the far negative tail
        err = np.abs(as_f32(got).astype(np.float64) - want)
        ulp = np.maximum(np.abs(want), 2.0 ** -126) * 2.0 ** -8
        assert np.all(err <= ulp + 2e-6 * np.maximum(1.0, np.abs(xs))), epi


def test_epilogue_bf16_rounds_every_op(oracle):
    L = oracle.lib()
    # bf16-typed dot: the accumulator 1 + 2^-9 is rounded to 1.0 before the bias add, and
    # 1 + 2^-9 + 2^-12 rounds to 1.0; with f32 ops the single final rounding sees
    # 1 + 2^-8 + 2^-12 and goes up to 1.0078125.
    acc, b = 1.0 + 2.0 ** -9, 2.0 ** -9 + 2.0 ** -12
    assert L.xo_epilogue_one(acc, 1, 1, 1, b, 0) == 0x3F80
    assert L.xo_epilogue_one(acc, 0, 0, 1, b, 0) == 0x3F81
    # bias itself is rounded to bf16 first when the add is bf16-typed
    assert L.xo_epilogue_one(0.0, 1, 1, 1, 1.0 + 2.0 ** -9, 0) == 0x3F80


# ---- dequant dot ----------------------------------------------------------------

def _dot_case(rng, B, M, K, N, group, w_bits):
    a = bf16(rng.standard_normal((B, M, K)))
    lo, hi = (-127, 128) if w_bits == 8 else (-8, 8)
    w = rng.integers(lo, hi, size=(B, K, N)).astype(np.int8)
    G = K // group
    return a, w, G


@pytest.mark.parametrize("w_bits", [8, 4])
def test_dequant_dot_one_hot_is_exact(oracle, w_bits):
    """One-hot activations select single dequantised weights: out = bf16(round_mul(w*s))."""
    rng = np.random.default_rng(11)
    B, K, N, group = 2, 64, 48, 16
    _, w, G = _dot_case(rng, B, K, K, N, group, w_bits)
    a = np.zeros((B, K, K), np.float32)
    a[:, np.arange(K), np.arange(K)] = 1.0
    s32 = rng.uniform(1e-3, 2e-2, size=(B, G, N)).astype(np.float32)
    wp = w if w_bits == 8 else dtypes.pack_s4(w)
    for scale_ty, mul_ty in (("f32", "f32"), ("bf16", "bf16"), ("bf16", "f32"), ("f32", "bf16")):
        s = bf16(s32) if scale_ty == "bf16" else s32
        out = oracle.dequant_dot(bf16(a), wp, w_bits, s, scale_ty, mul_ty, group=group)
        sv = as_f32(s) if scale_ty == "bf16" else s
        if mul_ty == "bf16":
            sv = as_f32(bf16(sv))
        prod = w.astype(np.float64) * np.repeat(sv, group, axis=1).astype(np.float64)
        prod32 = prod.astype(np.float32)                    # float64 product is exact; one rounding
        if mul_ty == "bf16":
            prod32 = as_f32(bf16(prod32))
        assert np.array_equal(out, bf16(prod32)), (scale_ty, mul_ty)


def test_dequant_dot_brute_force_float64(oracle):
    rng = np.random.default_rng(5)
    B, M, K, N, group = 2, 5, 96, 40, 32       # all different: a transposed operand cannot pass
    a, w, G = _dot_case(rng, B, M, K, N, group, 4)
    s = bf16(rng.uniform(1e-3, 2e-2, size=(B, G, N)))
    bias = bf16(rng.standard_normal(N))
    out = oracle.dequant_dot(a, dtypes.pack_s4(w), 4, s, "bf16", "bf16", bias=bias, group=group,
                             epilogue="silu")
    wd = as_f32(bf16((w.astype(np.float64) * np.repeat(as_f32(s), group, axis=1)).astype(np.float32)))
    ref = np.einsum("bmk,bkn->bmn", as_f32(a).astype(np.float64), wd.astype(np.float64))
    ref = _silu64(ref + as_f32(bias).astype(np.float64))
    err = np.abs(as_f32(out).astype(np.float64) - ref)
    assert np.all(err <= np.abs(ref) * 2.0 ** -8 + 1e-5)


def test_dequant_dot_integer_data_is_exact(oracle):
    """Small integers: every partial sum is exact in f32, so the result is order-free."""
    rng = np.random.default_rng(2)
    B, M, K, N = 1, 7, 128, 24
    a = rng.integers(-4, 5, size=(B, M, K)).astype(np.float32)
    w = rng.integers(-127, 128, size=(B, K, N)).astype(np.int8)
    s = np.full((B, 1, N), 0.5, np.float32)
    out = oracle.dequant_dot(bf16(a), w, 8, s, "f32", "f32")
    ref = np.einsum("bmk,bkn->bmn", a.astype(np.int64), w.astype(np.int64)) * 0.5
    assert np.array_equal(out, bf16(ref.astype(np.float32)))


def test_dot_adds_in_increasing_k(oracle):
    """Documents the (unpinned) order choice: 2^24 + 1 + 1 ... stays 2^24 left to right."""
    K = 64
    a = np.ones((1, K), np.float32)
    w = np.ones((K, 1), np.int8)
    a[0, 0] = 2.0 ** 12
    s = np.ones((K, 1), np.float32)          # group 1: a scale per row
    s[0, 0] = 2.0 ** 12
    out = oracle.dequant_dot(bf16(a), w, 8, s, "f32", "f32", group=1)
    assert as_f32(out)[0, 0] == 2.0 ** 24


# ---- fp8 scaled dot -------------------------------------------------------------

@pytest.mark.parametrize("b_is_nk", [False, True])
def test_fp8_dot_brute_force(oracle, b_is_nk):
    rng = np.random.default_rng(9)
    M, K, N = 6, 80, 10
    a8 = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((M, K)) * 64, -448, 448))
    b8 = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((K, N)) * 64, -448, 448))
    bias = bf16(rng.standard_normal(N))
    bmat = np.ascontiguousarray(b8.T) if b_is_nk else b8
    out = oracle.fp8_scaled_dot(a8, bmat, 1 / 64, 1 / 64, b_is_nk=b_is_nk, bias=bias,
                                epilogue="gelu_tanh")
    ref = (dtypes.f8e4m3fn_to_f32(a8).astype(np.float64) / 64) @ (dtypes.f8e4m3fn_to_f32(b8).astype(np.float64) / 64)
    ref = _gelu64(ref + as_f32(bias).astype(np.float64))
    err = np.abs(as_f32(out).astype(np.float64) - ref)
    assert np.all(err <= np.abs(ref) * 2.0 ** -8 + 1e-5)


def test_fp8_dot_one_hot(oracle):
    K, N = 32, 256
    a = np.zeros((K, K), np.float32)
    a[np.arange(K), np.arange(K)] = 1.0
    a8 = dtypes.f32_to_f8e4m3fn(a)
    b8 = np.tile(np.arange(256, dtype=np.uint8), (K, 1))
    b8[(b8 & 0x7F) == 0x7F] = 0
    out = oracle.fp8_scaled_dot(a8, b8, 1.0, 0.25)
    want = bf16(dtypes.f8e4m3fn_to_f32(b8) * np.float32(0.25))
    assert np.array_equal(as_f32(out), as_f32(want))       # value compare: -0 sums to +0


def test_fp8_dot_vector_scales(oracle):
    """Per-row a_scale and per-channel b_scale: a vector of equal values is the per-tensor
    case bit for bit; power-of-two vectors scale row m / column n exactly (so each output is
    the unscaled sum times sa[m]*sb[n] before the one rounding); general vectors against f64;
    and a transposed index (scales along the wrong axis) must change the result."""
    rng = np.random.default_rng(21)
    M, K, N = 7, 48, 9
    a8 = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((M, K)) * 32, -448, 448))
    b8 = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((K, N)) * 32, -448, 448))
    for nk in (False, True):
        bm = np.ascontiguousarray(b8.T) if nk else b8
        same = oracle.fp8_scaled_dot(a8, bm, np.full(M, 0.3, np.float32), np.full(N, 0.7, np.float32), b_is_nk=nk)
        assert np.array_equal(same, oracle.fp8_scaled_dot(a8, bm, np.float32(0.3), np.float32(0.7), b_is_nk=nk))
        sa = (2.0 ** rng.integers(-6, 3, M)).astype(np.float32)
        sb = (2.0 ** rng.integers(-6, 3, N)).astype(np.float32)
        got = as_f32(oracle.fp8_scaled_dot(a8, bm, sa, sb, b_is_nk=nk))
        unit = dtypes.f8e4m3fn_to_f32(a8).astype(np.float64) @ dtypes.f8e4m3fn_to_f32(b8).astype(np.float64)
        # |sum| < 2^24 * 2^-6 granularity: the f32 sums of these f8 products are exact
        want = as_f32(bf16((unit * sa[:, None] * sb[None, :]).astype(np.float32)))
        assert np.array_equal(got, want)
        sa = rng.uniform(0.01, 2.0, M).astype(np.float32)
        sb = rng.uniform(0.01, 2.0, N).astype(np.float32)
        got = as_f32(oracle.fp8_scaled_dot(a8, bm, sa, sb, b_is_nk=nk)).astype(np.float64)
        ref = unit * sa[:, None].astype(np.float64) * sb[None, :]
        assert np.all(np.abs(got - ref) <= np.abs(ref) * 2.0 ** -8 + 1e-6)
        if not nk:
            wrong = unit * sa[::-1, None].astype(np.float64) * sb[None, :]
            assert not np.all(np.abs(got - wrong) <= np.abs(wrong) * 2.0 ** -8 + 1e-6)


def test_fp8_dot_f8_result(oracle):
    """f8 result = convert(clamp(v / z)): v must be the bf16-result path's value before its
    rounding, the codes the numpy restatement of divide / clamp / cast on those v (the cast itself
    is pinned by the reference's vectors), multiply is not divide, and clamping saturates."""
    rng = np.random.default_rng(33)
    M, K, N = 9, 64, 12
    a8 = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((M, K)) * 32, -448, 448))
    b8 = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((K, N)) * 32, -448, 448))
    bias = bf16(rng.standard_normal(N))
    kw = dict(bias=bias, epilogue="gelu_tanh")
    z = np.float32(0.0137)
    codes, v = oracle.fp8_scaled_dot(a8, b8, 1 / 64, 1 / 64, d_scale=z, **kw)
    assert np.array_equal(bf16(v), oracle.fp8_scaled_dot(a8, b8, 1 / 64, 1 / 64, **kw))
    want = dtypes.f32_to_f8e4m3fn(np.clip((v / z).astype(np.float32), -448, 448))
    assert np.array_equal(codes, want)
    codes_m, v_m = oracle.fp8_scaled_dot(a8, b8, 1 / 64, 1 / 64, d_scale=z, d_scale_divides=False, **kw)
    assert np.array_equal(v_m, v)
    assert np.array_equal(codes_m, dtypes.f32_to_f8e4m3fn(np.clip((v * z).astype(np.float32), -448, 448)))
    assert not np.array_equal(codes_m, codes)
    sat, v2 = oracle.fp8_scaled_dot(a8, b8, 1.0, 1.0, d_scale=np.float32(1e-3))   # |v| / 1e-3 >> 448
    assert set(np.unique(sat[np.abs(v2) > 1.0])) <= {0x7E, 0xFE}                  # +-448, never NaN


def test_block_scaled_dot(oracle):
    """MXFP8: against f64 on the dequantised operands; all scales 1.0 is the plain dot of the two
    code matrices; doubling one block's scale adds exactly that block's contribution once more;
    scales along the wrong axis (transposed scale matrix semantics) must change the result."""
    rng = np.random.default_rng(44)
    M, K, N = 6, 128, 9
    a8 = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((M, K)) * 8, -448, 448).astype(np.float32))
    b8 = dtypes.f32_to_f8e4m3fn(np.clip(rng.standard_normal((N, K)) * 8, -448, 448).astype(np.float32))
    sa = rng.integers(120, 134, (M, K // 32)).astype(np.uint8)
    sb = rng.integers(120, 134, (N, K // 32)).astype(np.uint8)
    af, bf = dtypes.f8e4m3fn_to_f32(a8).astype(np.float64), dtypes.f8e4m3fn_to_f32(b8).astype(np.float64)
    ad = af * np.repeat(2.0 ** (sa.astype(np.float64) - 127), 32, axis=1)
    bd = bf * np.repeat(2.0 ** (sb.astype(np.float64) - 127), 32, axis=1)
    ref = ad @ bd.T
    got = as_f32(oracle.block_scaled_dot(a8, b8, sa, sb)).astype(np.float64)
    assert np.all(np.abs(got - ref) <= np.abs(ref) * 2.0 ** -8 + 1e-6)
    one_a, one_b = np.full_like(sa, 127), np.full_like(sb, 127)
    plain = oracle.block_scaled_dot(a8, b8, one_a, one_b)
    assert np.array_equal(plain, oracle.fp8_scaled_dot(a8, b8, 1.0, 1.0, b_is_nk=True))
    # small integers: every sum is exact, so doubling block 2 of row 3 adds its part exactly once more
    ai = dtypes.f32_to_f8e4m3fn(rng.integers(-3, 4, (M, K)).astype(np.float32))
    bi = dtypes.f32_to_f8e4m3fn(rng.integers(-3, 4, (N, K)).astype(np.float32))
    base = as_f32(oracle.block_scaled_dot(ai, bi, one_a, one_b))
    bumped = one_a.copy()
    bumped[3, 2] = 128
    part = dtypes.f8e4m3fn_to_f32(ai)[3, 64:96] @ dtypes.f8e4m3fn_to_f32(bi)[:, 64:96].T
    want = base.copy()
    want[3] += part
    assert np.array_equal(as_f32(oracle.block_scaled_dot(ai, bi, bumped, one_b)), want)
    wrong = (af * np.repeat(2.0 ** (sa[::-1].astype(np.float64) - 127), 32, axis=1)) @ bd.T
    assert not np.all(np.abs(got - wrong) <= np.abs(wrong) * 2.0 ** -8 + 1e-6)


# ---- RMSNorm + quantize -----------------------------------------------------------

def test_tree32_sum_order(oracle):
    v = np.arange(1, 1025, dtype=np.float32)
    assert oracle.tree32_sum(v) == 1024 * 1025 / 2              # exact: order-free
    # inside a window additions run left to right: 2^24 swallows 31 ones one at a time
    w = np.ones(64, np.float32)
    w[0] = 2.0 ** 24
    assert oracle.tree32_sum(w) == 2.0 ** 24 + 32.0             # second window sums to 32 first
    w2 = np.ones(64, np.float32)
    w2[31] = 2.0 ** 24
    assert oracle.tree32_sum(w2) == 2.0 ** 24 + 32.0 + 32.0     # 31 ones add up before the big one


def test_quantize_power_of_two_rows_closed_form(oracle):
    """x = +-2^k, eps = 0: x/sqrt(mean x^2) = +-1 exactly, so y = +-gamma, amax = max gamma."""
    rng = np.random.default_rng(4)
    rows, cols = 6, 160
    sign = rng.choice([-1.0, 1.0], size=(rows, cols))
    k = rng.integers(-3, 4, size=(rows, 1))
    x = (sign * 2.0 ** k).astype(np.float32)
    gamma = bf16(rng.uniform(0.5, 1.5, cols))
    q, s = oracle.rmsnorm_quantize_fp8(bf16(x), gamma, eps=0.0)
    g = as_f32(gamma)
    amax = g.max()
    assert np.all(s == np.float32(amax) / np.float32(448))
    want = dtypes.f32_to_f8e4m3fn(((sign * g).astype(np.float32) / s[:, None]).astype(np.float32))
    assert np.array_equal(q, want)
    assert np.all((q & 0x7F).max(axis=1) == 0x7E)                # amax maps to +-448


def test_quantize_invariants_and_float64(oracle):
    rng = np.random.default_rng(8)
    rows, cols = 16, 1000                                        # ragged: not a multiple of 32
    x = rng.standard_normal((rows, cols))
    x[rng.random((rows, cols)) < 0.01] *= 50
    xb, gamma = bf16(x), bf16(rng.uniform(0.5, 1.5, cols))
    q, s = oracle.rmsnorm_quantize_fp8(xb, gamma, eps=1e-6)
    assert not np.any((q & 0x7F) == 0x7F)
    assert np.all((q & 0x7F).max(axis=1) == 0x7E)
    xf = as_f32(xb).astype(np.float64)
    y = xf / np.sqrt((xf ** 2).mean(axis=1, keepdims=True) + 1e-6) * as_f32(gamma).astype(np.float64)
    amax = np.abs(y).max(axis=1)
    assert np.allclose(s, amax / 448, rtol=2.0 ** -7)             # y was rounded to bf16 first
    deq = dtypes.f8e4m3fn_to_f32(q).astype(np.float64) * s[:, None]
    # e4m3 has 3 mantissa bits: relative step 2^-3, half of it after rounding, plus bf16 noise
    assert np.all(np.abs(deq - y) <= np.abs(y) * (2.0 ** -4 + 2.0 ** -7) + amax[:, None] * 2.0 ** -10)


def test_quantize_zero_row_gives_nan_codes(oracle):
    x = np.zeros((1, 64), np.float32)
    q, s = oracle.rmsnorm_quantize_fp8(bf16(x), bf16(np.ones(64)), eps=1e-6)
    assert s[0] == 0.0 and np.all((q & 0x7F) == 0x7F)


# ---- u4 weights with zero points ------------------------------------------------

def _pack4(v):
    v = np.ascontiguousarray(v, np.uint8).reshape(-1)
    return (v[0::2] | (v[1::2] << 4)).astype(np.uint8)


def test_u4_zero_point_dequantisation_one_hot_and_brute_force(oracle):
    """(w - z) * s for unsigned 4-bit weights: one-hot activations read single dequantised weights
    back (nibble order of weights AND zero points, the group a row belongs to, unsignedness, the
    single bf16 rounding); a small dot against float64; and z = 8 turns u4 into s4 exactly."""
    rng = np.random.default_rng(21)
    K, N, g = 64, 24, 16
    w = rng.integers(0, 16, (K, N)).astype(np.uint8)
    w[:16, 0] = np.arange(16)                      # every code in one column
    z = rng.integers(0, 16, (K // g, N)).astype(np.uint8)
    s32 = (rng.integers(128, 256, (K // g, N)) / 128.0 * np.exp2(rng.integers(-8, 2, (K // g, N)))).astype(np.float32)
    s = dtypes.f32_to_bf16(s32)                    # exactly representable
    eye = dtypes.f32_to_bf16(np.eye(K, dtype=np.float32))
    got = oracle.dequant_dot(eye, _pack4(w), 4, s, "bf16", "bf16", group=g, unsigned=True, zero_points=_pack4(z))
    diff = w.astype(np.float32) - np.repeat(z, g, axis=0).astype(np.float32)
    want = dtypes.f32_to_bf16((diff * np.repeat(dtypes.bf16_to_f32(s), g, axis=0)).astype(np.float32))
    assert np.array_equal(got, want)
    # f32-typed multiply: no rounding of the product before the dot; one-hot rows still read it back,
    # rounded once by the final convert
    got32 = oracle.dequant_dot(eye, _pack4(w), 4, s32, "f32", "f32", group=g, unsigned=True, zero_points=_pack4(z))
    assert np.array_equal(got32, dtypes.f32_to_bf16((diff * np.repeat(s32, g, axis=0)).astype(np.float32)))
    # without zero points the unsigned code itself is the weight
    got0 = oracle.dequant_dot(eye, _pack4(w), 4, s, "bf16", "bf16", group=g, unsigned=True)
    assert np.array_equal(got0, dtypes.f32_to_bf16((w * np.repeat(dtypes.bf16_to_f32(s), g, axis=0)).astype(np.float32)))
    # z = 8 everywhere is the signed reading of the same bits with the sign bit flipped
    a = dtypes.f32_to_bf16(rng.standard_normal((5, K)).astype(np.float32))
    z8 = np.full((K // g, N), 8, np.uint8)
    as_u4 = oracle.dequant_dot(a, _pack4(w), 4, s, "bf16", "bf16", group=g, unsigned=True, zero_points=_pack4(z8))
    as_s4 = oracle.dequant_dot(a, _pack4(w ^ 8), 4, s, "bf16", "bf16", group=g)
    assert np.array_equal(as_u4, as_s4)
    # a dot against float64 on the dequantised weights
    got = dtypes.bf16_to_f32(oracle.dequant_dot(a, _pack4(w), 4, s, "bf16", "bf16", group=g, unsigned=True,
                                                zero_points=_pack4(z))).astype(np.float64)
    ref = dtypes.bf16_to_f32(a).astype(np.float64) @ dtypes.bf16_to_f32(want).astype(np.float64)
    assert np.max(np.abs(got - ref) / np.maximum(np.abs(ref), 1e-2)) < 2.0 ** -7


# ---- ragged dot -------------------------------------------------------------------

def test_ragged_dot_composition_is_pinned(oracle):
    """The ragged dot is one dense dot per group on that group's rows (ragged_dot_rewriter.cc:110-210).
    Equal group sizes must give the batched dot reshaped; every row must equal a one-row dot with
    its group's weights; rows past the last group are epilogue(0); float64 agrees."""
    from xla_amd import workloads
    G, K, N = 4, 64, 24
    w = workloads.ragged_s8_experts(M=12, K=K, N=N, groups=G, sizes=[3, 3, 3, 3])
    got = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", w["group_sizes"],
                                    bias=w["bias"])
    batched = oracle.dequant_dot(w["lhs"].reshape(G, 3, K), w["weights"], 8, w["scales"], "f32", "f32", bias=w["bias"])
    assert np.array_equal(got, batched.reshape(12, N))
    # uneven, with an empty group and unowned rows at the end
    sizes = [5, 0, 2, 1]
    got = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", sizes, bias=w["bias"])
    owner = [0] * 5 + [2] * 2 + [3]
    for m, g in enumerate(owner):
        one = oracle.dequant_dot(w["lhs"][m:m + 1], w["weights"][g], 8, w["scales"][g], "f32", "f32", bias=w["bias"])
        assert np.array_equal(got[m], one[0]), m
    assert np.array_equal(got[8:], np.broadcast_to(w["bias"], (4, N)))     # a dot of nothing, plus the bias
    a64 = dtypes.bf16_to_f32(w["lhs"]).astype(np.float64)
    for m, g in enumerate(owner):
        ref = a64[m] @ (w["weights"][g].astype(np.float64) * w["scales"][g].astype(np.float64)) + dtypes.bf16_to_f32(w["bias"])
        assert np.max(np.abs(dtypes.bf16_to_f32(got[m]) - ref) / np.maximum(np.abs(ref), 1e-2)) < 2.0 ** -7
    # sizes that overrun M are cut at M
    over = oracle.ragged_dequant_dot(w["lhs"], w["weights"], 8, w["scales"], "f32", "f32", [10, 10, 0, 0], bias=w["bias"])
    assert np.array_equal(over[:10], oracle.dequant_dot(w["lhs"][:10], w["weights"][0], 8, w["scales"][0], "f32", "f32", bias=w["bias"]))
    assert np.array_equal(over[10:], oracle.dequant_dot(w["lhs"][10:], w["weights"][1], 8, w["scales"][1], "f32", "f32", bias=w["bias"]))


# ---- f32 result of the dequantize-dot (the dot's own value is the module's result) ----------------

def test_dequant_dot_f32_result_is_the_value_before_the_final_convert(oracle):
    """fusion_emitter_int4_device_test.cc:101,205,320,508 end in an f32 dot.  The f32 result is pinned
    three ways: rounding it gives the bf16 result bit for bit (every epilogue); one-hot activations
    read single dequantised weights back exactly; and float64 on a small dot bounds it to f32
    summation noise -- with the rows of the weights reversed it must not."""
    rng = np.random.default_rng(5)
    M, K, N, g = 5, 256, 48, 64
    a = dtypes.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    w = rng.integers(-8, 8, size=(K, N)).astype(np.int8)
    sc = dtypes.f32_to_bf16(rng.uniform(1e-3, 2e-2, size=(K // g, N)).astype(np.float32))
    bias = dtypes.f32_to_bf16(rng.standard_normal((N,)).astype(np.float32))
    wp = dtypes.pack_s4(w)
    for epi in ("none", "relu", "gelu_tanh", "silu"):
        v32 = oracle.dequant_dot(a, wp, 4, sc, "bf16", "bf16", bias=bias, group=g, epilogue=epi, f32_result=True)
        v16 = oracle.dequant_dot(a, wp, 4, sc, "bf16", "bf16", bias=bias, group=g, epilogue=epi)
        assert v32.dtype == np.float32 and np.array_equal(dtypes.f32_to_bf16(v32), v16), epi
    # one-hot rows: out[m, n] = bf16(w[k_m, n] * s) exactly, as an f32
    hot = np.zeros((M, K), np.float32)
    ks = [0, 63, 64, 200, 255]
    hot[np.arange(M), ks] = 1.0
    got = oracle.dequant_dot(dtypes.f32_to_bf16(hot), wp, 4, sc, "bf16", "bf16", group=g, f32_result=True)
    s32 = dtypes.bf16_to_f32(sc)
    want = np.stack([dtypes.bf16_to_f32(dtypes.f32_to_bf16(w[k].astype(np.float32) * s32[k // g])) for k in ks])
    assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))
    # float64 on the rounded weights
    wd = dtypes.bf16_to_f32(dtypes.f32_to_bf16(w.astype(np.float32) * np.repeat(s32, g, axis=0))).astype(np.float64)
    a64 = dtypes.bf16_to_f32(a).astype(np.float64)
    ref = a64 @ wd
    v32 = oracle.dequant_dot(a, wp, 4, sc, "bf16", "bf16", group=g, f32_result=True)
    tol = 2.0 ** -22 * (np.abs(a64) @ np.abs(wd))
    assert np.all(np.abs(v32 - ref) <= tol)
    assert not np.all(np.abs(v32 - a64 @ wd[::-1]) <= tol)
