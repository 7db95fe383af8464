"""The weight-streaming kernels of xla_amd.fp8_scaled_dot (up to 64 rows of a per launch; rhs [K,N] or [N,K]) against
the CPU oracle, through the FFI handler: every token-tile count, ragged K and N, K-slices with and without
scratch, vector scales, f8 results with amax, batches, one-hot exactness and special values."""
import numpy as np
import pytest
import torch

from tests.gpu_util import check_dot, check_f8_result, dev_bf16, dev_f32, dev_u8, host_bf16
from tests.test_gpu_fp8_dot import EPI, floor_for, reference, say
from xla_amd import dtypes, ffi, ops, workloads

pytestmark = pytest.mark.gpu


def run(w, nk=False, slices=0, scratch="auto", force=3, batch=None, **kw):
    """force=3: the streaming kernels or an error; slices: K-slices (0: the launcher's choice)."""
    b = w["b"]
    if nk:
        b = np.ascontiguousarray(np.swapaxes(b, -1, -2))
    a, b = dev_u8(w["a"]), dev_u8(b)
    sa = dev_f32(np.array(w["a_scale"], np.float32))
    sb = dev_f32(np.array(w["b_scale"], np.float32))
    bias = dev_bf16(w["bias"]) if w.get("bias") is not None else None
    ffi.set_option("fp8_dot_kernel", force)
    ffi.set_option("fp8_decode_slices", slices)
    try:
        if scratch == "auto" and slices:   # the sizer is asked under the same option
            n = ffi.library().xla_amd_fp8_scaled_dot_workspace_bytes(w["a"].shape[-2], w["a"].shape[-1], w["b"].shape[-1], 1 if nk else 0)
            scratch = torch.empty(max(n * (batch or 1), 16), dtype=torch.uint8, device="cuda")
        out = ops.fp8_scaled_dot(a, b, sa, sb, bias, rhs_contracting_dim=1 if nk else 0, epilogue=w["epilogue"],
                                 scratch=scratch, **kw)
        torch.cuda.synchronize()
    finally:
        ffi.set_option("fp8_dot_kernel", 0)
        ffi.set_option("fp8_decode_slices", 0)
    return out, ffi.last_kernel()


def tile_name(nk, M):
    return "fp8_dot_decode_%s_m%d" % ("nk" if nk else "kn", 16 * ((M + 15) // 16))


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("M", [1, 8, 16, 17, 32, 33, 48, 64])
@pytest.mark.parametrize("K,N", [(1024, 256), (528, 136), (4096, 72)])
def test_every_tile_count_ragged_k_and_n(oracle, M, K, N, nk):
    """528 is no multiple of a step (32 rows, or 128 of the [N,K] kernel), 136 and 72 none of a strip."""
    if nk and M > 48:
        pytest.skip("the [N,K] streaming kernel takes up to 48 rows of a")
    say("fp8 streaming M=%d K=%d N=%d nk=%s" % (M, K, N, nk))
    w = workloads.c3_fp8(M, K, N)
    out, kern = run(w, nk=nk)
    assert kern == tile_name(nk, M), kern
    n_floor = check_dot(host_bf16(out), reference(oracle, w), floor_for(w), kern)
    assert n_floor <= max(4, out.numel() // 50)


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("slices", [2, 4, 8])
def test_k_slices(oracle, slices, nk):
    """K split over workgroups: sums through the scratch and the second kernel; without the scratch one
    slice.  The last slices of K = 2176 are short or empty."""
    say("fp8 streaming, %d K-slices, nk=%s" % (slices, nk))
    w = workloads.c3_fp8(24, 2176, 264)
    ref = reference(oracle, w)
    out, kern = run(w, nk=nk, slices=slices)
    assert kern == tile_name(nk, 24)
    check_dot(host_bf16(out), ref, floor_for(w), "%s, %d slices" % (kern, slices))
    out1, _ = run(w, nk=nk, slices=slices, scratch=None)
    check_dot(host_bf16(out1), ref, floor_for(w), "%s, no scratch" % kern)
    # two runs give the same bits: the slices are added in slice order
    out2, _ = run(w, nk=nk, slices=slices)
    assert torch.equal(out, out2)


@pytest.mark.parametrize("mode", ["kn", "nk", "mx"])
@pytest.mark.parametrize("cols", [2, 3])
def test_workgroups_that_walk_several_strips(oracle, mode, cols):
    """More strips than CUs: a workgroup takes `cols` strips in turn (forced here on five strips, the
    last one short and, with three per workgroup, the second workgroup's walk ending early); with
    K-slices beside it."""
    from tests.test_gpu_fp8_dot import mx_case, mx_floor
    say("fp8 streaming, %d strips per workgroup, %s" % (cols, mode))
    M, K, N = 24, 1024, 584
    ffi.set_option("fp8_decode_cols", cols)
    try:
        for slices in (0, 2):
            if mode == "mx":
                a, b, sa, sb = mx_case(M, K, N, 9)
                got, kern = run_mx(a, b, sa, sb, slices=slices)
                assert kern == "fp8_dot_decode_mx_m32:walk", kern
                check_dot(got, oracle.block_scaled_dot(a, b, sa, sb), mx_floor(a, b, sa, sb, False), kern)
            else:
                w = workloads.c3_fp8(M, K, N)
                out, kern = run(w, nk=mode == "nk", slices=slices)
                assert kern == tile_name(mode == "nk", M) + ":walk", kern
                check_dot(host_bf16(out), reference(oracle, w), floor_for(w), kern)
    finally:
        ffi.set_option("fp8_decode_cols", 0)


def test_the_launcher_splits_k_for_narrow_results(oracle):
    say("fp8 streaming, the launcher's own slices")
    M, K, N = 16, 4096, 512
    assert ffi.library().xla_amd_fp8_scaled_dot_workspace_bytes(M, K, N, 0) >= 2 * M * N * 4
    w = workloads.c3_fp8(M, K, N)
    out, kern = run(w, force=0)
    assert kern == tile_name(False, M)
    check_dot(host_bf16(out), reference(oracle, w), floor_for(w), kern)


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("which", ["a", "b", "ab"])
@pytest.mark.parametrize("slices", [0, 2])
def test_vector_scales(oracle, which, nk, slices):
    say("fp8 streaming, vector scales %s, nk=%s, slices=%d" % (which, nk, slices))
    M, K, N = 20, 1024, 200
    w = workloads.c3_fp8(M, K, N)
    rng = np.random.default_rng(5)
    if "a" in which:
        w["a_scale"] = rng.uniform(0.004, 0.04, M).astype(np.float32)
    if "b" in which:
        w["b_scale"] = rng.uniform(0.004, 0.04, N).astype(np.float32)
    out, kern = run(w, nk=nk, slices=slices)
    assert kern == tile_name(nk, M)
    check_dot(host_bf16(out), reference(oracle, w), floor_for(w), kern)


@pytest.mark.parametrize("epilogue,dot_ty,ep_ty", [("DEFAULT", "f32", "f32"), ("BIAS", "f32", "f32"), ("RELU", "f32", "f32"),
                                                  ("BIAS_SILU", "f32", "f32"), ("GELU", "f32", "bf16"), ("BIAS_RELU", "bf16", "bf16")])
def test_epilogues_and_rounding_points(oracle, epilogue, dot_ty, ep_ty):
    say("fp8 streaming, %s dot %s ops %s" % (epilogue, dot_ty, ep_ty))
    w = dict(workloads.c3_fp8(40, 512, 128), epilogue=epilogue)
    if "BIAS" not in epilogue:
        w["bias"] = None
    types = dict(dot_type=dot_ty, epilogue_type=ep_ty)
    out, kern = run(w, **types)
    ref = reference(oracle, w, **types)
    fl = floor_for(w)
    if "bf16" in (dot_ty, ep_ty):   # a difference far below one ulp can flip a bf16 rounding on the way
        fl = fl * 12 + np.abs(dtypes.bf16_to_f32(ref)) * 6 * 2.0 ** -8
    check_dot(host_bf16(out), ref, fl, kern)


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("divides", [True, False])
@pytest.mark.parametrize("slices", [0, 4])
def test_f8_result_with_amax(oracle, divides, nk, slices):
    say("fp8 streaming, f8 result, divides=%s nk=%s slices=%d" % (divides, nk, slices))
    M, K, N = 32, 1024, 136
    w = workloads.c3_fp8(M, K, N)
    s = np.float32(1 / 64)
    w["a_scale"] = w["b_scale"] = s
    z = np.float32(0.0171 if divides else 1 / 0.0171)
    (out, amax), kern = run(w, nk=nk, slices=slices, d_scale=dev_f32(np.array(z, np.float32)), d_scale_multiplies=not divides,
                            amax=True)
    assert kern == tile_name(nk, M)
    ref, val = oracle.fp8_scaled_dot(w["a"], w["b"], s, s, bias=w["bias"], epilogue=EPI[w["epilogue"]], d_scale=z,
                                     d_scale_divides=divides)
    check_f8_result(out.cpu().numpy(), ref, val, z, divides, floor_for(w), kern)
    want = float(np.max(np.abs(val)))
    got = float(amax.cpu())
    assert abs(got - want) <= 2.0 ** -7 * want + float(np.max(floor_for(w))), (got, want)


@pytest.mark.parametrize("nk", [False, True])
def test_batched(oracle, nk):
    say("fp8 streaming, batched, nk=%s" % nk)
    B, M, K, N = 3, 12, 640, 264
    ws = [workloads.c3_fp8(M, K, N) for _ in range(B)]
    for i, x in enumerate(ws):   # different data per batch
        x["a"] = np.roll(x["a"], 3 * i, axis=0)
        x["b"] = np.roll(x["b"], 5 * i, axis=1)
    w = dict(ws[0], a=np.stack([x["a"] for x in ws]), b=np.stack([x["b"] for x in ws]))
    for slices in (0, 2):
        out, kern = run(w, nk=nk, slices=slices, batch=B)
        assert kern == tile_name(nk, M)
        got = host_bf16(out)
        for i in range(B):
            check_dot(got[i], reference(oracle, ws[i]), floor_for(ws[i]), "%s batch %d" % (kern, i))


@pytest.mark.parametrize("nk", [False, True])
def test_one_hot_rows_read_single_values_back_exactly(oracle, nk):
    """a = selector rows of 1.0: every output is one rhs value times the scales, exactly -- every f8 code
    at every position of a 128-value step, so a transposed byte or a permuted k shows as a wrong value."""
    say("fp8 streaming, one-hot, nk=%s" % nk)
    M, K, N = 32, 384, 256
    ks = (np.arange(M) * 37 + 5) % K
    a = np.zeros((M, K), np.float32)
    a[np.arange(M), ks] = 1.0
    b8 = ((np.arange(K)[:, None] * 7 + np.arange(N)[None, :]) % 256).astype(np.uint8)
    b8[(b8 & 0x7F) == 0x7F] = 0x3A
    w = dict(a=dtypes.f32_to_f8e4m3fn(a), b=b8, a_scale=np.float32(0.5), b_scale=np.float32(0.25), bias=None,
             epilogue="DEFAULT")
    want = dtypes.f32_to_bf16(dtypes.f8e4m3fn_to_f32(b8[ks]) * np.float32(0.125))
    for slices in (0, 2):
        out, kern = run(w, nk=nk, slices=slices)
        assert kern == tile_name(nk, M)
        assert np.array_equal(dtypes.bf16_to_f32(host_bf16(out)), dtypes.bf16_to_f32(want)), (kern, slices)


@pytest.mark.parametrize("nk", [False, True])
def test_nan_codes_and_the_end_of_k(oracle, nk):
    """A NaN code makes its row or channel NaN and nothing else.  K = 144 ends inside a step, and what
    lies behind a row's end in memory (the start of the next row of a, or of the next channel of an
    [N,K] rhs) must not leak in even when it holds NaN codes."""
    say("fp8 streaming, NaN codes, nk=%s" % nk)
    M, K, N = 5, 144, 64
    w = dict(workloads.c3_fp8(M, K, N), epilogue="DEFAULT", bias=None)
    a8, b8 = w["a"].copy(), w["b"].copy()
    a8[1, :16] = 0x7F         # right behind row 0's end: row 1 is NaN, row 0 stays finite
    a8[3, 17] = 0xFF
    b8[:16, 1] = 0x7F         # right behind channel 0's end in an [N,K] rhs
    b8[100, 9] = 0x7F
    w["a"], w["b"] = a8, b8
    out, kern = run(w, nk=nk)
    got = dtypes.bf16_to_f32(host_bf16(out))
    ref = dtypes.bf16_to_f32(reference(oracle, w))
    assert np.array_equal(np.isnan(got), np.isnan(ref)), kern
    finite = np.ones((M, N), bool)
    finite[[1, 3], :] = False
    finite[:, [1, 9]] = False
    assert np.array_equal(~np.isnan(got), finite), kern
    assert np.allclose(got[finite], ref[finite], rtol=2.0 ** -7, atol=float(np.max(floor_for(w)[finite]))), kern


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("M", [16, 48, 100])
def test_bf16_typed_multiply(oracle, M, nk):
    """A bf16-typed dequantise multiply with per-tensor scales: powers of two round nothing, the streaming
    kernels serve the call and the result is that of the f32-typed call bit for bit; any other scale makes
    them return at once and the bf16-operand kernels launched behind them (or, without their scratch,
    the exact kernel) produce the result."""
    say("fp8 streaming, bf16-typed multiply, M=%d nk=%s" % (M, nk))
    K, N = (8192 if M > 64 else 1024), 264   # (100 rows: K long enough for passes to beat the two tiles)
    w = dict(workloads.c3_fp8(M, K, N), a_scale=np.float32(1 / 64), b_scale=np.float32(1 / 32))
    types = dict(dequant_type="bf16")
    # the streaming kernels' own form that rounds the scaled operands to bf16 stands behind the f8 form
    # ("|rounded"); it takes up to 32 rows of an [N,K] rhs per launch, so 48 rows go through in two passes there
    tag = "|rounded"
    out, kern = run(w, nk=nk, force=0, **types)
    assert kern.startswith("fp8_dot_decode_%s_m" % ("nk" if nk else "kn")) and kern.endswith(tag), kern
    plain, kern_plain = run(w, nk=nk, force=0)
    if nk and M > 32:
        assert kern == "fp8_dot_decode_nk_m32:x32|rounded", kern
        check_dot(host_bf16(out), reference(oracle, w), floor_for(w), kern)
    else:
        assert kern == kern_plain + tag, (kern, kern_plain)
        assert torch.equal(out, plain)
    w2 = dict(w, a_scale=np.float32(0.3), b_scale=np.float32(0.013))
    ref2 = reference(oracle, w2, **types)
    for slices in (0, 2):
        out2, kern2 = run(w2, nk=nk, force=0, slices=slices, **types)
        assert kern2 == kern, kern2
        n_floor = check_dot(host_bf16(out2), ref2, floor_for(w2, exact_kernel=True), "%s, %d slices" % (kern2, slices))
        assert n_floor <= max(8, out2.numel() // 50)
    out3, kern3 = run(w2, nk=nk, force=0, scratch=None, **types)     # no scratch: one K-slice
    assert kern3 == kern, kern3
    check_dot(host_bf16(out3), ref2, floor_for(w2, exact_kernel=True), kern3)
    out4, _ = run(w, nk=nk, force=0, scratch=None, **types)
    check_dot(host_bf16(out4), reference(oracle, w, **types), floor_for(w), "pow2 scales, no scratch")


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("which", ["a", "b", "ab"])
@pytest.mark.parametrize("M", [20, 64])
def test_bf16_typed_multiply_with_vector_scales(oracle, which, M, nk):
    """Per-row and per-channel scales under a bf16-typed multiply (no single test tells whether they round
    anything): the rounding form of the streaming kernels runs alone, each operand scaled by its row's or its
    channel's scale."""
    say("fp8 streaming, bf16-typed multiply, vector scales %s, M=%d" % (which, M))
    K, N = 1024, 200
    w = workloads.c3_fp8(M, K, N)
    rng = np.random.default_rng(5)
    if "a" in which:
        w["a_scale"] = rng.uniform(0.004, 0.04, M).astype(np.float32)
    if "b" in which:
        w["b_scale"] = rng.uniform(0.004, 0.04, N).astype(np.float32)
    types = dict(dequant_type="bf16")
    ref = reference(oracle, w, **types)
    for slices in (0, 2):
        out, kern = run(w, nk=nk, force=0, slices=slices, **types)
        assert kern == ("fp8_dot_decode_nk_m32:x32|rounded" if nk and M > 32 else tile_name(nk, M) + "|rounded"), kern
        n_floor = check_dot(host_bf16(out), ref, floor_for(w, exact_kernel=True), "%s, %d slices" % (kern, slices))
        assert n_floor <= max(8, out.numel() // 50)


@pytest.mark.parametrize("nk", [False, True])
def test_rounded_operands_read_every_code_back_exactly(nk):
    """The form that rounds the scaled operands, on one-hot rows: output [m, n] is
    bf16(bf16(1 * 0.75) * bf16(b[k_m, n] * 0.3125)) for every f8 code at every position of a step -- the
    hardware widening of each code, the rounding of the product and the k order of both operands."""
    say("fp8 streaming, rounded operands, one-hot")
    M, K, N = 32, 384, 256
    ks = (np.arange(M) * 37 + 5) % K
    a = np.zeros((M, K), np.float32)
    a[np.arange(M), ks] = 1.0
    b8 = ((np.arange(K)[:, None] * 7 + np.arange(N)[None, :]) % 256).astype(np.uint8)
    b8[(b8 & 0x7F) == 0x7F] = 0x3A
    w = dict(a=dtypes.f32_to_f8e4m3fn(a), b=b8, a_scale=np.float32(0.75), b_scale=np.float32(0.3125), bias=None,
             epilogue="DEFAULT")
    bs = dtypes.bf16_to_f32(dtypes.f32_to_bf16(dtypes.f8e4m3fn_to_f32(b8[ks]) * np.float32(0.3125)))
    want = dtypes.f32_to_bf16(np.float32(0.75) * bs)
    for slices in (0, 2):
        out, kern = run(w, nk=nk, slices=slices, force=0, dequant_type="bf16")
        assert kern == "fp8_dot_decode_%s_m32|rounded" % ("nk" if nk else "kn"), kern
        assert np.array_equal(dtypes.bf16_to_f32(host_bf16(out)), dtypes.bf16_to_f32(want)), slices


def test_scales_on_the_sum_option(oracle):
    """fp8_scales_on_sum = 1: a bf16-typed multiply with any scale is the f32-typed call (what the reference's
    GPU pipeline computes for that HLO), at decode size on the streaming kernels."""
    say("fp8 bf16-typed multiply computed with the scales on the sum")
    # (scales that are bf16 numbers, as the parameters of a bf16-typed module are, and no powers of two)
    w = dict(workloads.c3_fp8(16, 1024, 264), a_scale=np.float32(77 / 256), b_scale=np.float32(213 / 16384))
    plain, kern_plain = run(w, force=0)
    ffi.set_option("fp8_scales_on_sum", 1)
    try:
        out, kern = run(w, force=0, dequant_type="bf16")
    finally:
        ffi.set_option("fp8_scales_on_sum", 0)
    assert kern == kern_plain == "fp8_dot_decode_kn_m16", (kern, kern_plain)
    assert torch.equal(out, plain)
    # and close to the op-by-op value as a whole (that value rounds every a * a_scale and b * b_scale to bf16)
    ref = dtypes.bf16_to_f32(reference(oracle, w, dequant_type="bf16")).astype(np.float64)
    got = dtypes.bf16_to_f32(host_bf16(out)).astype(np.float64)
    assert np.linalg.norm(got - ref) <= 1e-2 * np.linalg.norm(ref), np.linalg.norm(got - ref) / np.linalg.norm(ref)


def test_what_the_streaming_kernels_do_not_take():
    a = torch.zeros((2, 80, 64), dtype=torch.uint8, device="cuda")
    b = torch.zeros((2, 64, 64), dtype=torch.uint8, device="cuda")
    one = torch.ones((), dtype=torch.float32, device="cuda")
    ffi.set_option("fp8_dot_kernel", 3)
    try:
        with pytest.raises(ffi.FfiError, match="only without a batch dimension"):
            ops.fp8_scaled_dot(a, b, one, one)      # 80 rows per batch
        with pytest.raises(ffi.FfiError, match="streaming kernels take"):
            ops.fp8_scaled_dot(a[0, :8], b[0, :, :60].contiguous(), one, one)   # N % 8 != 0
    finally:
        ffi.set_option("fp8_dot_kernel", 0)


@pytest.mark.parametrize("nk", [False, True])
@pytest.mark.parametrize("M", [65, 100, 130, 200])
def test_more_rows_go_through_in_equal_passes(oracle, M, nk):
    """More rows of a than one launch takes (64, or 48 with the rhs [N,K]): passes of equal row counts
    (multiples of 16), the last one with what is left; per-row scales and the bias follow the rows."""
    say("fp8 streaming, %d rows in passes, nk=%s" % (M, nk))
    K, N = 1024, 264
    w = workloads.c3_fp8(M, K, N)
    w["a_scale"] = np.random.default_rng(M).uniform(0.004, 0.04, M).astype(np.float32)
    most = 48 if nk else 64
    passes = -(-M // most)
    rows = -(-(-(-M // passes)) // 16) * 16
    for slices in (0, 2):
        out, kern = run(w, nk=nk, slices=slices)
        assert kern == "%s:x%d" % (tile_name(nk, rows), rows), kern
        check_dot(host_bf16(out), reference(oracle, w), floor_for(w), kern)


def test_passes_with_an_f8_result_fold_one_amax(oracle):
    say("fp8 streaming, 150 rows in passes, f8 result + amax")
    M, K, N = 150, 512, 136
    w = workloads.c3_fp8(M, K, N)
    s = np.float32(1 / 64)
    w["a_scale"] = w["b_scale"] = s
    z = np.float32(0.0171)
    (out, amax), kern = run(w, d_scale=dev_f32(np.array(z, np.float32)), amax=True)
    assert kern == "fp8_dot_decode_kn_m64:x64", kern
    ref, val = oracle.fp8_scaled_dot(w["a"], w["b"], s, s, bias=w["bias"], epilogue=EPI[w["epilogue"]], d_scale=z,
                                     d_scale_divides=True)
    check_f8_result(out.cpu().numpy(), ref, val, z, True, floor_for(w), kern)
    want = float(np.max(np.abs(val)))
    got = float(amax.cpu())
    assert abs(got - want) <= 2.0 ** -7 * want + float(np.max(floor_for(w))), (got, want)


def test_the_launcher_takes_passes_where_they_are_cheaper(oracle):
    """Few tiles of a long K: two passes of the streaming kernel instead of a handful of 256 x 256 tiles;
    many tiles: the tiled kernel."""
    say("fp8 streaming passes, the launcher's own choice")
    w = workloads.c3_fp8(96, 4096, 512)
    out, kern = run(w, force=0)
    assert kern == "fp8_dot_decode_kn_m48:x48", kern
    check_dot(host_bf16(out), reference(oracle, w), floor_for(w), kern)
    out, kern = run(w, nk=True, force=0)
    assert kern == "fp8_dot_decode_nk_m48:x48", kern
    check_dot(host_bf16(out), reference(oracle, w), floor_for(w), kern)
    big = workloads.c3_fp8(512, 256, 512)   # four passes of a short K against one round of tiles
    out, kern = run(big, force=0)
    assert kern.startswith("fp8_scaled_dot_tiled"), kern


# ---- block scales (MXFP8) on the [N,K] streaming kernel: up to 32 rows of a, K % 128 == 0 ---------------

def run_mx(a, b, sa, sb, bias=None, slices=0, batch=None, **kw):
    ffi.set_option("fp8_dot_kernel", 3)
    ffi.set_option("fp8_decode_slices", slices)
    try:
        scratch = "auto"
        if slices:
            n = ffi.library().xla_amd_fp8_scaled_dot_workspace_bytes(a.shape[-2], a.shape[-1], b.shape[-2], 1)
            scratch = torch.empty(max(n * (batch or 1), 16), dtype=torch.uint8, device="cuda")
        out = ops.fp8_scaled_dot(dev_u8(a), dev_u8(b), dev_u8(sa), dev_u8(sb), dev_bf16(bias) if bias is not None else None,
                                 rhs_contracting_dim=1, scratch=scratch, **kw)
        torch.cuda.synchronize()
    finally:
        ffi.set_option("fp8_dot_kernel", 0)
        ffi.set_option("fp8_decode_slices", 0)
    return host_bf16(out), ffi.last_kernel()


@pytest.mark.parametrize("M", [1, 16, 17, 32])
@pytest.mark.parametrize("K,N", [(512, 272), (1024, 136), (128, 64)])
@pytest.mark.parametrize("slices", [0, 2])
def test_mxfp8_block_scales(oracle, M, K, N, slices):
    from tests.test_gpu_fp8_dot import mx_case, mx_floor
    say("fp8 streaming MXFP8 M=%d K=%d N=%d slices=%d" % (M, K, N, slices))
    a, b, sa, sb = mx_case(M, K, N, 7)
    got, kern = run_mx(a, b, sa, sb, slices=slices)
    assert kern == "fp8_dot_decode_mx_m%d" % (16 * ((M + 15) // 16)), kern
    n_floor = check_dot(got, oracle.block_scaled_dot(a, b, sa, sb), mx_floor(a, b, sa, sb, False), kern)
    assert n_floor <= max(4, got.size // 50)


@pytest.mark.parametrize("M", [33, 64, 70])
@pytest.mark.parametrize("slices", [0, 2])
def test_mxfp8_more_rows_in_passes(oracle, M, slices):
    """More than 32 rows with block scales: passes of up to 32 rows, each with its rows' scales."""
    from tests.test_gpu_fp8_dot import mx_case, mx_floor
    say("fp8 streaming MXFP8 M=%d in passes, slices=%d" % (M, slices))
    K, N = 1024, 136
    a, b, sa, sb = mx_case(M, K, N, 11)
    sa[:] = ((np.arange(M)[:, None] * 3 + np.arange(K // 32)[None, :]) % 13 + 121).astype(np.uint8)   # scales that tell rows apart
    got, kern = run_mx(a, b, sa, sb, slices=slices)
    rows = -(-(-(-M // -(-M // 32))) // 16) * 16
    assert kern == "fp8_dot_decode_mx_m%d:x%d" % (rows, rows), kern
    n_floor = check_dot(got, oracle.block_scaled_dot(a, b, sa, sb), mx_floor(a, b, sa, sb, False), kern)
    assert n_floor <= max(4, got.size // 50)


@pytest.mark.parametrize("epilogue,dot_ty,ep_ty", [("BIAS_GELU", "f32", "f32"), ("BIAS_SILU", "bf16", "bf16"), ("RELU", "f32", "f32")])
def test_mxfp8_with_an_epilogue_and_batched(oracle, epilogue, dot_ty, ep_ty):
    from tests.test_gpu_fp8_dot import mx_case, mx_floor
    say("fp8 streaming MXFP8 %s dot %s ops %s, batched" % (epilogue, dot_ty, ep_ty))
    names = {"BIAS_GELU": "gelu_tanh", "BIAS_SILU": "silu", "RELU": "relu"}
    B, M, K, N = 2, 24, 384, 200
    cases = [mx_case(M, K, N, 30 + i) for i in range(B)]
    a, b, sa, sb = (np.stack([c[j] for c in cases]) for j in range(4))
    bias = dtypes.f32_to_bf16(np.random.default_rng(3).standard_normal(N).astype(np.float32)) if "BIAS" in epilogue else None
    got, kern = run_mx(a, b, sa, sb, bias, batch=B, epilogue=epilogue, dot_type=dot_ty, epilogue_type=ep_ty)
    assert kern == "fp8_dot_decode_mx_m32", kern
    for i in range(B):
        ref = oracle.block_scaled_dot(a[i], b[i], sa[i], sb[i], bias=bias, dot_ty=dot_ty, ep_ty=ep_ty, epilogue=names[epilogue])
        fl = 1.2 * mx_floor(a[i], b[i], sa[i], sb[i], False)
        if "bf16" in (dot_ty, ep_ty):
            fl = fl * 12 + np.abs(dtypes.bf16_to_f32(ref)) * 6 * 2.0 ** -8
        check_dot(got[i], ref, fl, "%s %s batch %d" % (kern, epilogue, i))


def test_mxfp8_one_block_at_a_time(oracle):
    """Data in a single 32-element block of K, a different scale on every block and channel: each block must
    come out multiplied by its own two scales exactly (products of small integers, exact sums) -- a scale
    byte taken from the wrong block, row or channel shows as a wrong power of two."""
    say("fp8 streaming MXFP8 block by block")
    M, K, N = 20, 256, 144
    rng = np.random.default_rng(2)
    ai = rng.integers(-3, 4, (M, K)).astype(np.float32)
    bi = rng.integers(-3, 4, (N, K)).astype(np.float32)
    sa = np.repeat((121 + np.arange(K // 32)).astype(np.uint8)[None, :], M, axis=0)
    sa[:, :] += (np.arange(M) % 5).astype(np.uint8)[:, None]
    sb = np.repeat((134 - 2 * np.arange(K // 32)).astype(np.uint8)[None, :], N, axis=0)   # sa + sb differs from block to block
    sb[:, :] += (np.arange(N) % 3).astype(np.uint8)[:, None]
    for j in range(K // 32):
        a1 = np.zeros_like(ai)
        a1[:, 32 * j:32 * j + 32] = ai[:, 32 * j:32 * j + 32]
        a8, b8 = dtypes.f32_to_f8e4m3fn(a1), dtypes.f32_to_f8e4m3fn(bi)
        got, kern = run_mx(a8, b8, sa, sb)
        assert kern == "fp8_dot_decode_mx_m32"
        assert np.array_equal(got, oracle.block_scaled_dot(a8, b8, sa, sb)), j
