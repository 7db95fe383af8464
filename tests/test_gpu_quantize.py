"""GPU parity of xla_amd.rowwise_quantize_fp8 against the CPU oracle: bit-exact f8e4m3fn
codes and f32 scales, called through the library's FFI handler symbol."""
import sys

import numpy as np
import pytest
import torch

from tests.gpu_util import dev_bf16
from xla_amd import dtypes, ffi, ops, workloads

pytestmark = pytest.mark.gpu


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def run(x_u16, gamma_u16, eps=1e-6):
    x = dev_bf16(x_u16)
    g = dev_bf16(gamma_u16) if gamma_u16 is not None else None
    q, s = ops.rowwise_quantize_fp8(x, g, eps=eps)
    torch.cuda.synchronize()
    return q.cpu().numpy(), s.cpu().numpy()


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
@pytest.mark.parametrize("rows,cols", [(64, 8192), (33, 4096), (7, 2048), (5, 1024), (3, 16384), (9, 256)])
def test_rmsnorm_quantize_bit_exact(oracle, variant, rows, cols):
    say("quantize rmsnorm variant=%d rows=%d cols=%d" % (variant, rows, cols))
    w = workloads.c4_quantize(rows, cols)
    ffi.set_option("quantize_variant", variant)
    try:
        q, s = run(w["x"], w["gamma"])
    finally:
        ffi.set_option("quantize_variant", 0)
    q_ref, s_ref = oracle.rmsnorm_quantize_fp8(w["x"], w["gamma"], eps=1e-6)
    assert np.array_equal(s.view(np.uint32), s_ref.view(np.uint32))
    assert np.array_equal(q, q_ref)


@pytest.mark.parametrize("rows,cols", [(4, 1000), (3, 37), (2, 8191), (5, 1), (1, 31), (6, 4104)])
def test_rmsnorm_quantize_ragged_columns(oracle, rows, cols):
    say("quantize rmsnorm ragged rows=%d cols=%d" % (rows, cols))
    w = workloads.c4_quantize(rows, cols)
    q, s = run(w["x"], w["gamma"])
    q_ref, s_ref = oracle.rmsnorm_quantize_fp8(w["x"], w["gamma"], eps=1e-6)
    assert np.array_equal(s.view(np.uint32), s_ref.view(np.uint32))
    assert np.array_equal(q, q_ref)


def test_plain_quantize_every_bf16_value_in_range():
    """Without RMSNorm and with amax = 448 the scale is exactly 1, so q = f8e4m3fn(x): sweeps the
    hardware convert over every bf16 value of magnitude <= 448 (ties, subnormals, both zeros)."""
    say("quantize plain exhaustive bf16")
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    v = dtypes.bf16_to_f32(h)
    keep = h[np.abs(v) <= 448.0]
    cols = 1024
    rows = (keep.size + cols - 2) // (cols - 1)
    x = np.zeros((rows, cols), np.uint16)
    flat = np.zeros(rows * (cols - 1), np.uint16)
    flat[:keep.size] = keep
    x[:, 1:] = flat.reshape(rows, cols - 1)
    x[:, 0] = 0x43E0                                      # 448.0 in every row
    q, s = run(x, None)
    assert np.all(s == 1.0)
    want = dtypes.f32_to_f8e4m3fn(dtypes.bf16_to_f32(x))
    bad = np.argwhere(q != want)
    assert bad.size == 0, [(hex(x[tuple(i)]), hex(q[tuple(i)]), hex(want[tuple(i)])) for i in bad[:12]]


def test_plain_quantize_matches_oracle_scale_path(oracle):
    say("quantize plain random")
    rng = np.random.default_rng(12)
    x = dtypes.f32_to_bf16((rng.standard_normal((40, 4096)) * rng.uniform(1e-3, 1e3, (40, 1))).astype(np.float32))
    q, s = run(x, None)
    xf = dtypes.bf16_to_f32(x)
    amax = np.abs(xf).max(axis=1)
    s_ref = (amax / np.float32(448)).astype(np.float32)
    assert np.array_equal(s.view(np.uint32), s_ref.view(np.uint32))
    d = np.clip((xf / s_ref[:, None]).astype(np.float32), -448, 448)
    assert np.array_equal(q, oracle.f32_to_f8e4m3fn(d))


def test_quantize_special_rows(oracle):
    """All-zero row (scale 0 -> NaN codes, as the unguarded HLO gives), tiny and huge rows: the
    IEEE-division fallback instead of the reciprocal shortcut."""
    say("quantize special rows")
    cols = 512
    rng = np.random.default_rng(5)
    base = rng.standard_normal((6, cols)).astype(np.float32)
    base[0] = 0.0
    base[1] *= 1e-30
    base[2] *= 1e30
    base[3] = np.clip(base[3], -1, 1)
    x = dtypes.f32_to_bf16(base)
    q, s = run(x, None)
    xf = dtypes.bf16_to_f32(x)
    amax = np.abs(xf).max(axis=1)
    s_ref = (amax / np.float32(448)).astype(np.float32)
    assert np.array_equal(s.view(np.uint32), s_ref.view(np.uint32))
    assert np.all((q[0] & 0x7F) == 0x7F)
    with np.errstate(all="ignore"):
        d = np.clip((xf[1:] / s_ref[1:, None]).astype(np.float32), -448, 448)
    assert np.array_equal(q[1:], oracle.f32_to_f8e4m3fn(d))


def test_quantize_empty_and_errors():
    say("quantize empty + error paths")
    x = torch.empty((0, 128), dtype=torch.bfloat16, device="cuda")
    g = torch.ones((128,), dtype=torch.bfloat16, device="cuda")
    q, s = ops.rowwise_quantize_fp8(x, g)
    assert q.shape == (0, 128) and s.shape == (0,)
    with pytest.raises(ffi.FfiError, match="gamma must have one entry per column"):
        ops.rowwise_quantize_fp8(torch.zeros((2, 64), dtype=torch.bfloat16, device="cuda"), g)
    with pytest.raises(ffi.FfiError, match="rows longer than 1048576 elements are not supported"):
        ops.rowwise_quantize_fp8(torch.zeros((1, (1 << 20) + 8), dtype=torch.bfloat16, device="cuda"), None)


@pytest.mark.parametrize("rows,cols,variant,kernel", [
    (9, 28672, 0, "lds_row"), (3, 16392, 0, "lds_row"), (2, 65536, 0, "lds_row"), (5, 40008, 0, "lds_row"),
    (9, 28672, 1, "long"), (2, 65544, 0, "long"), (4, 20001, 0, "long_unaligned"), (1, 1 << 20, 0, "long")])
def test_rmsnorm_quantize_long_rows(oracle, rows, cols, variant, kernel):
    """Rows past 16384 elements (an FFN activation of 28672, a vocabulary-sized row): up to 65536
    aligned elements the row is held in LDS by one workgroup, beyond that (and for unaligned rows) a
    kernel walks the row three times through L2; same codes and scales, bit for bit, windows of 32
    and the levels above them in the oracle's order."""
    say("quantize rmsnorm long rows=%d cols=%d variant=%d" % (rows, cols, variant))
    w = workloads.c4_quantize(rows, cols)
    ffi.set_option("quantize_variant", variant)
    try:
        q, s = run(w["x"], w["gamma"])
    finally:
        ffi.set_option("quantize_variant", 0)
    assert ffi.last_kernel() == "rowwise_quantize_fp8:" + kernel, ffi.last_kernel()
    q_ref, s_ref = oracle.rmsnorm_quantize_fp8(w["x"], w["gamma"], eps=1e-6)
    assert np.array_equal(s.view(np.uint32), s_ref.view(np.uint32))
    assert np.array_equal(q, q_ref)


def test_quantize_long_special_rows(oracle):
    """Long rows without RMSNorm: an all-zero row (NaN codes), a row with a NaN (NaN scale and codes),
    tiny and huge rows (the IEEE-division path)."""
    say("quantize long special rows")
    cols = 20480
    rng = np.random.default_rng(6)
    base = rng.standard_normal((5, cols)).astype(np.float32)
    base[0] = 0.0
    base[1] *= 1e-30
    base[2] *= 1e30
    base[4, 12345] = np.nan
    x = dtypes.f32_to_bf16(base)
    q, s = run(x, None)
    assert ffi.last_kernel() == "rowwise_quantize_fp8:lds_row", ffi.last_kernel()
    xf = dtypes.bf16_to_f32(x)
    amax = np.abs(xf[:4]).max(axis=1)
    s_ref = (amax / np.float32(448)).astype(np.float32)
    assert np.array_equal(s[:4].view(np.uint32), s_ref.view(np.uint32))
    assert np.all((q[0] & 0x7F) == 0x7F)
    with np.errstate(all="ignore"):
        d = np.clip((xf[1:4] / s_ref[1:, None]).astype(np.float32), -448, 448)
    assert np.array_equal(q[1:4], oracle.f32_to_f8e4m3fn(d))
    assert np.isnan(s[4]) and np.all((q[4] & 0x7F) == 0x7F)


def test_c4_full_size_bit_exact(oracle):
    """Configuration 4 (bf16 [16384,8192]) at full size, every code and scale against the oracle."""
    say("quantize C4 full 16384x8192")
    w = workloads.c4_quantize()
    q, s = run(w["x"], w["gamma"])
    q_ref, s_ref = oracle.rmsnorm_quantize_fp8(w["x"], w["gamma"], eps=1e-6)
    assert np.array_equal(s.view(np.uint32), s_ref.view(np.uint32))
    bad = np.argwhere(q != q_ref)
    assert bad.size == 0, (len(bad), [(tuple(i), hex(w["x"][tuple(i)]), hex(q[tuple(i)]), hex(q_ref[tuple(i)]),
                                       float(s[i[0]])) for i in bad[:12]])
    assert not np.any((q & 0x7F) == 0x7F)
    assert np.all((q & 0x7F).max(axis=1) == 0x7E)
