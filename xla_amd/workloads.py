"""Synthetic inputs for the five benchmark configurations (fixed seeds, numpy only).

Each generator takes the full shape by default and accepts smaller shapes so that parity
tests can run the same distributions at sizes a scalar CPU oracle finishes in seconds.
bf16 values are round-to-nearest-even from f32 draws and travel as uint16 bit patterns;
f8e4m3fn values travel as uint8 codes; s4 weights are returned both unpacked (int8) and
packed two per byte.  ``algorithmic_bytes`` / ``algorithmic_flops`` are the per-call figures
roofline fractions are computed from (operands and results once each; no padding, re-reads
or workspaces).
"""
import numpy as np

from . import dtypes


def _rng(seed):
    return np.random.default_rng(seed)


def c1_s8_channel(M=16, K=4096, N=4096):
    """bf16 A[M,K] . (convert(s8 W[K,N]) * f32 scale[N]) -> bf16 [M,N]; f32-typed multiply."""
    a = dtypes.f32_to_bf16(_rng(1).standard_normal((M, K)).astype(np.float32))
    w = _rng(2).integers(-127, 128, size=(K, N)).astype(np.int8)
    scale = _rng(3).uniform(1e-3, 1e-2, size=(N,)).astype(np.float32)
    return dict(name="C1", lhs=a, weights=w, scales=scale, bias=None, weight_dtype="s8",
                weight_shape=(K, N), group=K, dequant_type="f32", epilogue="DEFAULT",
                algorithmic_bytes=K * N + M * K * 2 + N * 4 + M * N * 2,
                algorithmic_flops=2 * M * K * N)


def c2_s4_group(M=1, K=8192, N=28672, group=128):
    """bf16 A[M,K] . bf16(convert(s4 W[K,N]) * bf16 scale[K/group,N]) + bias -> SiLU -> bf16."""
    a = dtypes.f32_to_bf16(_rng(10 + M).standard_normal((M, K)).astype(np.float32))
    w = _rng(20).integers(-8, 8, size=(K, N)).astype(np.int8)
    scale = dtypes.f32_to_bf16(_rng(21).uniform(1e-3, 2e-2, size=(K // group, N)).astype(np.float32))
    bias = dtypes.f32_to_bf16(_rng(22).standard_normal((N,)).astype(np.float32))
    return dict(name="C2", lhs=a, weights=w, weights_packed=dtypes.pack_s4(w), scales=scale,
                bias=bias, weight_dtype="s4", weight_shape=(K, N), group=group,
                dequant_type="bf16", epilogue="BIAS_SILU",
                algorithmic_bytes=K * N // 2 + (K // group) * N * 2 + N * 2 + M * K * 2 + M * N * 2,
                algorithmic_flops=2 * M * K * N)


def u4_zero_point_group(M=8, K=4096, N=4096, group=128):
    """bf16 A[M,K] . bf16((u4 W[K,N] - u4 zero[K/group,N]) * bf16 scale[K/group,N]) + bias -> bf16."""
    a = dtypes.f32_to_bf16(_rng(60 + M).standard_normal((M, K)).astype(np.float32))
    w = _rng(61).integers(0, 16, size=(K, N)).astype(np.uint8)
    zero = _rng(62).integers(0, 16, size=(K // group, N)).astype(np.uint8)
    scale = dtypes.f32_to_bf16(_rng(63).uniform(1e-3, 2e-2, size=(K // group, N)).astype(np.float32))
    bias = dtypes.f32_to_bf16(_rng(64).standard_normal((N,)).astype(np.float32))
    pack = lambda v: (v.reshape(-1)[0::2] | (v.reshape(-1)[1::2] << 4)).astype(np.uint8)
    return dict(name="u4zp", lhs=a, weights=w.astype(np.int8), weights_packed=pack(w), scales=scale,
                zero_points=zero, zero_points_packed=pack(zero), bias=bias, weight_dtype="u4",
                weight_shape=(K, N), group=group, dequant_type="bf16", epilogue="BIAS",
                algorithmic_bytes=K * N // 2 + (K // group) * N * 5 // 2 + N * 2 + M * K * 2 + M * N * 2,
                algorithmic_flops=2 * M * K * N)


def ragged_s8_experts(M=32, K=4096, N=4096, groups=8, sizes=None):
    """bf16 A[M,K] (rows sorted by expert) . (s8 W[G,K,N] * f32 scale[G,N]) + bias -> bf16 [M,N];
    `sizes`: rows per expert (default: a random split of M, some experts empty)."""
    rng = _rng(70 + M)
    a = dtypes.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    w = _rng(71).integers(-127, 128, size=(groups, K, N)).astype(np.int8)
    scale = _rng(72).uniform(1e-3, 1e-2, size=(groups, N)).astype(np.float32)
    bias = dtypes.f32_to_bf16(_rng(73).standard_normal((N,)).astype(np.float32))
    if sizes is None:
        cuts = np.sort(rng.integers(0, M + 1, size=groups - 1))
        sizes = np.diff(np.concatenate([[0], cuts, [M]]))
    return dict(name="ragged", lhs=a, weights=w, scales=scale, bias=bias, weight_dtype="s8",
                weight_shape=(groups, K, N), group=K, dequant_type="f32", epilogue="BIAS",
                group_sizes=np.asarray(sizes, np.int32),
                algorithmic_bytes=groups * K * N + groups * N * 4 + N * 2 + M * K * 2 + M * N * 2,
                algorithmic_flops=2 * M * K * N)


def ragged_s4_group_experts(M=32, K=4096, N=4096, groups=8, group=128, sizes=None):
    """bf16 A[M,K] (rows sorted by expert) . bf16(s4 W[G,K,N] * bf16 scale[G,K/group,N]) + bias -> bf16."""
    rng = _rng(80 + M)
    a = dtypes.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    w = _rng(81).integers(-8, 8, size=(groups, K, N)).astype(np.int8)
    scale = dtypes.f32_to_bf16(_rng(82).uniform(1e-3, 2e-2, size=(groups, K // group, N)).astype(np.float32))
    bias = dtypes.f32_to_bf16(_rng(83).standard_normal((N,)).astype(np.float32))
    if sizes is None:
        cuts = np.sort(rng.integers(0, M + 1, size=groups - 1))
        sizes = np.diff(np.concatenate([[0], cuts, [M]]))
    return dict(name="ragged_s4", lhs=a, weights=w, weights_packed=dtypes.pack_s4(w), scales=scale, bias=bias,
                weight_dtype="s4", weight_shape=(groups, K, N), group=group, dequant_type="bf16", epilogue="BIAS",
                group_sizes=np.asarray(sizes, np.int32),
                algorithmic_bytes=groups * K * N // 2 + groups * (K // group) * N * 2 + N * 2 + M * K * 2 + M * N * 2,
                algorithmic_flops=2 * M * K * N)


def batched_s4_group(B=4, M=8, K=1024, N=512, group=128):
    """bf16 A[B,M,K] . bf16(s4 W[B,K,N] * bf16 scale[B,K/group,N]) -> bf16 [B,M,N]."""
    a = dtypes.f32_to_bf16(_rng(90 + M).standard_normal((B, M, K)).astype(np.float32))
    w = _rng(91).integers(-8, 8, size=(B, K, N)).astype(np.int8)
    scale = dtypes.f32_to_bf16(_rng(92).uniform(1e-3, 2e-2, size=(B, K // group, N)).astype(np.float32))
    return dict(name="batched_s4", lhs=a, weights=w, weights_packed=dtypes.pack_s4(w), scales=scale, bias=None,
                weight_dtype="s4", weight_shape=(B, K, N), group=group, dequant_type="bf16", epilogue="DEFAULT",
                algorithmic_bytes=B * (K * N // 2 + (K // group) * N * 2 + M * K * 2 + M * N * 2),
                algorithmic_flops=2 * B * M * K * N)


def k_minor(w):
    """The same dequantize-dot with its weights stored [N,K] (or [B,N,K]) -- the contracting dimension
    minor -- and scales / zero points [N,K/group] (per-channel scales stay [N] / [B,N]).  4-bit values are
    re-packed along K.  Returns a copy of the workload with `rhs_contracting_dim` = 1; the values of the
    dot are those of `w`."""
    v = dict(w)
    wt = np.ascontiguousarray(np.swapaxes(w["weights"], -1, -2))
    v["weights"] = wt
    v["weight_shape"] = tuple(wt.shape)
    K = w["lhs"].shape[-1]
    pack = lambda x: (x.reshape(-1)[0::2] | (x.reshape(-1)[1::2] << 4)).astype(np.uint8)
    if w["weight_dtype"] in ("s4", "u4"):
        v["weights_packed"] = pack(wt.astype(np.int8).view(np.uint8) & 0xF)
    if w["group"] != K:
        v["scales"] = np.ascontiguousarray(np.swapaxes(w["scales"], -1, -2))
        if w.get("zero_points") is not None:
            z = np.ascontiguousarray(np.swapaxes(w["zero_points"], -1, -2))
            v["zero_points"] = z
            v["zero_points_packed"] = pack(z)
    v["rhs_contracting_dim"] = 1
    return v


def c3_fp8(M=8192, K=8192, N=8192):
    """f8 A[M,K] . f8 B[K,N], per-tensor f32 scales 1/64, + bias, GELU(tanh) -> bf16."""
    def f8(seed, shape):
        v = np.clip(_rng(seed).standard_normal(shape, dtype=np.float32) * 64.0, -448.0, 448.0)
        return dtypes.f32_to_f8e4m3fn(v)
    a = f8(30, (M, K))
    b = f8(31, (K, N))
    bias = dtypes.f32_to_bf16(_rng(32).standard_normal((N,)).astype(np.float32))
    return dict(name="C3", a=a, b=b, a_scale=np.float32(1 / 64), b_scale=np.float32(1 / 64),
                bias=bias, rhs_contracting_dim=0, epilogue="BIAS_GELU",
                algorithmic_bytes=M * K + K * N + M * N * 2 + N * 2,
                algorithmic_flops=2 * M * K * N)


def c4_quantize(rows=16384, cols=8192):
    """bf16 x[rows,cols] ~N(0,1) with 1% outliers x50, bf16 gamma ~U[0.5,1.5]."""
    x = _rng(40).standard_normal((rows, cols), dtype=np.float32)
    mask = _rng(41).random((rows, cols), dtype=np.float32) < 0.01
    x = np.where(mask, x * 50.0, x).astype(np.float32)
    gamma = dtypes.f32_to_bf16(_rng(42).uniform(0.5, 1.5, size=(cols,)).astype(np.float32))
    return dict(name="C4", x=dtypes.f32_to_bf16(x), gamma=gamma, eps=1e-6,
                algorithmic_bytes=rows * cols * 2 + rows * cols + rows * 4 + cols * 2)


def c5_s8_batched(B=8, M=512, K=4096, N=14336):
    """bf16 A[B,M,K] . (convert(s8 W[B,K,N]) * f32 scale[B,N]), batch dim 0 -> bf16 [B,M,N]."""
    a = dtypes.f32_to_bf16(_rng(50).standard_normal((B, M, K), dtype=np.float32))
    w = _rng(51).integers(-127, 128, size=(B, K, N), dtype=np.int8)
    scale = _rng(52).uniform(1e-3, 1e-2, size=(B, N)).astype(np.float32)
    return dict(name="C5", lhs=a, weights=w, scales=scale, bias=None, weight_dtype="s8",
                weight_shape=(B, K, N), group=K, dequant_type="f32", epilogue="DEFAULT",
                algorithmic_bytes=B * (K * N + M * K * 2 + N * 4 + M * N * 2),
                algorithmic_flops=2 * B * M * K * N)
