"""The allocation-free launcher (xla_amd_launch_dequant_dot_static_scratch) against the launcher
that takes a workspace, through the C ABI: same kernels, same summation order, so the outputs
must be bit-identical -- on two calls in a row, the second on a smaller input (the static array
then still holds the first call's partial sums beyond what the second overwrites)."""
import ctypes as C

import numpy as np
import pytest
import torch

from tests.gpu_util import check_dot, dev_bf16, dev_f32, dev_s8, dev_u8, dot_floor, host_bf16
from xla_amd import dtypes, ffi, workloads

pytestmark = pytest.mark.gpu

EPI = {"DEFAULT": 0, "BIAS_SILU": 7}


def _params(lhs, weights, scales, bias, out, M, K, N, group, wdt, sdt, dequant, epilogue):
    p = ffi.LaunchDequantDot()
    p.lhs, p.weights, p.scales = lhs.data_ptr(), weights.data_ptr(), scales.data_ptr()
    p.bias = bias.data_ptr() if bias is not None else None
    p.out = out.data_ptr()
    p.workspace, p.workspace_bytes = None, 0
    p.batch, p.M, p.K, p.N, p.group, p.scale_batch = 1, M, K, N, group, 1
    p.weight_dtype, p.scale_dtype, p.bias_dtype = wdt, sdt, dtypes.BF16
    p.dequant_type, p.dot_type, p.epilogue_type, p.epilogue = dequant, dtypes.F32, dtypes.F32, EPI[epilogue]
    return p


def _both(p, need):
    """Runs p through the workspace launcher and the static-scratch one; returns both outputs."""
    L = ffi.library()
    stream = torch.cuda.current_stream().cuda_stream
    n_out = p.M * p.N
    out_ws = torch.full((n_out,), 0x7fc0, dtype=torch.int16, device="cuda")
    out_st = torch.full((n_out,), 0x7fc1, dtype=torch.int16, device="cuda")
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    p.out, p.workspace, p.workspace_bytes = out_ws.data_ptr(), ws.data_ptr(), need
    rc = L.xla_amd_launch_dequant_dot(C.byref(p), stream)
    assert rc == 0, L.xla_amd_last_error()
    kernel_ws = L.xla_amd_last_kernel()
    p.out, p.workspace, p.workspace_bytes = out_st.data_ptr(), None, 0
    rc = L.xla_amd_launch_dequant_dot_static_scratch(C.byref(p), stream)
    assert rc == 0, L.xla_amd_last_error()
    assert L.xla_amd_last_kernel() == kernel_ws
    torch.cuda.synchronize()
    return out_ws.cpu().numpy().view(np.uint16), out_st.cpu().numpy().view(np.uint16)


def test_static_scratch_matches_workspace_launcher(oracle):
    L = ffi.library()
    # first call: configuration 1 (s8 per channel, 16 tokens): K is split four ways
    c1 = workloads.c1_s8_channel()
    M, K, N = 16, 4096, 4096
    need = L.xla_amd_dequant_dot_workspace_bytes(1, M, K, N, dtypes.S8)
    assert need > 0, "configuration 1 is expected to split K through the scratch"
    lhs, w, sc = dev_bf16(c1["lhs"]), dev_s8(c1["weights"]), dev_f32(c1["scales"])
    p = _params(lhs, w, sc, None, lhs, M, K, N, K, dtypes.S8, dtypes.F32, dtypes.F32, "DEFAULT")
    got_ws, got_st = _both(p, need)
    assert np.array_equal(got_ws, got_st)
    ref = oracle.dequant_dot(c1["lhs"], c1["weights"], 8, c1["scales"], "f32", "f32")
    a = np.abs(dtypes.bf16_to_f32(c1["lhs"]).astype(np.float64))
    wd = np.abs(c1["weights"].astype(np.float64)) * c1["scales"].astype(np.float64)[None, :]
    check_dot(got_st.reshape(M, N), ref, dot_floor(a, wd, K), "static scratch, configuration 1")

    # second call, smaller: s4 group scales, 4 tokens (split in two)
    M2, K2, N2 = 4, 2048, 1024
    c2 = workloads.c2_s4_group(M=M2, K=K2, N=N2)
    need2 = L.xla_amd_dequant_dot_workspace_bytes(1, M2, K2, N2, dtypes.S4)
    assert 0 < need2 < need
    lhs2, w2, sc2, b2 = dev_bf16(c2["lhs"]), dev_u8(c2["weights_packed"]), dev_bf16(c2["scales"]), dev_bf16(c2["bias"])
    p2 = _params(lhs2, w2, sc2, b2, lhs2, M2, K2, N2, 128, dtypes.S4, dtypes.BF16, dtypes.BF16, "BIAS_SILU")
    got_ws2, got_st2 = _both(p2, need2)
    assert np.array_equal(got_ws2, got_st2)
    ref2 = oracle.dequant_dot(c2["lhs"], c2["weights_packed"], 4, c2["scales"], "bf16", "bf16", bias=c2["bias"],
                              group=128, epilogue="silu")
    a2 = np.abs(dtypes.bf16_to_f32(c2["lhs"]).astype(np.float64))
    wd2 = np.abs(c2["weights"].astype(np.float64)) * np.repeat(
        dtypes.bf16_to_f32(c2["scales"]).astype(np.float64), 128, axis=0)
    check_dot(got_st2.reshape(M2, N2), ref2, dot_floor(a2, wd2, K2), "static scratch, s4 group scales")


def test_static_scratch_refuses_oversized_partial_sums():
    L = ffi.library()
    # 64 tokens on 40 strips of a long K, cut into eight K-slices: 10 MiB of f32 partial sums
    M, K, N = 64, 32768, 5120
    ffi.set_option("dequant_dot_slices", 8)
    try:
        need = L.xla_amd_dequant_dot_workspace_bytes(1, M, K, N, dtypes.S4)
        assert need > 8 << 20, need
        t = torch.zeros(16, dtype=torch.uint8, device="cuda")
        p = _params(t, t, t, None, t, M, K, N, 128, dtypes.S4, dtypes.BF16, dtypes.BF16, "DEFAULT")
        rc = L.xla_amd_launch_dequant_dot_static_scratch(C.byref(p), torch.cuda.current_stream().cuda_stream)
        assert rc == 8 and b"static scratch holds" in L.xla_amd_last_error()
    finally:
        ffi.set_option("dequant_dot_slices", 0)


def test_static_scratch_with_weights_stored_k_minor(oracle):
    """Weights [N,K] (rhs_contracting_dim = 1): the K-slices of the [N,K] kernel go through the static
    array as well, bit-identical to the workspace launcher."""
    L = ffi.library()
    M, K, N = 8, 4096, 512
    c1 = workloads.c1_s8_channel(M=M, K=K, N=N)
    v = workloads.k_minor(c1)
    need = L.xla_amd_dequant_dot_workspace_bytes_nk(1, M, K, N, dtypes.S8)
    assert need > 0, "few channels: K is expected to be cut into slices"
    lhs, w, sc = dev_bf16(v["lhs"]), dev_s8(v["weights"]), dev_f32(v["scales"])
    p = _params(lhs, w, sc, None, lhs, M, K, N, K, dtypes.S8, dtypes.F32, dtypes.F32, "DEFAULT")
    p.rhs_contracting_dim = 1
    got_ws, got_st = _both(p, need)
    assert np.array_equal(got_ws, got_st)
    ref = oracle.dequant_dot(c1["lhs"], c1["weights"], 8, c1["scales"], "f32", "f32")
    a = np.abs(dtypes.bf16_to_f32(c1["lhs"]).astype(np.float64))
    wd = np.abs(c1["weights"].astype(np.float64)) * c1["scales"].astype(np.float64)[None, :]
    check_dot(got_st.reshape(M, N), ref, dot_floor(a, wd, K), "static scratch, weights [N,K]")


def test_static_scratch_with_more_than_64_tokens(oracle):
    """More than 64 tokens of s8 weights run on the tiled kernel, whose short last round is split along
    K through the scratch: the static array must be sized for that too.  A shape whose split fits is
    bit-identical to the workspace launcher (same split, same order of the two halves); one whose
    split needs more than the array is refused, as the [N,K] spelling of it is."""
    L = ffi.library()
    M, K, N = 128, 2048, 2048      # 8 tiles, all split in two: 8 x (256 KiB + 16)
    need = L.xla_amd_dequant_dot_workspace_bytes(1, M, K, N, dtypes.S8)
    assert 0 < need <= 8 << 20, need
    c = workloads.c1_s8_channel(M=M, K=K, N=N)
    lhs, w, sc = dev_bf16(c["lhs"]), dev_s8(c["weights"]), dev_f32(c["scales"])
    p = _params(lhs, w, sc, None, lhs, M, K, N, K, dtypes.S8, dtypes.F32, dtypes.F32, "DEFAULT")
    ffi.set_option("dequant_dot_kernel", 3)   # (a matrix this small would otherwise go through the decode kernel twice)
    try:
        got_ws, got_st = _both(p, need)
    finally:
        ffi.set_option("dequant_dot_kernel", 0)
    assert L.xla_amd_last_kernel().endswith(b":tail2"), L.xla_amd_last_kernel()
    assert np.array_equal(got_ws, got_st)
    ref = oracle.dequant_dot(c["lhs"], c["weights"], 8, c["scales"], "f32", "f32")
    a = np.abs(dtypes.bf16_to_f32(c["lhs"]).astype(np.float64))
    wd = np.abs(c["weights"].astype(np.float64)) * c["scales"].astype(np.float64)[None, :]
    check_dot(got_st.reshape(M, N), ref, dot_floor(a, wd, K), "static scratch, split last round")

    M2, N2 = 1024, 4096            # 64 tiles split in two: 16 MiB
    need2 = L.xla_amd_dequant_dot_workspace_bytes(1, M2, K, N2, dtypes.S8)
    assert need2 > 8 << 20, need2
    t = torch.zeros(16, dtype=torch.uint8, device="cuda")
    for rcd in (0, 1):
        p2 = _params(t, t, t, None, t, M2, K, N2, K, dtypes.S8, dtypes.F32, dtypes.F32, "DEFAULT")
        p2.rhs_contracting_dim = rcd
        rc = L.xla_amd_launch_dequant_dot_static_scratch(C.byref(p2), torch.cuda.current_stream().cuda_stream)
        assert rc == 8 and b"static scratch holds" in L.xla_amd_last_error(), (rcd, rc, L.xla_amd_last_error())
