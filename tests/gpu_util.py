"""Helpers shared by the GPU parity tests: numpy <-> device tensors for the narrow types and
the comparison rules of the parity contract."""
import numpy as np
import torch

from xla_amd import dtypes


def dev_bf16(u16):
    return torch.from_numpy(np.ascontiguousarray(u16).view(np.int16).copy()).view(torch.bfloat16).cuda()


def dev_u8(a):
    return torch.from_numpy(np.ascontiguousarray(a, np.uint8).copy()).cuda()


def dev_s8(a):
    return torch.from_numpy(np.ascontiguousarray(a, np.int8).copy()).cuda()


def dev_f32(a):
    return torch.from_numpy(np.array(a, np.float32, order="C")).cuda()  # keeps a 0-d array 0-d


def host_bf16(t):
    return t.detach().cpu().view(torch.int16).numpy().view(np.uint16)


def bf16_ordinal(u16):
    """Signed-magnitude ordinal of a bf16 pattern: adjacent values differ by 1, +-0 coincide."""
    u = np.asarray(u16, np.int32)
    mag = u & 0x7FFF
    return np.where(u & 0x8000, -mag, mag)


def check_dot(got_u16, ref_u16, abs_floor, what=""):
    """Parity rule for f32-accumulated dots: every output within 2 bf16 ulp of the oracle's, or
    within `abs_floor` (per element) where cancellation makes ulps meaningless.  Returns the
    number of elements that needed the floor."""
    got_u16 = np.asarray(got_u16)
    ref_u16 = np.asarray(ref_u16)
    assert got_u16.shape == ref_u16.shape, (got_u16.shape, ref_u16.shape)
    dist = np.abs(bf16_ordinal(got_u16) - bf16_ordinal(ref_u16))
    ok = dist <= 2
    g = dtypes.bf16_to_f32(got_u16).astype(np.float64)
    r = dtypes.bf16_to_f32(ref_u16).astype(np.float64)
    both_nan = np.isnan(g) & np.isnan(r)
    near = np.abs(g - r) <= abs_floor
    bad = ~(ok | near | both_nan)
    if bad.any():
        idx = np.argwhere(bad)[:8]
        detail = [(tuple(i), float(g[tuple(i)]), float(r[tuple(i)]), int(dist[tuple(i)])) for i in idx]
        raise AssertionError("%s: %d of %d outputs differ by more than 2 bf16 ulp (and the floor): %s"
                             % (what, int(bad.sum()), bad.size, detail))
    return int((~ok & near).sum())


def dot_floor(abs_a, abs_w, K):
    """2^-24 * sqrt(K) * sum_k |a_k w_kn|: the scale of the difference between two f32 summation
    orders of the same products (float64 inputs, [..,M,K] @ [..,K,N])."""
    return (2.0 ** -24) * np.sqrt(K) * (abs_a @ abs_w) * 1.25
