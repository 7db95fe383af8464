"""Helpers shared by the GPU parity tests: numpy <-> device tensors for the narrow types and
the comparison rules of the parity contract."""
import numpy as np
import torch

from xla_amd import dtypes


# (test id or label, outputs that passed only through the absolute floor / codes that differ from the
# oracle's, outputs compared): printed as a table at the end of the run by tests/conftest.py, so that
# how far the 2-ulp rule had to lean on its floor is visible in every test log
FLOOR_LOG = []


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
    n_floor = int((~ok & near).sum())
    FLOOR_LOG.append((what or "dot", "within the floor only", n_floor, int(bad.size)))
    return n_floor


def dot_floor(abs_a, abs_w, K):
    """2^-24 * sqrt(K) * sum_k |a_k w_kn|: the scale of the difference between two f32 summation
    orders of the same products (float64 inputs, [..,M,K] @ [..,K,N])."""
    return (2.0 ** -24) * np.sqrt(K) * (abs_a @ abs_w) * 1.25


def f8_value(codes):
    return dtypes.f8e4m3fn_to_f32(np.asarray(codes, np.uint8)).astype(np.float64)


def check_f8_result(got_codes, ref_codes, ref_value, d_scale, divides, abs_floor, what=""):
    """Parity rule for an f8 result convert(clamp(v / z)) of a dot: the oracle's v is only matched
    to 2 bf16 ulp (or the floor), so a code is accepted when some value within that window of
    the oracle's v is scaled, clamped and cast to it -- the cast is monotonic, so the code must
    lie between the codes of the window's ends.  Returns how many codes differ from the oracle's."""
    got_codes, ref_codes = np.asarray(got_codes, np.uint8), np.asarray(ref_codes, np.uint8)
    v = np.asarray(ref_value, np.float64)
    tol = np.maximum(np.abs(v) * 2.0 ** -7, abs_floor)      # 2 ulp of an 8-bit significand
    z = float(d_scale)
    def cast(x):
        t = (x / z if divides else x * z).astype(np.float32)
        return f8_value(dtypes.f32_to_f8e4m3fn(np.clip(t, -448, 448)))
    lo, hi = cast(v - tol), cast(v + tol)
    lo, hi = np.minimum(lo, hi), np.maximum(lo, hi)
    g = f8_value(got_codes)
    both_nan = np.isnan(g) & np.isnan(f8_value(ref_codes))
    bad = ~(((g >= lo) & (g <= hi)) | both_nan)
    if bad.any():
        idx = np.argwhere(bad)[:8]
        raise AssertionError("%s: %d of %d f8 codes outside the window: %s" % (
            what, int(bad.sum()), bad.size,
            [(tuple(i), float(g[tuple(i)]), float(lo[tuple(i)]), float(hi[tuple(i)])) for i in idx]))
    differ = int((got_codes != ref_codes).sum())
    FLOOR_LOG.append((what or "f8 result", "codes other than the oracle's (inside the window)", differ, int(bad.size)))
    return differ


def check_dot_f32(got_f32, ref_f32, abs_floor, what=""):
    """The same rule for a dot whose f32 value is the result itself: within 2 bf16 ulp of the oracle's
    value (2**-7 of its magnitude bounds that from below), or within `abs_floor`."""
    g = np.asarray(got_f32, np.float64)
    r = np.asarray(ref_f32, np.float64)
    assert g.shape == r.shape, (g.shape, r.shape)
    ok = np.abs(g - r) <= np.abs(r) * 2.0 ** -7
    near = np.abs(g - r) <= abs_floor
    both_nan = np.isnan(g) & np.isnan(r)
    bad = ~(ok | near | both_nan)
    if bad.any():
        idx = np.argwhere(bad)[:8]
        raise AssertionError("%s: %d of %d f32 outputs differ by more than 2 bf16 ulp (and the floor): %s"
                             % (what, int(bad.sum()), bad.size, [(tuple(i), float(g[tuple(i)]), float(r[tuple(i)])) for i in idx]))
    n_floor = int((~ok & near).sum())
    FLOOR_LOG.append((what or "dot (f32 result)", "within the floor only", n_floor, int(bad.size)))
    return n_floor
