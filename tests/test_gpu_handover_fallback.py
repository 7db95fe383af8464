"""The bounded waits of the kernels that hand partial sums over between workgroups, on purpose: with
option "handover_test" = 1 the producing workgroups finish their work but never raise their flags and
the waiting workgroup gives up after a few polls, so its fallback -- the whole strip by a plain loop
(decode kernels), the second half of K by the same workgroup (tiled kernel) -- computes the result.
Every kernel exits normally; nothing spins without bound.  The result must match the oracle like any
other, and the next ordinary call on the same scratch must not take the abandoned run's flags or
sums for its own (the slot's generation has moved on)."""
import numpy as np
import pytest
import torch

from tests.test_gpu_dequant_dot import compare, run_dot, say
from xla_amd import ffi, workloads

pytestmark = pytest.mark.gpu


def run_with_dropped_flags(w, **kw):
    ffi.set_option("handover_test", 1)
    try:
        return run_dot(w, **kw)
    finally:
        ffi.set_option("handover_test", 0)


@pytest.mark.parametrize("M,K,N,group", [(8, 2048, 512, 128), (3, 1024 + 128, 800, 64), (16, 4096, 256, 128)])
def test_s4_pair_finisher_recomputes_its_strip(oracle, M, K, N, group):
    say("hand-over give-up, s4 pair M=%d K=%d N=%d" % (M, K, N))
    w = workloads.c2_s4_group(M=M, K=K, N=N, group=group)
    normal, kern = run_dot(w, pair=1)
    assert kern == "dequant_dot_decode_s4x_m16_pair", kern
    compare(oracle, w, normal, "s4 pair, ordinary run")
    alone, kern = run_with_dropped_flags(w, pair=1)
    assert kern == "dequant_dot_decode_s4x_m16_pair", kern
    compare(oracle, w, alone, "s4 pair, finisher gave up")
    again, _ = run_dot(w, pair=1)    # same scratch, next generation: the ordinary result, bit for bit
    assert np.array_equal(again, normal)


def test_u4_pair_finisher_recomputes_its_strip(oracle):
    say("hand-over give-up, u4 pair with zero points")
    w = workloads.u4_zero_point_group(M=8, K=2048, N=512, group=128)
    normal, kern = run_dot(w, pair=1)
    assert kern == "dequant_dot_decode_u4x_m16_pair", kern
    compare(oracle, w, normal, "u4 pair, ordinary run")
    alone, kern = run_with_dropped_flags(w, pair=1)
    assert kern == "dequant_dot_decode_u4x_m16_pair", kern
    compare(oracle, w, alone, "u4 pair, finisher gave up")


@pytest.mark.parametrize("strip", [128, 64])
@pytest.mark.parametrize("M,K,N,steps", [(16, 1024, 256, 1), (5, 2048, 136, 2), (16, 4096, 384, 4)])
def test_s8_last_slice_recomputes_its_strip(oracle, M, K, N, steps, strip):
    say("hand-over give-up, s8 slices M=%d K=%d N=%d steps=%d strip=%d" % (M, K, N, steps, strip))
    w = workloads.c1_s8_channel(M=M, K=K, N=N)
    name = "dequant_dot_decode_s8x_m16_%ss%d" % ("n64_" if strip == 64 else "", steps)
    normal, kern = run_dot(w, steps=steps, strip=strip)
    assert kern == name, kern
    compare(oracle, w, normal, "s8 slices, ordinary run")
    alone, kern = run_with_dropped_flags(w, steps=steps, strip=strip)
    assert kern == name, kern
    compare(oracle, w, alone, "s8 slices, last slice gave up")
    again, _ = run_dot(w, steps=steps, strip=strip)
    assert np.array_equal(again, normal)


@pytest.mark.parametrize("dtype", ["s8", "s4"])
def test_tiled_first_half_does_the_second_half_itself(oracle, dtype):
    say("hand-over give-up, tiled kernel split last round, %s" % dtype)
    M, K, N = 128, 2048, 1024       # 4 tiles, every one split along K
    w = workloads.c1_s8_channel(M=M, K=K, N=N) if dtype == "s8" else workloads.c2_s4_group(M=M, K=K, N=N, group=128)
    normal, kern = run_dot(w, force_kernel=3)
    assert kern.endswith(":tail2"), kern
    compare(oracle, w, normal, "tiled split tail, ordinary run")
    alone, kern = run_with_dropped_flags(w, force_kernel=3)
    assert kern.endswith(":tail2"), kern
    compare(oracle, w, alone, "tiled split tail, first half gave up")
    whole, kern = run_dot(w, force_kernel=3, tail=1)   # unsplit tiles sum K in the order the give-up path uses
    assert not kern.endswith(":tail2"), kern
    assert np.array_equal(alone, whole)
    again, _ = run_dot(w, force_kernel=3)
    assert np.array_equal(again, normal)
