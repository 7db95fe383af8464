"""Exhaustive device-side checks of numerics shortcuts, through the library's self-check entry."""
import sys

import pytest

from xla_amd import ffi

pytestmark = pytest.mark.gpu


def test_tanh_scaling_free_division_equals_ieee_division_on_every_f32():
    """tanh_xla's quotient p / q through div_well_scaled against the plain f32 division, on all 2^32
    inputs: the epilogue keeps the reference's op-by-op value bit for bit."""
    print("[case] tanh division, all f32 inputs", flush=True)
    sys.stdout.flush()
    assert ffi.selfcheck_library().xla_amd_selfcheck_tanh_division_mismatches() == 0
