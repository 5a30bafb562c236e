"""The arithmetic shortcuts of the activation quantizers, checked on the device itself."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_division_shortcuts_equal_ieee_division_for_every_float_in_their_range(hip):
    """rcp_rn / div_rn (a reciprocal approximation plus fused multiply-add corrections) stand in for the IEEE divisions
    of the Q8_0 and Q8_K quantizers: amax / 127, 1 / d, -127 / max, 1 / iscale.  The library's self-test kernel compares
    them with true division for all 1 677 721 601 floats between 2^-100 and 2^100, both signs: no bit may differ."""
    print("psn_selftest_arith", flush=True)
    counts = hip.selftest_arith()
    assert counts == [0] * 8, counts
