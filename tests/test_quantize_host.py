"""The numpy quantizers that feed benchmarks must produce exactly the oracle's bytes."""
import numpy as np

import ggufref as G
from openagents_amd import quantize


def test_numpy_q4_0_and_q8_0_match_oracle_bit_for_bit(orc):
    w = G.seeded_weights(700, 64, 2048)
    w[0, :32] = 0
    w[1, :32] = np.float32(0.5) * (np.arange(32) % 16 - 8)
    w[2, :4] = [8, -7, -8, 0]
    w[3, 5] = 1.0
    w[3, 9] = -1.0                     # equal magnitudes: the first one sets the sign of d
    assert np.array_equal(quantize.quantize_q4_0(w), orc.quantize(orc.Q4_0, w))
    assert np.array_equal(quantize.quantize_q8_0(w), orc.quantize(orc.Q8_0, w))
    x = G.seeded_acts(701, 4, 4096)
    assert np.array_equal(quantize.quantize_q8_0(x), orc.quantize(orc.Q8_0, x))
    assert np.array_equal(quantize.quantize_q4_0(x), orc.quantize(orc.Q4_0, x))
