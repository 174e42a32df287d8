"""The product's rotary frequencies, on the host, against values worked by hand from the
reference's rule (J/inference/operation/RoPE.java:13-28): no twin of the formula is involved."""
import math

import pytest

from gpullama3_java_amd.config import Llama3RopeScaling
from gpullama3_java_amd.parts.rotary import frequencies

SC_8 = Llama3RopeScaling(8.0, 1.0, 4.0, 64)
SC_32 = Llama3RopeScaling(32.0, 1.0, 4.0, 8192)


def ratio(wavelen, sc):
    """Scaled over unscaled frequency of the second pair of a head of 4 whose wavelength is ``wavelen``
    (theta ** -0.5 == 2 pi / wavelen)."""
    theta = (wavelen / (2 * math.pi)) ** 2
    return float(frequencies(4, theta, sc)[1]) / float(frequencies(4, theta, None)[1])


# smooth = (old/wavelen - lo)/(hi - lo); scaled/base = (1 - smooth)/factor + smooth (RoPE.java:25-26):
# old 64, band 16..64: wavelen 32 -> smooth 1/3 -> 5/12; 25.6 -> 1/2 -> 9/16; 64/3 -> 2/3 -> 17/24.
# old 8192, factor 32: wavelen 4096 -> smooth 1/3 -> (2/3)/32 + 1/3 = 17/48.
@pytest.mark.parametrize("sc, wavelen, expect", [(SC_8, 32.0, 5 / 12), (SC_8, 25.6, 9 / 16), (SC_8, 64 / 3, 17 / 24),
                                                 (SC_32, 4096.0, 17 / 48)])
def test_interpolated_frequencies_at_points_worked_by_hand(sc, wavelen, expect):
    assert abs(ratio(wavelen, sc) - expect) < 2e-6


def test_the_three_branches_and_their_edges():
    assert ratio(8.0, SC_8) == 1.0 and ratio(15.99, SC_8) == 1.0            # short wavelengths keep their frequency
    assert abs(ratio(100.0, SC_8) - 1 / 8) < 1e-7                           # long ones are divided by the factor
    assert abs(ratio(16.01, SC_8) - 1.0) < 1e-3 and abs(ratio(63.99, SC_8) - 1 / 8) < 1e-4   # continuous at both edges
    last = 1.0
    for i in range(1, 48):                                                   # and falling in between
        r = ratio(16.0 + i, SC_8)
        assert r < last
        last = r


def test_unscaled_frequencies_are_powers_of_theta():
    f = frequencies(8, 10000.0, None)
    for n in range(4):
        assert abs(float(f[n]) - 10000.0 ** (-2 * n / 8)) < 1e-7 * float(f[n]) + 1e-12


def test_tables_are_shared_while_held_and_freed_with_their_last_holder():
    import gc

    from gpullama3_java_amd.config import RotarySpec
    from gpullama3_java_amd.parts.rotary import Rotary
    spec = RotarySpec(head_dim=8, theta=10000.0, scaling=None, pairing="half", max_positions=33)
    a, b = Rotary(spec, "cpu"), Rotary(spec, "cpu")
    assert a.cos is b.cos and a.cos.shape == (33, 4)
    n = len(Rotary._tables)
    del a, b
    gc.collect()
    assert len(Rotary._tables) == n - 1
