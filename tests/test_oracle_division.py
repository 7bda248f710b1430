"""The GPU computes sf = amax / 448 (or / 6) as q = a*y, q + fma(-C, q, a)*y with y = fl(1/C) instead
of an IEEE division.  This pins that shortcut: over EVERY positive float whose quotient is a normal
number the two agree bit for bit (checked on the CPU with a correctly rounded fmaf)."""
import pytest

from oracle import cref


@pytest.mark.parametrize('c', [448.0, 6.0])
def test_three_instruction_division_equals_ieee_division_for_every_float(c):
    # all positive normal floats: bit patterns 0x00800000 .. 0x7F800000, in 8 slices
    lo, hi = 0x00800000, 0x7F800000
    step = (hi - lo) // 8
    bad = 0
    for i in range(8):
        a = lo + i * step
        b = hi if i == 7 else a + step
        bad += cref.count_div_mismatches(c, a, b)
    assert bad == 0


@pytest.mark.parametrize('c', [448.0, 6.0])
def test_the_check_can_fail(c):
    """Negative control: without the fma correction (a * fl(1/C) alone) a large share of one binade
    differs from the IEEE quotient, and the same counter sees it."""
    n = 0x40000000 - 0x3F800000
    assert cref.count_div_mismatches(c, 0x3F800000, 0x40000000, uncorrected=True) > n // 10
