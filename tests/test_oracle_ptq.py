"""The oracle's restatement of N2D2's float -> integer scaling approximation (src/DeepNetQuantization.cpp:1043-1134)
against cases worked out by hand from the definitions and against the identities the construction guarantees; then
the C++ host code (DeepNetQuantization in the Frame_HIP glue) against the oracle.  No GPU involved."""
import math

import numpy as np
import pytest

from oracle import ptq_scaling as ref


def test_fixed_point_hand_cases():
    # max 0.5, int16 limit 32767: 0.5 * 2^15 = 16384 fits, 0.5 * 2^16 = 32768 does not
    assert ref.approximate_scaling_with_fixed_point("FixedMult16", [0.5, 0.25]) == ("FixedMult16", 15, [16384, 8192])
    # int32 limit: 0.5 * 2^31 = 2^30 fits, 2^32 * 0.5 does not
    assert ref.approximate_scaling_with_fixed_point("FixedMult32", [0.5, 0.125]) == ("FixedMult32", 31, [2 ** 30, 2 ** 28])
    # does not fit 16 bits at all: falls back to 32; 40000 * 2^15 = 1310720000 < 2^31 <= 40000 * 2^16
    assert ref.approximate_scaling_with_fixed_point("FixedMult16", [40000.0]) == ("FixedMult32", 15, [1310720000])
    # rounding is half away from zero: 0.3 * 2^16 = 19660.8 -> 19661; max 0.45 -> 2^16 * 0.45 = 29491.2 fits, 2^17 * 0.45 does not
    mode, bits, vals = ref.approximate_scaling_with_fixed_point("FixedMult16", [0.3, 0.45])
    assert (mode, bits) == ("FixedMult16", 16) and vals == [19661, 29491]
    # tiny scalings stop at 50 fractional bits
    assert ref.approximate_scaling_with_fixed_point("FixedMult32", [2.0 ** -40])[1] == 50
    with pytest.raises(RuntimeError):
        ref.approximate_scaling_with_fixed_point("FixedMult32", [3e9])


def test_fixed_point_takes_the_largest_bit_count_that_fits():
    rng = np.random.default_rng(5)
    for mode, limit in (("FixedMult16", 32767), ("FixedMult32", 2 ** 31 - 1)):
        for _ in range(200):
            sc = np.exp(rng.uniform(-12, 4, size=int(rng.integers(1, 9)))).astype(np.float32)
            m, bits, vals = ref.approximate_scaling_with_fixed_point(mode, sc)
            assert m == mode
            top = float(sc.max())
            assert top * 2.0 ** bits <= limit and (bits == 50 or top * 2.0 ** (bits + 1) > limit)
            assert all(abs(v - float(s) * 2.0 ** bits) <= 0.5 for v, s in zip(vals, sc))


def test_power_of_2_hand_cases():
    f = ref.approximate_scaling_with_power_of_2_divs
    # 0.5 = 2^-1 exactly
    assert f(0.5, 1) == ([1], 1.0)
    # 0.3: the first power of two not above it is 2^-2 = 0.25 (83 % of it, below the 98 % threshold), so the term is
    # doubled: 2^-1 = 0.5, which overshoots by 0.5 / 0.3
    e, p = f(0.3, 1)
    assert e == [1] and p == pytest.approx(0.5 / float(np.float32(0.3)), rel=1e-12)
    # 0.75 = 2^-1 + 2^-2
    assert f(0.75, 2) == ([1, 2], 1.0)
    # 1 = 2^0 is exact after one term: it is split into 2^-1 + 2^-1
    assert f(1.0, 2) == ([1, 1], 1.0)
    # 0.1: 2^-4 + 2^-5 = 0.09375 is 93.75 % of it: the last term is doubled, 2^-4 + 2^-4 = 0.125 = 1.25 x 0.1
    e, p = f(0.1, 2)
    assert e == [4, 4] and p == pytest.approx(0.125 / float(np.float32(0.1)), rel=1e-12)
    # 0.99 * 2^-3: one term 2^-3 would be 1 / 0.99 too much, so the greedy term is 2^-4 (50.5 %), then 2^-5 (+25.25 %):
    # 75.8 % < 98 %, the last term is doubled: 2^-4 + 2^-4 = 2^-3
    e, p = f(0.99 / 8, 2)
    assert e == [4, 4] and p == pytest.approx(1 / 0.99, rel=1e-6)


def test_power_of_2_terms_sum_to_scaling_times_precision():
    rng = np.random.default_rng(6)
    for nb in (1, 2, 3):
        for _ in range(300):
            s = float(np.float32(np.exp(rng.uniform(-9, 0))))
            e, p = ref.approximate_scaling_with_power_of_2_divs(s, nb)
            total = sum(2.0 ** -k for k in e)
            assert len(e) == nb and all(k >= 0 for k in e) and e == sorted(e)
            if p == 1.0:
                assert 0.98 * s <= total * (1 + 1e-12) and total <= s * (1 + 1e-12)     # snapped: within 2 % below
            else:
                assert p > 1.0 and total == pytest.approx(s * p, rel=1e-9)               # overshoots by exactly p
            assert total <= 2.0 * s                                                      # never more than double


def test_host_code_matches_the_oracle():
    fh = pytest.importorskip("n2d2_amd.frame_hip")
    rng = np.random.default_rng(7)
    for mode in ("FixedMult16", "FixedMult32"):
        for _ in range(100):
            sc = np.exp(rng.uniform(-12, 12, size=int(rng.integers(1, 9)))).astype(np.float32)
            want = ref.approximate_scaling_with_fixed_point(mode, sc)
            got = fh.approximate_scaling_with_fixed_point(mode, sc)
            assert got[0] == want[0] and got[1] == want[1] and list(got[2]) == want[2], (mode, sc)
    with pytest.raises(fh.FrameHipError) as e:
        fh.approximate_scaling_with_fixed_point("FixedMult32", [3e9])
    assert "does not fit a 32-bit multiplier" in str(e.value)      # a std::runtime_error, as in the reference
    for nb in (1, 2):
        for _ in range(300):
            s = float(np.float32(np.exp(rng.uniform(-9, 0))))
            want = ref.approximate_scaling_with_power_of_2_divs(s, nb)
            got = fh.approximate_scaling_with_power_of_2_divs(s, nb)
            assert got[0] == want[0] and got[1] == pytest.approx(want[1], rel=1e-12), (s, nb)
    assert math.isclose(fh.approximate_scaling_with_power_of_2_divs(1.0, 2)[1], 1.0)
