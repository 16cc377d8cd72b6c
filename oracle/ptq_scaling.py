"""TEST INFRASTRUCTURE, not product code: CPU restatement of the step of N2D2's post-training quantization that replaces a
floating-point rescale by an integer Scaling (src/DeepNetQuantization.cpp:1043-1134, 1147-1178, 1240-1278).  Only
tests import this module.

Pinned in tests/test_oracle_ptq.py by cases worked out by hand from the definitions (which a ceil/floor mix-up, a
dropped doubling or a wrong limit fail) and by the identities the construction guarantees: the fixed-point bit count is
the largest that fits, and the power-of-two terms sum to scaling * precision.  The reference holds no golden vectors
for these functions.
"""
import math

import numpy as np

INT16_MAX = 32767
INT32_MAX = 2147483647


def _round_half_away(x):
    """std::round."""
    return math.floor(x + 0.5) if x >= 0 else -math.floor(-x + 0.5)


def approximate_scaling_with_fixed_point(mode, scaling_per_output):
    """(mode, nbFractionalBits, int32 factors); mode is "FixedMult16" or "FixedMult32" and may come back changed
    (ref: src/DeepNetQuantization.cpp:1043-1093)."""
    sc = np.asarray(scaling_per_output, dtype=np.float32)
    limit = INT16_MAX if mode == "FixedMult16" else INT32_MAX
    max_scaling = float(sc.max())
    if max_scaling >= limit:
        if mode == "FixedMult16":
            return approximate_scaling_with_fixed_point("FixedMult32", scaling_per_output)
        raise RuntimeError("Max scaling (%g) doesn't fit in FIXED_MULT32." % max_scaling)
    nb_bits = min(int(math.floor(math.log(limit / max_scaling) / math.log(2.0))), 50)
    # float * 2^n is exact in binary floating point, whatever the width
    values = [int(_round_half_away(float(s) * float(1 << nb_bits))) for s in sc]
    return mode, nb_bits, values


def approximate_scaling_with_power_of_2_divs(scaling, nb_divisions):
    """(exponents, precision): scaling <= 1 as a sum of nb_divisions terms 2^-e, precision = sum / scaling
    (ref: src/DeepNetQuantization.cpp:1095-1134)."""
    scaling = float(np.float32(scaling))
    assert nb_divisions > 0 and 0.0 < scaling <= 1.0
    precision = 0.0
    exps = [0] * nb_divisions
    for i in range(nb_divisions):
        if precision == 1.0:
            exps[i - 1] += 1
            exps[i] = exps[i - 1]
        else:
            e = int(math.ceil(math.log2(1.0 / (scaling * (1.0 - precision)))))
            precision += 1.0 / (scaling * 2.0 ** e)
            exps[i] = e
    if precision >= 0.98:
        precision = 1.0
    elif precision < 1.0:
        precision += 1.0 / (scaling * 2.0 ** exps[-1])
        exps[-1] -= 1
    return exps, precision


def approximate_activation_scaling(scaling_per_output, mode):
    """What approximateActivationScaling leaves: (mode, scaling values, frac_bits, per-output factor applied to the
    cell's weights and biases) (ref: src/DeepNetQuantization.cpp:1147-1178, 1201-1287)."""
    sc = np.asarray(scaling_per_output, dtype=np.float32)
    if mode in ("SingleShift", "DoubleShift") and bool((sc > 1.0).any()):
        mode = "FixedMult16"
    ones = np.ones(len(sc), dtype=np.float32)
    if mode == "FloatMult":
        return mode, sc, 0, ones
    if mode in ("FixedMult16", "FixedMult32"):
        mode, nb_bits, values = approximate_scaling_with_fixed_point(mode, sc)
        return mode, np.asarray(values, dtype=np.int64), nb_bits, ones
    nb_div = 1 if mode == "SingleShift" else 2
    shifts, rescale = [], []
    for s in sc:
        exps, precision = approximate_scaling_with_power_of_2_divs(s, nb_div)
        rescale.append(np.float32(1 / precision))
        shifts.append(exps[0] if nb_div == 1 else (exps[1] - exps[0], exps[1]))
    return mode, np.asarray(shifts, dtype=np.int64), 0, np.asarray(rescale, dtype=np.float32)
