"""Pins the SAT / LSQ part of the CPU oracle: closed forms restated by the
reference's own unit tests, data files held by the reference's tests,
structural invariants and finite differences."""
import os

import numpy as np
import pytest

import refmath as rm
from oracle import oracle as orc

RNG = np.random.default_rng(77)
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sat_lenet4b")


# ------------------------------------------------------------ SAT weights

def test_sat_default_matches_reference_unit_test_formula():
    # tests/Quantizer/QAT/Cell/class_SATQuantizerCell_Frame_CUDA.cpp:108-146
    w = RNG.uniform(-1, 1, size=(8, 4, 3, 3)).astype(np.float32)
    rng = 2.0 ** 4
    t = np.tanh(w.astype(np.float64))
    m = np.abs(t).max()
    wq = 2.0 * ((1.0 / rng) * np.rint(0.5 * ((t / m) + 1.0) * rng)) - 1.0
    got, tmax, _ = orc.sat_weight_forward(w, rng, "default")
    assert abs(tmax - m) < 1e-6
    assert np.max(np.abs(got - wq)) < 1e-6        # reference test uses 1e-3
    # with SAT scaling: divide by sqrt(var_unbiased * dimB*dimY*dimX)
    outputs_size = 8 * 3 * 3
    scal = np.sqrt(wq.var(ddof=1) * outputs_size)
    got_s, _, s = orc.sat_weight_forward(w, rng, "default", apply_scaling=True, outputs_size=outputs_size)
    assert abs(s - scal) / scal < 1e-5
    assert np.max(np.abs(got_s - wq / scal)) < 1e-5
    # backward: dW = dWq * sech^2(w) / (tanh_max * scaling)
    dwq = RNG.normal(size=w.shape).astype(np.float32)
    want = dwq / np.cosh(w.astype(np.float64)) ** 2 / (m * scal)
    got_b = orc.sat_weight_backward(dwq, w, rng, tmax * s, "default")
    assert np.max(np.abs(got_b - want) / (np.abs(want) + 1e-6)) < 1e-5


@pytest.mark.parametrize("mode,rng", [("symrange", 15.0), ("symrange", 255.0), ("default", 15.0), ("default", 255.0),
                                      ("fullrange", 15.0), ("asymrange", 15.0)])
def test_sat_weight_grid_and_invariants(mode, rng):
    w = RNG.normal(0, 0.05, size=(16, 8, 3, 3)).astype(np.float32)
    wq, tmax, _ = orc.sat_weight_forward(w, rng, mode)
    assert abs(tmax - np.abs(np.tanh(w.astype(np.float64))).max()) < 1e-7
    if mode == "symrange":
        r2 = np.floor(rng / 2)
        levels = wq.astype(np.float64) * r2
        assert np.max(np.abs(levels - np.rint(levels))) < 1e-5
        assert np.abs(wq).max() == pytest.approx(1.0, abs=1e-6)          # the max maps to +-1
        neg, _, _ = orc.sat_weight_forward(-w, rng, mode)
        assert np.array_equal(neg, -wq)                                   # odd function
        assert len(np.unique(np.rint(levels))) <= 2 * r2 + 1
    if mode == "default":
        levels = (wq.astype(np.float64) + 1.0) / 2.0 * rng
        assert np.max(np.abs(levels - np.rint(levels))) < 1e-4
        assert wq.min() >= -1.0 and wq.max() <= 1.0
    if mode == "fullrange":
        assert wq.min() >= -1.0 - 1e-6 and wq.max() <= 1.0 + 1e-6
    if mode == "asymrange":
        r2 = np.floor(rng / 2)
        assert wq.min() >= -1.0 - 1.0 / r2 - 1e-6 and wq.max() <= 1.0 + 1e-6
    # unquantized twin: |wq - w_noq| is at most half a level (symrange / default)
    if mode in ("symrange", "default"):
        noq, _, _ = orc.sat_weight_forward(w, rng, "none")
        step = 1.0 / np.floor(rng / 2) if mode == "symrange" else 2.0 / rng
        assert np.max(np.abs(wq - noq)) <= step / 2 + 1e-6


def _weights_for_normalised(qn, wmax=1.2):
    """float32 weights whose tanh(w) / max|tanh w| equals qn (float64 target), the maximum supplied by a first element."""
    w = np.arctanh(np.clip(np.asarray(qn, np.float64), -1, 1) * np.tanh(wmax) * (1 - 1e-12))
    return np.concatenate([[wmax], w]).astype(np.float32)


@pytest.mark.parametrize("rng", [15.0, 255.0, 3.0])
def test_sat_fullrange_forward_closed_form(rng):
    """quantize_weight_fullrange_propagate (src/Quantizer/QAT/Kernel/SATQuantizer_Frame_Kernels.cpp:117-146) in float64:
    q = (t/m + 1)/2; level = rint((R + 0.9998) q - 0.4999); w_q = 2 level / R - 1.  Exact values away from ties, the grid,
    and probes on both sides of the first and last bin edges, which sit at q = (k + 0.9999) / (R + 0.9998): with the
    offset dropped, with 1/(2R) in its place, or with the slope 1 + 1/R, a probe lands on the other level."""
    w = RNG.normal(0, 0.6, size=6000).astype(np.float32)
    t = np.tanh(w.astype(np.float64))
    m = np.abs(t).max()
    arg = (rng + 0.9998) * (0.5 * (t / m + 1.0)) - 0.4999
    safe = np.abs(arg - np.floor(arg) - 0.5) > 1e-3
    want = 2.0 * np.rint(arg) / rng - 1.0
    got, tmax, _ = orc.sat_weight_forward(w, rng, "fullrange")
    assert abs(tmax - m) < 1e-7 and safe.sum() > 0.99 * w.size
    assert np.max(np.abs(got[safe] - want[safe])) < 5e-7
    lev = (got.astype(np.float64) + 1.0) / 2.0 * rng
    assert np.max(np.abs(lev - np.rint(lev))) < 1e-4
    seen = set(np.rint(lev).astype(int).tolist())
    assert seen <= set(range(int(rng) + 1)) and (rng > 15 or len(seen) == rng + 1)    # levels 0..R, nothing outside
    # the ends: t/m = -1 -> level 0, t/m = +1 -> level R, i.e. exactly -1 and +1
    ends, _, _ = orc.sat_weight_forward(np.array([-1.2, 1.2], np.float32), rng, "fullrange")
    assert ends.tolist() == [-1.0, 1.0]
    # probes 3e-5 of a level on either side of every bin edge
    k = np.arange(int(rng))
    for side, expect in ((-3e-5, k), (3e-5, k + 1)):
        q = (k + 0.9999 + side) / (rng + 0.9998)
        probe, _, _ = orc.sat_weight_forward(_weights_for_normalised(2 * q - 1), rng, "fullrange")
        lv = np.rint((probe[1:].astype(np.float64) + 1.0) / 2.0 * rng).astype(int)
        assert lv.tolist() == expect.tolist(), (side, rng)
    # the edges are NOT those of the plain rounding of the default mode (q = (k + 0.5) / R): on those the two modes differ
    q = (k + 0.5 + 0.2 * (0.5 - (k + 0.5) / rng)) / rng        # between the default edge and the full-range edge
    pr_f, _, _ = orc.sat_weight_forward(_weights_for_normalised(2 * q - 1), rng, "fullrange")
    pr_d, _, _ = orc.sat_weight_forward(_weights_for_normalised(2 * q - 1), rng, "default")
    assert np.count_nonzero(pr_f[1:] != pr_d[1:]) >= k.size - 1


@pytest.mark.parametrize("rng", [15.0, 255.0, 7.0])
def test_sat_asymrange_forward_closed_form(rng):
    """quantize_weight_asymrange_propagate (SATQuantizer_Frame_Kernels.cpp:188-214) in float64: R' = floor(R/2);
    level = rint((R' + 1/2) t/m - 1/2) in [-R'-1, R']; w_q = level / R'.  Bin edges at t/m = (k + 1) / (R' + 1/2)."""
    r2 = np.floor(rng / 2)
    w = RNG.normal(0, 0.6, size=6000).astype(np.float32)
    t = np.tanh(w.astype(np.float64))
    m = np.abs(t).max()
    arg = (r2 + 0.5) * (t / m) - 0.5
    safe = np.abs(arg - np.floor(arg) - 0.5) > 1e-3
    want = np.rint(arg) / r2
    got, tmax, _ = orc.sat_weight_forward(w, rng, "asymrange")
    assert abs(tmax - m) < 1e-7 and safe.sum() > 0.99 * w.size
    assert np.max(np.abs(got[safe] - want[safe])) < 5e-7
    lev = got.astype(np.float64) * r2
    assert np.max(np.abs(lev - np.rint(lev))) < 1e-4
    seen = set(np.rint(lev).astype(int).tolist())
    assert seen <= set(range(-int(r2) - 1, int(r2) + 1)) and (rng > 15 or len(seen) == rng + 1)   # R + 1 levels, one more below
    ends, _, _ = orc.sat_weight_forward(np.array([-1.2, 1.2], np.float32), rng, "asymrange")
    assert ends.tolist() == [float(np.float32(-r2 - 1) * (np.float32(1.0) / np.float32(r2))), 1.0]
    k = np.arange(-int(r2) - 1, int(r2))
    for side, expect in ((-3e-5, k), (3e-5, k + 1)):
        qn = (k + 1 + side) / (r2 + 0.5)
        probe, _, _ = orc.sat_weight_forward(_weights_for_normalised(qn), rng, "asymrange")
        assert np.rint(probe[1:].astype(np.float64) * r2).astype(int).tolist() == expect.tolist(), (side, rng)
    # the un-rounded twin is the same affine map
    noq, _, _ = orc.sat_weight_forward(w, rng, "none_asym")
    assert np.max(np.abs(noq - (arg / r2))) < 1e-6



def test_sat_symrange_rint_is_half_to_even():
    # Find float32 inputs whose normalised value times 7 is an exact tie k+0.5 and
    # check they land on the even neighbour (rintf), not away from zero (roundf).
    r2 = np.float32(7.0)
    wmax = np.float32(1.2)
    centers = np.arctanh(np.array([0.5, 1.5, 2.5, 3.5, 4.5]) / 7.0 * np.tanh(1.2))
    cand = np.concatenate([c + np.linspace(-2e-5, 2e-5, 200001) for c in centers]).astype(np.float32)
    w = np.concatenate([[wmax], cand, -cand]).astype(np.float32)
    noq, _, _ = orc.sat_weight_forward(w, 15.0, "none")              # tanh(w)/max as the oracle computes it
    scaled = (noq * r2).astype(np.float32)                            # the argument handed to rintf
    ties = np.flatnonzero(np.abs(scaled - np.trunc(scaled)) == 0.5)
    assert ties.size >= 4
    wq, _, _ = orc.sat_weight_forward(w, 15.0, "symrange")
    even = np.rint(scaled[ties])                                      # numpy rint: half to even
    assert not np.array_equal(even, rm.round_half_away(scaled[ties]))  # the two roundings differ on this set
    assert np.array_equal(wq[ties], (np.float32(1.0) / r2) * even.astype(np.float32))


@pytest.mark.parametrize("layer,rng,max_frac", [("conv1", 255.0, 0.10), ("conv2", 15.0, 0.005)])
def test_sat_symrange_reproduces_reference_exported_weights(layer, rng, max_frac):
    """Data held by the reference's tests: full-precision and exported quantized
    weights of a SAT-trained LeNet (QuantMode=Symmetric). The exported quantized
    tensor is one SGD step staler, so a small fraction may sit one level off."""
    w = rm.read_syntxt(os.path.join(GOLD, layer + "_weights.syntxt")).astype(np.float32)
    ref = rm.read_syntxt(os.path.join(GOLD, layer + "_quant_weights.syntxt"))
    wq, _, _ = orc.sat_weight_forward(w, rng, "symrange")
    r2 = np.floor(rng / 2)
    d = np.rint((wq.astype(np.float64) - ref) * r2)
    assert np.max(np.abs((wq - ref) * r2 - d)) < 1e-3       # differences are whole levels
    assert np.abs(d).max() <= 1
    assert np.count_nonzero(d) <= max_frac * w.size


def test_sat_scaling_reproduces_reference_exported_fc_weights():
    # fc2: Range=255 (final classifier), Symmetric, ApplyScaling=1; mOutputsSize = dimB*dimY*dimX = nbOutputs
    w = rm.read_syntxt(os.path.join(GOLD, "fc2_weights.syntxt")).astype(np.float32)
    ref = rm.read_syntxt(os.path.join(GOLD, "fc2_quant_weights_quant.syntxt"))
    wq, _, scal = orc.sat_weight_forward(w, 255.0, "symrange", apply_scaling=True, outputs_size=10)
    lev = np.rint((wq.astype(np.float64) - ref) * scal * 127.0)
    assert np.abs(lev).max() <= 1
    assert np.count_nonzero(lev) <= 0.10 * w.size
    assert np.max(np.abs((wq - ref) * scal * 127.0 - lev)) < 2e-2


@pytest.mark.parametrize("mode", ["default", "fullrange", "asymrange"])
def test_sat_weight_backward_matches_finite_differences_of_unrounded_map(mode):
    w = RNG.normal(0, 0.3, size=200)
    rng = 15.0
    eps = 1e-6
    k = int(np.argmax(np.abs(w)))          # the element that sets tanh_max: its derivative has an extra term
    twin = {"default": "none", "fullrange": "none", "asymrange": "none_asym"}[mode]

    def f(v):
        # un-rounded forward with tanh_max frozen (the reference treats it as a constant)
        t = np.tanh(v) / np.abs(np.tanh(w)).max()
        if mode == "default":
            return t
        if mode == "fullrange":
            return (1.0 + 0.9998 / rng) * t          # 2q-1 with q affine in t: slope factor on t
        r2 = np.floor(rng / 2)
        return (1.0 + 1.0 / (2 * r2)) * t - 1.0 / (2 * r2)
    num = (f(w + eps) - f(w - eps)) / (2 * eps)
    tmax = np.abs(np.tanh(w)).max()
    got = orc.sat_weight_backward(np.ones_like(w), w, rng, tmax, mode)
    mask = np.ones(w.size, bool)
    mask[k] = False
    assert np.max(np.abs(got[mask] - num[mask])) < 1e-6
    # the oracle's unquantized forward agrees with f (so f is the map being differentiated)
    if mode != "fullrange":
        noq, _, _ = orc.sat_weight_forward(w, rng, twin)
        assert np.max(np.abs(noq - f(w))) < 1e-7       # mode constants are float32 in the reference


# -------------------------------------------------------- SAT activations

@pytest.mark.parametrize("nb_bits,alpha", [(4, 6.0), (8, 2.0), (3, 1.5), (4, -1.5)])
def test_sat_activation_forward_reference_formula(nb_bits, alpha):
    # tests/Quantizer/QAT/Activation/class_SATQuantizerActivation_Frame.cpp:105-116
    rng = float(2 ** nb_bits - 1)
    x = RNG.uniform(-3, 9, size=5000).astype(np.float32)
    a = abs(alpha)
    hard = np.clip(x.astype(np.float64), 0.0, a)
    want = a * (1.0 / rng) * rm.round_half_away(rng * (hard / a))
    y, fp = orc.sat_act_forward(x, rng, alpha, inference=False)
    assert np.array_equal(fp, x)
    assert np.max(np.abs(y - want)) < 1e-5 * a
    lev = y.astype(np.float64) / a * rng
    assert np.max(np.abs(lev - np.rint(lev))) < 1e-4 and lev.min() >= 0 and lev.max() <= rng + 1e-4
    y2, none = orc.sat_act_forward(x, rng, alpha, inference=True)
    assert none is None and np.array_equal(y, y2)
    y3, _ = orc.sat_act_forward(y, rng, alpha)      # idempotent on the grid
    assert np.max(np.abs(y3 - y)) < 1e-6 * a


def test_sat_activation_round_is_half_away():
    rng, alpha = 16.0, 8.0                                       # powers of two: the ties are exact
    x = (np.array([0.5, 1.5, 2.5, 13.5]) * alpha / rng).astype(np.float32)
    y, _ = orc.sat_act_forward(x, rng, alpha)
    assert (y / alpha * rng).tolist() == [1, 2, 3, 14]


def test_sat_activation_backward_ste_edges_and_alpha_gradient():
    rng, alpha = 15.0, 6.0
    x = np.array([-1.0, 0.0, 1e-3, 3.0, 6.0, 6.0 + 1e-3, 2.2], dtype=np.float32)
    g = np.array([1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0], dtype=np.float32)
    dx, dalpha, terms = orc.sat_act_backward(g, x, rng, alpha)
    assert dx.tolist() == [0, 0, 3, 4, 5, 0, 7]                      # 0 < x <= alpha passes
    q = np.clip(x.astype(np.float64), 0, alpha) / alpha
    qr = rm.round_half_away(rng * q) / rng
    want_terms = np.where(x >= alpha, 1.0, qr - q) * g
    assert np.max(np.abs(terms - want_terms)) < 1e-6
    assert abs(dalpha - want_terms.sum()) < 1e-5
    _, d2, _ = orc.sat_act_backward(g, x, rng, alpha, beta=1.0, prev_diff_alpha=10.0)
    assert abs(d2 - (want_terms.sum() + 10.0)) < 1e-5


# -------------------------------------------------------------------- LSQ

def test_lsq_forward_backward_reference_formulas():
    # tests/Quantizer/QAT/Cell/class_LSQQuantizerCell_Frame.cpp:121-200 restates the same forms
    R = 15
    lo, hi = -((R + 1) >> 1), (R - 1) >> 1
    assert (lo, hi) == (-8, 7)
    step = 0.037
    w = RNG.normal(0, 0.2, size=4099).astype(np.float32)
    q = w.astype(np.float64) / np.float32(step)
    want = np.where(q <= lo, lo * step, np.where(q >= hi, hi * step, rm.round_half_away(q) * step))
    got = orc.lsq_forward(w, step, lo, hi)
    assert np.max(np.abs(got - want)) < 1e-6
    assert got.min() >= lo * step - 1e-6 and got.max() <= hi * step + 1e-6
    g = RNG.normal(size=w.size).astype(np.float32)
    dfp, ds = orc.lsq_backward(g, w, step, lo, hi)
    mask = (q > lo) & (q < hi)
    assert np.array_equal(dfp, np.where(mask, g, 0).astype(np.float32))
    terms = np.where(q <= lo, lo, np.where(q >= hi, hi, rm.round_half_away(q) - q)) * g
    assert abs(ds - terms.sum()) < 1e-5 * np.abs(terms).sum()
    # activation flavour: range [0, R]
    x = np.abs(w) * 3
    got = orc.lsq_forward(x, step, 0, R)
    qx = x.astype(np.float64) / np.float32(step)
    want = np.where(qx <= 0, 0.0, np.where(qx >= R, R * step, rm.round_half_away(qx) * step))
    assert np.max(np.abs(got - want)) < 1e-6


def test_lsq_round_half_away_and_strict_ste_bounds():
    step, lo, hi = 0.5, -8, 7
    x = np.array([0.25, 0.75, -0.25, -0.75, 3.5, -4.0, 3.4999, 10.0])     # /0.5 -> .5 ties and the bounds
    got = orc.lsq_forward(x, step, lo, hi)
    assert got.tolist() == [0.5, 1.0, -0.5, -1.0, 3.5, -4.0, 3.5, 3.5]
    dfp, _ = orc.lsq_backward(np.ones_like(x), x, step, lo, hi)
    assert dfp.tolist() == [1, 1, 1, 1, 0, 0, 1, 0]                      # q == lo or q == hi is masked
