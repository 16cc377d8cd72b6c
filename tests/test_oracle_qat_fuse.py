"""Pins the oracle's restatement of the pass from a SAT-trained float graph to integer cells (oracle/qat_fuse.py) on the
trained LeNet-with-BatchNorm parameters N2D2's own test of that pass loads (tests/Quantizer/QAT/Optimization/
class_DeepNetQAT.cpp:96-140 checks that the recognition rate survives the pass; without the MNIST images the same claim
is checked here on the levels themselves): every fused stage, run on the oracle's integer cells, must give the levels the
float stage (convolution with the quantized weights, BatchNorm in inference, SAT activation quantizer) gives from the
same input.  The two differ only where rounding the weights, the bias and the clip to integers moves a value across a
rounding boundary: by one level, rarely.  A wrong sign, a dropped term or swapped (range, alpha) pairs move every output."""
import numpy as np
import pytest

import sat_lenet as sl
from oracle import cells, oracle as o, qat_fuse as qf


@pytest.mark.parametrize("name", ["w8a8", "w4a4"])
def test_trained_weights_quantize_onto_the_exported_level_grid(name):
    # the *_quant_weights files are one solver step older than the weights: same grid, a few elements one level apart
    d = sl.load(name)
    for conv, _, shape, w_range in sl.conv_stages(name)[:2]:
        wq = sl.quantized_conv_weights(d, conv, shape, w_range)
        exported = d[conv + "_quant_weights"].reshape(shape)
        levels = (wq - exported) * np.float32(w_range / 2.0)
        assert np.abs(levels - np.rint(levels)).max() < 1e-3
        assert np.abs(levels).max() <= 1.001 and (np.rint(levels) == 0).mean() > 0.75


@pytest.mark.parametrize("name", ["w8a8", "w4a4"])
def test_fused_conv_stages_reproduce_the_float_graph(name):
    d = sl.load(name)
    fused = sl.fuse_with_oracle(d, name)
    x = sl.images(16, seed=5)
    y = sl.integer_graph(fused, x)
    R = sl.act_range(name)
    chain = (x / np.float32(255)).astype(np.float32)             # the float graph end to end, from the [0, 1] stimuli
    for (conv, bn, shape, w_range), src in zip(sl.conv_stages(name), ("input", "pool1", "pool2")):
        f = fused[conv]
        xin = x if src == "input" else y[src]
        alpha = float(d[bn + "_QAct_SAT_Alpha"][0])
        assert (f["in_range"], f["out_range"]) == (255 if src == "input" else R, R)
        assert np.array_equal(f["w"], np.rint(f["w"])) and np.array_equal(f["bias"], np.rint(f["bias"]))
        xf = (xin * np.float32(f["in_alpha"] / f["in_range"])).astype(np.float32)
        # (1) the float stage with the weights the integer cell holds, mapped back: only bias and clip rounding differ
        wsf = 15.0 if w_range == 15 else np.floor(w_range / 2.0)
        exact = sl.float_conv_stage(xf, (f["w"] / np.float32(wsf)).astype(np.float32), sl.bn_of(d, bn), alpha, R)
        diff = y[conv] - exact
        assert np.abs(diff).max() <= 1 and (diff != 0).mean() < 0.004, (conv, np.abs(diff).max(), (diff != 0).mean())
        # (2) the float stage as trained: 8-bit default-mode weights (2k-255)/255 are not multiples of 1/127, so
        # rounding them moves more outputs by a level; 4-bit ones are kept exactly (the 15 / 31 correction)
        trained = sl.float_conv_stage(xf, f["wq"], sl.bn_of(d, bn), alpha, R)
        diff = y[conv] - trained
        assert np.abs(diff).max() <= (2 if w_range == 255 else 1)
        assert (diff != 0).mean() < (0.12 if w_range == 255 else 0.004), (conv, (diff != 0).mean())
        # (3) end to end
        chain = sl.float_conv_stage(chain, f["wq"], sl.bn_of(d, bn), alpha, R)
        assert np.abs(y[conv] - chain).max() <= 2 and (y[conv] != chain).mean() < 0.2
        assert np.unique(y[conv]).size > 4                       # the comparison is not between constant maps
        chain = (chain * np.float32(alpha / R)).astype(np.float32)
        if conv != "conv3":
            chain = o.pool_forward(chain, (2, 2), (2, 2), kind="max", quantized=False)


def test_four_bit_default_mode_weights_are_carried_on_five_bits():
    d = sl.load("w4a4")
    fused = sl.fuse_with_oracle(d, "w4a4")
    for conv in ("conv2", "conv3"):
        w = fused[conv]["w"]
        assert np.all(np.abs(w) % 2 == 1) and np.abs(w).max() == 15          # odd multiples of 1/15, times 15
        assert np.array_equal(w, np.rint(fused[conv]["wq"] * np.float32(15)))
        assert fused[conv]["weight_bits"] == 4 and fused[conv]["act_bits"] == 4
    assert fused["conv1"]["weight_bits"] == 8 and np.abs(fused["conv1"]["w"]).max() == 127


def test_negative_and_vanishing_batchnorm_factors():
    d = sl.load("w4a4")
    conv, bn, shape, w_range = sl.conv_stages("w4a4")[1]
    scales, biases, means, variances = [v.copy() for v in sl.bn_of(d, bn)]
    scales[::2] *= -1                      # every other channel: negative gamma
    biases[::2] = np.abs(biases[::2]) + 1  # ... whose outputs would otherwise all clamp to 0
    variances[5] = 0.0                     # a channel that never saw data
    wq = sl.quantized_conv_weights(d, conv, shape, w_range)
    alpha, a1 = float(d[bn + "_QAct_SAT_Alpha"][0]), float(d["bn1_QAct_SAT_Alpha"][0])
    W, B, S, Cl, _, ab, ranges, alphas = qf.quantize_and_fuse_batchnorm_with_conv(
        (15, 15), (a1, a1), wq, None, w_range, True, scales, biases, means, variances, sl.EPS, 15, alpha)
    assert np.all(S[np.arange(16) != 5] > 0) and np.all(Cl[np.arange(16) != 5] > 0) and (S[5], B[5], Cl[5]) == (0, 0, 0)
    assert np.array_equal(W[0], -np.rint(wq[0] * np.float32(15))) and np.array_equal(W[1], np.rint(wq[1] * np.float32(15)))
    x = np.random.default_rng(8).integers(0, 16, size=(8, 6, 14, 14)).astype(np.float32)
    y = cells.conv_cell(x, W, B, cells.ActSpec("Rectifier", "FloatMult", S, 0, Cl, ab, True))
    keep = np.arange(16) != 5
    want = sl.float_conv_stage((x * np.float32(a1 / 15)).astype(np.float32), wq, (scales, biases, means, variances), alpha, 15)
    diff = (y - want)[:, keep]
    assert np.abs(diff).max() <= 1 and (diff != 0).mean() < 0.004
    assert np.unique(y[:, 0]).size > 2 and np.all(y[:, 5] == 0)
    assert ranges == (15, 15) and alphas == (np.float32(alpha), np.float32(alpha))


@pytest.mark.parametrize("name", ["w8a8", "w4a4"])
def test_fused_fc_stages_follow_the_float_graph_up_to_the_signed_saturation(name):
    # The Fc cells keep their Linear activation, whose output N2D2 takes as signed: the clip keeps [0, alpha] as the float
    # graph does, and the saturation then cuts at 2^(bits-1) - 1 (127 of 255 levels, 7 of 15).
    d = sl.load(name)
    fused = sl.fuse_with_oracle(d, name)
    y = sl.integer_graph(fused, sl.images(64, seed=6))
    for (fc, shape, w_range, a_range), src in zip(sl.fc_stages(name), ("conv3", "fc1")):
        f = fused[fc]
        alpha = float(d[fc + "_QAct_SAT_Alpha"][0])
        xf = (y[src] * np.float32(f["in_alpha"] / f["in_range"])).astype(np.float32).reshape(64, -1, 1, 1)
        wsf = np.floor(w_range / 2.0)
        w_back = (f["w"].astype(np.float64) / (wsf * f["sat"])).astype(np.float32)
        z = o.conv_forward(xf, w_back.reshape(shape + (1, 1)))
        a, _ = o.sat_act_forward(z, a_range, alpha, True)
        top = (1 << (f["act_bits"] - 1)) - 1
        want = np.minimum(np.rint(a * np.float32(a_range / alpha)), top)
        diff = y[fc] - want
        assert np.abs(diff).max() <= 1 and (diff != 0).mean() < 0.01, (fc, np.abs(diff).max(), (diff != 0).mean())
        assert y[fc].min() == 0 and y[fc].max() == top and np.unique(y[fc]).size > 4
        assert np.array_equal(f["w"], np.rint(f["w"])) and np.abs(f["w"]).max() <= wsf        # the SAT divisor cancels


def test_fc_without_activation_quantizer_and_with_bias():
    rng = np.random.default_rng(9)
    wq = (rng.integers(-7, 8, size=(5, 12)) / 7.0).astype(np.float32)
    bias = rng.normal(0, 0.5, size=5).astype(np.float32)
    W, B, S, Cl, clipped, wb, ab, ranges, alphas = qf.quantize_fc((15, 255), (4.0, 1.0), wq, bias, 15, 1.0, None, None)
    assert not clipped and (wb, ab) == (4, 32) and ranges == (255, 255) and alphas == (1.0, 1.0)
    x = rng.integers(0, 16, size=(3, 12)).astype(np.float64)
    # without an activation quantizer the outputs are the float graph's times the input range (not range / alpha:
    # `scaleFactorOutput = rangeOpFc.first`, DeepNetQAT.cpp:760); the integer cell holds them times 7 before the Scaling
    want = ((x * 4.0 / 15) @ wq.astype(np.float64).T + bias) * 15
    got = (x @ W.astype(np.float64).T + B) * S[0]
    assert np.allclose(got, want, atol=0.5 * 4 / 7 + 1e-6) and np.abs(want).max() > 50      # half a unit of the rounded bias
    assert np.array_equal(W, np.rint(wq * 7)) and np.array_equal(B, np.rint(bias * np.float32(15 / 4.0 * 7)))


def test_elemwise_sum_takes_its_first_parent_s_levels():
    s, c, bits, ranges, alphas = qf.quantize_elemwise((255, 255), (9.0, 9.0), 15, 3.0, 4, 15, 5.0)
    assert bits == 4 and ranges == (15, 15) and alphas == (5.0, 5.0)
    a = np.arange(0, 16, dtype=np.float64)[:, None]
    b = np.arange(0, 16, dtype=np.float64)[None, :]
    want = np.rint(np.clip((a + b) * 3.0 / 15, 0, 5.0) / 5.0 * 15)           # the float graph on levels of alpha 3, range 15
    got = np.rint(np.clip(a + b, 0, c[0]) * s[0])
    assert np.array_equal(got, want) and c[0] == np.float32(25.0) and s[0] == np.float32(0.6)
