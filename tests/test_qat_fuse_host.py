"""The library's DeepNetQAT (C++, host only) against the oracle's restatement on the trained LeNet-with-BatchNorm
parameters: both follow the reference's operand order and types, so every installed value must be identical."""
import numpy as np
import pytest

import sat_lenet as sl
from oracle import qat_fuse as qf


@pytest.fixture(scope="module")
def fh():
    from n2d2_amd import frame_hip
    return frame_hip


@pytest.mark.parametrize("name", ["w8a8", "w4a4"])
def test_the_pass_installs_the_oracle_s_values(fh, name):
    d = sl.load(name)
    want = sl.fuse_with_oracle(d, name)
    net = sl.fuse_with_library(fh, d, name, batch=2)
    for cell, f in want.items():
        assert np.array_equal(net.weights(cell).reshape(f["w"].shape), f["w"]), cell
        mode, frac, scaling = net.scaling(cell)
        assert mode == "FloatMult" and np.array_equal(scaling.astype(np.float32), f["scaling"]), cell
        assert np.array_equal(net.clipping(cell), f["clipping"]), cell
        assert net.quantized(cell) == (f["weight_bits"], f["act_bits"], f["kind"]), cell
        if f["bias"] is not None:
            assert np.array_equal(net.biases(cell), f["bias"]), cell
    # without an export precision nothing is unsigned; with the 8 bits fuseQATGraph sets, the Rectifier cells are
    try:
        fh.set_globals(8, True, True)
        assert [net.cell_info(c)["unsigned"] for c in ("conv1", "pool1", "conv3", "fc1", "fc2")] == [True, True, True, False, False]
    finally:
        fh.set_globals(0, True, False)


def test_fixed_point_and_shift_modes_of_the_conv_fuse(fh):
    d = sl.load("w4a4")
    want = sl.fuse_with_oracle(d, "w4a4")
    net = sl.fuse_with_library(fh, d, "w4a4", batch=2, mode="FixedMult16")
    for conv in ("conv1", "conv2", "conv3"):
        mode, frac, scaling = net.scaling(conv)
        # std::round(sc * 2^16) on the Float_T scaling, 16 fractional bits whatever the factor (DeepNetQAT.cpp:1248-1265)
        assert (mode, frac) == ("FixedMult16", 16)
        assert np.array_equal(scaling, np.floor(want[conv]["scaling"].astype(np.float64) * 65536 + 0.5))
        assert np.array_equal(net.clipping(conv), want[conv]["clipping"])
    net = sl.fuse_with_library(fh, d, "w4a4", batch=2, mode="SingleShift")
    for conv in ("conv2", "conv3"):
        mode, _, shifts = net.scaling(conv)
        # approximateScalingWithPowerOf2Divs with one division, per output
        assert mode == "SingleShift"
        assert [fh.approximate_scaling_with_power_of_2_divs(float(v), 1)[0][0] for v in want[conv]["scaling"]] == list(shifts)


def test_the_pass_declines_what_the_reference_declines(fh):
    d = sl.load("w4a4")
    conv, bn, shape, w_range = sl.conv_stages("w4a4")[0]
    wq = sl.quantized_conv_weights(d, conv, shape, w_range)
    net = fh.Net(sl.INI % 2)
    # a BatchNorm whose activation has no SAT quantizer is not fused, and the cell is left alone
    fused, ranges, alphas = net.fuse_batchnorm_with_conv(conv, (255, 255), (1.0, 1.0), wq, None, w_range, True, *sl.bn_of(d, bn), sl.EPS, None, None)
    assert not fused and ranges == (255, 255) and net.quantized(conv) == (0, 0, "Linear") and net.weights(conv).size == 0
    # a convolution with a non-linear activation neither
    net2 = fh.Net((sl.INI % 2).replace("NbOutputs=6\nActivationFunction=Linear", "NbOutputs=6\nActivationFunction=Rectifier"))
    fused, _, _ = net2.fuse_batchnorm_with_conv(conv, (255, 255), (1.0, 1.0), wq, None, w_range, True, *sl.bn_of(d, bn), sl.EPS, 15, 5.0)
    assert not fused
    with pytest.raises(fh.FrameHipError) as e:              # weights of another cell
        net.fuse_batchnorm_with_conv("conv2", (255, 255), (1.0, 1.0), wq[:5], None, w_range, True, *sl.bn_of(d, "bn2"), sl.EPS, 15, 5.0)
    assert "do not match the outputs of conv2" in str(e.value)
    with pytest.raises(fh.FrameHipError):
        net.quantize_fc("conv1", (15, 15), (1.0, 1.0), np.zeros((6, 25)), None, 15, 1.0, 15, 5.0)


def test_without_rounding_the_pass_installs_the_unscaled_values(fh):
    # WeightsApprox::NONE keeps the quantized weights as they are (floats): the pass installs them as the reference
    # does; the integer cells refuse them at initialize (covered with the GPU tests)
    d = sl.load("w4a4")
    net = sl.fuse_with_library(fh, d, "w4a4", batch=2, rounding=False)
    want = sl.fuse_with_oracle(d, "w4a4", rounding=False)
    for cell, f in want.items():
        assert np.array_equal(net.weights(cell).reshape(f["w"].shape), f["w"]) and not np.array_equal(f["w"], np.rint(f["w"])), cell
        assert np.array_equal(net.scaling(cell)[2].astype(np.float32), f["scaling"]), cell
        assert np.array_equal(net.clipping(cell), f["clipping"]), cell


def test_elemwise_pass(fh):
    ini = (sl.INI % 2) + "\n[sum]\nInput=pool1,pool1\nType=ElemWise\nNbOutputs=6\nOperation=Sum\nActivationFunction=Linear\n"
    net = fh.Net(ini)
    ranges, alphas = net.quantize_elemwise("sum", (255, 255), (9.0, 9.0), 15, 3.0, 15, 5.0)
    s, c, bits, r, a = qf.quantize_elemwise((255, 255), (9.0, 9.0), 15, 3.0, 6, 15, 5.0)
    assert (ranges, alphas) == (r, a) == ((15, 15), (5.0, 5.0))
    assert np.array_equal(net.scaling("sum")[2].astype(np.float32), s) and np.array_equal(net.clipping("sum"), c)
    assert net.quantized("sum") == (bits, 0, "Rectifier")
