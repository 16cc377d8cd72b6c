"""The integer LeNet that the library's DeepNetQAT pass makes of the trained SAT parameters, run on the GPU through the
C++ Frame_HIP cells: every cell's output must equal, bit for bit, what the CPU oracle's integer cells compute from the
parameters the pass installed; and the whole chain, float graph -> pass -> GPU, must keep the float graph's levels."""
import numpy as np
import pytest

import sat_lenet as sl
from oracle import cells

pytestmark = pytest.mark.gpu

_DT = {"FloatMult": np.float32, "FixedMult16": np.int32, "FixedMult32": np.int32, "SingleShift": np.uint8}


@pytest.fixture(scope="module")
def fh():
    from n2d2_amd import frame_hip
    frame_hip.set_globals(8, True, True)          # fuseQATGraph sets CellExport::mPrecision to 8; stimuli are u8
    yield frame_hip
    frame_hip.set_globals(0, True, False)


def _oracle_graph(net, x):
    """The net's own parameters on the oracle's integer cells."""
    def act(cell):
        mode, frac, scaling = net.scaling(cell)
        _, ab, kind = net.quantized(cell)
        return cells.ActSpec(kind, mode, scaling.astype(_DT[mode]), frac, net.clipping(cell), ab, net.cell_info(cell)["unsigned"])

    def w(cell, shape):
        return net.weights(cell).reshape(shape)

    y = {}
    y["conv1"] = cells.conv_cell(x, w("conv1", (6, 1, 5, 5)), net.biases("conv1"), act("conv1"))
    y["pool1"] = cells.pool_cell(y["conv1"], "max", (2, 2), (2, 2))
    y["conv2"] = cells.conv_cell(y["pool1"], w("conv2", (16, 6, 5, 5)), net.biases("conv2"), act("conv2"))
    y["pool2"] = cells.pool_cell(y["conv2"], "max", (2, 2), (2, 2))
    y["conv3"] = cells.conv_cell(y["pool2"], w("conv3", (120, 16, 5, 5)), net.biases("conv3"), act("conv3"))
    y["fc1"] = cells.fc_cell(y["conv3"], w("fc1", (84, 120)), None, act("fc1"))
    y["fc2"] = cells.fc_cell(y["fc1"], w("fc2", (10, 84)), None, act("fc2"))
    return y


@pytest.mark.parametrize("name,mode", [("w8a8", "FloatMult"), ("w4a4", "FloatMult"), ("w4a4", "FixedMult16"), ("w4a4", "SingleShift")])
def test_fused_lenet_on_the_gpu_is_the_oracle_s_integer_graph(fh, name, mode):
    d = sl.load(name)
    x = sl.images(32, seed=11)
    net = sl.fuse_with_library(fh, d, name, batch=32, mode=mode)
    net.set_fusion(False)
    net.initialize()
    net.set_stimuli(x)
    net.propagate()
    want = _oracle_graph(net, x)
    for cell in ("conv1", "pool1", "conv2", "pool2", "conv3", "fc1", "fc2"):
        got = net.outputs(cell)
        assert np.array_equal(got, want[cell].reshape(got.shape)), cell
    assert np.unique(want["fc2"]).size > 4
    if mode == "FloatMult":
        # ... and those are the levels of the float graph, up to the rounding of weights, biases and clips
        R = sl.act_range(name)
        chain = (x / np.float32(255)).astype(np.float32)
        for (conv, bn, shape, w_range), pool in zip(sl.conv_stages(name), ("pool1", "pool2", None)):
            alpha = float(d[bn + "_QAct_SAT_Alpha"][0])
            levels = sl.float_conv_stage(chain, sl.quantized_conv_weights(d, conv, shape, w_range), sl.bn_of(d, bn), alpha, R)
            got = net.outputs(conv)
            # end to end the deviations add up: a few of 255 levels after three stages of rounded 8-bit weights, one of
            # 15 with the 4-bit weights, which the pass keeps exactly
            dev = np.abs(got - levels)
            assert dev.max() <= (6 if R == 255 else 1) and dev.mean() < (0.3 if R == 255 else 0.06), conv
            chain = (levels * np.float32(alpha / R)).astype(np.float32)
            if pool:
                from oracle import oracle as o
                chain = o.pool_forward(chain, (2, 2), (2, 2), kind="max", quantized=False)


def test_unrounded_weights_are_refused_at_initialize(fh):
    d = sl.load("w4a4")
    net = sl.fuse_with_library(fh, d, "w4a4", batch=2, rounding=False)
    with pytest.raises(fh.FrameHipError) as e:
        net.initialize()
        net.set_stimuli(sl.images(2, seed=1))
        net.propagate()
    assert "is not an integer" in str(e.value) and "quantize the network" in str(e.value)
