"""Helper of the QAT-fuse tests (not a test module): the LeNet with BatchNorm that N2D2's own test of the fuse pass loads
(tests/tests_data/mnist_model/LeNet-bn-SAT-8b.ini and LeNet-bn-SAT.ini), its trained parameters from
tests/golden/sat_lenet_bn, the float graph in inference and the pass over it with the CPU oracle."""
import os

import numpy as np

from oracle import cells, oracle as o, qat_fuse as qf

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sat_lenet_bn")
EPS = 1.0e-5     # BatchNormCell's default Epsilon (src/Cell/BatchNormCell.cpp:33)


def load(name):
    return dict(np.load(os.path.join(GOLDEN, name + ".npz")))


def act_range(name):
    return 255 if name == "w8a8" else 15


def conv_stages(name):
    """(conv, bn, weight shape [O, C, kH, kW], weight range): QWeight.Range is 255 for conv1 in both files."""
    R = act_range(name)
    return [("conv1", "bn1", (6, 1, 5, 5), 255), ("conv2", "bn2", (16, 6, 5, 5), R), ("conv3", "bn3", (120, 16, 5, 5), R)]


def fc_stages(name):
    """(fc, weight shape [O, K], weight range, activation range): fc2 keeps 255 / 255 in both files."""
    R = act_range(name)
    return [("fc1", (84, 120), R, R), ("fc2", (10, 84), 255, 255)]


def quantized_conv_weights(d, conv, shape, w_range):
    """What SATQuantizerCell (Default mode, ApplyScaling=0) makes of the trained weights at a propagate."""
    O, _, kH, kW = shape
    return o.sat_weight_forward(d[conv + "_weights"].reshape(shape), w_range, "default", False, O * kH * kW)[0]


def quantized_fc_weights(d, fc, shape, w_range):
    """ApplyScaling=1: (quantized weights, the divisor applied)."""
    wq, _, sat = o.sat_weight_forward(d[fc + "_weights"].reshape(shape + (1, 1)), w_range, "default", True, shape[0])
    return wq.reshape(shape), sat


def bn_of(d, bn):
    return d[bn + "_scales"], d[bn + "_biases"], d[bn + "_means"], d[bn + "_variances"]


def float_conv_stage(x, wq, bn, alpha, R):
    """Conv (no bias, Linear) -> BatchNorm (inference) -> SAT activation quantizer; returns the output levels."""
    z = qf.batchnorm_inference(o.conv_forward(x, wq), *bn, eps=EPS)
    a, _ = o.sat_act_forward(z, R, alpha, True)
    return np.rint(a * np.float32(R / alpha))


def images(n, seed):
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, size=(n, 1, 32, 32)) * (rng.random((n, 1, 32, 32)) < 0.3)
    return x.astype(np.float32)


def fuse_with_oracle(d, name, rounding=True):
    """The pass over the whole net as fuseQATGraph threads it (src/Quantizer/QAT/Optimization/DeepNetQAT.cpp:87-520):
    (ranges, alphas) start at (255, 255) / (1, 1); pooling cells leave them alone.  Returns {cell: dict}."""
    ranges, alphas = (255, 255), (1.0, 1.0)
    out = {}
    for conv, bn, shape, w_range in conv_stages(name):
        wq = quantized_conv_weights(d, conv, shape, w_range)
        r1, a1 = ranges[0], alphas[0]
        W, B, S, Cl, wb, ab, ranges, alphas = qf.quantize_and_fuse_batchnorm_with_conv(
            ranges, alphas, wq, None, w_range, True, *bn_of(d, bn), EPS, act_range(name), float(d[bn + "_QAct_SAT_Alpha"][0]),
            rounding, rounding, rounding)
        out[conv] = dict(w=W, bias=B, scaling=S, clipping=Cl, weight_bits=wb, act_bits=ab, wq=wq, in_range=r1, in_alpha=a1,
                         out_range=ranges[0], out_alpha=alphas[0], kind="Rectifier", unsigned=True)
    for fc, shape, w_range, a_range in fc_stages(name):
        wq, sat = quantized_fc_weights(d, fc, shape, w_range)
        r1, a1 = ranges[0], alphas[0]
        W, B, S, Cl, clipped, wb, ab, ranges, alphas = qf.quantize_fc(
            ranges, alphas, wq, None, w_range, sat, a_range, float(d[fc + "_QAct_SAT_Alpha"][0]), rounding, rounding, rounding)
        out[fc] = dict(w=W, bias=B, scaling=S, clipping=Cl if clipped else None, weight_bits=wb, act_bits=ab, wq=wq, sat=sat, in_range=r1,
                       in_alpha=a1, out_range=ranges[0], out_alpha=alphas[0], kind="Linear", unsigned=False)
    return out


def act_spec(f):
    return cells.ActSpec(f["kind"], "FloatMult", f["scaling"], 0, f["clipping"], f["act_bits"], f["unsigned"])


def integer_graph(fused, x):
    """The fused net on the oracle's integer cells; returns {cell: output} including the pooling cells."""
    y = {}
    y["conv1"] = cells.conv_cell(x, fused["conv1"]["w"], fused["conv1"]["bias"], act_spec(fused["conv1"]))
    y["pool1"] = cells.pool_cell(y["conv1"], "max", (2, 2), (2, 2))
    y["conv2"] = cells.conv_cell(y["pool1"], fused["conv2"]["w"], fused["conv2"]["bias"], act_spec(fused["conv2"]))
    y["pool2"] = cells.pool_cell(y["conv2"], "max", (2, 2), (2, 2))
    y["conv3"] = cells.conv_cell(y["pool2"], fused["conv3"]["w"], fused["conv3"]["bias"], act_spec(fused["conv3"]))
    y["fc1"] = cells.fc_cell(y["conv3"], fused["fc1"]["w"], fused["fc1"]["bias"], act_spec(fused["fc1"]))
    y["fc2"] = cells.fc_cell(y["fc1"], fused["fc2"]["w"], fused["fc2"]["bias"], act_spec(fused["fc2"]))
    return y


INI = """
DefaultModel=Frame_HIP

[sp]
SizeX=32
SizeY=32
NbChannels=1
BatchSize=%d

[conv1]
Input=sp
Type=Conv
KernelDims=5 5
NbOutputs=6
ActivationFunction=Linear

[pool1]
Input=conv1
Type=Pool
Mapping.ChannelsPerGroup=1
PoolDims=2 2
NbOutputs=6
Stride=2
Pooling=Max

[conv2]
Input=pool1
Type=Conv
KernelDims=5 5
NbOutputs=16
ActivationFunction=Linear

[pool2]
Input=conv2
Type=Pool
Mapping.ChannelsPerGroup=1
PoolDims=2 2
NbOutputs=16
Stride=2
Pooling=Max

[conv3]
Input=pool2
Type=Conv
KernelDims=5 5
NbOutputs=120
ActivationFunction=Linear

[fc1]
Input=conv3
Type=Fc
NbOutputs=84
ActivationFunction=Linear

[fc2]
Input=fc1
Type=Fc
NbOutputs=10
ActivationFunction=Linear
"""


def fuse_with_library(fh, d, name, batch, mode="FloatMult", rounding=True):
    """The same pass through the C++ DeepNetQAT of the library, into a net of Frame_HIP cells built from INI text."""
    net = fh.Net(INI % batch)
    ranges, alphas = (255, 255), (1.0, 1.0)
    for conv, bn, shape, w_range in conv_stages(name):
        wq = quantized_conv_weights(d, conv, shape, w_range)
        fused, ranges, alphas = net.fuse_batchnorm_with_conv(conv, ranges, alphas, wq, None, w_range, True, *bn_of(d, bn), EPS, act_range(name),
                                                             float(d[bn + "_QAct_SAT_Alpha"][0]), mode, rounding, rounding, rounding)
        assert fused
    for fc, shape, w_range, a_range in fc_stages(name):
        wq, sat = quantized_fc_weights(d, fc, shape, w_range)
        ranges, alphas = net.quantize_fc(fc, ranges, alphas, wq, None, w_range, sat, a_range, float(d[fc + "_QAct_SAT_Alpha"][0]), rounding,
                                         rounding, rounding)
    for pool in ("pool1", "pool2"):
        net.set_quantized(pool, 8)
    return net
