"""Synthetic quantized networks (the benchmark configurations) and their
execution through the C ABI.

A network is a layer-ordered list of cells as N2D2's post-training quantization
leaves them: integer weights and biases, a Scaling in each activation, stand-alone
ScalingCells on residual shortcuts, ElemWise sums with unit weights.  Parameters
are seeded random draws; the per-layer rescale magnitudes are calibrated on one
image with numpy so that activations keep a healthy dynamic range through the
depth of the net (a stand-in for N2D2's calibration pass, not part of inference).
"""
import math

import numpy as np


class ActDesc:
    """Activation of a cell: kind, Scaling parameters, bits and signedness."""

    def __init__(self, kind="Linear", mode="None", scaling=None, frac_bits=0, clipping=None, nb_bits=8, unsigned_out=False):
        self.kind, self.mode, self.scaling, self.frac_bits = kind, mode, scaling, frac_bits
        self.clipping, self.nb_bits, self.unsigned_out = clipping, nb_bits, unsigned_out

    def kwargs(self):
        return dict(kind=self.kind, mode=self.mode, scaling=self.scaling, frac_bits=self.frac_bits,
                    clipping=self.clipping, nb_bits=self.nb_bits, unsigned_out=self.unsigned_out)

    def bounds(self):
        if self.unsigned_out:
            lo, hi = 0, (1 << self.nb_bits) - 1
        else:
            lo, hi = -(1 << (self.nb_bits - 1)), (1 << (self.nb_bits - 1)) - 1
        if self.kind == "Rectifier":
            lo = max(lo, 0)
        return lo, hi

    def apply_np(self, acc, channel_axis=1):
        """Exact integer form of the rescale on an int64 array (calibration only)."""
        if self.mode == "None":
            return np.maximum(acc, 0) if self.kind == "Rectifier" else acc
        shape = [1] * acc.ndim
        shape[channel_axis] = -1
        v = acc.astype(np.int64)
        if self.clipping is not None and self.mode in ("FixedMult16", "FixedMult32", "FloatMult"):
            cl = np.rint(np.asarray(self.clipping, dtype=np.float64)).astype(np.int64).reshape(shape)
            v = np.where(cl > 0, np.clip(v, 0, np.maximum(cl, 0)), np.clip(v, np.minimum(cl, 0), 0))
        if self.mode == "FloatMult":
            r = v.astype(np.float32) * np.asarray(self.scaling, dtype=np.float32).reshape(shape)
            r = (np.sign(r) * np.floor(np.abs(r.astype(np.float64)) + 0.5)).astype(np.int64)
        else:
            if self.mode == "SingleShift":
                m = np.ones(len(self.scaling), dtype=np.int64)
                p = np.asarray(self.scaling, dtype=np.int64)
            elif self.mode == "DoubleShift":
                s = np.asarray(self.scaling, dtype=np.int64).reshape(-1, 2)
                m = 1 + (1 << s[:, 0])
                p = s[:, 1]
            else:
                m = np.asarray(self.scaling, dtype=np.int64)
                p = np.full(len(m), self.frac_bits, dtype=np.int64)
            half = np.where(p > 0, 1 << np.maximum(p - 1, 0), 0)
            r = (v * m.reshape(shape) + half.reshape(shape)) >> p.reshape(shape)
        lo, hi = self.bounds()
        return np.clip(r, lo, hi)


class Layer:
    def __init__(self, name, type_, inputs, **kw):
        self.name, self.type, self.inputs = name, type_, inputs
        self.__dict__.update(kw)


class NetSpec:
    def __init__(self, name, in_shape, input_unsigned=True):
        self.name, self.in_shape, self.input_unsigned = name, in_shape, input_unsigned
        self.layers = []
        self.shapes = {"input": in_shape}
        self.unsigned = {"input": input_unsigned}

    def add(self, layer, out_shape, unsigned_out):
        layer.out_shape = out_shape
        layer.unsigned_out = unsigned_out
        self.layers.append(layer)
        self.shapes[layer.name] = out_shape
        self.unsigned[layer.name] = unsigned_out
        return layer.name

    @property
    def output(self):
        return self.layers[-1].name

    def macs_per_image(self):
        total = 0
        for l in self.layers:
            if l.type == "conv":
                O, Cg, kH, kW = l.w.shape
                total += l.out_shape[1] * l.out_shape[2] * O * Cg * kH * kW
            elif l.type == "fc":
                total += l.w.size
        return total

    def conv_macs_per_image(self):
        return sum(l.out_shape[1] * l.out_shape[2] * l.w.size for l in self.layers if l.type == "conv" and l.groups == 1)


# ------------------------------------------------------------ numpy helpers (calibration only)

def _out_dim(n, k, s, p0, p1, d=1):
    return int((n + p0 + p1 - d * (k - 1) - 1 + s) / float(s))


def _conv_acc_np(x, w, stride, pad, groups):
    """x [C,H,W] ints, w [O,C/g,kH,kW]; zero-padded correlation through im2col + BLAS (exact in float64)."""
    C, H, W = x.shape
    O, Cg, kH, kW = w.shape
    sx, sy = stride
    oH, oW = _out_dim(H, kH, sy, pad[1], pad[3]), _out_dim(W, kW, sx, pad[0], pad[2])
    xp = np.zeros((C, H + pad[1] + pad[3] + kH, W + pad[0] + pad[2] + kW), dtype=np.float64)
    xp[:, pad[1]:pad[1] + H, pad[0]:pad[0] + W] = x
    out = np.empty((O, oH, oW), dtype=np.float64)
    og = O // groups
    for g in range(groups):
        cols = np.empty((Cg, kH, kW, oH, oW), dtype=np.float64)
        for ky in range(kH):
            for kx in range(kW):
                cols[:, ky, kx] = xp[g * Cg:(g + 1) * Cg, ky:ky + sy * (oH - 1) + 1:sy, kx:kx + sx * (oW - 1) + 1:sx]
        out[g * og:(g + 1) * og] = (w[g * og:(g + 1) * og].reshape(og, -1).astype(np.float64)
                                    @ cols.reshape(Cg * kH * kW, oH * oW)).reshape(og, oH, oW)
    return np.rint(out).astype(np.int64)


def _pool_np(x, kind, pool, stride, pad):
    C, H, W = x.shape
    oH = int((H + 2 * pad[1] - pool[1] + stride[1]) / float(stride[1]))
    oW = int((W + 2 * pad[0] - pool[0] + stride[0]) / float(stride[0]))
    out = np.zeros((C, oH, oW), dtype=np.int64)
    for oy in range(oH):
        for ox in range(oW):
            y0, x0 = oy * stride[1] - pad[1], ox * stride[0] - pad[0]
            win = x[:, max(y0, 0):min(y0 + pool[1], H), max(x0, 0):min(x0 + pool[0], W)]
            if kind == "max":
                out[:, oy, ox] = win.max(axis=(1, 2))
            else:
                s = win.sum(axis=(1, 2))
                out[:, oy, ox] = np.sign(s) * (np.abs(s) // (pool[0] * pool[1]))
    return out


class _Builder:
    """Adds cells to a NetSpec while pushing one calibration image through them."""

    def __init__(self, name, in_shape, seed, scaling_mode, nb_bits=8, unsigned_data=True, frac_bits=16):
        self.rng = np.random.default_rng(seed)
        self.spec = NetSpec(name, in_shape, input_unsigned=True)
        self.mode, self.nb_bits, self.unsigned_data, self.frac_bits = scaling_mode, nb_bits, unsigned_data, frac_bits
        self.values = {"input": self.rng.integers(0, 256, size=in_shape).astype(np.int64)}

    # per-channel Scaling parameters approximating the float factors s (one per channel)
    def _scaling_params(self, s, mode=None):
        mode = mode or self.mode
        if mode == "SingleShift":
            return np.clip(np.rint(-np.log2(s)), 0, 31).astype(np.uint8), 0
        if mode == "DoubleShift":
            best = None
            for a in range(0, 5):
                b = np.clip(np.rint(np.log2((1 + 2.0 ** a) / s)), 0, 31)
                err = np.abs((1 + 2.0 ** a) / 2.0 ** b - s) / s
                if best is None:
                    best = (np.full(len(s), a), b, err)
                else:
                    take = err < best[2]
                    best = (np.where(take, a, best[0]), np.where(take, b, best[1]), np.where(take, err, best[2]))
            return np.stack([best[0], best[1]], 1).astype(np.uint8), 0
        if mode in ("FixedMult16", "FixedMult32"):
            p = self.frac_bits
            return np.maximum(np.rint(s * 2.0 ** p), 1).astype(np.int32), p
        return s.astype(np.float32), 0

    def _make_act(self, acc, kind, O, nb_bits=None, mode=None, clip=False, target=None):
        nb_bits = nb_bits or self.nb_bits
        mode = mode or self.mode
        unsigned = self.unsigned_data and kind == "Rectifier"
        if mode == "None":
            return ActDesc(kind, "None", nb_bits=nb_bits, unsigned_out=unsigned)
        full = (1 << nb_bits) - 1 if unsigned else (1 << (nb_bits - 1)) - 1
        target = target or 0.8 * full
        ref = max(float(np.percentile(np.abs(acc), 99.5)), 1.0)
        s = (target / ref) * self.rng.uniform(0.75, 1.3, size=O)
        scaling, frac = self._scaling_params(s, mode)
        clipping = None
        if clip:
            clipping = (ref * self.rng.uniform(0.9, 1.6, size=O)).astype(np.float32)
        return ActDesc(kind, mode, scaling, frac, clipping, nb_bits, unsigned)

    def _weights(self, shape, wstd, wmax, uniform):
        if uniform:
            return self.rng.integers(-wmax, wmax + 1, size=shape).astype(np.int8)
        return np.clip(np.rint(self.rng.normal(0, wstd, size=shape)), -wmax, wmax).astype(np.int8)

    def conv(self, name, inp, O, k, stride=1, pad=0, kind="Rectifier", groups=1, wstd=30.0, wmax=127, weight_bits=8,
             bias=True, nb_bits=None, mode=None, clip=False, uniform=False, sub=(1, 1)):
        inps = list(inp) if isinstance(inp, (list, tuple)) else [inp]     # several inputs: their channels one behind the other
        C, (H, W) = sum(self.spec.shapes[i][0] for i in inps), self.spec.shapes[inps[0]][1:]
        w = self._weights((O, C // groups, k, k), wstd, wmax, uniform)
        p4 = (pad, pad, pad, pad)
        acc = _conv_acc_np(np.concatenate([self.values[i] for i in inps], 0), w.astype(np.int64), (stride, stride), p4, groups)
        if tuple(sub) != (1, 1):
            # ConvCell's SubSample: the sums of sub[0] x sub[1] neighbouring positions added up, ragged last windows included
            summed = np.zeros((O, -(-acc.shape[1] // sub[1]), -(-acc.shape[2] // sub[0])), dtype=np.int64)
            for oy in range(acc.shape[1]):
                for ox in range(acc.shape[2]):
                    summed[:, oy // sub[1], ox // sub[0]] += acc[:, oy, ox]
            acc = summed
        b = None
        if bias:
            mag = max(int(np.percentile(np.abs(acc), 90) / 4), 16)
            b = self.rng.integers(-mag, mag + 1, size=O).astype(np.int32)
            acc = acc + b[:, None, None]
        act = self._make_act(acc, kind, O, nb_bits, mode, clip)
        self.values[name] = act.apply_np(acc, 0)
        l = Layer(name, "conv", inps, w=w, bias=b, stride=(stride, stride), pad=p4, dil=(1, 1), groups=groups,
                  weight_bits=weight_bits, act=act, sub=tuple(sub))
        return self.spec.add(l, (O,) + acc.shape[1:], act.unsigned_out)

    def fc(self, name, inp, O, kind="Linear", wstd=30.0, wmax=127, weight_bits=8, mode=None, nb_bits=None, uniform=False):
        inps = list(inp) if isinstance(inp, (list, tuple)) else [inp]     # several inputs: their values one input behind the other
        flat = np.concatenate([self.values[i].reshape(-1) for i in inps])
        w = self._weights((O, flat.size), wstd, wmax, uniform)
        acc = w.astype(np.int64) @ flat
        mag = max(int(np.percentile(np.abs(acc), 90) / 4), 16)
        b = self.rng.integers(-mag, mag + 1, size=O).astype(np.int32)
        acc = (acc + len(inps) * b.astype(np.int64)).reshape(O, 1, 1)     # FcCell_Frame.cpp:309: the bias once per input
        act = self._make_act(acc, kind, O, nb_bits, mode)
        self.values[name] = act.apply_np(acc, 0)
        l = Layer(name, "fc", inps, w=w, bias=b, weight_bits=weight_bits, act=act)
        return self.spec.add(l, (O, 1, 1), act.unsigned_out)

    def pool(self, name, inp, kind, pool, stride, pad=0):
        inps = list(inp) if isinstance(inp, (list, tuple)) else [inp]     # several inputs: their channels one behind the other
        v = _pool_np(np.concatenate([self.values[i] for i in inps], 0), kind, (pool, pool), (stride, stride), (pad, pad))
        self.values[name] = v
        l = Layer(name, "pool", inps, kind=kind, pool=(pool, pool), stride=(stride, stride), pad=(pad, pad))
        # no activation: range of the parents (PoolCell::getOutputsRange)
        return self.spec.add(l, v.shape, all(self.spec.unsigned[i] for i in inps))

    def scaling(self, name, inp, frac_bits=14):
        """Stand-alone ScalingCell as `_rescale_branch` leaves it: FIXED_MULT16, factor <= 1, no activation."""
        C = self.spec.shapes[inp][0]
        s = self.rng.uniform(0.55, 1.0, size=C)
        mult = np.maximum(np.rint(s * 2.0 ** frac_bits), 1).astype(np.int32)
        # ScalingCell::getOutputsRange: unsigned iff the parent is and every factor is >= 0
        unsigned = self.spec.unsigned[inp]
        act = ActDesc("Linear", "FixedMult16", mult, frac_bits, None, self.nb_bits, unsigned)
        self.values[name] = act.apply_np(self.values[inp], 0)
        return self.spec.add(Layer(name, "scaling", [inp], act=act), self.spec.shapes[inp], unsigned)

    def sum(self, name, inps, kind="Rectifier", nb_bits=None, weights=None, shifts=None):
        """weights / shifts: one integer per input (ElemWise CoeffMode PerInput), 1 and 0 by default."""
        w = [1] * len(inps) if weights is None else [int(v) for v in weights]
        sh = [0] * len(inps) if shifts is None else [int(v) for v in shifts]
        acc = sum(w[k] * self.values[i] + sh[k] for k, i in enumerate(inps))
        C = acc.shape[0]
        act = self._make_act(acc, kind, C, nb_bits, target=None)
        self.values[name] = act.apply_np(acc, 0)
        plain = weights is None and shifts is None
        l = Layer(name, "elemwise", list(inps), act=act, weights=None if plain else np.array(w, dtype=np.float32),
                  shifts=None if plain else np.array(sh, dtype=np.float32), coeff_mode="PerLayer" if plain else "PerInput")
        return self.spec.add(l, acc.shape, act.unsigned_out)


# --------------------------------------------------------------- the configurations

def lenet(seed=1):
    """LeNet-style 8-bit PTQ net: 1x32x32 u8, conv 6@5x5, maxpool 2, conv 16@5x5, maxpool 2, FC 120-84-10;
    weights U[-127,127], per-layer fixed-point rescale with shift 20, integer logits."""
    b = _Builder("lenet", (1, 32, 32), seed, "FixedMult32", frac_bits=20)
    x = b.conv("conv1", "input", 6, 5, uniform=True)
    x = b.pool("pool1", x, "max", 2, 2)
    x = b.conv("conv2", x, 16, 5, uniform=True)
    x = b.pool("pool2", x, "max", 2, 2)
    x = b.fc("fc1", x, 120, kind="Rectifier", uniform=True)
    x = b.fc("fc2", x, 84, kind="Rectifier", uniform=True)
    b.fc("fc3", x, 10, kind="Linear", uniform=True, mode="None")
    return b.spec


def resnet50(seed=4, pool_pad=1, unsigned_data=True, image=224):
    """ResNet-50, 8-bit PTQ: 7x7 s2 stem, 3x3 s2 max-pool (pad 1 -> 56x56; pad 0 is N2D2's own model file),
    bottlenecks [3,4,6,3] with the stride in the 3x3, per-channel double-shift rescales, FIXED_MULT16 ScalingCells
    on identity shortcuts, ElemWise sums, global average pool, FC 1000 with raw int32 logits."""
    b = _Builder("resnet50", (3, image, image), seed, "DoubleShift", unsigned_data=unsigned_data)
    x = b.conv("conv1", "input", 64, 7, 2, 3)
    x = b.pool("pool1", x, "max", 3, 2, pool_pad)
    stage = 2
    for nf, blocks, stride in ((64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)):
        for i in range(blocks):
            n = "conv%d.%d" % (stage, i + 1)
            s = stride if i == 0 else 1
            y = b.conv(n + "_1x1", x, nf, 1)
            y = b.conv(n + "_3x3", y, nf, 3, s, 1)
            y = b.conv(n + "_1x1_x4", y, 4 * nf, 1, kind="Linear")
            if i == 0:
                sc = b.conv(n + "_1x1_proj", x, 4 * nf, 1, s, 0, kind="Linear")
            else:
                sc = b.scaling(n + "_shortcut_rescale", x)
            x = b.sum(n + "_sum", [y, sc])
        stage += 1
    C, H, W = b.spec.shapes[x]
    x = b.pool("pool", x, "avg", H, H)
    b.fc("fc", x, 1000, mode="None")
    return b.spec


def mobilenet_v1(seed=3, image=224):
    """MobileNet-v1 1.0, 8-bit PTQ: 3x3 s2 stem, 13 depthwise 3x3 + pointwise 1x1 blocks, per-channel fixed-point
    rescale (one shift per cell), ReLU6 == saturation at 255, global average pool, FC 1000."""
    b = _Builder("mobilenet_v1", (3, image, image), seed, "FixedMult32", frac_bits=16)
    x = b.conv("conv1", "input", 32, 3, 2, 1)
    cfg = [(64, 1), (128, 2), (128, 1), (256, 2), (256, 1), (512, 2), (512, 1), (512, 1), (512, 1), (512, 1), (512, 1),
           (1024, 2), (1024, 1)]
    for i, (O, s) in enumerate(cfg):
        C = b.spec.shapes[x][0]
        b.frac_bits = 16 + (i % 9)
        x = b.conv("conv%d_dw" % (i + 2), x, C, 3, s, 1, groups=C, wstd=50.0)
        x = b.conv("conv%d_pw" % (i + 2), x, O, 1)
    C, H, W = b.spec.shapes[x]
    x = b.pool("pool", x, "avg", H, H)
    b.fc("fc", x, 1000, mode="None")
    return b.spec


def resnet18_w4a4(seed=5, image=224):
    """ResNet-18 with 4-bit weights in [-7,7] (nibble-packed) and 4-bit activations in [0,15] as the SAT export
    leaves it: per-channel fixed-point rescale (16 fractional bits) with clipping; first and last layer 8-bit."""
    b = _Builder("resnet18_w4a4", (3, image, image), seed, "FixedMult32", frac_bits=16)
    x = b.conv("conv1", "input", 64, 7, 2, 3, nb_bits=4, clip=True)          # 8-bit weights, 4-bit activations out
    x = b.pool("pool1", x, "max", 3, 2, 1)
    stage = 2
    for nf, stride in ((64, 1), (128, 2), (256, 2), (512, 2)):
        for i in range(2):
            n = "conv%d.%d" % (stage, i + 1)
            s = stride if i == 0 else 1
            y = b.conv(n + "_a", x, nf, 3, s, 1, wstd=3.0, wmax=7, weight_bits=4, nb_bits=4, clip=True)
            y = b.conv(n + "_b", y, nf, 3, 1, 1, kind="Linear", wstd=3.0, wmax=7, weight_bits=4, nb_bits=4, clip=True)
            if s != 1 or b.spec.shapes[x][0] != nf:
                sc = b.conv(n + "_proj", x, nf, 1, s, 0, kind="Linear", wstd=3.0, wmax=7, weight_bits=4, nb_bits=4, clip=True)
            else:
                sc = x
            x = b.sum(n + "_sum", [y, sc], nb_bits=4)
        stage += 1
    C, H, W = b.spec.shapes[x]
    x = b.pool("pool", x, "avg", H, H)
    b.fc("fc", x, 1000, mode="None")
    return b.spec


def branches_net(seed=43):
    """A small net whose cells read several cells at once (N2D2 writes a concatenation this way: the reader's channels are
    its inputs' channels one behind the other): three branches off a stem joined by a 3x3 convolution, that and one branch
    joined again by a 1x1 convolution, a residual sum, a global average and a global maximum over two cells each, an FC
    over both."""
    b = _Builder("branches", (3, 24, 24), seed, "SingleShift")
    stem = b.conv("stem", "input", 64, 3, stride=2, pad=1)
    a = b.conv("a3", stem, 64, 3, pad=1)
    c = b.conv("b1", stem, 32, 1)
    d = b.pool("bpool", stem, "max", 3, 1, pad=1)
    j = b.conv("join", [a, c, d], 128, 3, pad=1)
    k = b.conv("join1", [j, c], 64, 1, kind="Linear")
    t = b.sum("sum", [k, stem])
    t = b.pool("pool", [t, c], "avg", 12, 12)
    u = b.pool("pool_b", [a, d], "max", 12, 12)
    b.fc("fc", [t, u], 10, mode="None")
    return b.spec


def single_conv_stage(seed=2):
    """One ResNet-18 stage conv: 3x3 s1 p1 64->64 on 56x56, u8 input, N(0,40) weights, per-channel single shift in
    [8,12], ReLU clip [0,255]."""
    spec = NetSpec("conv3x3_64", (64, 56, 56))
    rng = np.random.default_rng(seed)
    w = np.clip(np.rint(rng.normal(0, 40, size=(64, 64, 3, 3))), -127, 127).astype(np.int8)
    act = ActDesc("Rectifier", "SingleShift", rng.integers(8, 13, size=64).astype(np.uint8), nb_bits=8, unsigned_out=True)
    spec.add(Layer("conv", "conv", ["input"], w=w, bias=None, stride=(1, 1), pad=(1, 1, 1, 1), dil=(1, 1), groups=1,
                   weight_bits=8, act=act), (64, 56, 56), True)
    return spec


# ------------------------------------------------------------------ execution on the GPU

class GpuNet:
    """Instantiates every cell of a NetSpec through the C ABI and runs them in layer order on the current stream.
    Activations stay on the device in the private NHWC form between cells; all buffers are allocated once."""

    def __init__(self, spec, batch, fuse=True, halo=True, kernel_choice=0, bottlenecks="projection", stem_pool=True,
                 dw_pw=True, s2d=True, chains=True, fc_chains=True):
        """fuse: fold a ScalingCell whose only consumer is an ElemWise sum into that sum (one pass instead of two;
        the rescaled tensor is never written), and a two-input sum into the 1x1 convolution that feeds it.
        halo: a tensor written by a convolution and read only by convolutions is stored with the readers' padding as
        a border of zeros around every image, which lets a padded KxK reader fetch every tap without a validity test.
        kernel_choice: capi.KERNEL_* bits handed to every convolution (which kernel runs, never what it computes).
        bottlenecks: run a residual block 1x1 -> 3x3 -> 1x1 + sum (+ projection) whose cells qualify as one launch
        (n2d2hip_bottleneck_*); its input tensor then carries a border of one pixel.  True / "all", "projection" (only the
        blocks with a projection shortcut, where one launch replaces four), or False.
        stem_pool: compute the max pooling behind a first-layer convolution in that convolution's launch
        (n2d2hip_conv_forward_maxpool) where the library takes the pair.
        dw_pw: run a 3x3 depthwise convolution and the 1x1 convolution that alone reads it as one launch (n2d2hip_dw_pw_*)
        where the library takes the pair and expects the launch to be faster than the two (n2d2hip_dw_pw_pays); "all":
        wherever the library takes the pair.
        s2d: store the network input space-to-depth (16-byte pixels of 2 x 2 input pixels, with a border of zeros) when the
        one cell reading it is a first-layer convolution the library serves that way (n2d2hip_conv_s2d_halo).
        fc_chains: run two or three fully-connected cells, each the only reader of the one before, as one launch
        (n2d2hip_fc_chain_*) where the library takes them.
        chains: run a block's 3x3 convolution in the launch of the expanding 1x1 convolution + sum that alone reads it
        (n2d2hip_conv_chain_*) where the library takes the pair: the 3x3 convolution's output stays on the chip."""
        from . import capi, runtime as rt
        self.spec, self.B, self.rt, self.capi = spec, batch, rt, capi
        consumers = {}
        for l in spec.layers:
            for i in l.inputs:
                consumers.setdefault(i, []).append(l)
        self.folded = set()
        self.fused_sums = {}
        by_name = {l.name: l for l in spec.layers}
        order = {l.name: k for k, l in enumerate(spec.layers)}
        order["input"] = -1
        C, H, W = spec.in_shape

        def reads_halo(m):
            # (asked of the library, from the layer's shape: the reader's cell does not exist yet when its input is allocated)
            return (m.type == "conv" and len(m.inputs) == 1
                    and rt.Conv.shape_reads_halo(m.w.shape, m.stride, m.pad, m.dil, m.groups, m.weight_bits, kernel_choice,
                                                 getattr(m, "sub", (1, 1))))

        def halo_of(l, cell):
            """Border to store around l's output: the largest padding among its readers, if all of them can use it."""
            readers = consumers.get(l.name, [])
            if not halo or not readers or not all(reads_halo(m) for m in readers) or not cell.accepts_halo():
                return 0
            return max(max(m.pad) for m in readers)
        self.input = rt.DTensor(batch, C, H, W, capi.U8B if spec.input_unsigned else capi.I8)
        self.tensors = {"input": self.input}
        self.steps = []
        ins_of = {}
        for l in spec.layers:
            ins = [self.tensors[i] for i in l.inputs]
            Co, Ho, Wo = l.out_shape
            if l.type in ("conv", "fc"):
                act = rt.Act(Co, **l.act.kwargs())
                if l.type == "conv":
                    cell = rt.Conv(l.w, l.bias, act, ins[0].dtype, l.stride, l.pad, l.dil, l.groups, l.weight_bits, kernel_choice,
                                   getattr(l, "sub", (1, 1)))
                else:
                    # several inputs: each inner product starts from the bias and they are added up (FcCell_Frame.cpp:309)
                    cell = rt.Fc(l.w, None if l.bias is None else l.bias * len(ins), act, ins[0].dtype,
                                 (sum(t.C for t in ins), ins[0].H, ins[0].W), l.weight_bits)
                if ins[0].halo and not (l.type == "conv" and cell.accepts_halo()):
                    raise RuntimeError("layer %s cannot read the halo its input was given (GpuNet(halo=False) avoids it)" % l.name)
                out = rt.DTensor(batch, Co, Ho, Wo, act.out_dtype(), halo=halo_of(l, cell) if l.type == "conv" else 0)
                if len(ins) > 1:
                    # a cell with several inputs: one launch gathers their channels, the convolution reads that
                    gathered = rt.DTensor(batch, sum(t.C for t in ins), ins[0].H, ins[0].W, ins[0].dtype)
                    self.steps.append((l, cell, (lambda c, i, o, g=gathered: c.forward(rt.concat_channels(i, g), o))))
                else:
                    self.steps.append((l, cell, (lambda c, i, o: c.forward(i[0], o))))
            elif l.type == "pool":
                cell = rt.Pool(l.kind, l.pool, l.stride, l.pad)
                out = rt.DTensor(batch, Co, Ho, Wo, ins[0].dtype)
                if len(ins) > 1:
                    gathered = rt.DTensor(batch, sum(t.C for t in ins), ins[0].H, ins[0].W, ins[0].dtype)
                    self.steps.append((l, cell, (lambda c, i, o, g=gathered: c.forward(rt.concat_channels(i, g), o))))
                else:
                    self.steps.append((l, cell, (lambda c, i, o: c.forward(i[0], o))))
            elif l.type == "scaling":
                cell = rt.Act(Co, **l.act.kwargs())
                out = rt.DTensor(batch, Co, Ho, Wo, cell.out_dtype())
                self.steps.append((l, cell, (lambda c, i, o: rt.check(rt.lib.n2d2hip_scaling_forward(c.handle, i[0].ref, o.ref, rt.stream_ptr())))))
            elif l.type == "elemwise":
                act = rt.Act(Co, **l.act.kwargs())
                cell = rt.ElemWiseSum(len(ins), Co, act, l.weights, l.shifts, l.coeff_mode)
                out = rt.DTensor(batch, Co, Ho, Wo, act.out_dtype())
                if fuse:
                    for k, name in enumerate(l.inputs):
                        prod = next((m for m in spec.layers if m.name == name), None)
                        if prod is not None and prod.type == "scaling" and len(consumers[name]) == 1 and not self.folded & set(l.inputs):
                            sc_cell = next(c for (m, c, f) in self.steps if m is prod)
                            if cell.fold_input_scaling(k, sc_cell):
                                self.folded.add(name)
                                ins[k] = self.tensors[prod.inputs[0]]
                step = (l, cell, (lambda c, i, o: c.forward(i, o)))
                if fuse and len(ins) == 2:
                    # the convolution that runs last among the inputs takes the sum into its epilogue
                    for k in (1, 0):
                        prod = by_name.get(l.inputs[k])
                        other = l.inputs[1 - k]
                        if (prod is None or prod.type != "conv" or prod.groups != 1 or len(prod.inputs) != 1 or len(consumers[prod.name]) != 1
                                or prod.name in self.folded or other in self.folded and by_name[other].type != "scaling"):
                            continue
                        other_src = by_name[other].inputs[0] if other in self.folded else other
                        if order[other_src] > order[prod.name]:
                            continue
                        conv_cell = next(c for (m, c, f) in self.steps if m is prod)
                        if conv_cell.fuse_sum(cell, k, ins[1 - k].dtype):
                            self.folded.add(prod.name)
                            self.fused_sums[l.name] = (cell, prod)  # keeps the sum cell alive
                            ins = [ins_of[prod.name][0], ins[1 - k]]
                            step = (l, conv_cell, (lambda c, i, o: c.forward_sum(i[0], i[1], o)))
                            break
                self.steps.append(step)
            else:
                raise ValueError(l.type)
            self.tensors[l.name] = out
            ins_of[l.name] = ins
        # a network input that only padded convolutions of this kind read carries their padding too (the graph-edge
        # conversion fills the interior)
        first = consumers.get("input", [])
        if halo and first and all(reads_halo(m) for m in first) and all(c.accepts_halo() for (m, c, f) in self.steps if m in first):
            h = max(max(m.pad) for m in first)
            if h > 0:
                nx = rt.DTensor(batch, C, H, W, self.input.dtype, halo=h)
                for lst in ins_of.values():
                    for k, t in enumerate(lst):
                        if t is self.input:
                            lst[k] = nx
                self.input = self.tensors["input"] = nx
        # a first-layer convolution and the max pooling behind it as one launch (the convolution's output is never written)
        self.stem_pools = {}
        if fuse and stem_pool:
            step_index = {l.name: k for k, (l, c, f) in enumerate(self.steps)}
            for l in spec.layers:
                if l.type != "pool" or l.kind != "max" or len(l.inputs) != 1:
                    continue
                conv = by_name.get(l.inputs[0])
                if conv is None or conv.type != "conv" or len(conv.inputs) != 1 or len(consumers[conv.name]) != 1 or conv.name in self.folded:
                    continue
                conv_cell, pool_cell = self.steps[step_index[conv.name]][1], self.steps[step_index[l.name]][1]
                x = ins_of[conv.name][0]
                if x.halo or not conv_cell.accepts_maxpool(pool_cell, x.H, x.W):
                    continue
                self.steps[step_index[l.name]] = (l, conv_cell, (lambda c, i, o, pool=pool_cell: c.forward_maxpool(pool, i[0], o)))
                ins_of[l.name] = ins_of[conv.name]
                self.folded.add(conv.name)
                self.stem_pools[l.name] = conv
        # a 3x3 depthwise convolution and the 1x1 convolution that alone reads it as one launch (the depthwise output is
        # never written)
        self.dw_pws = {}
        if fuse and dw_pw:
            step_index = {l.name: k for k, (l, c, f) in enumerate(self.steps)}
            for l in spec.layers:
                if l.type != "conv" or len(l.inputs) != 1 or l.groups != 1 or l.w.shape[2:] != (1, 1) or l.name in self.folded:
                    continue
                dw = by_name.get(l.inputs[0])
                if (dw is None or dw.type != "conv" or len(dw.inputs) != 1 or dw.groups == 1 or len(consumers[dw.name]) != 1 or dw.name in self.folded
                        or ins_of[dw.name][0].halo or self.tensors[l.name].halo):
                    continue
                fused_cell = rt.DwPw.create(self.steps[step_index[dw.name]][1], self.steps[step_index[l.name]][1])
                if fused_cell is None:
                    continue
                # the library knows where one launch is faster than two (large tensors between the cells; small images
                # with 512 outputs per work-group)
                x = ins_of[dw.name][0]
                if dw_pw != "all" and not fused_cell.pays(batch, x.H, x.W):
                    continue
                self.steps[step_index[l.name]] = (l, fused_cell, (lambda c, i, o: c.forward(i[0], o)))
                ins_of[l.name] = ins_of[dw.name]
                self.folded.add(dw.name)
                self.dw_pws[l.name] = dw
        # A tensor read by padded convolutions and, as the other input, by sums that a convolution has taken into its
        # epilogue may carry the convolutions' padding too (the epilogue finds the other input's pixels past its borders),
        # when its producer can write it: ResNet-18's block inputs, which a max pooling or such a sum produces.
        if fuse and halo:
            step_index = {l.name: k for k, (l, c, f) in enumerate(self.steps)}
            for l in spec.layers:
                t = self.tensors.get(l.name)
                readers = consumers.get(l.name, [])
                if t is None or t.halo or l.name in self.folded or l.name == spec.output or not readers:
                    continue
                convs = [m for m in readers if m.type == "conv"]
                sums = [m for m in readers if m.type == "elemwise"]
                if not convs or len(convs) + len(sums) != len(readers):
                    continue
                # (a sum that reads it directly because the convolution holding the sum has it as its own input, a
                # projection shortcut, is that convolution reading it)
                if not all(m.name in self.fused_sums and (ins_of[m.name][1] is t) != (ins_of[m.name][0] is t) for m in sums):
                    continue
                if not all(reads_halo(m) and (m.name in self.folded or self.steps[step_index[m.name]][1].accepts_halo()) for m in convs):
                    continue
                h = max(max(m.pad) for m in convs)
                if h == 0:
                    continue
                producer_cell = self.steps[step_index[l.name]][1]
                writes = (l.name in self.fused_sums or l.name in self.stem_pools
                          or (l.type == "conv" and producer_cell.accepts_halo())
                          or (l.type == "pool" and len(l.inputs) == 1 and producer_cell.writes_halo(ins_of[l.name][0])))
                if not writes:
                    continue
                nx = rt.DTensor(t.B, t.C, t.H, t.W, t.dtype, halo=h)
                for lst in ins_of.values():
                    for k, u in enumerate(lst):
                        if u is t:
                            lst[k] = nx
                self.tensors[l.name] = nx
        # The network input in space-to-depth form, when its one reader takes it (with its pooling, if the two are one launch)
        if s2d and halo and len(first) == 1 and first[0].type == "conv" and len(first[0].inputs) == 1 and self.input.halo == 0:
            m = first[0]
            step_index = {l.name: k for k, (l, c, f) in enumerate(self.steps)}
            pooled = next((p for p, conv in self.stem_pools.items() if conv is m), None)
            conv_cell = self.steps[step_index[pooled if pooled else m.name]][1]
            pool_cell = rt.Pool(by_name[pooled].kind, by_name[pooled].pool, by_name[pooled].stride, by_name[pooled].pad) if pooled else None
            h = conv_cell.s2d_halo(H, W, pool_cell) if isinstance(conv_cell, rt.Conv) else -1
            out_t = self.tensors[pooled if pooled else m.name]
            if h >= 0 and (pooled or out_t.halo == 0):
                nx = rt.DTensor(batch, C, H, W, self.input.dtype, capi.S2D, halo=h)
                for lst in ins_of.values():
                    for k, t in enumerate(lst):
                        if t is self.input:
                            lst[k] = nx
                self.input = self.tensors["input"] = nx
        self.bottlenecks, self.bottleneck_layers = {}, {}
        self._bottleneck_mode = "all" if bottlenecks is True else bottlenecks
        if fuse and halo and bottlenecks:
            self._plan_bottlenecks(consumers, by_name, ins_of)
        # 3x3 convolutions computed by the launch of the expansion and sum that alone read them (their tensors are never written)
        self.chains = {}
        if fuse and halo and chains:
            self._plan_chains(consumers, by_name, ins_of)
        # fully-connected cells in a row as one launch (the vectors between them are never written)
        self.fc_chains = {}
        if fuse and fc_chains:
            step_index = {l.name: k for k, (l, c, f) in enumerate(self.steps)}
            for l in spec.layers:
                if l.type != "fc" or len(l.inputs) != 1 or l.name in self.folded:
                    continue
                readers = consumers.get(l.name, [])
                if l.name != spec.output and len(readers) == 1 and readers[0].type == "fc" and len(readers[0].inputs) == 1:
                    continue        # not the last of its run
                run = [l]
                while len(run) < 3:
                    prev = by_name.get(run[0].inputs[0])
                    if (prev is None or prev.type != "fc" or len(prev.inputs) != 1 or len(consumers[prev.name]) != 1 or prev.name in self.folded
                            or prev.name == spec.output):
                        break
                    run.insert(0, prev)
                if len(run) < 2 or any(m.name in self.folded for m in run):
                    continue
                cells = [self.steps[step_index[m.name]][1] for m in run]
                if not all(isinstance(c, rt.Fc) for c in cells):
                    continue
                fused = rt.FcChain.create(cells)
                if fused is None:
                    continue
                self.steps[step_index[l.name]] = (l, fused, (lambda c, i, o: c.forward(i[0], o)))
                ins_of[l.name] = ins_of[run[0].name]
                for m in run[:-1]:
                    self.folded.add(m.name)
                self.fc_chains[l.name] = run[:-1]
        self._io = [(ins_of[l.name], self.tensors[l.name]) for l in spec.layers]
        # folded ScalingCells are not launched and their output is never materialised
        for name in self.folded:
            del self.tensors[name]
        keep = [k for k, l in enumerate(spec.layers) if l.name not in self.folded]
        self.steps = [self.steps[k] for k in keep]
        self._io = [self._io[k] for k in keep]
        self.launched = [spec.layers[k] for k in keep]

    def _plan_chains(self, consumers, by_name, ins_of):
        """For every sum folded into the expanding 1x1 convolution of a block (and not part of a whole-block launch): the 3x3
        convolution whose output only that convolution reads runs in the same launch, where the library takes the pair
        (n2d2hip_conv_chain_supported) and the 3x3 convolution's input carries its padding as a border."""
        step_index = {l.name: k for k, (l, c, f) in enumerate(self.steps)}
        for sum_name, (sum_cell, expand) in list(self.fused_sums.items()):
            if sum_name in self.bottlenecks or len(expand.inputs) != 1:
                continue
            c3 = by_name.get(expand.inputs[0])
            if (c3 is None or c3.type != "conv" or len(c3.inputs) != 1 or len(consumers[c3.name]) != 1 or c3.name in self.folded
                    or c3.name == self.spec.output):
                continue
            k = step_index[sum_name]
            c3_cell, expand_cell = self.steps[step_index[c3.name]][1], self.steps[k][1]
            if not isinstance(c3_cell, self.rt.Conv) or not isinstance(expand_cell, self.rt.Conv) or not expand_cell.chain_supported(c3_cell):
                continue
            x = ins_of[c3.name][0]
            if x.halo < 1 or ins_of[sum_name][0] is not self.tensors[c3.name]:
                continue
            ins_of[sum_name] = [x, ins_of[sum_name][1]]
            self.steps[k] = (self.steps[k][0], expand_cell, (lambda c, i, o, c3c=c3_cell: c.forward_chain(c3c, i[0], i[1], o)))
            self.folded.add(c3.name)
            self.chains[sum_name] = c3

    def _plan_bottlenecks(self, consumers, by_name, ins_of):
        """For every sum folded into a 1x1 convolution: reduce -> 3x3 -> expand (+ projection) as one launch, if the
        library takes them (n2d2hip_bottleneck_create).  The sum may sit in the expansion (the other input is the block's
        input, plain or through a folded ScalingCell) or in the projection, which runs last (the sum is then moved into the
        expansion).  The block's input gets a border of one pixel, which its producer must be able to write (a max
        pooling, a folded sum, another bottleneck).  self.bottlenecks: "all", "projection" (only blocks with a projection:
        the others are as fast cell by cell) or False."""
        rt = self.rt
        cell_of = {m.name: c for (m, c, f) in self.steps}
        step_index = {m.name: k for k, (m, c, f) in enumerate(self.steps)}
        for sum_name, (sum_cell, holder) in list(self.fused_sums.items()):
            sum_layer = by_name[sum_name]
            other_name = [i for i in sum_layer.inputs if i != holder.name][0]
            other_layer = by_name.get(other_name)
            expand, proj = holder, None
            if by_name.get(holder.inputs[0]) is None or by_name[holder.inputs[0]].type != "conv":
                # the sum sits in the projection: the expansion is the sum's other input
                if other_layer is None or other_layer.type != "conv" or other_name in self.folded or len(consumers[other_name]) != 1:
                    continue
                expand, proj = other_layer, holder
            conv_b = by_name.get(expand.inputs[0])
            conv_a = by_name.get(conv_b.inputs[0]) if conv_b is not None and conv_b.type == "conv" else None
            if (conv_a is None or conv_a.type != "conv" or len(consumers[conv_a.name]) != 1 or len(consumers[conv_b.name]) != 1
                    or len(conv_a.inputs) != 1 or len(conv_b.inputs) != 1 or len(expand.inputs) != 1):
                continue
            xname = conv_a.inputs[0]
            x = self.tensors.get(xname)
            scaled = proj is None and other_name in self.folded and other_layer is not None and other_layer.type == "scaling"
            if proj is None:
                other_src = other_layer.inputs[0] if scaled else other_name
                if other_src != xname:
                    cand = by_name.get(other_src)
                    if cand is None or cand.type != "conv" or cand.inputs[0] != xname or len(consumers[cand.name]) != 1 or scaled:
                        continue
                    proj = cand
            elif proj.inputs[0] != xname:
                continue
            readers = {conv_a.name, proj.name if proj is not None else sum_name} | ({other_name} if scaled else set())
            if x is None or xname == "input" or not {m.name for m in consumers[xname]} <= readers | {sum_name}:
                continue
            producer = by_name[xname]
            can_write_halo = (xname in self.fused_sums or xname in self.bottlenecks or xname in self.stem_pools
                              or (producer.type == "pool" and len(producer.inputs) == 1 and cell_of[xname].writes_halo(ins_of[xname][0])))
            if x.halo not in (0, 1) or (x.halo == 0 and not can_write_halo):
                continue
            moved = False
            if holder is not expand:
                # move the sum from the projection into the expansion (undone below if the library declines)
                k_exp = sum_layer.inputs.index(expand.name)
                if not cell_of[expand.name].fuse_sum(sum_cell, k_exp, self.tensors[proj.name].dtype):
                    continue
                moved = True
            bn = rt.Bottleneck.create(cell_of[conv_a.name], cell_of[conv_b.name], cell_of[expand.name],
                                      cell_of[proj.name] if proj is not None else None)
            # the library takes the block or not, and knows where the one launch is the faster plan
            if bn is None or (self._bottleneck_mode != "all" and not bn.pays(x.B, x.H, x.W)):
                if moved:
                    cell_of[expand.name].fuse_sum(None, 0, 0)       # (the projection still holds the sum)
                continue
            if moved:
                cell_of[proj.name].fuse_sum(None, 0, 0)
            if x.halo == 0:
                nx = rt.DTensor(x.B, x.C, x.H, x.W, x.dtype, halo=1)
                for lst in ins_of.values():
                    for k, t in enumerate(lst):
                        if t is x:
                            lst[k] = nx
                self.tensors[xname] = nx
                x = nx
            self.bottlenecks[sum_name] = bn
            self.bottleneck_layers[sum_name] = [conv_a, conv_b, expand] + ([proj] if proj is not None else [])
            k = step_index[sum_name]
            ins_of[sum_name] = [x]
            self.steps[k] = (sum_layer, bn, (lambda c, i, o: c.forward(i[0], o)))
            for gone in [conv_a.name, conv_b.name, expand.name] + ([proj.name] if proj is not None else []):
                self.folded.add(gone)

    def set_input(self, x):
        """x: integer NCHW numpy array [B,C,H,W].  It is uploaded as the byte planes a caller would hand over (uint8 NCHW, int8
        for a signed input) and converted on the device (convert_input)."""
        np_t, dt = (np.uint8, self.capi.U8) if self.spec.input_unsigned else (np.int8, self.capi.I8)
        import torch
        lo, hi = (0, 255) if self.spec.input_unsigned else (-128, 127)          # (values outside the type saturate, as n2d2hip_convert does)
        flat = torch.from_numpy(np.clip(np.ascontiguousarray(x), lo, hi).astype(np_t).reshape(-1)).cuda()
        self.input_src = self.rt.DTensor(x.shape[0], x.shape[1], x.shape[2], x.shape[3], dt, self.capi.NCHW,
                                         flat)
        self._input_plain = None
        if self.input.layout == self.capi.NHWC and self.input.halo:
            self._input_plain = self.rt.DTensor(self.input.B, self.input.C, self.input.H, self.input.W, self.input.dtype)
        self.convert_input()

    def convert_input(self):
        """The graph-edge conversion: the caller's byte planes (NCHW) into the form the first cell reads (NHWC with a channel
        stride of 4 or 16, or space-to-depth), one launch of n2d2hip_convert."""
        if self._input_plain is not None:
            # an NHWC input with a border: converted without it, then copied into the interior (no configuration has one)
            t, h = self._input_plain.convert_from(self.input_src), self.input.halo
            self.input.buf.view(t.B, t.H + 2 * h, t.W + 2 * h, t.cs)[:, h:t.H + h, h:t.W + h, :] = t.buf.view(t.B, t.H, t.W, t.cs)
        else:
            self.input.convert_from(self.input_src)

    def forward(self):
        for (l, cell, fn), (ins, out) in zip(self.steps, self._io):
            fn(cell, ins, out)
        return self.tensors[self.spec.output]

    def capture(self, forwards=1, with_input_conversion=False):
        """Records `forwards` forwards, one behind the other, into a HIP graph (every launch of the C ABI goes to the
        capturing stream and none of them allocates or clears memory) and returns a callable that replays it.  More than
        one forward per graph spreads the cost of launching a graph over them: a network of one or two kernels is
        otherwise timed by that cost.  with_input_conversion: each forward is preceded by the graph-edge conversion of the
        byte planes set_input() left on the device."""
        import torch
        self.forward()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for _ in range(forwards):
                    if with_input_conversion:
                        self.convert_input()
                    self.forward()
        torch.cuda.synchronize()
        self._graph = graph

        def replay():
            graph.replay()
            return self.tensors[self.spec.output]
        return replay

    def forward_subset(self, indices):
        """Replays only the launches with these indices into self.launched (their inputs keep the values of the last
        full forward)."""
        for k in indices:
            l, cell, fn = self.steps[k]
            ins, out = self._io[k]
            fn(cell, ins, out)

    def kernel_names(self):
        """One forward with the library's launch log open around every cell: [[kernel name, ...]] per entry of
        self.launched, as the library itself names what it launched (template arguments included)."""
        names = []
        for (l, cell, fn), (ins, out) in zip(self.steps, self._io):
            with self.capi.launch_log() as log:
                fn(cell, ins, out)
            names.append([e[0] for e in log.entries])
        return names

    def forward_timed(self):
        """One forward with a pair of events around every cell launch, recorded on the stream the kernels run on.
        Returns [(layer, milliseconds)]."""
        import torch
        evs = []
        for (l, cell, fn), (ins, out) in zip(self.steps, self._io):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn(cell, ins, out)
            e1.record()
            evs.append((l, e0, e1))
        torch.cuda.synchronize()
        return [(l, e0.elapsed_time(e1)) for l, e0, e1 in evs]

    def layer_bytes(self, l):
        """Algorithmic HBM bytes of one cell: inputs and output once at storage width, weights once."""
        ins, out = self._io[self.launched.index(l)]
        total = sum(t.B * t.C * t.H * t.W * (4 if t.dtype == self.capi.I32 else 1) for t in ins)
        total += out.B * out.C * out.H * out.W * (4 if out.dtype == self.capi.I32 else 1)
        if l.type in ("conv", "fc"):
            total += l.w.size // (2 if l.weight_bits == 4 else 1)
        if l.name in self.bottleneck_layers:
            total += sum(m.w.size for m in self.bottleneck_layers[l.name])
        elif l.name in self.fused_sums:
            total += self.fused_sums[l.name][1].w.size
        if l.name in self.chains:           # the 3x3 convolution's weights; its output never leaves the chip
            total += self.chains[l.name].w.size
        if l.name in self.fc_chains:        # the earlier cells' weights; their outputs never leave the chip
            total += sum(m.w.size for m in self.fc_chains[l.name])
        if l.name in self.stem_pools:       # the convolution's weights; its output never leaves the chip
            total += self.stem_pools[l.name].w.size
        if l.name in self.dw_pws:           # the depthwise weights; its output never leaves the chip
            total += self.dw_pws[l.name].w.size
        return total

    def layer_macs(self, l):
        if l.name in self.bottleneck_layers:
            return sum(self.B * m.out_shape[1] * m.out_shape[2] * m.w.size for m in self.bottleneck_layers[l.name])
        if l.name in self.fused_sums:
            c3 = self.chains.get(l.name)
            return self.layer_macs(self.fused_sums[l.name][1]) + (self.layer_macs(c3) if c3 is not None else 0)
        if l.name in self.stem_pools:
            return self.layer_macs(self.stem_pools[l.name])
        if l.name in self.dw_pws:
            dw = self.dw_pws[l.name]
            return self.B * l.out_shape[1] * l.out_shape[2] * l.w.size + self.B * dw.out_shape[1] * dw.out_shape[2] * dw.w.size
        if l.type == "conv":
            return self.B * l.out_shape[1] * l.out_shape[2] * l.w.size
        if l.type == "fc":
            return self.B * (l.w.size + sum(m.w.size for m in self.fc_chains.get(l.name, [])))
        return 0

    def activation_bytes(self):
        """Algorithmic HBM bytes of one forward: every cell reads its inputs and writes its output once, plus weights."""
        return sum(self.layer_bytes(l) for l in self.launched)
