"""GPU parity of the integer cells: every result is compared bit-for-bit with
the CPU oracle on the same seeded inputs, calling through the C ABI."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(2024)


@pytest.fixture(scope="module")
def rt():
    from n2d2_amd import runtime
    return runtime


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _u8(shape):
    return RNG.integers(0, 256, size=shape).astype(np.int32)


def _i8(shape, lo=-127, hi=127):
    return RNG.integers(lo, hi + 1, size=shape).astype(np.int32)


def _acts(O, bits=8):
    """One activation spec per rescale mode / signedness, with per-channel parameters."""
    from oracle.cells import ActSpec
    hi = 2 ** bits
    return {
        "none_linear": ActSpec("Linear", "None"),
        "none_relu": ActSpec("Rectifier", "None"),
        "sshift_relu_u": ActSpec("Rectifier", "SingleShift", RNG.integers(8, 13, size=O), nb_bits=bits, unsigned_out=True),
        "sshift_lin_s": ActSpec("Linear", "SingleShift", RNG.integers(7, 12, size=O), nb_bits=bits, unsigned_out=False),
        "dshift_relu_u": ActSpec("Rectifier", "DoubleShift", np.stack([RNG.integers(0, 6, size=O), RNG.integers(9, 15, size=O)], 1),
                                 nb_bits=bits, unsigned_out=True),
        "dshift_lin_s": ActSpec("Linear", "DoubleShift", np.stack([RNG.integers(1, 4, size=O), RNG.integers(10, 14, size=O)], 1),
                                nb_bits=bits, unsigned_out=False),
        "fixed_relu_u": ActSpec("Rectifier", "FixedMult32", RNG.integers(2 ** 14, 2 ** 15, size=O), frac_bits=24,
                                nb_bits=bits, unsigned_out=True),
        "fixed_clip_s": ActSpec("Linear", "FixedMult16", RNG.integers(2 ** 10, 2 ** 12, size=O), frac_bits=20,
                                clipping=RNG.uniform(2000.0, 60000.0, size=O).astype(np.float32), nb_bits=bits, unsigned_out=False),
        "fixed_wide": ActSpec("Linear", "FixedMult32", RNG.integers(2 ** 28, 2 ** 30, size=O), frac_bits=40,
                              nb_bits=bits, unsigned_out=False),                    # needs the 64-bit product
        "fixed_neg": ActSpec("Linear", "FixedMult32", -RNG.integers(2 ** 10, 2 ** 12, size=O), frac_bits=20,
                             nb_bits=bits, unsigned_out=False),                     # negative multiplier
        "float_relu_u": ActSpec("Rectifier", "FloatMult", RNG.uniform(2e-4, 4e-3, size=O).astype(np.float32),
                                nb_bits=bits, unsigned_out=True),
        "float_clip_s": ActSpec("Linear", "FloatMult", RNG.uniform(2e-4, 4e-3, size=O).astype(np.float32),
                                clipping=np.where(RNG.random(O) < 0.5, 30000.5, -20000.0).astype(np.float32),
                                nb_bits=bits, unsigned_out=False),
    }


# ------------------------------------------------------------ conversion

def test_convert_round_trips(rt):
    from n2d2_amd import capi
    for Cc in (3, 16, 20, 64):
        x = _u8((2, Cc, 5, 7))
        for dt, vals in ((capi.U8B, x), (capi.U8, x), (capi.I8, x - 128), (capi.I32, x * 1000 - 7)):
            for layout in (capi.NHWC, capi.NCHW):
                t = rt.DTensor.from_numpy(vals, dt, layout)
                assert np.array_equal(t.to_numpy(), vals), (Cc, dt, layout)
        # F32 graph edge
        t = rt.DTensor.from_numpy(x.astype(np.float32), capi.U8B)
        assert np.array_equal(t.to_numpy(), x)
    # raw NHWC U8B bytes: value - 128, channel fastest, padded channels hold logical zero
    x = _u8((1, 3, 2, 2))
    raw = rt.DTensor.from_numpy(x, capi.U8B).raw().reshape(1, 2, 2, 4)
    assert np.array_equal(raw[..., :3].astype(np.int64) + 128, x.transpose(0, 2, 3, 1))
    assert (raw[..., 3] == -128).all()


# --------------------------------------------------------------- scaling

@pytest.mark.parametrize("layout", ["NHWC", "NCHW"])
def test_scaling_cell_all_modes(rt, layout):
    from n2d2_amd import capi
    lay = capi.NHWC if layout == "NHWC" else capi.NCHW
    Cc = 24
    acc = RNG.integers(-200000, 200001, size=(3, Cc, 6, 5)).astype(np.int32)
    acc[0, :, 0, 0] = 2 ** 24 - 1
    acc[0, :, 0, 1] = -(2 ** 24 - 1)
    acc[0, :, 0, 2] = 0
    for name, spec in _acts(Cc).items():
        _say("scaling %s %s" % (layout, name))
        act = rt.Act(Cc, **spec.kwargs())
        x = rt.DTensor.from_numpy(acc, capi.I32, lay)
        got = rt.scaling_forward(act, x).to_numpy()
        want = spec.apply(acc.astype(np.float32))
        assert np.array_equal(got, want.astype(np.int64)), name
    for bits, uns in ((4, True), (4, False)):
        spec = _acts(Cc, bits)["sshift_relu_u" if uns else "dshift_lin_s"]
        act = rt.Act(Cc, **spec.kwargs())
        got = rt.scaling_forward(act, rt.DTensor.from_numpy(acc, capi.I32, lay)).to_numpy()
        assert np.array_equal(got, spec.apply(acc.astype(np.float32)).astype(np.int64))
        assert got.max() <= (15 if uns else 7)


def test_scaling_on_byte_inputs_is_the_residual_branch_rescale(rt):
    from n2d2_amd import capi
    from oracle.cells import ActSpec
    Cc = 32
    x = _i8((2, Cc, 7, 7), -128, 127)
    spec = ActSpec("Linear", "FixedMult16", RNG.integers(2 ** 13, 2 ** 15, size=Cc), frac_bits=14, nb_bits=8, unsigned_out=False)
    act = rt.Act(Cc, **spec.kwargs())
    got = rt.scaling_forward(act, rt.DTensor.from_numpy(x, capi.I8)).to_numpy()
    assert np.array_equal(got, spec.apply(x.astype(np.float32)).astype(np.int64))


def test_error_behaviour_matches_reference(rt):
    from n2d2_amd import capi
    with pytest.raises(capi.N2D2HipError) as e:
        rt.Act(4, "Linear", "SingleShift", [1, 1, 1, 1], nb_bits=0)
    assert e.value.status == capi.ERR_NOT_QUANTIZED and "can only be used on quantized network" in str(e.value)
    # a leaky Rectifier gives non-integers below zero on signed or un-rescaled cells ...
    with pytest.raises(capi.N2D2HipError, match="non-integer"):
        rt.Act(4, "Rectifier", "SingleShift", [1, 1, 1, 1], leak_slope=0.1)
    with pytest.raises(capi.N2D2HipError, match="non-integer"):
        rt.Act(4, "Rectifier", "None", None, leak_slope=0.1, unsigned_out=True)
    # ... and changes nothing behind a rescale that saturates to an unsigned range, as in the reference
    from oracle.cells import ActSpec
    leaky = ActSpec("Rectifier", "SingleShift", np.array([1, 2, 3, 4]), nb_bits=8, unsigned_out=True, leak_slope=0.1)
    xl = RNG.integers(-3000, 3000, size=(2, 4, 3, 3)).astype(np.int32)
    got = rt.scaling_forward(rt.Act(4, **leaky.kwargs()), rt.DTensor.from_numpy(xl, capi.I32)).to_numpy()
    assert np.array_equal(got, leaky.apply(xl.astype(np.float32)).astype(np.int64)) and got.min() == 0
    act = rt.Act(4, "Linear", "SingleShift", [1, 1, 1, 1], nb_bits=8, unsigned_out=False)
    x = rt.DTensor.from_numpy(_u8((1, 5, 2, 2)), capi.I32)
    with pytest.raises(capi.N2D2HipError):            # channel mismatch: nothing is written
        rt.scaling_forward(act, x)
    with pytest.raises(capi.N2D2HipError):            # signed range into an unsigned store
        rt.scaling_forward(act, rt.DTensor.from_numpy(_u8((1, 4, 2, 2)), capi.I32), out_dtype=capi.U8B)


# ------------------------------------------------------------------ conv

CONV_CASES = [
    # name, B, C, H, W, O, (kW,kH), (sx,sy), (L,T,R,B), (dx,dy), input kind
    ("3x3_c64", 2, 64, 14, 14, 64, (3, 3), (1, 1), (1, 1, 1, 1), (1, 1), "u8"),
    ("1x1_c64_o256", 3, 64, 9, 11, 256, (1, 1), (1, 1), (0, 0, 0, 0), (1, 1), "u8"),
    ("1x1_s2", 2, 128, 14, 14, 96, (1, 1), (2, 2), (0, 0, 0, 0), (1, 1), "i8"),
    ("3x3_s2_c32", 2, 32, 15, 17, 48, (3, 3), (2, 2), (1, 1, 1, 1), (1, 1), "u8"),
    ("stem7x7_c3", 2, 3, 37, 41, 64, (7, 7), (2, 2), (3, 3, 3, 3), (1, 1), "u8"),
    ("stem3x3_c3", 2, 3, 20, 20, 32, (3, 3), (2, 2), (1, 1, 1, 1), (1, 1), "u8"),
    ("stem5x5_c3_o20", 3, 3, 45, 301, 20, (5, 5), (2, 2), (2, 2, 2, 2), (1, 1), "i8"),
    ("lenet5x5_c1", 4, 1, 32, 32, 6, (5, 5), (1, 1), (0, 0, 0, 0), (1, 1), "u8"),
    ("lenet5x5_c6", 4, 6, 14, 14, 16, (5, 5), (1, 1), (0, 0, 0, 0), (1, 1), "u8"),
    ("c20_o10_asym", 2, 20, 9, 8, 10, (2, 5), (1, 3), (1, 2, 0, 1), (1, 1), "i8"),
    ("dilated_nopad", 2, 16, 17, 17, 16, (3, 3), (1, 1), (0, 0, 0, 0), (2, 3), "u8"),
    ("dilated_pad_quirk", 2, 16, 12, 12, 16, (3, 3), (1, 3), (2, 2, 2, 2), (3, 3), "u8"),
    ("big_k", 1, 512, 7, 7, 130, (3, 3), (1, 1), (1, 1, 1, 1), (1, 1), "u8"),
    ("tall_m", 5, 16, 33, 31, 16, (3, 3), (1, 1), (1, 1, 1, 1), (1, 1), "u8"),
    # channel counts that are multiples of 64 (the pipelined kernel): every window quirk again, both K step widths
    ("c64_dilated_pad_quirk", 2, 64, 12, 12, 70, (3, 3), (1, 3), (2, 2, 2, 2), (3, 3), "u8"),
    ("c128_asym", 3, 128, 9, 8, 40, (2, 5), (2, 3), (1, 2, 0, 1), (1, 1), "i8"),
    ("c64_5x5", 2, 64, 11, 13, 64, (5, 5), (1, 1), (2, 2, 2, 2), (1, 1), "u8"),
    ("c192_1x7", 2, 192, 9, 15, 130, (7, 1), (1, 1), (3, 0, 3, 0), (1, 1), "u8"),
    ("c320_dil2", 1, 320, 13, 13, 300, (3, 3), (2, 2), (2, 2, 2, 2), (2, 2), "i8"),
    ("c256_ragged_m", 7, 256, 5, 7, 128, (3, 3), (1, 1), (1, 1, 1, 1), (1, 1), "u8"),
    # the reference's hand-unrolled 3x3 window met by a dilated kernel (bounds [0,3) x [0,3) at the last pixel)
    ("c16_dil2_unrolled_window", 2, 16, 13, 13, 16, (3, 3), (2, 2), (2, 2, 2, 2), (2, 2), "u8"),
    ("c3_dily2_unrolled_window", 2, 3, 13, 13, 16, (3, 3), (2, 2), (1, 2, 1, 2), (1, 2), "u8"),
    ("c128_1x1_many_tiles", 6, 128, 23, 21, 256, (1, 1), (1, 1), (0, 0, 0, 0), (1, 1), "u8"),
]


@pytest.mark.parametrize("case", CONV_CASES, ids=[c[0] for c in CONV_CASES])
def test_conv_cell_bit_exact(rt, case):
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    name, B, Cc, H, W, O, k, s, p, d, kind = case
    x = _u8((B, Cc, H, W)) if kind == "u8" else _i8((B, Cc, H, W), -128, 127)
    w = np.clip(np.rint(RNG.normal(0, 40, size=(O, Cc, k[1], k[0]))), -127, 127).astype(np.int32)
    bias = RNG.integers(-4096, 4097, size=O).astype(np.int32)
    in_dt = capi.U8B if kind == "u8" else capi.I8
    xd = rt.DTensor.from_numpy(x, in_dt)
    acts = _acts(O)
    names = list(acts) if name in ("3x3_c64", "c20_o10_asym") else ["none_linear", "sshift_relu_u", "dshift_lin_s", "fixed_relu_u", "float_relu_u"]
    if Cc % 64 == 0 and "fixed_wide" not in names:
        names.append("fixed_wide")         # (a multiplier of 30 bits on the pipelined kernel: the 64-bit product)
    for an in names:
        spec = acts[an]
        _say("conv %s %s" % (name, an))
        want = cells_ref.conv_cell(x, w, bias, spec, stride=s, pad=p, dil=d)
        assert np.abs(want).max() < 2 ** 24
        conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), in_dt, stride=s, pad=p, dil=d)
        got = conv.forward(xd).to_numpy()
        assert got.shape == want.shape
        assert np.array_equal(got, want.astype(np.int64)), (name, an)
    # NoBias
    spec = acts["sshift_relu_u"]
    conv = rt.Conv(w, None, rt.Act(O, **spec.kwargs()), in_dt, stride=s, pad=p, dil=d)
    want = cells_ref.conv_cell(x, w, None, spec, stride=s, pad=p, dil=d)
    assert np.array_equal(conv.forward(xd).to_numpy(), want.astype(np.int64))


def test_conv_config2_resnet18_stage_single_shift(rt):
    """3x3 s1 p1 64->64 on 56x56, uint8 input, N(0,40) weights, per-channel single shift in [8,12], ReLU clip [0,255];
    the oracle runs a 4-image slice, the GPU the same slice."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    from oracle.cells import ActSpec
    B = 4
    x = _u8((B, 64, 56, 56))
    w = np.clip(np.rint(RNG.normal(0, 40, size=(64, 64, 3, 3))), -127, 127).astype(np.int32)
    spec = ActSpec("Rectifier", "SingleShift", RNG.integers(8, 13, size=64), nb_bits=8, unsigned_out=True)
    want = cells_ref.conv_cell(x, w, None, spec, pad=(1, 1, 1, 1))
    conv = rt.Conv(w, None, rt.Act(64, **spec.kwargs()), capi.U8B, pad=(1, 1, 1, 1))
    got = conv.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy()
    assert np.array_equal(got, want.astype(np.int64))
    assert got.min() == 0 and got.max() == 255


@pytest.mark.parametrize("stride", [1, 2])
def test_depthwise_conv_bit_exact(rt, stride):
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    Cc = 48
    x = _u8((3, Cc, 13, 12))
    w = _i8((Cc, 1, 3, 3))
    bias = RNG.integers(-2000, 2001, size=Cc).astype(np.int32)
    acts = _acts(Cc)
    for an in ("fixed_relu_u", "sshift_lin_s", "none_linear", "float_relu_u"):
        spec = acts[an]
        if an == "fixed_relu_u":
            spec.scaling = RNG.integers(2 ** 13, 2 ** 14, size=Cc)
            spec.frac_bits = 18
        want = cells_ref.conv_cell(x, w, bias, spec, stride=(stride, stride), pad=(1, 1, 1, 1), groups=Cc)
        conv = rt.Conv(w, bias, rt.Act(Cc, **spec.kwargs()), capi.U8B, stride=(stride, stride), pad=(1, 1, 1, 1), groups=Cc)
        got = conv.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy()
        assert np.array_equal(got, want.astype(np.int64)), an
    # dilated depthwise whose last pixel meets the reference's hand-unrolled 3x3 window
    x = _u8((2, Cc, 13, 13))
    spec = acts["sshift_lin_s"]
    want = cells_ref.conv_cell(x, w, bias, spec, stride=(stride, stride), pad=(2, 2, 2, 2), dil=(2, 2), groups=Cc)
    conv = rt.Conv(w, bias, rt.Act(Cc, **spec.kwargs()), capi.U8B, stride=(stride, stride), pad=(2, 2, 2, 2), dil=(2, 2), groups=Cc)
    assert np.array_equal(conv.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy(), want.astype(np.int64))


def test_grouped_convolutions_bit_exact(rt):
    """G equal groups with 1 < G that are not the depthwise case (ConvCell_Frame_Kernels.cpp:89-96,132: the weight of a
    connected channel is found by its position among the connected ones): shapes for the pipelined, the first-layer-free
    general and the 4-bit kernels, a depth multiplier (G == C, O == 2 C), a 1x1."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    cases = (  # B, C, O, G, k, stride, pad, weight_bits
        (3, 64, 128, 2, 3, 1, 1, 8), (2, 12, 18, 3, 5, 2, 2, 8), (2, 32, 64, 32, 3, 1, 1, 8), (2, 128, 64, 4, 1, 1, 0, 8),
        (2, 64, 64, 4, 3, 1, 1, 4), (1, 6, 20, 2, 3, 2, 0, 8))
    for (B, Cc, O, G, k, stride, pad, bits) in cases:
        x = _u8((B, Cc, 11, 9))
        w = _i8((O, Cc // G, k, k)) if bits == 8 else RNG.integers(-7, 8, size=(O, Cc // G, k, k)).astype(np.int8)
        bias = RNG.integers(-2000, 2001, size=O).astype(np.int32)
        spec = _acts(O)["sshift_lin_s" if bits == 8 else "fixed_relu_u"]
        want = cells_ref.conv_cell(x, w, bias, spec, stride=(stride, stride), pad=(pad,) * 4, groups=G)
        conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, stride=(stride, stride), pad=(pad,) * 4, groups=G,
                       weight_bits=bits)
        got = conv.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy()
        assert np.array_equal(got, want.astype(np.int64)), (B, Cc, O, G, k, stride, pad, bits)
    with pytest.raises(capi.N2D2HipError, match="do not divide"):
        rt.Conv(_i8((6, 2, 3, 3)), None, rt.Act(6, **_acts(6)["sshift_lin_s"].kwargs()), capi.U8B, groups=4)


def test_conv_sub_sampling_bit_exact(rt):
    """ConvCell's SubSample (src/Cell/ConvCell_Frame_Kernels.cpp:46-52,135-140): the sums of subX x subY neighbouring positions
    added up (ragged last windows included), the bias added once, then the activation; shapes that run the pipelined, the
    first-layer, the direct, the general and the depthwise kernel underneath; every rescale mode and raw int32 outputs."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    cases = (  # B, C, O, H, W, k, stride, pad, groups, (subX, subY), activations
        (2, 64, 64, 9, 12, 3, 1, 1, 1, (2, 2), ("sshift_relu_u", "none_linear", "fixed_wide")),
        (3, 3, 32, 21, 23, 5, 2, 2, 1, (3, 2), ("fixed_relu_u", "float_relu_u")),
        (2, 1, 6, 16, 16, 5, 1, 0, 1, (2, 2), ("sshift_relu_u", "dshift_lin_s")),
        (2, 20, 10, 10, 7, 3, 1, 1, 1, (1, 3), ("sshift_lin_s",)),
        (2, 32, 32, 11, 9, 3, 1, 1, 32, (2, 2), ("sshift_lin_s",)),
        (1, 128, 40, 6, 6, 1, 1, 0, 1, (6, 6), ("sshift_relu_u",)))
    for (B, Cc, O, H, W, k, stride, pad, G, sub, names) in cases:
        x = _u8((B, Cc, H, W))
        w = _i8((O, Cc // G, k, k))
        bias = RNG.integers(-2000, 2001, size=O).astype(np.int32)
        for an in names:
            spec = _acts(O)[an]
            _say("sub-sampled conv %s %s" % ((B, Cc, O, H, W, k, stride, pad, G, sub), an))
            want = cells_ref.conv_cell(x, w, bias, spec, stride=(stride, stride), pad=(pad,) * 4, groups=G, sub=sub).astype(np.int64)
            conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, stride=(stride, stride), pad=(pad,) * 4, groups=G, sub=sub)
            assert conv.out_shape(H, W) == want.shape[2:]
            assert not conv.accepts_halo()
            got = conv.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy()
            assert got.shape == want.shape and np.array_equal(got, want), (Cc, O, k, sub, an, np.count_nonzero(got != want))
            # a second call on a larger batch (the sums' buffer grows) and without a bias
            if an == names[0]:
                x2 = _u8((B + 2, Cc, H, W))
                nb = rt.Conv(w, None, rt.Act(O, **spec.kwargs()), capi.U8B, stride=(stride, stride), pad=(pad,) * 4, groups=G, sub=sub)
                for xx in (x, x2):
                    w2 = cells_ref.conv_cell(xx, w, None, spec, stride=(stride, stride), pad=(pad,) * 4, groups=G, sub=sub).astype(np.int64)
                    assert np.array_equal(nb.forward(rt.DTensor.from_numpy(xx, capi.U8B)).to_numpy(), w2)


def test_direct_kernel_for_a_handful_of_channels(rt):
    """Layers with at most 16 input channels and 32 outputs can run one thread per output pixel (the library's own choice
    for at most 4 input channels: LeNet's first convolution): against the oracle and against the matrix-core kernel on the
    same cell, over kernel sizes, strides, paddings, a dilation, both
    input types and the rescale modes."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    cases = (  # B, C, O, H, W, k, stride, pad, dil, input type, activation
        (5, 1, 6, 32, 32, 5, 1, 0, 1, capi.U8B, "fixed_relu_u"), (5, 6, 16, 14, 14, 5, 1, 0, 1, capi.U8B, "fixed_relu_u"),
        (2, 3, 32, 17, 15, 3, 2, 1, 1, capi.U8B, "sshift_lin_s"), (2, 16, 20, 9, 11, 7, 1, 3, 1, capi.I8, "float_relu_u"),
        (3, 5, 8, 12, 12, 3, 1, 0, 2, capi.I8, "sshift_lin_s"), (2, 9, 5, 8, 8, 1, 1, 0, 1, capi.U8B, "fixed_relu_u"),
        (1, 2, 17, 6, 40, 3, (1, 2), 1, 1, capi.U8B, "dshift_relu_u"))
    for (B, Cc, O, H, W, k, stride, pad, dil, in_dtype, an) in cases:
        stride = stride if isinstance(stride, tuple) else (stride, stride)
        x = _u8((B, Cc, H, W)) if in_dtype == capi.U8B else _i8((B, Cc, H, W))
        w = _i8((O, Cc, k, k))
        bias = RNG.integers(-2000, 2001, size=O).astype(np.int32)
        acts = _acts(O)
        spec = acts[an if an in acts else "sshift_lin_s"]
        want = cells_ref.conv_cell(x, w, bias, spec, stride=stride, pad=(pad,) * 4, dil=(dil, dil))
        got = {}
        for choice in (0, capi.KERNEL_DIRECT, capi.KERNEL_NO_DIRECT):
            conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), in_dtype, stride=stride, pad=(pad,) * 4, dil=(dil, dil),
                           kernel_choice=choice)
            got[choice] = conv.forward(rt.DTensor.from_numpy(x, in_dtype)).to_numpy()
        assert np.array_equal(got[capi.KERNEL_DIRECT], want.astype(np.int64)), (B, Cc, O, H, W, k, stride, pad, dil)
        assert np.array_equal(got[capi.KERNEL_NO_DIRECT], got[capi.KERNEL_DIRECT]) and np.array_equal(got[0], got[capi.KERNEL_DIRECT])


def test_concat_channels_and_convolution_of_several_inputs(rt):
    """n2d2hip_concat_channels against numpy (odd channel counts, inputs and output with borders, both byte types; the
    channels past the last one hold the stored form of 0), and a ConvCell with three inputs (src/Cell/ConvCell_Frame.cpp:
    438-459: one weighted sum per input, added up) as the convolution of the gathered channels, against the oracle."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    for dtype, make in ((capi.U8B, _u8), (capi.I8, _i8)):
        xs = [make((2, 5, 7, 6)), make((2, 16, 7, 6)), make((2, 3, 7, 6))]
        ts = [rt.DTensor.from_numpy(x, dtype) for x in xs]
        ts[1] = ts[1].with_halo(1)
        want = np.concatenate(xs, 1).astype(np.int64)
        for halo in (0, 2):
            out = rt.concat_channels(ts, halo=halo)
            assert np.array_equal(out.to_numpy(), want), (dtype, halo)
            raw = out.raw().reshape(2, 7 + 2 * halo, 6 + 2 * halo, out.cs)[:, halo:7 + halo, halo:6 + halo, 24:]
            assert np.all(raw.view(np.uint8) == (0x80 if dtype == capi.U8B else 0)), (dtype, halo)
    xs = [_u8((2, 5, 7, 6)), _u8((2, 16, 7, 6)), _u8((2, 3, 7, 6))]
    w = _i8((20, 24, 3, 3))
    bias = RNG.integers(-2000, 2001, size=20).astype(np.int32)
    spec = _acts(20)["sshift_lin_s"]
    want = cells_ref.conv_cell(xs, w, bias, spec, pad=(1, 1, 1, 1))
    conv = rt.Conv(w, bias, rt.Act(20, **spec.kwargs()), capi.U8B, pad=(1, 1, 1, 1))
    got = conv.forward(rt.concat_channels([rt.DTensor.from_numpy(x, capi.U8B) for x in xs])).to_numpy()
    assert np.array_equal(got, want.astype(np.int64))
    with pytest.raises(capi.N2D2HipError, match="one byte type"):
        rt.concat_channels([rt.DTensor.from_numpy(xs[0], capi.U8B), rt.DTensor.from_numpy(_i8((2, 3, 7, 6)), capi.I8)])
    with pytest.raises(capi.N2D2HipError, match="channels"):
        rt.concat_channels([rt.DTensor.from_numpy(xs[0], capi.U8B)], out=rt.DTensor(2, 6, 7, 6, capi.U8B))


@pytest.mark.parametrize("stride", [1, 2])
def test_depthwise3x3_strip_kernel_against_general_kernel(rt, stride):
    """The 3x3 depthwise kernel (threads walk down strips of rows) against the oracle and against the general depthwise
    kernel, on shapes whose strips end unevenly, with and without padding, unsigned and signed inputs."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    for (B, Cc, H, W, pad, in_dtype) in ((5, 32, 37, 29, 1, capi.U8B), (2, 130, 9, 11, 1, capi.I8), (3, 64, 14, 14, 0, capi.U8B),
                                         (1, 8, 3, 3, 1, capi.U8B)):
        x = _u8((B, Cc, H, W)) if in_dtype == capi.U8B else _i8((B, Cc, H, W))
        w = _i8((Cc, 1, 3, 3))
        bias = RNG.integers(-2000, 2001, size=Cc).astype(np.int32)
        spec = _acts(Cc)["fixed_relu_u"]
        spec.scaling = RNG.integers(2 ** 13, 2 ** 14, size=Cc)
        spec.frac_bits = 21
        want = cells_ref.conv_cell(x, w, bias, spec, stride=(stride, stride), pad=(pad,) * 4, groups=Cc)
        got = {}
        for choice in (0, capi.KERNEL_NO_PIPE):
            conv = rt.Conv(w, bias, rt.Act(Cc, **spec.kwargs()), in_dtype, stride=(stride, stride), pad=(pad,) * 4, groups=Cc,
                           kernel_choice=choice)
            got[choice] = conv.forward(rt.DTensor.from_numpy(x, in_dtype)).to_numpy()
        assert np.array_equal(got[0], want.astype(np.int64)), (B, Cc, H, W, pad)
        assert np.array_equal(got[capi.KERNEL_NO_PIPE], got[0])


def test_conv_int4_weights_uint4_activations(rt):
    """Weights in [-7,7] nibble-packed, activations in [0,15], fixed-point rescale with clip, 4-bit unsigned output."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    from oracle.cells import ActSpec
    for (Cc, O, k, s, p) in ((64, 64, 3, 1, 1), (64, 128, 3, 2, 1), (64, 128, 1, 2, 0), (32, 40, 5, 1, 2)):
        x = RNG.integers(0, 16, size=(2, Cc, 14, 14)).astype(np.int32)
        w = RNG.integers(-7, 8, size=(O, Cc, k, k)).astype(np.int32)
        bias = RNG.integers(-300, 301, size=O).astype(np.int32)
        spec = ActSpec("Rectifier", "FixedMult32", RNG.integers(300, 900, size=O), frac_bits=16,
                       clipping=RNG.uniform(500.0, 3000.0, size=O).astype(np.float32), nb_bits=4, unsigned_out=True)
        want = cells_ref.conv_cell(x, w, bias, spec, stride=(s, s), pad=(p, p, p, p))
        conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, stride=(s, s), pad=(p, p, p, p), weight_bits=4)
        got = conv.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy()
        assert np.array_equal(got, want.astype(np.int64)), (Cc, O, k, s)
        assert got.max() <= 15 and len(np.unique(got)) > 4
        # same weights through the 8-bit path give the same cell
        conv8 = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, stride=(s, s), pad=(p, p, p, p))
        assert np.array_equal(conv8.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy(), got)


def test_conv_int4_weights_pipelined_kernel_tiles(rt):
    """4-bit weights on the pipelined kernel (packed in memory and in LDS, widened on the way to the matrix core): each of
    its three tile shapes, with the plain and the scaled-up rescale tables, a strided 1x1 and weights at both ends of
    the 4-bit range ([-8, 7]), against the oracle and against the general kernel."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    from oracle.cells import ActSpec
    cases = ((3, 64, 64, 3, 1, 1, 30, 0), (3, 128, 128, 3, 1, 1, 19, capi.KERNEL_TILE_M128), (3, 128, 128, 3, 1, 1, 19, capi.KERNEL_TILE_M64),
             (2, 256, 192, 1, 2, 0, 15, capi.KERNEL_TILE_M128 | capi.KERNEL_NO_HI16), (2, 64, 200, 3, 2, 1, 23, capi.KERNEL_TILE_M64),
             (1, 192, 64, 1, 1, 0, 9, capi.KERNEL_NO_HI16))
    for (B, Cc, O, k, s, p, H, choice) in cases:
        x = RNG.integers(0, 16, size=(B, Cc, H, H + 3)).astype(np.int32)
        w = RNG.integers(-8, 8, size=(O, Cc, k, k)).astype(np.int32)
        bias = RNG.integers(-300, 301, size=O).astype(np.int32)
        spec = ActSpec("Rectifier", "FixedMult32", RNG.integers(300, 900, size=O), frac_bits=16,
                       clipping=RNG.uniform(500.0, 3000.0, size=O).astype(np.float32), nb_bits=4, unsigned_out=True)
        want = cells_ref.conv_cell(x, w, bias, spec, stride=(s, s), pad=(p, p, p, p))
        xd = rt.DTensor.from_numpy(x, capi.U8B)
        got = {}
        for ch in (choice, capi.KERNEL_NO_PIPE):
            conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, stride=(s, s), pad=(p, p, p, p), weight_bits=4, kernel_choice=ch)
            got[ch] = conv.forward(xd).to_numpy()
        assert np.array_equal(got[choice], want.astype(np.int64)), (B, Cc, O, k, s, p, H, choice)
        assert np.array_equal(got[capi.KERNEL_NO_PIPE], got[choice])
    # full-range 8-bit activations and an unclipped rescale (the accumulators are 16 times the sums before they are divided)
    x = _u8((2, 128, 12, 12))
    w = RNG.integers(-8, 8, size=(128, 128, 3, 3)).astype(np.int32)
    spec = ActSpec("Rectifier", "SingleShift", RNG.integers(7, 11, size=128), nb_bits=8, unsigned_out=True)
    want = cells_ref.conv_cell(x, w, None, spec, pad=(1, 1, 1, 1))
    conv = rt.Conv(w, None, rt.Act(128, **spec.kwargs()), capi.U8B, pad=(1, 1, 1, 1), weight_bits=4)
    assert np.array_equal(conv.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy(), want.astype(np.int64))


def test_conv_linearity_and_batch_independence_at_full_width(rt):
    """Size-independent properties at a ResNet-50 layer shape (1x1, 256->64 on 56x56, batch 16): raw sums are additive in
    the weights, and an image's result does not depend on its position in the batch."""
    from n2d2_amd import capi
    B, Cc, O, H = 16, 256, 64, 56
    x = _u8((B, Cc, H, H))
    x[5] = x[0]
    w1 = _i8((O, Cc, 1, 1), -60, 60)
    w2 = _i8((O, Cc, 1, 1), -60, 60)
    xd = rt.DTensor.from_numpy(x, capi.U8B)
    raw = lambda w: rt.Conv(w, None, rt.Act(O, "Linear", "None"), capi.U8B).forward(xd).to_numpy()
    a, b, ab = raw(w1), raw(w2), raw(w1 + w2)
    assert np.array_equal(a + b, ab)
    assert np.array_equal(a[0], a[5])
    ref = np.einsum("chw,oc->ohw", x[3].astype(np.int64), w1[:, :, 0, 0].astype(np.int64))
    assert np.array_equal(a[3], ref)


# -------------------------------------------------------------------- fc

@pytest.mark.parametrize("shape", [(16, 5, 5, 120), (120, 1, 1, 84), (84, 1, 1, 10), (2048, 1, 1, 1000), (1, 6, 6, 20)])
def test_fc_cell_bit_exact(rt, shape):
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    Cc, H, W, O = shape
    B = 9
    x = _u8((B, Cc, H, W))
    w = np.clip(np.rint(RNG.normal(0, 30, size=(O, Cc * H * W))), -127, 127).astype(np.int32)
    bias = RNG.integers(-4096, 4097, size=O).astype(np.int32)
    acts = _acts(O)
    for an in ("none_linear", "fixed_relu_u", "dshift_lin_s"):
        spec = acts[an]
        want = cells_ref.fc_cell(x, w, bias, spec)
        assert np.abs(want).max() < 2 ** 24
        fc = rt.Fc(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, (Cc, H, W))
        got = fc.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy()
        assert np.array_equal(got, want.astype(np.int64)), an


def test_cells_with_at_most_four_outputs(rt):
    """Convolutions and FCs with 1 to 4 outputs (a binary classifier's last layer, a segmentation head): their output pixel
    is one dword.  From 3, 20 and 64 input channels, byte and raw int32 outputs, and a convolution that reads such a
    tensor."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    for O in (1, 2, 3, 4):
        for (Cc, k, pad, choice) in ((3, 3, 1, 0), (3, 3, 1, capi.KERNEL_NO_DIRECT), (20, 3, 1, 0), (64, 1, 0, 0), (128, 3, 1, 0)):
            x = _u8((3, Cc, 9, 7))
            w = _i8((O, Cc, k, k))
            bias = RNG.integers(-2000, 2001, size=O).astype(np.int32)
            for an in ("sshift_relu_u", "none_linear", "fixed_clip_s"):
                spec = _acts(O)[an]
                want = cells_ref.conv_cell(x, w, bias, spec, pad=(pad,) * 4)
                conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, pad=(pad,) * 4, kernel_choice=choice)
                got = conv.forward(rt.DTensor.from_numpy(x, capi.U8B))
                assert got.cs == 4 and np.array_equal(got.to_numpy(), want.astype(np.int64)), (O, Cc, k, an)
        x = _u8((5, 84, 1, 1))
        w = _i8((O, 84))
        bias = RNG.integers(-4096, 4097, size=O).astype(np.int32)
        for an in ("none_linear", "fixed_relu_u"):
            spec = _acts(O)[an]
            fc = rt.Fc(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, (84, 1, 1))
            assert np.array_equal(fc.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy(), cells_ref.fc_cell(x, w, bias, spec).astype(np.int64)), (O, an)
    # depthwise on 3 channels (3x3 and 5x5, stride 1 and 2)
    for k, stride in ((3, 1), (3, 2), (5, 1)):
        x = _u8((2, 3, 9, 8))
        w = _i8((3, 1, k, k))
        spec = _acts(3)["sshift_relu_u"]
        want = cells_ref.conv_cell(x, w, None, spec, stride=(stride, stride), pad=(k // 2,) * 4, groups=3)
        conv = rt.Conv(w, None, rt.Act(3, **spec.kwargs()), capi.U8B, stride=(stride, stride), pad=(k // 2,) * 4, groups=3)
        assert np.array_equal(conv.forward(rt.DTensor.from_numpy(x, capi.U8B)).to_numpy(), want.astype(np.int64)), (k, stride)
    # two layers: 16 -> 2 -> 8 channels
    x = _u8((2, 16, 8, 8))
    w1, w2 = _i8((2, 16, 3, 3)), _i8((8, 2, 3, 3))
    s1, s2 = _acts(2)["sshift_relu_u"], _acts(8)["sshift_lin_s"]
    mid = cells_ref.conv_cell(x, w1, None, s1, pad=(1,) * 4)
    want = cells_ref.conv_cell(mid, w2, None, s2, pad=(1,) * 4)
    c1 = rt.Conv(w1, None, rt.Act(2, **s1.kwargs()), capi.U8B, pad=(1,) * 4)
    c2 = rt.Conv(w2, None, rt.Act(8, **s2.kwargs()), capi.U8B, pad=(1,) * 4)
    assert np.array_equal(c2.forward(c1.forward(rt.DTensor.from_numpy(x, capi.U8B))).to_numpy(), want.astype(np.int64))


# ------------------------------------------------------------------ pool

@pytest.mark.parametrize("kind,pool,stride,pad", [("max", (2, 2), (2, 2), (0, 0)), ("max", (3, 3), (2, 2), (0, 0)),
                                                  ("max", (3, 3), (2, 2), (1, 1)), ("avg", (7, 7), (7, 7), (0, 0)),
                                                  ("avg", (3, 3), (2, 2), (1, 1)), ("avg", (2, 2), (2, 2), (0, 0)),
                                                  ("max", (3, 3), (1, 1), (1, 1)), ("max", (2, 2), (1, 1), (1, 1)),
                                                  ("max", (3, 3), (3, 2), (2, 0)), ("max", (3, 2), (2, 2), (1, 1))])
def test_pool_cell_bit_exact(rt, kind, pool, stride, pad):
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    for dt, x in ((capi.U8B, _u8((3, 24, 14, 15))), (capi.I8, _i8((3, 24, 14, 15), -128, 127)), (capi.U8, _u8((2, 3, 14, 14))),
                  (capi.U8, _u8((2, 16, 9, 14))), (capi.U8B, _u8((2, 64, 13, 13)))):
        want = cells_ref.pool_cell(x, kind, pool, stride, pad)
        got = rt.Pool(kind, pool, stride, pad).forward(rt.DTensor.from_numpy(x, dt)).to_numpy()
        assert np.array_equal(got, want.astype(np.int64)), (kind, dt)


def test_pool_cell_with_a_connection_map_bit_exact(rt):
    """Outputs that pool several channels (PoolCell_Frame_Kernels.cpp:60-75,150-185): the full map a Pool section without
    Mapping keys gets, groups, a hand-made map with an unconnected output."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    rng = np.random.default_rng(77)
    for dt, x in ((capi.U8B, _u8((2, 12, 9, 10))), (capi.I8, _i8((2, 12, 9, 10), -128, 127)), (capi.U8, _u8((2, 3, 8, 8))),
                  (capi.U8B, _u8((1, 40, 7, 7)))):
        Cn = x.shape[1]
        groups = np.zeros((Cn, 3), dtype=np.uint8)
        for c in range(Cn):
            groups[c, c * 3 // Cn] = 1
        hand = (rng.random((Cn, 5)) < 0.4).astype(np.uint8)
        hand[:, 2] = 0                                       # an output no channel feeds
        for maps in (np.ones((Cn, 4), dtype=np.uint8), groups, hand, np.ones((Cn, 20), dtype=np.uint8)):
            for kind, pool, stride, pad in (("max", (2, 2), (2, 2), (0, 0)), ("max", (3, 3), (2, 2), (1, 1)), ("avg", (3, 3), (2, 2), (1, 1)),
                                            ("avg", (2, 3), (1, 2), (0, 0)), ("max", (3, 3), (3, 2), (2, 0))):
                want = cells_ref.pool_cell(x, kind, pool, stride, pad, maps=maps)
                got = rt.Pool(kind, pool, stride, pad, maps=maps).forward(rt.DTensor.from_numpy(x, dt)).to_numpy()
                assert got.shape == want.shape and np.array_equal(got, want.astype(np.int64)), (dt, kind, pool, maps.shape)


def test_pool_with_a_connection_map_refuses_tensors_that_do_not_fit(rt):
    from n2d2_amd import capi
    x = rt.DTensor.from_numpy(_u8((2, 6, 8, 8)), capi.U8B)
    pool = rt.Pool("max", (2, 2), (2, 2), maps=np.ones((6, 3), dtype=np.uint8))
    assert pool.forward(x).to_numpy().shape == (2, 3, 4, 4)
    with pytest.raises(capi.N2D2HipError, match="expected"):              # output of the wrong size
        pool.forward(x, rt.DTensor(2, 3, 5, 4, capi.U8B))
    with pytest.raises(capi.N2D2HipError, match="one dtype"):             # output of another storage type
        pool.forward(x, rt.DTensor(2, 3, 4, 4, capi.I8))
    with pytest.raises(ValueError, match="the map is"):                   # a map for another number of channels
        rt.Pool("max", (2, 2), (2, 2), maps=np.ones((5, 3), dtype=np.uint8)).forward(x)
    with pytest.raises(capi.N2D2HipError, match="null descriptor or map"):
        capi.check(rt.lib.n2d2hip_pool_forward_mapped(rt.C.byref(pool.desc), None, 0, 0, x.ref, pool.make_output(x).ref, rt.stream_ptr()))


def test_global_average_pool_bit_exact(rt):
    """Whole-input average window (the classifier head's pooling): negative sums must truncate toward zero."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    for dt, x in ((capi.U8B, _u8((5, 2048, 7, 7))), (capi.I8, _i8((3, 300, 7, 5), -128, 127)), (capi.I8, _i8((2, 24, 3, 3), -128, 0)),
                  (capi.U8, _u8((2, 3, 6, 6)))):
        H, W = x.shape[2:]
        want = cells_ref.pool_cell(x, "avg", (W, H), (W, H), (0, 0))
        got = rt.Pool("avg", (W, H), (W, H), (0, 0)).forward(rt.DTensor.from_numpy(x, dt)).to_numpy()
        assert got.shape == want.shape and np.array_equal(got, want.astype(np.int64)), (dt, x.shape)


# -------------------------------------------------------------- elemwise

def test_elemwise_sum_cell_bit_exact(rt):
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    from oracle.cells import ActSpec
    Cc = 40
    a, b, c = _u8((2, Cc, 7, 9)), _i8((2, Cc, 7, 9), -128, 127), _u8((2, Cc, 7, 9))
    da, db, dc = rt.DTensor.from_numpy(a, capi.U8B), rt.DTensor.from_numpy(b, capi.I8), rt.DTensor.from_numpy(c, capi.U8B)
    acts = _acts(Cc)
    # residual add as PTQ leaves it: unit weights, zero shifts, rescale in the activation
    for an, spec in (("dshift", ActSpec("Rectifier", "DoubleShift", np.stack([RNG.integers(0, 3, size=Cc), RNG.integers(1, 4, size=Cc)], 1),
                                        nb_bits=8, unsigned_out=True)),
                     ("fixed", ActSpec("Rectifier", "FixedMult16", RNG.integers(2 ** 12, 2 ** 14, size=Cc), frac_bits=14, nb_bits=8, unsigned_out=True)),
                     ("float", ActSpec("Linear", "FloatMult", RNG.uniform(0.2, 0.9, size=Cc).astype(np.float32), nb_bits=8, unsigned_out=False)),
                     ("none", acts["none_relu"])):
        want = cells_ref.elemwise_cell([a, b], spec)
        ew = rt.ElemWiseSum(2, Cc, rt.Act(Cc, **spec.kwargs()))
        assert np.array_equal(ew.forward([da, db]).to_numpy(), want.astype(np.int64)), an
    # general coefficients, three inputs, float arithmetic as the reference
    spec = ActSpec("Linear", "FixedMult16", RNG.integers(2 ** 10, 2 ** 12, size=Cc), frac_bits=13, nb_bits=8, unsigned_out=False)
    w = np.array([1.5, -0.75, 2.0], dtype=np.float32)
    s = np.array([3.0, -10.5, 0.25], dtype=np.float32)
    want = cells_ref.elemwise_cell([a, b, c], spec, w, s, "PerInput")
    ew = rt.ElemWiseSum(3, Cc, rt.Act(Cc, **spec.kwargs()), w, s, "PerInput")
    assert np.array_equal(ew.forward([da, db, dc]).to_numpy(), want.astype(np.int64))
    wc = RNG.uniform(-2, 2, size=Cc).astype(np.float32)
    sc = RNG.uniform(-20, 20, size=Cc).astype(np.float32)
    want = cells_ref.elemwise_cell([a, b], spec, wc, sc, "PerChannel")
    ew = rt.ElemWiseSum(2, Cc, rt.Act(Cc, **spec.kwargs()), wc, sc, "PerChannel")
    assert np.array_equal(ew.forward([da, db]).to_numpy(), want.astype(np.int64))


def test_elemwise_with_folded_scaling_cell(rt):
    """ScalingCell -> ElemWise sum in one launch equals the two reference cells run one after the other."""
    from n2d2_amd import capi
    from oracle.cells import ActSpec
    from oracle import cells as cells_ref
    for Cc, shape in ((40, (2, 40, 7, 9)), (256, (3, 256, 14, 14))):
        a, b = _u8(shape), _u8(shape)
        da, db = rt.DTensor.from_numpy(a, capi.U8B), rt.DTensor.from_numpy(b, capi.U8B)
        sum_spec = ActSpec("Rectifier", "DoubleShift", np.stack([RNG.integers(0, 3, size=Cc), RNG.integers(1, 4, size=Cc)], 1),
                           nb_bits=8, unsigned_out=True)
        for mode, sc_spec in (("fixed16", ActSpec("Linear", "FixedMult16", RNG.integers(2 ** 12, 2 ** 15, size=Cc), frac_bits=14, nb_bits=8, unsigned_out=True)),
                              ("sshift", ActSpec("Linear", "SingleShift", RNG.integers(0, 3, size=Cc), nb_bits=8, unsigned_out=False)),
                              ("dshift", ActSpec("Linear", "DoubleShift", np.stack([RNG.integers(0, 3, size=Cc), RNG.integers(1, 4, size=Cc)], 1),
                                                 nb_bits=8, unsigned_out=True))):
            for k in (0, 1):
                xs = [a, b]
                xs[k] = sc_spec.apply(xs[k].astype(np.float32))
                want = cells_ref.elemwise_cell(xs, sum_spec)
                sc = rt.Act(Cc, **sc_spec.kwargs())
                ew = rt.ElemWiseSum(2, Cc, rt.Act(Cc, **sum_spec.kwargs()))
                assert ew.fold_input_scaling(k, sc), mode
                assert np.array_equal(ew.forward([da, db]).to_numpy(), want.astype(np.int64)), (mode, k, Cc)
                assert ew.fold_input_scaling(k, None)      # undo: plain sum again
                assert np.array_equal(ew.forward([da, db]).to_numpy(), cells_ref.elemwise_cell([a, b], sum_spec).astype(np.int64))
    # a float Scaling or a weighted sum is left to the caller as a separate launch
    fl = rt.Act(Cc, **ActSpec("Linear", "FloatMult", np.full(Cc, 0.5, np.float32), nb_bits=8, unsigned_out=True).kwargs())
    ew = rt.ElemWiseSum(2, Cc, rt.Act(Cc, **sum_spec.kwargs()))
    assert ew.fold_input_scaling(0, fl) is False
    ew = rt.ElemWiseSum(2, Cc, rt.Act(Cc, **sum_spec.kwargs()), np.array([2.0, 1.0], np.float32), np.zeros(2, np.float32), "PerInput")
    assert ew.fold_input_scaling(0, sc) is False


def test_conv_with_folded_residual_sum(rt):
    """1x1 convolution + ElemWise sum (+ ScalingCell on the shortcut) in one launch equals the reference cells run in turn."""
    from n2d2_amd import capi
    from oracle.cells import ActSpec
    from oracle import cells as cells_ref
    rng = np.random.default_rng(77)
    cases = [  # C, O, H, stride, B
        (64, 256, 9, 1, 3), (256, 128, 7, 1, 2), (128, 512, 8, 2, 2), (64, 64, 5, 1, 2), (256, 64, 6, 1, 3), (512, 1024, 7, 2, 5)]
    for C, O, H, stride, B in cases:
        x = rng.integers(0, 256, size=(B, C, H, H))
        w = np.clip(np.rint(rng.normal(0, 20, size=(O, C, 1, 1))), -127, 127).astype(np.int64)
        bias = rng.integers(-2000, 2000, size=O)
        conv_spec = ActSpec("Linear", "DoubleShift", np.stack([rng.integers(0, 3, size=O), rng.integers(8, 12, size=O)], 1),
                            nb_bits=8, unsigned_out=False)
        sum_spec = ActSpec("Rectifier", "DoubleShift", np.stack([rng.integers(0, 3, size=O), rng.integers(0, 3, size=O)], 1),
                           nb_bits=8, unsigned_out=True)
        y = cells_ref.conv_cell(x, w, bias, conv_spec, stride=(stride, stride))
        OH = y.shape[2]
        dx = rt.DTensor.from_numpy(x, capi.U8B)
        for other_dtype, other in ((capi.U8B, rng.integers(0, 256, size=(B, O, OH, OH))), (capi.I8, rng.integers(-128, 128, size=(B, O, OH, OH))),
                                   (capi.U8B, rng.choice([0, 1, 254, 255], size=(B, O, OH, OH))), (capi.I8, rng.choice([-128, -1, 0, 127], size=(B, O, OH, OH)))):
            dother = rt.DTensor.from_numpy(other, other_dtype)
            for pre_mode in (None, "FixedMult16", "SingleShift"):
                if pre_mode == "FixedMult16":
                    pre_spec = ActSpec("Linear", "FixedMult16", rng.integers(2 ** 12, 2 ** 15, size=O), frac_bits=14, nb_bits=8,
                                       unsigned_out=other_dtype == capi.U8B)
                elif pre_mode == "SingleShift":
                    pre_spec = ActSpec("Linear", "SingleShift", rng.integers(0, 3, size=O), nb_bits=8, unsigned_out=other_dtype == capi.U8B)
                else:
                    pre_spec = None
                o2 = other.astype(np.float32) if pre_spec is None else pre_spec.apply(other.astype(np.float32))
                for k in (0, 1):
                    ins = [y, o2] if k == 0 else [o2, y]
                    want = cells_ref.elemwise_cell(ins, sum_spec).astype(np.int64)
                    ew = rt.ElemWiseSum(2, O, rt.Act(O, **sum_spec.kwargs()))
                    pre = None
                    if pre_spec is not None:
                        pre = rt.Act(O, **pre_spec.kwargs())
                        assert ew.fold_input_scaling(1 - k, pre)
                    # twice: with the sum's arithmetic on 16-bit pairs where the tables allow it, and on 32 bits
                    for no16 in (0, capi.KERNEL_NO_SUM16):
                        conv = rt.Conv(w, bias, rt.Act(O, **conv_spec.kwargs()), capi.U8B, stride=(stride, stride), kernel_choice=no16)
                        assert conv.fuse_sum(ew, k, other_dtype), (C, O)
                        out = rt.DTensor(B, O, OH, OH, capi.U8B)
                        conv.forward_sum(dx, dother, out)
                        got = out.to_numpy()
                        assert np.array_equal(got, want), (C, O, H, stride, other_dtype, pre_mode, k, no16, np.count_nonzero(got != want))
                    # the other input and the output may each carry a border of their own
                    if pre_mode is None and k == 0:
                        for oh, rh in ((0, 1), (1, 2), (2, 0)):
                            dother_h = rt.DTensor(B, O, OH, OH, other_dtype, halo=rh)
                            if rh:
                                dother_h.buf.view(B, OH + 2 * rh, OH + 2 * rh, dother_h.cs)[:, rh:OH + rh, rh:OH + rh, :] = \
                                    dother.buf.view(B, OH, OH, dother.cs)
                            else:
                                dother_h.buf.copy_(dother.buf)
                            out = rt.DTensor(B, O, OH, OH, capi.U8B, halo=oh)
                            conv.forward_sum(dx, dother_h, out)
                            assert np.array_equal(out.to_numpy(), want), (C, O, H, stride, other_dtype, oh, rh)
                    # the plain convolution is still available on the same handle
                    assert np.array_equal(conv.forward(dx).to_numpy(), y.astype(np.int64))
    # what cannot be folded is reported, and the cells then run separately
    w3 = np.clip(np.rint(rng.normal(0, 20, size=(64, 64, 3, 3))), -127, 127).astype(np.int64)
    conv3 = rt.Conv(w3, None, rt.Act(64, **conv_spec_for(64, rng).kwargs()), capi.U8B, pad=(1, 1, 1, 1))
    ew = rt.ElemWiseSum(2, 64, rt.Act(64, **sum_spec_for(64, rng).kwargs()))
    assert conv3.fuse_sum(ew, 0, capi.U8B) is False
    wc = np.clip(np.rint(rng.normal(0, 20, size=(64, 48, 1, 1))), -127, 127).astype(np.int64)
    conv48 = rt.Conv(wc, None, rt.Act(64, **conv_spec_for(64, rng).kwargs()), capi.U8B)
    assert conv48.fuse_sum(ew, 0, capi.U8B) is False
    w1 = np.clip(np.rint(rng.normal(0, 20, size=(64, 64, 1, 1))), -127, 127).astype(np.int64)
    conv1 = rt.Conv(w1, None, rt.Act(64, **conv_spec_for(64, rng).kwargs()), capi.U8B)
    ewf = rt.ElemWiseSum(2, 64, rt.Act(64, "Linear", "FloatMult", np.full(64, 0.5, np.float32), nb_bits=8, unsigned_out=True))
    assert conv1.fuse_sum(ewf, 0, capi.U8B) is False
    with pytest.raises(capi.N2D2HipError):
        conv1.forward_sum(rt.DTensor(1, 64, 4, 4, capi.U8B), rt.DTensor(1, 64, 4, 4, capi.U8B), rt.DTensor(1, 64, 4, 4, capi.U8B))


def test_conv_rescale_variants_agree(rt):
    """The pipelined kernel has two integer epilogues (32-bit multiply-shift-saturate, and scaled-up tables whose result is
    the upper register half, saturated as 16-bit pairs); both must give the oracle's bytes, for either output signedness."""
    from n2d2_amd import capi
    from oracle.cells import ActSpec
    from oracle import cells as cells_ref
    rng = np.random.default_rng(123)
    for C, O, H, k, pad, stride in ((64, 256, 9, 1, 0, 1), (128, 64, 7, 3, 1, 1), (64, 192, 6, 3, 0, 1), (3, 64, 45, 7, 3, 2)):
        x = rng.integers(0, 256, size=(3, C, H, H))
        w = np.clip(np.rint(rng.normal(0, 25, size=(O, C, k, k))), -127, 127).astype(np.int64)
        bias = rng.integers(-3000, 3000, size=O)
        for spec in (ActSpec("Rectifier", "DoubleShift", np.stack([rng.integers(0, 3, size=O), rng.integers(6, 13, size=O)], 1), nb_bits=8, unsigned_out=True),
                     ActSpec("Linear", "SingleShift", rng.integers(5, 16, size=O), nb_bits=8, unsigned_out=False),
                     ActSpec("Linear", "FixedMult16", rng.integers(2 ** 8, 2 ** 12, size=O), frac_bits=16, nb_bits=8, unsigned_out=False),
                     ActSpec("Rectifier", "FixedMult32", rng.integers(2 ** 18, 2 ** 22, size=O), frac_bits=28, nb_bits=8, unsigned_out=True)):
            want = cells_ref.conv_cell(x, w, bias, spec, stride=(stride, stride), pad=(pad, pad, pad, pad)).astype(np.int64)
            dx = rt.DTensor.from_numpy(x, capi.U8B)
            for no16 in (0, capi.KERNEL_NO_HI16):
                conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, stride=(stride, stride), pad=(pad, pad, pad, pad),
                               kernel_choice=no16)
                got = conv.forward(dx).to_numpy()
                assert np.array_equal(got, want), (C, O, k, spec.mode, no16, np.count_nonzero(got != want))


def test_conv_reads_and_writes_halo_tensors(rt):
    """A tensor stored with its reader's padding as a border of zeros: a convolution writes it (plain and with a folded sum),
    a padded KxK convolution reads it, the graph-edge conversion reads it, and every result equals the plain tensors'."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    rng = np.random.default_rng(91)
    for C, O, O2, H, W, k, stride, pad, halo, B in ((64, 64, 64, 9, 7, 3, 1, 1, 1, 3), (128, 128, 192, 8, 8, 3, 2, 1, 1, 2),
                                                     (64, 128, 64, 6, 10, 5, 1, 2, 2, 2), (256, 64, 64, 7, 7, 3, 1, 1, 2, 2),
                                                     (64, 64, 128, 12, 12, 1, 2, 0, 1, 2)):
        x = rng.integers(0, 256, size=(B, C, H, W))
        w1 = np.clip(np.rint(rng.normal(0, 20, size=(O, C, 1, 1))), -127, 127).astype(np.int64)
        w2 = np.clip(np.rint(rng.normal(0, 20, size=(O2, O, k, k))), -127, 127).astype(np.int64)
        s1, s2 = conv_spec_for(O, rng), conv_spec_for(O2, rng)
        s1.kind, s1.unsigned_out = "Rectifier", True
        b1, b2 = rng.integers(-500, 500, size=O), rng.integers(-500, 500, size=O2)
        y1 = cells_ref.conv_cell(x, w1, b1, s1)
        y2 = cells_ref.conv_cell(y1, w2, b2, s2, stride=(stride, stride), pad=(pad, pad, pad, pad))
        c1 = rt.Conv(w1, b1, rt.Act(O, **s1.kwargs()), capi.U8B)
        c2 = rt.Conv(w2, b2, rt.Act(O2, **s2.kwargs()), capi.U8B, stride=(stride, stride), pad=(pad, pad, pad, pad))
        assert c1.accepts_halo() and c2.accepts_halo()
        dx = rt.DTensor.from_numpy(x, capi.U8B)
        mid = c1.make_output(dx, halo=halo)
        assert mid.buf.numel() == B * (H + 2 * halo) * (W + 2 * halo) * mid.cs
        c1.forward(dx, mid)
        assert np.array_equal(mid.to_numpy(), y1.astype(np.int64)), (C, O, "written with a halo")
        border = mid.buf.view(B, H + 2 * halo, W + 2 * halo, mid.cs).clone()
        border[:, halo:H + halo, halo:W + halo, :] = -128
        assert bool((border == -128).all()), "the border keeps the stored form of 0"
        got = c2.forward(mid).to_numpy()
        assert np.array_equal(got, y2.astype(np.int64)), (C, O, O2, k, stride, pad, halo)
        # a reader with no padding of its own skips the border
        w3 = np.clip(np.rint(rng.normal(0, 20, size=(64, O, 1, 1))), -127, 127).astype(np.int64)
        s3 = conv_spec_for(64, rng)
        c3 = rt.Conv(w3, None, rt.Act(64, **s3.kwargs()), capi.U8B)
        assert np.array_equal(c3.forward(mid).to_numpy(), cells_ref.conv_cell(y1, w3, None, s3).astype(np.int64))
        # the folded residual sum writes a halo too
        ssum = sum_spec_for(O, rng)
        other = rng.integers(0, 256, size=(B, O, H, W))
        ew = rt.ElemWiseSum(2, O, rt.Act(O, **ssum.kwargs()))
        c1b = rt.Conv(w1, b1, rt.Act(O, **conv_spec_for(O, rng).kwargs()), capi.U8B)
        ylin = cells_ref.conv_cell(x, w1, b1, conv_spec_for(O, np.random.default_rng(5)))
        c1b = rt.Conv(w1, b1, rt.Act(O, **conv_spec_for(O, np.random.default_rng(5)).kwargs()), capi.U8B)
        assert c1b.fuse_sum(ew, 0, capi.U8B)
        want = cells_ref.elemwise_cell([ylin, other.astype(np.float32)], ssum).astype(np.int64)
        out = rt.DTensor(B, O, H, W, capi.U8B, halo=halo)
        c1b.forward_sum(dx, rt.DTensor.from_numpy(other, capi.U8B), out)
        assert np.array_equal(out.to_numpy(), want)
    # multipliers of 30 bits (the 64-bit product): written with a border, read from one
    from oracle.cells import ActSpec
    x = rng.integers(0, 256, size=(2, 64, 9, 7))
    w1 = np.clip(np.rint(rng.normal(0, 20, size=(128, 64, 1, 1))), -127, 127).astype(np.int64)
    w2 = np.clip(np.rint(rng.normal(0, 20, size=(64, 128, 3, 3))), -127, 127).astype(np.int64)
    s1 = ActSpec("Rectifier", "FixedMult32", rng.integers(2 ** 28, 2 ** 30, size=128), frac_bits=37, nb_bits=8, unsigned_out=True)
    s2 = ActSpec("Linear", "FixedMult32", rng.integers(2 ** 28, 2 ** 30, size=64), frac_bits=40, nb_bits=8, unsigned_out=False)
    y1 = cells_ref.conv_cell(x, w1, None, s1)
    y2 = cells_ref.conv_cell(y1, w2, None, s2, pad=(1, 1, 1, 1))
    c1 = rt.Conv(w1, None, rt.Act(128, **s1.kwargs()), capi.U8B)
    c2 = rt.Conv(w2, None, rt.Act(64, **s2.kwargs()), capi.U8B, pad=(1, 1, 1, 1))
    assert c1.accepts_halo() and c2.accepts_halo() and len(np.unique(y2)) > 50
    mid = c1.make_output(rt.DTensor.from_numpy(x, capi.U8B), halo=1)
    c1.forward(rt.DTensor.from_numpy(x, capi.U8B), mid)
    assert np.array_equal(mid.to_numpy(), y1.astype(np.int64)) and np.array_equal(c2.forward(mid).to_numpy(), y2.astype(np.int64))
    # cells that do not take a halo say so
    xh = rt.DTensor(1, 64, 4, 4, capi.U8B, halo=1)
    with pytest.raises(capi.N2D2HipError):
        rt.Pool("max", (2, 2), (2, 2), (0, 0)).forward(xh)
    wd = np.clip(np.rint(rng.normal(0, 20, size=(64, 48, 3, 3))), -127, 127).astype(np.int64)
    c48 = rt.Conv(wd, None, rt.Act(64, **conv_spec_for(64, rng).kwargs()), capi.U8B, pad=(1, 1, 1, 1))
    assert not c48.accepts_halo()


def test_conv3x3_patch_kernel_bit_exact(rt):
    """3x3, stride 1, padding 1 on an input that carries its padding: the kernel that reads one patch of pixels at nine
    shifts (weights straight to registers in fragment order), against the oracle and against the pipelined kernel, over
    image sizes whose rows are shorter and longer than a tile, tiles that straddle images, channel counts that take the
    two-wave and the four-wave block, tiles of 128 and of 256 positions, several 64-channel steps, both epilogues, outputs
    with and without a border."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    from oracle.cells import ActSpec
    rng = np.random.default_rng(123)
    cases = ((64, 64, 9, 7, 3), (64, 128, 28, 28, 2), (128, 64, 14, 14, 5), (192, 128, 7, 7, 9), (64, 64, 56, 56, 1),
             (128, 256, 5, 33, 2), (256, 128, 30, 3, 3), (64, 192, 1, 1, 70), (128, 128, 60, 4, 1))
    for C, O, H, W, B in cases:
        x = rng.integers(0, 256, size=(B, C, H, W))
        w = np.clip(np.rint(rng.normal(0, 25, size=(O, C, 3, 3))), -127, 127).astype(np.int64)
        bias = rng.integers(-3000, 3000, size=O)
        specs = (ActSpec("Rectifier", "DoubleShift", np.stack([rng.integers(0, 3, size=O), rng.integers(9, 13, size=O)], 1), nb_bits=8, unsigned_out=True),
                 ActSpec("Linear", "SingleShift", rng.integers(9, 15, size=O), nb_bits=8, unsigned_out=False),
                 ActSpec("Rectifier", "FixedMult16", rng.integers(2 ** 6, 2 ** 10, size=O), frac_bits=20, nb_bits=8, unsigned_out=True))
        dx = rt.DTensor.from_numpy(x, capi.U8B).with_halo(1)
        for spec in specs:
            want = cells_ref.conv_cell(x, w, bias, spec, pad=(1, 1, 1, 1)).astype(np.int64)
            for choice in (capi.KERNEL_PATCH | capi.KERNEL_TILE_M256, capi.KERNEL_PATCH | capi.KERNEL_TILE_M128, capi.KERNEL_PATCH | capi.KERNEL_TILE_M64,
                           capi.KERNEL_PATCH | capi.KERNEL_NO_HI16 | capi.KERNEL_TILE_M256, capi.KERNEL_PATCH | capi.KERNEL_NO_HI16 | capi.KERNEL_TILE_M128,
                           capi.KERNEL_PATCH, 0, capi.KERNEL_NO_PATCH):
                print("patch conv", (C, O, H, W, B), spec.mode, choice, flush=True)
                conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, pad=(1, 1, 1, 1), kernel_choice=choice)
                assert conv.accepts_halo()
                for out_halo in (0, 1):
                    out = conv.make_output(dx, halo=out_halo)
                    conv.forward(dx, out)
                    got = out.to_numpy()
                    assert np.array_equal(got, want), (C, O, H, W, B, spec.mode, choice, out_halo, np.count_nonzero(got != want))
                    if out_halo:
                        border = out.buf.view(B, H + 2, W + 2, out.cs).clone()
                        border[:, 1:H + 1, 1:W + 1, :] = out.buf.view(-1)[0]
                        assert bool((border == out.buf.view(-1)[0]).all()), "the output's border is left alone"


def test_bottleneck_in_one_launch_bit_exact(rt):
    """n2d2hip_bottleneck_*: 1x1 -> 3x3 (-> 1x1 + sum with the block's input, plain or through a folded ScalingCell, or with
    a projection of it) in one launch equals the reference cells run in turn; the cells stay usable on their own.  Images
    narrower and wider than a tile's reach, tiles that straddle images, outputs with and without a border."""
    from n2d2_amd import capi
    from oracle.cells import ActSpec
    from oracle import cells as cells_ref
    rng = np.random.default_rng(4242)

    def relu_spec(O):
        return ActSpec("Rectifier", "DoubleShift", np.stack([rng.integers(0, 3, size=O), rng.integers(8, 12, size=O)], 1), nb_bits=8, unsigned_out=True)

    def lin_spec(O):
        return ActSpec("Linear", "SingleShift", rng.integers(8, 12, size=O), nb_bits=8, unsigned_out=False)

    def weights(O, Cc, k, std):
        return np.clip(np.rint(rng.normal(0, std, size=(O, Cc, k, k))), -127, 127).astype(np.int64)
    for cin, H, W, B, variant in ((256, 9, 7, 3, "identity"), (64, 9, 7, 3, "projection"), (256, 12, 20, 2, "scaled identity"),
                                  (256, 56, 56, 1, "identity"), (64, 30, 58, 2, "projection"), (64, 5, 61, 2, "two cells"),
                                  (256, 3, 1, 40, "two cells"), (256, 1, 1, 150, "scaled identity")):
        print("bottleneck", cin, H, W, B, variant, flush=True)
        x = rng.integers(0, 256, size=(B, cin, H, W))
        wa, wb, wc, wp = weights(64, cin, 1, 12), weights(64, 64, 3, 10), weights(256, 64, 1, 25), weights(256, cin, 1, 25)
        ba, bb, bc, bp = (rng.integers(-2000, 2000, size=n) for n in (64, 64, 256, 256))
        sa, sb, sc, sp = relu_spec(64), relu_spec(64), lin_spec(256), lin_spec(256)
        ssum = sum_spec_for(256, rng)
        t1 = cells_ref.conv_cell(x, wa, ba, sa)
        t2 = cells_ref.conv_cell(t1, wb, bb, sb, pad=(1, 1, 1, 1))
        ca = rt.Conv(wa, ba, rt.Act(64, **sa.kwargs()), capi.U8B)
        cb = rt.Conv(wb, bb, rt.Act(64, **sb.kwargs()), capi.U8B, pad=(1, 1, 1, 1))
        dx = rt.DTensor.from_numpy(x, capi.U8B).with_halo(1)
        if variant == "two cells":
            bn = rt.Bottleneck.create(ca, cb)
            assert bn is not None
            for out_halo in (0, 1):
                out = rt.DTensor(B, 64, H, W, capi.U8B, halo=out_halo)
                got = bn.forward(dx, out).to_numpy()
                assert np.array_equal(got, t2.astype(np.int64)), (cin, H, W, B, variant, out_halo, np.count_nonzero(got != t2))
            continue
        t3 = cells_ref.conv_cell(t2, wc, bc, sc)
        cc = rt.Conv(wc, bc, rt.Act(256, **sc.kwargs()), capi.U8B)
        ew = rt.ElemWiseSum(2, 256, rt.Act(256, **ssum.kwargs()))
        cp_, pre = None, None
        if variant == "projection":
            other = cells_ref.conv_cell(x, wp, bp, sp)
            cp_ = rt.Conv(wp, bp, rt.Act(256, **sp.kwargs()), capi.U8B)
            assert cc.fuse_sum(ew, 0, capi.I8)
        else:
            other = x.astype(np.float32)
            if variant == "scaled identity":
                pre_spec = ActSpec("Linear", "FixedMult16", rng.integers(2 ** 12, 2 ** 15, size=256), frac_bits=14, nb_bits=8, unsigned_out=True)
                other = pre_spec.apply(other)
                pre = rt.Act(256, **pre_spec.kwargs())
                assert ew.fold_input_scaling(1, pre)
            assert cc.fuse_sum(ew, 0, capi.U8B)
        want = cells_ref.elemwise_cell([t3, other], ssum).astype(np.int64)
        bn = rt.Bottleneck.create(ca, cb, cc, cp_)
        assert bn is not None, variant
        for out_halo in (1, 0):
            out = rt.DTensor(B, 256, H, W, capi.U8B, halo=out_halo)
            got = bn.forward(dx, out).to_numpy()
            assert np.array_equal(got, want), (cin, H, W, B, variant, out_halo, np.count_nonzero(got != want))
        # the cells still run on their own
        assert np.array_equal(cb.forward(ca.forward(dx, ca.make_output(dx, halo=1))).to_numpy(), t2.astype(np.int64))
    # what does not qualify is reported
    w128 = weights(128, 256, 1, 12)
    c128 = rt.Conv(w128, None, rt.Act(128, **relu_spec(128).kwargs()), capi.U8B)
    assert rt.Bottleneck.create(c128, cb) is None


def test_first_layer_conv_with_max_pool_in_one_launch_bit_exact(rt):
    """n2d2hip_conv_forward_maxpool: a first-layer convolution and the 3x3 stride-2 max pooling behind it in one launch equal
    the two reference cells; 7x7 / 5x5 / 3x3 kernels, pooling padding 1 and 0, odd sizes (strips that end unevenly, last
    rows and columns clamped), signed and unsigned outputs, pooled outputs with and without a border."""
    from n2d2_amd import capi
    from oracle.cells import ActSpec
    from oracle import cells as cells_ref
    rng = np.random.default_rng(99)
    for (B, H, W, k, pad, ppad, unsigned) in ((3, 224, 224, 7, 3, 1, True), (2, 64, 64, 7, 3, 0, True), (5, 37, 45, 3, 1, 1, True),
                                              (70, 30, 22, 5, 2, 1, False), (1, 9, 250, 3, 1, 0, True), (2, 224, 224, 7, 3, 0, False)):
        print("stem+pool", B, H, W, k, pad, ppad, unsigned, flush=True)
        x = rng.integers(0, 256, size=(B, 3, H, W))
        w = np.clip(np.rint(rng.normal(0, 30, size=(64, 3, k, k))), -127, 127).astype(np.int64)
        bias = rng.integers(-3000, 3000, size=64)
        if unsigned:
            spec = ActSpec("Rectifier", "DoubleShift", np.stack([rng.integers(0, 3, size=64), rng.integers(8, 11, size=64)], 1), nb_bits=8, unsigned_out=True)
        else:
            spec = ActSpec("Linear", "SingleShift", rng.integers(8, 11, size=64), nb_bits=8, unsigned_out=False)
        conv = rt.Conv(w, bias, rt.Act(64, **spec.kwargs()), capi.U8B, stride=(2, 2), pad=(pad,) * 4)
        pool = rt.Pool("max", (3, 3), (2, 2), (ppad, ppad))
        t = cells_ref.conv_cell(x, w, bias, spec, stride=(2, 2), pad=(pad,) * 4)
        want = cells_ref.pool_cell(t, "max", (3, 3), (2, 2), (ppad, ppad)).astype(np.int64)
        dx = rt.DTensor.from_numpy(x, capi.U8B)
        assert conv.accepts_maxpool(pool, H, W)
        for halo in (0, 1):
            out = rt.DTensor(B, 64, want.shape[2], want.shape[3], capi.U8B if unsigned else capi.I8, halo=halo)
            got = conv.forward_maxpool(pool, dx, out).to_numpy()
            assert np.array_equal(got, want), (B, H, W, k, pad, ppad, halo, np.count_nonzero(got != want))
        # the two cells on their own give the same
        assert np.array_equal(pool.forward(conv.forward(dx)).to_numpy(), want)
    # what does not qualify is reported: a 2x2 pooling, a convolution with 64 input channels
    assert not conv.accepts_maxpool(rt.Pool("max", (2, 2), (2, 2)), 224, 224)
    c64 = rt.Conv(np.ones((64, 64, 3, 3), dtype=np.int64), None, rt.Act(64, **spec.kwargs()), capi.U8B, stride=(2, 2), pad=(1,) * 4)
    assert not c64.accepts_maxpool(pool, 56, 56)


def test_first_layer_conv_on_space_to_depth_input_bit_exact(rt):
    """A first-layer convolution of stride 2 reading the network input in its space-to-depth form (n2d2hip_convert into
    N2D2HIP_S2D, n2d2hip_conv_s2d_halo) equals the reference cell, alone and with the 3x3 stride-2 max pooling behind it in
    the same launch: 7x7 / 5x5 / 3x3 kernels, even and odd paddings, odd image sizes (a last row / column that half exists),
    1 to 4 input channels, 64 / 32 / 48 outputs, scaled-up and full integer rescales (a Clip), signed inputs and outputs,
    batches that give a block several strips, pooled outputs with a border, conversion from int32, float and byte planes."""
    from n2d2_amd import capi
    from oracle.cells import ActSpec
    from oracle import cells as cells_ref
    import torch
    rng = np.random.default_rng(2718)
    cases = (  # B, C, H, W, O, k, pad, pool padding (None: no pooling), unsigned output, clip, source dtype
        (3, 3, 224, 224, 64, 7, 3, 1, True, False, "u8"), (2, 3, 224, 224, 64, 7, 3, None, True, False, "i32"),
        (2, 3, 64, 64, 64, 7, 3, 0, True, False, "f32"), (5, 3, 37, 45, 64, 3, 1, 1, True, False, "u8"),
        (70, 3, 30, 22, 64, 5, 2, 1, False, False, "i32"), (1, 3, 9, 222, 64, 3, 1, 0, True, False, "u8"),
        (2, 3, 224, 224, 32, 3, 1, None, True, False, "u8"), (3, 4, 50, 34, 48, 3, 0, None, True, False, "i32"),
        (2, 3, 224, 224, 64, 7, 3, None, True, True, "u8"), (4, 1, 33, 33, 16, 5, 1, None, False, False, "i32"),
        (2, 2, 96, 96, 64, 7, 2, 1, True, False, "u8"), (600, 3, 16, 16, 64, 3, 1, 1, True, False, "u8"),
        (130, 3, 40, 40, 32, 7, 3, None, True, True, "u8"))
    for (B, Cc, H, W, O, k, pad, ppad, unsigned, clip, src_kind) in cases:
        print("s2d stem", B, Cc, H, W, O, k, pad, ppad, unsigned, clip, src_kind, flush=True)
        x = rng.integers(0, 256, size=(B, Cc, H, W))
        w = np.clip(np.rint(rng.normal(0, 30, size=(O, Cc, k, k))), -127, 127).astype(np.int64)
        bias = rng.integers(-3000, 3000, size=O)
        if clip:
            spec = ActSpec("Rectifier", "FixedMult16", rng.integers(64, 256, size=O), frac_bits=16,
                           clipping=rng.uniform(3e4, 9e4, size=O).astype(np.float32), nb_bits=8, unsigned_out=True)
        elif unsigned:
            spec = ActSpec("Rectifier", "DoubleShift", np.stack([rng.integers(0, 3, size=O), rng.integers(8, 11, size=O)], 1), nb_bits=8, unsigned_out=True)
        else:
            spec = ActSpec("Linear", "SingleShift", rng.integers(8, 11, size=O), nb_bits=8, unsigned_out=False)
        conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), capi.U8B, stride=(2, 2), pad=(pad,) * 4)
        pool = rt.Pool("max", (3, 3), (2, 2), (ppad, ppad)) if ppad is not None else None
        want = cells_ref.conv_cell(x, w, bias, spec, stride=(2, 2), pad=(pad,) * 4)
        if pool is not None:
            want = cells_ref.pool_cell(want, "max", (3, 3), (2, 2), (ppad, ppad))
        want = want.astype(np.int64)
        halo = conv.s2d_halo(H, W, pool)
        assert halo >= 0, (B, Cc, H, W, O, k, pad, ppad)
        if src_kind == "u8":
            src = rt.DTensor(B, Cc, H, W, capi.U8, capi.NCHW, torch.from_numpy(x.astype(np.uint8).reshape(-1)).cuda())
        elif src_kind == "f32":
            src = rt.DTensor.from_numpy(x.astype(np.float32), capi.F32, capi.NCHW)
        else:
            src = rt.DTensor.from_numpy(x, capi.I32, capi.NCHW)
        for extra in (0, 1):          # a larger border than needed is as good
            dx = rt.DTensor(B, Cc, H, W, capi.U8B, capi.S2D, halo=halo + extra)
            dx.buf.fill_(77)          # the conversion writes every byte of it, border included
            dx.convert_from(src)
            for out_halo in ((0, 1) if pool is not None else (0,)):
                out = rt.DTensor(B, O, want.shape[2], want.shape[3], capi.U8B if unsigned else capi.I8, halo=out_halo)
                got = (conv.forward_maxpool(pool, dx, out) if pool is not None else conv.forward(dx, out)).to_numpy()
                assert np.array_equal(got, want), (B, Cc, H, W, O, k, pad, ppad, extra, out_halo, np.count_nonzero(got != want))
    # what is not served says so: stride 1, a 64-channel input, a row too long
    act = rt.Act(O, **spec.kwargs())
    assert rt.Conv(w, bias, act, capi.U8B, stride=(1, 1), pad=(pad,) * 4).s2d_halo(64, 64) == -1
    assert conv.s2d_halo(64, 600) == -1
    # ... and a border that is too small is refused with a message
    dx = rt.DTensor(2, 3, 40, 40, capi.U8B, capi.S2D, halo=0)
    with pytest.raises(capi.N2D2HipError, match="border"):
        conv.forward(dx, rt.DTensor(2, 32, 20, 20, capi.U8B))


def test_conv3x3_expansion_and_sum_in_one_launch_bit_exact(rt):
    """n2d2hip_conv_chain_forward: 3x3 convolution -> 1x1 expansion -> sum with another tensor (plain, or through a folded
    ScalingCell) in one launch equals the reference cells run in turn, and the two launches of the library.  64, 128 and 256
    middle channels, stride 1 and 2, tiles that end inside the tensor, inputs, shortcuts and outputs with and without
    a border."""
    from n2d2_amd import capi
    from oracle.cells import ActSpec
    from oracle import cells as cells_ref
    rng = np.random.default_rng(777)

    def relu_spec(O):
        return ActSpec("Rectifier", "DoubleShift", np.stack([rng.integers(0, 3, size=O), rng.integers(8, 12, size=O)], 1), nb_bits=8, unsigned_out=True)

    def lin_spec(O):
        return ActSpec("Linear", "SingleShift", rng.integers(8, 12, size=O), nb_bits=8, unsigned_out=False)

    def sum_spec(O):
        return ActSpec("Rectifier", "DoubleShift", np.stack([rng.integers(0, 3, size=O), rng.integers(0, 3, size=O)], 1), nb_bits=8, unsigned_out=True)

    def weights(O, Cc, k, std):
        return np.clip(np.rint(rng.normal(0, std, size=(O, Cc, k, k))), -127, 127).astype(np.int64)
    cases = ((64, 9, 7, 3, 1, "plain", 1, 0, 0), (64, 20, 20, 2, 1, "scaled", 1, 1, 1), (64, 13, 11, 2, 2, "plain", 1, 0, 1),
             (128, 10, 9, 3, 1, "scaled", 1, 0, 0), (128, 14, 14, 2, 2, "plain", 2, 1, 0), (128, 7, 5, 9, 1, "plain", 1, 1, 1),
             (256, 7, 7, 3, 1, "scaled", 1, 0, 0), (256, 14, 14, 2, 1, "plain", 1, 1, 1), (256, 9, 12, 2, 2, "scaled", 1, 0, 1),
             (256, 1, 1, 70, 1, "plain", 1, 0, 0))
    for cm, H, W, B, stride, variant, in_halo, other_halo, out_halo in cases:
        print("chain", cm, H, W, B, stride, variant, in_halo, other_halo, out_halo, flush=True)
        oc = 4 * cm
        x = rng.integers(0, 256, size=(B, cm, H, W))
        wb, wc = weights(cm, cm, 3, 6 if cm > 64 else 10), weights(oc, cm, 1, 18)
        bb, bc = rng.integers(-2000, 2000, size=cm), rng.integers(-2000, 2000, size=oc)
        sb, sc, ssum = relu_spec(cm), lin_spec(oc), sum_spec(oc)
        t2 = cells_ref.conv_cell(x, wb, bb, sb, stride=(stride, stride), pad=(1, 1, 1, 1))
        t3 = cells_ref.conv_cell(t2, wc, bc, sc)
        OH, OW = t2.shape[2], t2.shape[3]
        other_src = rng.integers(0, 256, size=(B, oc, OH, OW))
        cb = rt.Conv(wb, bb, rt.Act(cm, **sb.kwargs()), capi.U8B, stride=(stride, stride), pad=(1, 1, 1, 1))
        cc = rt.Conv(wc, bc, rt.Act(oc, **sc.kwargs()), capi.U8B)
        ew = rt.ElemWiseSum(2, oc, rt.Act(oc, **ssum.kwargs()))
        other = other_src.astype(np.float32)
        if variant == "scaled":
            pre_spec = ActSpec("Linear", "FixedMult16", rng.integers(2 ** 12, 2 ** 15, size=oc), frac_bits=14, nb_bits=8, unsigned_out=True)
            other = pre_spec.apply(other)
            assert ew.fold_input_scaling(1, rt.Act(oc, **pre_spec.kwargs()))
        assert cc.fuse_sum(ew, 0, capi.U8B)
        want = cells_ref.elemwise_cell([t3, other], ssum).astype(np.int64)
        assert cc.chain_supported(cb), (cm, variant)
        dx = rt.DTensor.from_numpy(x, capi.U8B).with_halo(in_halo)
        dother = rt.DTensor.from_numpy(other_src, capi.U8B)
        if other_halo:
            dother = dother.with_halo(other_halo)
        out = rt.DTensor(B, oc, OH, OW, capi.U8B, halo=out_halo)
        got = cc.forward_chain(cb, dx, dother, out).to_numpy()
        assert np.array_equal(got, want), (cm, H, W, B, stride, variant, np.count_nonzero(got != want))
        # the two cells still run on their own, to the same result
        mid = cb.forward(dx, cb.make_output(dx))
        assert np.array_equal(mid.to_numpy(), t2.astype(np.int64))
        two = cc.forward_sum(mid, dother, rt.DTensor(B, oc, OH, OW, capi.U8B)).to_numpy()
        assert np.array_equal(two, want)
    # what does not qualify is reported: an expansion to twice the channels, a 3x3 convolution with a dilation
    w2 = weights(128, 64, 1, 18)
    c2 = rt.Conv(w2, None, rt.Act(128, **lin_spec(128).kwargs()), capi.U8B)
    wb = weights(64, 64, 3, 10)
    cb = rt.Conv(wb, None, rt.Act(64, **relu_spec(64).kwargs()), capi.U8B, pad=(1, 1, 1, 1))
    assert not c2.chain_supported(cb)


def conv_spec_for(O, rng):
    from oracle.cells import ActSpec
    return ActSpec("Linear", "DoubleShift", np.stack([rng.integers(0, 3, size=O), rng.integers(8, 12, size=O)], 1), nb_bits=8, unsigned_out=False)


def sum_spec_for(O, rng):
    from oracle.cells import ActSpec
    return ActSpec("Rectifier", "DoubleShift", np.stack([rng.integers(0, 3, size=O), rng.integers(0, 3, size=O)], 1), nb_bits=8, unsigned_out=True)


@pytest.mark.parametrize("case", [(3, 32, 64, 1, 19, 21, 1), (2, 64, 128, 2, 23, 17, 1), (2, 128, 128, 1, 14, 14, 1), (2, 128, 256, 2, 28, 28, 1),
                                  (1, 256, 512, 2, 9, 10, 0), (2, 192, 64, 1, 8, 16, 1), (1, 32, 128, 2, 33, 41, 1),
                                  (1, 64, 256, 1, 11, 37, 0), (1, 512, 1024, 1, 5, 6, 1), (3, 128, 512, 1, 14, 14, 1),
                                  (2, 512, 512, 2, 15, 13, 1), (2, 64, 512, 1, 6, 18, 0)],
                         ids=lambda c: "x".join(str(v) for v in c))
def test_depthwise_and_pointwise_in_one_launch_bit_exact(rt, case):
    """n2d2hip_dw_pw_*: a 3x3 depthwise convolution and the 1x1 convolution reading it as one launch, against the oracle
    running the two cells and against the two separate launches; shapes whose tiles end unevenly in both directions,
    every chunk width and channel-tile count, unsigned and signed depthwise outputs."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    B, Cc, O, stride, H, W, pad = case
    _say("dw_pw %s" % (case,))
    signed_mid = Cc == 128 and O == 128
    x = _u8((B, Cc, H, W))
    wd = _i8((Cc, 1, 3, 3))
    bd = RNG.integers(-2000, 2001, size=Cc).astype(np.int32)
    wp = _i8((O, Cc, 1, 1))
    bp = RNG.integers(-20000, 20001, size=O).astype(np.int32)
    from oracle.cells import ActSpec
    # multipliers small enough that no accumulator can overflow the 32-bit multiply-add (the kernel's short rescale) on the
    # stride-1 cases, larger ones (a clamp comes first) on the others
    small = stride == 1 and not signed_mid
    if signed_mid:
        sd = ActSpec("Linear", "FixedMult32", RNG.integers(2 ** 13, 2 ** 14, size=Cc), frac_bits=21, nb_bits=8, unsigned_out=False)
    elif small:
        sd = ActSpec("Rectifier", "FixedMult32", RNG.integers(2 ** 11, 2 ** 12, size=Cc), frac_bits=18, nb_bits=8, unsigned_out=True)
    else:
        sd = ActSpec("Rectifier", "FixedMult32", RNG.integers(2 ** 13, 2 ** 14, size=Cc), frac_bits=20, nb_bits=8, unsigned_out=True)
    if small:
        sp = ActSpec("Rectifier", "FixedMult32", RNG.integers(2 ** 7, 2 ** 8, size=O), frac_bits=15 + (Cc // 64) % 3, nb_bits=8, unsigned_out=True)
    else:
        sp = ActSpec("Rectifier", "FixedMult32", RNG.integers(2 ** 13, 2 ** 14, size=O), frac_bits=16 + (Cc // 32) % 6, nb_bits=8, unsigned_out=True)
    mid = cells_ref.conv_cell(x, wd, bd, sd, stride=(stride, stride), pad=(pad,) * 4, groups=Cc)
    want = cells_ref.conv_cell(mid, wp, bp, sp)
    mid_dtype = capi.I8 if signed_mid else capi.U8B
    dw = rt.Conv(wd, bd, rt.Act(Cc, **sd.kwargs()), capi.U8B, stride=(stride, stride), pad=(pad,) * 4, groups=Cc)
    pw = rt.Conv(wp, bp, rt.Act(O, **sp.kwargs()), mid_dtype)
    xin = rt.DTensor.from_numpy(x, capi.U8B)
    separate = pw.forward(dw.forward(xin)).to_numpy()
    assert np.array_equal(separate, want.astype(np.int64))
    fused = rt.DwPw.create(dw, pw)
    assert fused is not None
    out = rt.DTensor(B, O, want.shape[2], want.shape[3], capi.U8B)
    got = fused.forward(xin, out).to_numpy()
    bad = np.count_nonzero(got != want)
    assert bad == 0, "%d of %d values differ" % (bad, want.size)
    # a pair the kernel is not written for is declined, not run: a 5-channel-wide 1x1 convolution
    narrow = rt.Conv(_i8((40, Cc, 1, 1)), None, rt.Act(40, **ActSpec("Rectifier", "SingleShift", RNG.integers(8, 12, size=40), nb_bits=8,
                                                                       unsigned_out=True).kwargs()), mid_dtype)
    assert rt.DwPw.create(dw, narrow) is None


def test_conv_randomized_sweep(rt):
    """Seeded sweep over the pipelined kernel's shape space (channel counts that are multiples of 64, kernel sizes, strides,
    paddings, dilations, ragged pixel counts, both input types, every integer rescale and both output signednesses, inputs
    and outputs with and without a border of zeros), each case against the oracle bit for bit."""
    from n2d2_amd import capi
    from oracle.cells import ActSpec
    from oracle import cells as cells_ref
    rng = np.random.default_rng(20240607)
    ncase = 0
    for it in range(48):
        C = int(rng.choice([64, 128, 192, 256, 320]))
        O = int(rng.choice([16, 64, 96, 128, 192, 256]))
        k = int(rng.choice([1, 1, 3, 3, 5]))
        kh = k if rng.random() < 0.8 else int(rng.choice([1, 3]))
        stride = int(rng.choice([1, 1, 2]))
        pad = int(rng.integers(0, k // 2 + 2)) if k > 1 else int(rng.integers(0, 2))
        dil = 2 if (k == 3 and rng.random() < 0.15) else 1
        H, W = int(rng.integers(dil * (kh - 1) + 1, 15)), int(rng.integers(dil * (k - 1) + 1, 15))
        B = int(rng.integers(1, 5))
        signed_in = rng.random() < 0.3
        x = rng.integers(-128, 128, size=(B, C, H, W)) if signed_in else rng.integers(0, 256, size=(B, C, H, W))
        in_dt = capi.I8 if signed_in else capi.U8B
        w = np.clip(np.rint(rng.normal(0, rng.choice([4, 20, 60]), size=(O, C, kh, k))), -127, 127).astype(np.int64)
        bias = rng.integers(-5000, 5000, size=O) if rng.random() < 0.8 else None
        unsigned_out = bool(rng.random() < 0.5)
        kind = "Rectifier" if unsigned_out else "Linear"
        mode = str(rng.choice(["SingleShift", "DoubleShift", "FixedMult16", "FixedMult32", "None"]))
        if mode == "SingleShift":
            spec = ActSpec(kind, mode, rng.integers(4, 18, size=O), nb_bits=8, unsigned_out=unsigned_out)
        elif mode == "DoubleShift":
            spec = ActSpec(kind, mode, np.stack([rng.integers(0, 5, size=O), rng.integers(6, 17, size=O)], 1), nb_bits=8, unsigned_out=unsigned_out)
        elif mode == "FixedMult16":
            spec = ActSpec(kind, mode, rng.integers(2 ** 6, 2 ** 15, size=O), frac_bits=int(rng.integers(14, 24)), nb_bits=8, unsigned_out=unsigned_out)
        elif mode == "FixedMult32":
            spec = ActSpec(kind, mode, rng.integers(2 ** 16, 2 ** 26, size=O), frac_bits=int(rng.integers(26, 36)), nb_bits=8, unsigned_out=unsigned_out)
        else:
            spec = ActSpec(kind, "None")
        p4 = (pad, pad, pad, pad)
        want = cells_ref.conv_cell(x.astype(np.float32), w, bias, spec, stride=(stride, stride), pad=p4, dil=(dil, dil))
        if np.abs(want).max() >= 2 ** 24:
            continue                                                    # the float-typed reference is exact below 2^24 only
        want = want.astype(np.int64)
        conv = rt.Conv(w, bias, rt.Act(O, **spec.kwargs()), in_dt, stride=(stride, stride), pad=p4, dil=(dil, dil))
        tag = (it, C, O, k, kh, stride, pad, dil, H, W, B, mode, unsigned_out, signed_in)
        _say("sweep %s" % (tag,))
        dx = rt.DTensor.from_numpy(x, in_dt)
        got = conv.forward(dx).to_numpy()
        assert got.shape == want.shape and np.array_equal(got, want), tag
        ncase += 1
        if conv.accepts_halo() and dil == 1 and mode != "None":
            # the same input stored with a border of zeros at least as wide as the padding, and a bordered output
            halo_in, halo_out = max(pad, 1) + int(rng.integers(0, 2)), int(rng.integers(1, 3))
            xin = rt.DTensor(B, C, H, W, in_dt, halo=halo_in)
            view = xin.buf.view(B, H + 2 * halo_in, W + 2 * halo_in, xin.cs)
            view[:, halo_in:H + halo_in, halo_in:W + halo_in, :] = dx.buf.view(B, H, W, dx.cs)
            out = conv.make_output(dx, halo=halo_out)
            conv.forward(xin, out)
            assert np.array_equal(out.to_numpy(), want), ("halo", halo_in, halo_out) + tag
    assert ncase >= 40


def test_fc_cells_in_a_row_in_one_launch_bit_exact(rt):
    """n2d2hip_fc_chain_*: two or three FcCells, each reading the one before, in one launch equal the reference cells run in
    turn: every rescale mode between the cells, raw int32 and byte outputs, signed and unsigned vectors, an input with
    height and width, a batch that does not fill the last work-group."""
    from n2d2_amd import capi
    from oracle import cells as cells_ref
    rng = np.random.default_rng(99)
    for B, shape, widths, modes in ((37, (16, 5, 5), (120, 84, 10), ("fixed_relu_u", "dshift_relu_u", "none_linear")),
                                    (5, (250, 1, 1), (128, 17), ("float_clip_s", "sshift_lin_s")),
                                    (64, (8, 3, 2), (33, 128, 7), ("dshift_lin_s", "fixed_clip_s", "fixed_wide")),
                                    (3, (1024, 1, 1), (64, 64), ("sshift_relu_u", "none_relu"))):
        print("fc chain", B, shape, widths, modes, flush=True)
        Cc, H, W = shape
        x = rng.integers(0, 256, size=(B, Cc, H, W))
        want = x
        cells, specs = [], []
        in_dtype, in_shape = capi.U8B, shape
        for O, mode in zip(widths, modes):
            K = in_shape[0] * in_shape[1] * in_shape[2]
            w = rng.integers(-20, 21, size=(O, K))
            bias = rng.integers(-500, 500, size=O)
            spec = _acts(O)[mode]
            act = rt.Act(O, **spec.kwargs())
            cells.append(rt.Fc(w, bias, act, in_dtype, in_shape))
            want = cells_ref.fc_cell(want, w, bias, spec)
            in_dtype, in_shape = act.out_dtype(), (O, 1, 1)
        chain = rt.FcChain.create(cells)
        assert chain is not None
        dx = rt.DTensor.from_numpy(x, capi.U8B)
        out = rt.DTensor(B, widths[-1], 1, 1, cells[-1].act.out_dtype())
        got = chain.forward(dx, out).to_numpy()
        assert np.array_equal(got, np.asarray(want).astype(np.int64).reshape(got.shape)), (B, shape, widths, modes)
        # the cells still run on their own, to the same result
        t = dx
        for c in cells:
            t = c.forward(t)
        assert np.array_equal(t.to_numpy(), got)
    # what does not qualify is reported: a cell with more than 128 outputs
    act = rt.Act(200, **_acts(200)["sshift_relu_u"].kwargs())
    wide = rt.Fc(rng.integers(-5, 6, size=(200, 64)), None, act, capi.U8B, (64, 1, 1))
    narrow = rt.Fc(rng.integers(-5, 6, size=(10, 200)), None, rt.Act(10, **_acts(10)["none_linear"].kwargs()), capi.U8B, (200, 1, 1))
    assert rt.FcChain.create([wide, narrow]) is None
