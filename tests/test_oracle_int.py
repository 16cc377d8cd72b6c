"""Pins the integer part of the CPU oracle against independent mathematics:
textbook cross-correlation, the brute-force loop of the reference's own conv
unit test, GEMM/FC equivalences, exact rational forms of the rescales."""
import itertools

import numpy as np
import pytest

import refmath as rm
from oracle import oracle as orc

RNG = np.random.default_rng(1234)


def _u8(shape):
    return RNG.integers(0, 256, size=shape).astype(np.float32)


def _i8(shape):
    return RNG.integers(-127, 128, size=shape).astype(np.float32)


# ------------------------------------------------------------------- conv

@pytest.mark.parametrize("k,s,p", [((3, 3), (1, 1), (1, 1)), ((5, 5), (1, 1), (0, 0)), ((7, 7), (2, 2), (3, 3)),
                                   ((1, 1), (2, 2), (0, 0)), ((3, 3), (2, 2), (1, 1)), ((2, 5), (1, 3), (1, 2)),
                                   ((3, 3), (1, 1), (2, 2)), ((3, 1), (2, 1), (0, 0))])
def test_conv_matches_zero_padded_correlation(k, s, p):
    kw, kh = k
    x = _u8((2, 5, 13, 11))
    w = _i8((4, 5, kh, kw))
    got = orc.conv_forward(x, w, stride=s, pad=(p[0], p[1], p[0], p[1]))
    want = rm.conv_int(x, w, stride=s, pad=p)
    assert got.shape == want.shape
    assert np.array_equal(got.astype(np.int64), want)
    # Frame<double> gives the same integers
    got64 = orc.conv_forward(x.astype(np.float64), w.astype(np.float64), stride=s, pad=(p[0], p[1], p[0], p[1]))
    assert np.array_equal(got64.astype(np.int64), want)


@pytest.mark.parametrize("d", [(2, 2), (3, 1), (1, 2)])
def test_conv_dilation_without_padding(d):
    x = _u8((1, 3, 15, 14))
    w = _i8((2, 3, 3, 3))
    got = orc.conv_forward(x, w, dil=d)
    assert np.array_equal(got.astype(np.int64), rm.conv_int(x, w, dil=d))


def test_conv_unrolled_3x3_window_ignores_dilation():
    """ConvCell_Frame_Kernels.cpp:95-117 unrolls "sxMin == syMin == 0 and sxMax == syMax == 3" by hand, without the
    dilation.  A dilated kernel meets those bounds where W + pad - ox*stride == 3: there the reference sums the first
    3x3 taps over the undilated window; everywhere else the taps whose INDEX is at least pad - o*stride (lines 72-75,
    also undilated) and whose dilated position is below the input's far edge."""
    x = _u8((1, 4, 13, 13))
    w = _i8((3, 4, 3, 3))
    got = orc.conv_forward(x, w, stride=(2, 2), pad=(2, 2, 2, 2), dil=(2, 2)).astype(np.int64)
    xi, wi = x.astype(np.int64), w.astype(np.int64)
    assert got.shape == (1, 3, 7, 7)
    for oy in range(7):
        for ox in range(7):
            iy0, ix0 = 2 * oy - 2, 2 * ox - 2
            want = np.zeros(3, dtype=np.int64)
            if (oy, ox) == (6, 6):          # 13 + 2 - 12 == 3 in both directions
                for ky in range(3):
                    for kx in range(3):
                        want += wi[:, :, ky, kx] @ xi[0, :, iy0 + ky, ix0 + kx]
            else:
                for ky in range(3):
                    for kx in range(3):
                        iy, ix = iy0 + 2 * ky, ix0 + 2 * kx
                        if ky >= max(2 - 2 * oy, 0) and kx >= max(2 - 2 * ox, 0) and iy < 13 and ix < 13:
                            want += wi[:, :, ky, kx] @ xi[0, :, iy, ix]
            assert np.array_equal(got[0, :, oy, ox], want), (oy, ox)


# (kW, kH, subX, subY, strideX, strideY, padX, padY, dilX, dilY): the tuples of
# tests/Cell/class_ConvCell_Frame.cpp:402-438 (channel sizes reduced).
REF_GRID = [
    (3, 3, 1, 1, 1, 1, 0, 0, 1, 1), (2, 5, 1, 1, 1, 1, 0, 0, 1, 1), (3, 3, 1, 1, 2, 2, 0, 0, 1, 1),
    (3, 3, 1, 1, 1, 3, 0, 0, 1, 1), (3, 3, 1, 1, 1, 1, 2, 2, 1, 1), (3, 3, 1, 1, 1, 1, 1, 3, 1, 1),
    (2, 5, 1, 1, 2, 2, 0, 0, 1, 1), (2, 5, 1, 1, 1, 3, 0, 0, 1, 1), (2, 5, 1, 1, 1, 1, 2, 2, 1, 1),
    (2, 5, 1, 1, 1, 1, 1, 3, 1, 1), (3, 3, 1, 1, 1, 3, 2, 2, 1, 1), (3, 3, 1, 1, 1, 3, 1, 3, 1, 1),
    (2, 5, 1, 1, 1, 3, 0, 0, 2, 2), (3, 3, 1, 1, 1, 3, 0, 0, 2, 2), (3, 3, 1, 1, 1, 3, 0, 0, 2, 1),
    (3, 3, 1, 1, 1, 3, 0, 0, 1, 2), (3, 3, 1, 1, 1, 3, 2, 2, 3, 3), (3, 3, 1, 1, 1, 3, 1, 3, 2, 2),
]


@pytest.mark.parametrize("case", REF_GRID)
def test_conv_matches_reference_unit_test_formula(case):
    kw, kh, _, _, sx, sy, px, py, dx, dy = case
    x = _u8((2, 2, 16, 14))
    w = _i8((3, 2, kh, kw))
    got = orc.conv_forward(x, w, stride=(sx, sy), pad=(px, py, px, py), dil=(dx, dy))
    want = rm.conv_reference_test_formula(x, w, (sx, sy), (px, py), (dx, dy))
    assert got.shape == want.shape
    assert np.array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("groups", [2, 8])
def test_conv_groups_and_depthwise(groups):
    C, O = 8, 8 if groups == 8 else 6
    x = _u8((2, C, 9, 9))
    w = _i8((O, C // groups, 3, 3))
    maps = orc.group_maps(C, O, groups)
    assert orc.get_nb_groups(maps) == groups
    got = orc.conv_forward(x, w, pad=(1, 1, 1, 1), maps=maps)
    want = rm.conv_int(x, w, pad=(1, 1), groups=groups)
    assert np.array_equal(got.astype(np.int64), want)


def test_conv_cell_with_several_inputs_is_the_convolution_of_their_concatenated_channels():
    """ConvCell_Frame<T>::propagate (src/Cell/ConvCell_Frame.cpp:438-459) adds one weighted sum per input, each with its
    slice of the weights: against the textbook correlation over all channels, with stride, padding and a bias."""
    from oracle import cells

    class Identity:
        def apply(self, y):
            return y
    xs = [_u8((2, 5, 9, 8)), _u8((2, 3, 9, 8)), _u8((2, 16, 9, 8))]
    w = _i8((7, 24, 3, 3))
    bias = np.arange(-3, 4, dtype=np.int32) * 1000
    got = cells.conv_cell(xs, w, bias, Identity(), stride=(2, 1), pad=(1, 1, 1, 1))
    want = rm.conv_int(np.concatenate(xs, 1), w, stride=(2, 1), pad=(1, 1)) + bias[None, :, None, None]
    assert np.array_equal(got.astype(np.int64), want)


def test_fc_cell_with_several_inputs_adds_the_bias_once_per_input():
    """FcCell_Frame<T>::propagate (src/Cell/FcCell_Frame.cpp:273-336): one inner product per input, each seeded with the
    bias (`:309`), added up: the product over all inputs' values plus as many biases as there are inputs."""
    from oracle import cells

    class Identity:
        def apply(self, y):
            return y
    xs = [_u8((3, 5, 2, 2)), _i8((3, 3, 2, 2)), _u8((3, 1, 2, 2))]
    w = _i8((4, 36))
    bias = np.array([5, -7, 100, 0], dtype=np.int32)
    got = cells.fc_cell(xs, w, bias, Identity()).reshape(3, 4).astype(np.int64)
    flat = np.concatenate([x.reshape(3, -1) for x in xs], 1).astype(np.int64)
    assert np.array_equal(got, flat @ w.astype(np.int64).T + 3 * bias)
    assert np.array_equal(cells.fc_cell(xs[:1], w[:, :20], bias, Identity()).reshape(3, 4).astype(np.int64),
                          flat[:, :20] @ w[:, :20].astype(np.int64).T + bias)


def test_nb_groups_irregular_mapping_is_flagged():
    m = orc.group_maps(4, 4, 2)
    m[3, 0] = 1
    assert orc.get_nb_groups(m) == -1
    assert orc.get_nb_groups(np.ones((4, 6), dtype=np.uint8)) == 1
    assert orc.get_nb_groups(np.zeros((4, 6), dtype=np.uint8)) == 0


def test_hand_made_group_count_is_the_number_of_connected_sets():
    """Cell::getNbGroupsHandMade (src/Cell/Cell.cpp:178-249) counts the sets of outputs tied together by shared channels: known
    small maps, then random ones against scipy's connected components of the bipartite graph (an independent algorithm)."""
    from scipy.sparse import csr_matrix
    from scipy.sparse.csgraph import connected_components
    m = np.zeros((8, 6), dtype=np.uint8)            # [channels, outputs]
    m[0:4, 0:2] = 1
    m[4:8, 2:6] = 1                                  # two unequal blocks: not "regular", two groups by hand
    assert orc.get_nb_groups(m) == -1 and orc.get_nb_groups_hand_made(m) == 2 and orc.nb_groups_of(m) == 2
    m[3, 5] = 1                                      # one shared channel ties them together
    assert orc.get_nb_groups_hand_made(m) == 1
    chain = np.zeros((5, 4), dtype=np.uint8)         # 0-1 share channel 1, 1-2 share channel 2, 3 on its own
    chain[0, 0] = chain[1, 0] = chain[1, 1] = chain[2, 1] = chain[2, 2] = chain[4, 3] = 1
    assert orc.get_nb_groups_hand_made(chain) == 2
    assert orc.get_nb_groups_hand_made(np.zeros((3, 3), dtype=np.uint8)) == 0
    lead = np.zeros((4, 4), dtype=np.uint8)          # outputs without a connection in front of the first connected one are skipped
    lead[0, 2] = lead[1, 3] = 1
    assert orc.get_nb_groups_hand_made(lead) == 2
    hole = lead.copy()
    hole[:, 3] = 0                                   # ... behind it: the reference's loop does not end
    with pytest.raises(ValueError):
        orc.get_nb_groups_hand_made(hole)
    rng = np.random.default_rng(77)
    for _ in range(60):
        nch, nout = rng.integers(2, 12), rng.integers(2, 12)
        m = (rng.random((nch, nout)) < rng.uniform(0.1, 0.5)).astype(np.uint8)
        for o in range(nout):                        # every output connected somewhere
            if not m[:, o].any():
                m[rng.integers(nch), o] = 1
        graph = np.zeros((nch + nout, nch + nout), dtype=np.uint8)
        graph[:nch, nch:] = m
        _, labels = connected_components(csr_matrix(graph), directed=False)
        assert orc.get_nb_groups_hand_made(m) == len(set(labels[nch:])), m


def test_conv_with_an_irregular_connection_map():
    """ConvCell_Frame_Kernels::forward under a map that is not a set of equal groups (src/Cell/ConvCell_Frame_Kernels.cpp:93-97):
    unconnected channels are skipped; with one hand-counted group the weights are indexed by channel, with several by the
    count of connected channels so far.  Against the plain convolution of weights scattered into a full tensor."""
    rng = np.random.default_rng(78)
    x = _u8((2, 8, 7, 9))
    # one group: overlapping connections
    m = (rng.random((8, 6)) < 0.5).astype(np.uint8)
    m[0, :] = 1
    m[1, 0] = 0                                      # (the first output does not see a leading block that divides the channels)
    m[2, 0] = 1
    assert orc.get_nb_groups(m) == -1 and orc.nb_groups_of(m) == 1
    w = _i8((6, 8, 3, 3))
    got = orc.conv_forward(x, w, pad=(1, 1, 1, 1), maps=m)
    want = rm.conv_int(x, w * m.T[:, :, None, None], pad=(1, 1))
    assert np.array_equal(got.astype(np.int64), want)
    # two unequal groups: packed slices
    m = np.zeros((8, 6), dtype=np.uint8)
    m[0:4, 0:2] = 1
    m[4:8, 2:6] = 1
    m[5, 3] = 0                                      # (an output may use fewer slices than there are)
    w = _i8((6, 4, 3, 3))
    full = np.zeros((6, 8, 3, 3), dtype=w.dtype)
    for o in range(6):
        for n, ch in enumerate(np.flatnonzero(m[:, o])):
            full[o, ch] = w[o, n]
    got = orc.conv_forward(x, w, stride=(2, 1), pad=(1, 1, 1, 1), maps=m)
    assert np.array_equal(got.astype(np.int64), rm.conv_int(x, full, stride=(2, 1), pad=(1, 1)))
    with pytest.raises(ValueError):                  # more connections than slices: the reference would read past its weights
        m2 = np.zeros((8, 6), dtype=np.uint8)
        m2[0:5, 0:2] = 1                             # two groups still (8 / 2 = 4 slices), five connections for outputs 0 and 1
        m2[5:8, 2:6] = 1
        assert orc.nb_groups_of(m2) == 2
        orc.conv_forward(x, w, pad=(1, 1, 1, 1), maps=m2)


def test_conv_identity_kernel_copies_input():
    x = _u8((2, 3, 7, 6))
    w = np.zeros((3, 3, 3, 3), dtype=np.float32)
    for c in range(3):
        w[c, c, 1, 1] = 1
    assert np.array_equal(orc.conv_forward(x, w, pad=(1, 1, 1, 1)), x)


def test_conv_1x1_is_gemm_is_fc():
    x = _u8((3, 6, 4, 5))
    w = _i8((7, 6, 1, 1))
    conv = orc.conv_forward(x, w)
    gemm = np.einsum("bchw,oc->bohw", x.astype(np.int64), w[:, :, 0, 0].astype(np.int64))
    assert np.array_equal(conv.astype(np.int64), gemm)
    # an FC over the flattened CHW tensor is a conv whose kernel spans the input
    wf = _i8((5, 6 * 4 * 5))
    bias = RNG.integers(-4096, 4097, size=5).astype(np.float32)
    fc = orc.fc_forward(x, wf, bias)
    conv_full = orc.conv_forward(x, wf.reshape(5, 6, 4, 5))
    orc.conv_forward_bias(conv_full, bias)
    assert np.array_equal(fc, conv_full.reshape(3, 5))
    want = x.reshape(3, -1).astype(np.int64) @ wf.astype(np.int64).T + bias.astype(np.int64)
    assert np.array_equal(fc.astype(np.int64), want)


def test_conv_beta_accumulation_over_split_inputs():
    x = _u8((2, 6, 8, 8))
    w = _i8((4, 6, 3, 3))
    whole = orc.conv_forward(x, w, pad=(1, 1, 1, 1))
    part = orc.conv_forward(x[:, :2], w[:, :2], pad=(1, 1, 1, 1))
    part = orc.conv_forward(np.ascontiguousarray(x[:, 2:]), np.ascontiguousarray(w[:, 2:]),
                            pad=(1, 1, 1, 1), out=part, beta=1.0)
    assert np.array_equal(whole, part)


def test_conv_float_accumulator_guard():
    """Sums of magnitude >= 2^24 are outside the bit-exact contract: float32 and
    float64 oracles disagree there, and agree below it."""
    x = np.full((1, 600, 3, 3), 255, dtype=np.float32)
    w = np.full((1, 600, 3, 3), 127, dtype=np.float32)
    w[0, ::7] = 126
    big32 = orc.conv_forward(x, w)
    big64 = orc.conv_forward(x.astype(np.float64), w.astype(np.float64))
    assert abs(big64[0, 0, 0, 0]) > 2 ** 24
    assert big32[0, 0, 0, 0] != big64[0, 0, 0, 0]
    small32 = orc.conv_forward(x[:, :50], w[:, :50])
    small64 = orc.conv_forward(x[:, :50].astype(np.float64), w[:, :50].astype(np.float64))
    assert np.array_equal(small32.astype(np.float64), small64)


def test_conv_output_dims_follow_reference_formulas():
    assert orc.conv_out_dim(224, 7, 2, 3) == 112
    assert orc.conv_out_dim(56, 3, 1, 1) == 56
    assert orc.conv_out_dim(56, 1, 2, 0) == 28
    assert orc.pool_out_dim(112, 3, 2, 0) == 55     # N2D2's own ResNet-50: unpadded pool
    assert orc.pool_out_dim(112, 3, 2, 1) == 56
    assert orc.pool_out_dim(7, 7, 7, 0) == 1


# ------------------------------------------------------------------- pool

@pytest.mark.parametrize("pool,stride,pad", [((2, 2), (2, 2), (0, 0)), ((3, 3), (2, 2), (0, 0)),
                                             ((3, 3), (2, 2), (1, 1)), ((7, 7), (7, 7), (0, 0)), ((3, 2), (1, 2), (1, 0))])
def test_pool_max_and_average(pool, stride, pad):
    x = RNG.integers(-128, 256, size=(2, 3, 15, 14)).astype(np.float32)
    B, C, H, W = x.shape
    mx = orc.pool_forward(x, pool, stride, pad, kind="max")
    av = orc.pool_forward(x, pool, stride, pad, kind="avg", quantized=True)
    oH, oW = mx.shape[2:]
    xi = x.astype(np.int64)
    for oy, ox in itertools.product(range(oH), range(oW)):
        y0, x0 = oy * stride[1] - pad[1], ox * stride[0] - pad[0]
        win = xi[:, :, max(y0, 0):min(y0 + pool[1], H), max(x0, 0):min(x0 + pool[0], W)]
        assert np.array_equal(mx[:, :, oy, ox].astype(np.int64), win.max(axis=(2, 3)))
        s = win.sum(axis=(2, 3))
        n = pool[0] * pool[1]          # count includes padding
        want = np.sign(s) * (np.abs(s) // n)    # integer division toward zero
        assert np.array_equal(av[:, :, oy, ox].astype(np.int64), want)


def test_pool_with_a_connection_map_pools_over_the_connected_channels():
    """PoolCell_Frame_Kernels.cpp:60-75,150-185 with a map: the maximum over window and connected channels; the sum over
    both divided by window size x connected channels, truncated; 0 for an output nothing feeds."""
    from oracle import cells
    x = RNG.integers(-128, 256, size=(2, 6, 9, 8)).astype(np.float32)
    xi = x.astype(np.int64)
    maps = np.array([[1, 0, 1, 0], [1, 0, 0, 0], [1, 1, 0, 0], [1, 1, 0, 0], [1, 0, 0, 0], [1, 0, 1, 0]], dtype=np.uint8)   # [channel, output]
    pool, stride, pad = (3, 3), (2, 2), (1, 1)
    mx = cells.pool_cell(x, "max", pool, stride, pad, maps=maps)
    av = cells.pool_cell(x, "avg", pool, stride, pad, maps=maps)
    assert mx.shape == av.shape == (2, 4, 5, 4)
    for oy, ox, o in itertools.product(range(5), range(4), range(4)):
        y0, x0 = oy * 2 - 1, ox * 2 - 1
        chans = np.flatnonzero(maps[:, o])
        if len(chans) == 0:
            assert not mx[:, o, oy, ox].any() and not av[:, o, oy, ox].any()
            continue
        win = xi[:, chans, max(y0, 0):min(y0 + 3, 9), max(x0, 0):min(x0 + 3, 8)]
        assert np.array_equal(mx[:, o, oy, ox].astype(np.int64), win.max(axis=(1, 2, 3)))
        s = win.sum(axis=(1, 2, 3))
        assert np.array_equal(av[:, o, oy, ox].astype(np.int64), np.sign(s) * (np.abs(s) // (9 * len(chans))))


def test_pool_cell_with_several_inputs_pools_every_input_on_its_own_channels():
    """PoolCell_Frame<T>::propagate (src/Cell/PoolCell_Frame.cpp:123-174) over several inputs, unit map over all their
    channels: window maxima / truncated window means of each input, written behind each other."""
    from oracle import cells
    xs = [RNG.integers(-128, 256, size=(2, 3, 9, 8)).astype(np.float32), RNG.integers(-128, 256, size=(2, 5, 9, 8)).astype(np.float32)]
    xi = np.concatenate(xs, 1).astype(np.int64)
    pool, stride, pad = (3, 3), (2, 2), (1, 1)
    mx = cells.pool_cell(xs, "max", pool, stride, pad)
    av = cells.pool_cell(xs, "avg", pool, stride, pad)
    assert mx.shape == av.shape == (2, 8, 5, 4)
    for oy, ox in itertools.product(range(5), range(4)):
        y0, x0 = oy * 2 - 1, ox * 2 - 1
        win = xi[:, :, max(y0, 0):min(y0 + 3, 9), max(x0, 0):min(x0 + 3, 8)]
        assert np.array_equal(mx[:, :, oy, ox].astype(np.int64), win.max(axis=(2, 3)))
        s = win.sum(axis=(2, 3))
        assert np.array_equal(av[:, :, oy, ox].astype(np.int64), np.sign(s) * (np.abs(s) // 9))


def test_pool_average_exhaustive_rounding_toward_zero():
    # every u8 / i8 window sum a 2x2, 3x3 or 7x7 pool can produce
    for n in (4, 9, 49):
        sums = np.arange(-128 * n, 255 * n + 1, dtype=np.int64)
        # build windows whose sum is the wanted value: first cell carries it
        x = np.zeros((sums.size, 1, 1, n), dtype=np.float32)
        x[:, 0, 0, 0] = sums
        got = orc.pool_forward(x, (n, 1), (n, 1), kind="avg", quantized=True)[:, 0, 0, 0]
        want = np.sign(sums) * (np.abs(sums) // n)
        assert np.array_equal(got.astype(np.int64), want)


def test_pool_max_first_element_and_argmax():
    x = np.full((1, 1, 2, 2), -5, dtype=np.float32)
    out, am = orc.pool_forward(x, (2, 2), (2, 2), kind="max", argmax=True)
    assert out[0, 0, 0, 0] == -5           # first element is always taken
    assert am[0, 0, 0, 0].tolist() == [0, 0, 0, 1]


# --------------------------------------------------------------- elemwise

def test_elemwise_sum_closed_form():
    # tests/Cell/class_ElemWiseCell_Frame.cpp:198-202: wA*a + wB*b + wC*c
    a, b, c = _u8((2, 3, 4, 5)), _i8((2, 3, 4, 5)), _u8((2, 3, 4, 5))
    assert np.array_equal(orc.elemwise_sum([a, b]), a + b)
    w = np.array([2.0, -3.0, 5.0], dtype=np.float32)
    s = np.array([1.0, 0.0, -7.0], dtype=np.float32)
    got = orc.elemwise_sum([a, b, c], w, s, "PerInput")
    assert np.array_equal(got, (w[0] * a + s[0]) + (w[1] * b + s[1]) + (w[2] * c + s[2]))
    # PerLayer: input 0 uses index 0, input k uses index k (the reference resizes both vectors to nbInputs)
    got = orc.elemwise_sum([a, b], np.array([3.0, 3.0]), np.array([2.0, 2.0]), "PerLayer")
    assert np.array_equal(got, 3 * a + 2 + 3 * b + 2)
    wc = np.array([1.0, 2.0, 4.0], dtype=np.float32)
    sc = np.array([0.0, 1.0, -1.0], dtype=np.float32)
    got = orc.elemwise_sum([a, b], wc, sc, "PerChannel")
    want = wc[None, :, None, None] * a + sc[None, :, None, None] + wc[None, :, None, None] * b + sc[None, :, None, None]
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- scaling

ACC = np.concatenate([np.arange(-70000, 70001, 7), np.arange(-600, 601),
                      np.array([2 ** 23, -2 ** 23, 2 ** 24 - 1, -(2 ** 24 - 1)])]).astype(np.int64)


@pytest.mark.parametrize("nb_bits,unsigned", [(8, True), (8, False), (4, True), (4, False)])
def test_fixed_point_exact(nb_bits, unsigned):
    for mult, p in [(2 ** 14, 20), (2 ** 15 - 1, 20), (23170, 16), (1, 0), (3, 1), (65535, 24), (-20000, 18), (2 ** 31 - 1, 31)]:
        x = ACC.astype(np.float64).reshape(1, 1, 1, -1)
        got = orc.scaling_fixed(x, [mult], p, nb_bits, unsigned)[0, 0, 0]
        want = np.array([rm.fixed_point(v, mult, p, nb_bits, unsigned) for v in ACC])
        assert np.array_equal(got.astype(np.int64), want)
        x32 = ACC.astype(np.float32).reshape(1, 1, 1, -1)
        got32 = orc.scaling_fixed(x32, [mult], p, nb_bits, unsigned)[0, 0, 0]
        assert np.array_equal(got32.astype(np.int64), want)


@pytest.mark.parametrize("nb_bits,unsigned", [(8, True), (8, False), (4, True)])
def test_single_and_double_shift_exact_all_shifts(nb_bits, unsigned):
    small = np.arange(-3000, 3001, dtype=np.int64)
    for s in range(0, 32):
        vals = small if s < 8 else small * (1 << (s - 7)) + 3
        vals = vals[np.abs(vals) < 2 ** 24]
        x = vals.astype(np.float32).reshape(1, 1, 1, -1)
        got = orc.scaling_single_shift(x, [s], nb_bits, unsigned)[0, 0, 0]
        want = np.array([rm.single_shift(v, s, nb_bits, unsigned) for v in vals])
        assert np.array_equal(got.astype(np.int64), want), s
    for a, b in [(0, 0), (1, 3), (2, 9), (3, 10), (5, 12), (7, 16), (4, 0), (8, 20)]:
        x = ACC.astype(np.float32).reshape(1, 1, 1, -1)
        got = orc.scaling_double_shift(x, [[a, b]], nb_bits, unsigned)[0, 0, 0]
        want = np.array([rm.double_shift(v, a, b, nb_bits, unsigned) for v in ACC])
        assert np.array_equal(got.astype(np.int64), want), (a, b)


def test_shift_rounding_is_floor_of_value_plus_half():
    # negative inputs: arithmetic shift floors, so -2.5 -> -2 and -3.5 -> -3
    x = np.array([-5, -7, 5, 7, -1, 1, 0], dtype=np.float32).reshape(1, 1, 1, -1)
    got = orc.scaling_single_shift(x, [1], 8, False)[0, 0, 0]
    assert got.tolist() == [-2, -3, 3, 4, 0, 1, 0]


def test_scaling_is_per_channel_in_nchw_order():
    x = np.full((2, 3, 2, 2), 1000, dtype=np.float32)
    got = orc.scaling_single_shift(x, [2, 3, 4], 8, True)
    assert got[:, 0].tolist() == [[[250, 250], [250, 250]]] * 2
    assert (got[:, 1] == 125).all() and (got[:, 2] == 63).all()


def test_fixed_point_clip_both_branches_and_rounding_of_clip():
    x = np.array([-9, -3, 0, 4, 6, 7, 100], dtype=np.float32).reshape(1, 1, 1, -1)
    # positive clip 5.5: values above it become 5.5 and are then rounded half away -> 6
    got = orc.scaling_fixed(x, [1], 0, 8, False, clip=[5.5])[0, 0, 0]
    assert got.tolist() == [0, 0, 0, 4, 6, 6, 6]
    got = orc.scaling_fixed(x, [1], 0, 8, False, clip=[5.4])[0, 0, 0]
    assert got.tolist() == [0, 0, 0, 4, 5, 5, 5]
    # negative clip: clamp to [clip, 0]
    got = orc.scaling_fixed(x, [1], 0, 8, False, clip=[-4.0])[0, 0, 0]
    assert got.tolist() == [-4, -3, 0, 0, 0, 0, 0]


def test_fixed_point_requires_quantized_cell():
    x = np.zeros((1, 1, 1, 1), dtype=np.float32)
    for f in (lambda: orc.scaling_fixed(x, [1], 0, 0, True),
              lambda: orc.scaling_single_shift(x, [1], 0, True),
              lambda: orc.scaling_double_shift(x, [[1, 1]], 0, True)):
        with pytest.raises(RuntimeError):
            f()


@pytest.mark.parametrize("nb_bits,unsigned", [(8, True), (8, False), (4, True)])
def test_floating_point_scaling_is_float32_product_rounded_half_away(nb_bits, unsigned):
    acc = np.arange(-2 ** 15, 2 ** 15 + 1, dtype=np.int64)
    scales = RNG.uniform(1e-4, 0.05, size=6).astype(np.float32)
    scales[0] = np.float32(0.5)        # exact ties
    scales[1] = np.float32(0.25)
    x = np.broadcast_to(acc.astype(np.float32), (1, 6, 1, acc.size)).copy()
    got = orc.scaling_float(x, scales, nb_bits, unsigned)
    lo, hi = (0, 2 ** nb_bits - 1) if unsigned else (-2 ** (nb_bits - 1), 2 ** (nb_bits - 1) - 1)
    for c in range(6):
        prod = (acc.astype(np.float32) * scales[c]).astype(np.float32)   # one IEEE float32 multiply
        want = np.clip(rm.round_half_away(prod), lo, hi)
        assert np.array_equal(got[0, c, 0].astype(np.float64), want)
    # not quantized: plain product, no rounding, no saturation
    raw = orc.scaling_float(x, scales, 0, unsigned)
    assert np.array_equal(raw[0, 2, 0], acc.astype(np.float32) * scales[2])
    # clip happens before the multiply
    cl = orc.scaling_float(x, scales, nb_bits, unsigned, clip=np.full(6, 1000.0, dtype=np.float32))
    prod = (np.clip(acc, 0, 1000).astype(np.float32) * scales[3]).astype(np.float32)
    assert np.array_equal(cl[0, 3, 0].astype(np.float64), np.clip(rm.round_half_away(prod), lo, hi))


def test_activations_after_scaling():
    x = np.array([-4, -1, 0, 3, 300], dtype=np.float32)
    assert orc.rectifier(x).tolist() == [0, 0, 0, 3, 300]
    # Clipping only applies to a cell that is not quantized
    assert orc.rectifier(x, clipping=6.0, cell_quantized=True).tolist() == [0, 0, 0, 3, 300]
    assert orc.rectifier(x, clipping=6.0, cell_quantized=False).tolist() == [0, 0, 0, 3, 6]
    assert orc.rectifier(x, leak=0.5).tolist() == [-2, -0.5, 0, 3, 300]
    assert orc.linear(x, clipping=2.0, cell_quantized=True).tolist() == x.tolist()
    assert orc.linear(x, clipping=2.0, cell_quantized=False).tolist() == [-2, -1, 0, 2, 2]


def test_conv_sub_sampling_adds_up_neighbouring_positions():
    """ConvCell_Frame_Kernels::forward with subSample > 1 (src/Cell/ConvCell_Frame_Kernels.cpp:46-52,135-140): output
    (ox / subX, oy / subY) collects the sums of its positions, the last window of a row or column holding what is left; against
    block sums of the plain convolution, on sizes that do and do not divide."""
    for (H, W, sub, stride, pad) in ((9, 12, (2, 2), (1, 1), 1), (10, 7, (3, 2), (1, 1), 0), (13, 13, (2, 3), (2, 1), 1), (8, 8, (1, 2), (1, 1), 1)):
        x = _u8((2, 3, H, W))
        w = _i8((4, 3, 3, 3))
        plain = orc.conv_forward(x, w, stride=stride, pad=(pad,) * 4).astype(np.int64)
        got = orc.conv_forward(x, w, stride=stride, pad=(pad,) * 4, sub=sub).astype(np.int64)
        oH, oW = plain.shape[2:]
        want = np.zeros((2, 4, -(-oH // sub[1]), -(-oW // sub[0])), dtype=np.int64)
        for oy in range(oH):
            for ox in range(oW):
                want[:, :, oy // sub[1], ox // sub[0]] += plain[:, :, oy, ox]
        assert got.shape == want.shape and np.array_equal(got, want), (H, W, sub)
        assert want.shape[2] == orc._lib.oracle_conv_out_dim(H, 3, stride[1], pad, 1, sub[1])
