"""Independent mathematical definitions used to pin the CPU oracle.

Nothing here shares code or loop structure with ``oracle/``: convolutions are
evaluated as zero-padded integer cross-correlations with numpy int64, the
integer rescales as exact rational floor divisions on Python integers.
"""
import numpy as np


def conv_int(x, w, stride=(1, 1), pad=(0, 0), dil=(1, 1), groups=1):
    """Textbook zero-padded cross-correlation, int64. x [B,C,H,W], w [O,C/g,kH,kW];
    stride/pad/dil are (x, y)."""
    x = np.asarray(x, dtype=np.int64)
    w = np.asarray(w, dtype=np.int64)
    B, C, H, W = x.shape
    O, Cg, kH, kW = w.shape
    sx, sy = stride
    px, py = pad
    dx, dy = dil
    xp = np.zeros((B, C, H + 2 * py, W + 2 * px), dtype=np.int64)
    xp[:, :, py:py + H, px:px + W] = x
    oH = (H + 2 * py - dy * (kH - 1) - 1) // sy + 1
    oW = (W + 2 * px - dx * (kW - 1) - 1) // sx + 1
    out = np.zeros((B, O, oH, oW), dtype=np.int64)
    og = O // groups
    for g in range(groups):
        xs = xp[:, g * Cg:(g + 1) * Cg]
        ws = w[g * og:(g + 1) * og]
        for ky in range(kH):
            for kx in range(kW):
                patch = xs[:, :, ky * dy: ky * dy + sy * (oH - 1) + 1: sy,
                           kx * dx: kx * dx + sx * (oW - 1) + 1: sx]
                out[:, g * og:(g + 1) * og] += np.einsum("bchw,oc->bohw", patch, ws[:, :, ky, kx])
    return out


def conv_reference_test_formula(x, w, stride, pad, dil):
    """The brute-force loop the reference's own unit test compares against
    (tests/Cell/class_ConvCell_Frame.cpp:495-535): window limits sxMin/sxMax are
    computed exactly as there, including for dilation > 1. Pure Python: tiny
    shapes only."""
    B, C, H, W = x.shape
    O, _, kH, kW = w.shape
    sx_, sy_ = stride
    px, py = pad
    dx, dy = dil
    oW = int((W + 2 * px - dx * (kW - 1) - 1 + sx_) / float(sx_))
    oH = int((H + 2 * py - dy * (kH - 1) - 1 + sy_) / float(sy_))
    out = np.zeros((B, O, oH, oW), dtype=np.int64)
    for b in range(B):
        for o in range(O):
            for oy in range(oH):
                for ox in range(oW):
                    sxMin = max(px - ox * sx_, 0)
                    syMin = max(py - oy * sy_, 0)
                    sxMax = min(max(W + px - ox * sx_, 0), kW + (dx - 1) * (kW - 1))
                    syMax = min(max(H + py - oy * sy_, 0), kH + (dy - 1) * (kH - 1))
                    s = 0
                    for c in range(C):
                        sy = syMin
                        while sy * dy < syMax:
                            sx = sxMin
                            while sx * dx < sxMax:
                                ix = ox * sx_ + sx * dx - px
                                iy = oy * sy_ + sy * dy - py
                                s += int(x[b, c, iy, ix]) * int(w[o, c, sy, sx])
                                sx += 1
                            sy += 1
                    out[b, o, oy, ox] = s
    return out


def saturate(v, nb_bits, unsigned):
    lo, hi = (0, (1 << nb_bits) - 1) if unsigned else (-(1 << (nb_bits - 1)), (1 << (nb_bits - 1)) - 1)
    return min(max(v, lo), hi)


def floor_div_pow2(n, p):
    """floor(n / 2**p) on Python integers (what an arithmetic right shift does)."""
    return n // (1 << p)


def fixed_point(v, mult, p, nb_bits, unsigned):
    """include/Scaling.hpp:122-128: (data*scale + HALF) >> frac, HALF = 2^(frac-1)."""
    half = (1 << (p - 1)) if p > 0 else 0
    return saturate(floor_div_pow2(int(v) * int(mult) + half, p), nb_bits, unsigned)


def single_shift(v, s, nb_bits, unsigned):
    """include/Scaling.hpp:196-202."""
    half = (1 << (s - 1)) if s > 0 else 0
    return saturate(floor_div_pow2(int(v) + half, s), nb_bits, unsigned)


def double_shift(v, a, b, nb_bits, unsigned):
    """include/Scaling.hpp:264-270."""
    half = (1 << (b - 1)) if b > 0 else 0
    v = int(v)
    return saturate(floor_div_pow2(v + v * (1 << a) + half, b), nb_bits, unsigned)


def round_half_away(x):
    """std::round on an exactly known real (numpy float64 input)."""
    x = np.asarray(x, dtype=np.float64)
    return np.sign(x) * np.floor(np.abs(x) + 0.5)


def read_syntxt(path):
    with open(path) as f:
        return np.array(f.read().split(), dtype=np.float64)
