"""ctypes front-end of the CPU oracle (TEST INFRASTRUCTURE, not the product).

Only tests, the smoke check and the benchmark's CPU-baseline leg import this
module.  Arrays are numpy, NCHW / OCHW as in N2D2 (Tensor dims {X,Y,Z,B} with
X fastest, include/containers/Tensor.hpp:162-193); integer-valued data is held
in float32 (or float64) exactly as the reference Frame cells hold it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libframe_oracle.so")


def build(force=False):
    """Compile the C restatement with gcc (make -C oracle)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()

_SFX = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64"}
_CT = {np.dtype(np.float32): C.c_float, np.dtype(np.float64): C.c_double}


def _fn(name, dtype):
    return getattr(_lib, "oracle_%s_%s" % (name, _SFX[np.dtype(dtype)]))


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _ia(vals):
    return (C.c_int * len(vals))(*[int(v) for v in vals])


def conv_out_dim(n, k, stride, pad, dil=1, sub=1):
    _lib.oracle_conv_out_dim.restype = C.c_uint
    return int(_lib.oracle_conv_out_dim(C.c_uint(n), C.c_uint(k), C.c_uint(stride),
                                        C.c_uint(pad), C.c_uint(dil), C.c_uint(sub)))


def pool_out_dim(n, pool, stride, pad):
    _lib.oracle_pool_out_dim.restype = C.c_uint
    return int(_lib.oracle_pool_out_dim(C.c_uint(n), C.c_uint(pool), C.c_uint(stride), C.c_uint(pad)))


def get_nb_groups(maps):
    """maps: bool array [C, O] (Tensor<bool> {O,C}: maps(o,c) = maps[c, o])."""
    m = np.ascontiguousarray(maps, dtype=np.uint8)
    nch, nout = m.shape
    _lib.oracle_get_nb_groups.restype = C.c_long
    return int(_lib.oracle_get_nb_groups(_p(m), C.c_size_t(nout), C.c_size_t(nch)))


def get_nb_groups_hand_made(maps):
    """Cell::getNbGroupsHandMade (src/Cell/Cell.cpp:178-249), walked the way the reference walks it: from the first output
    that has a connection, take an unclassified output, collect every output reachable from it through shared channels
    (`:213-236`), count one group, go on with the next unclassified output.  maps: bool [C, O].  0 for a map without any
    connection (`:196-199`).  An output without connections behind the first connected one makes the reference's loop spin
    (`:212-215`: `continue` without advancing): ValueError here."""
    m = np.asarray(maps) != 0
    nch, nout = m.shape
    first = next((o for o in range(nout) if m[:, o].any()), None)
    if first is None:
        return 0
    classified = set()
    groups = 0
    current = first
    while current < nout:
        if not m[:, current].any():
            raise ValueError("output %d has no connection: the reference does not return on such a map" % current)
        pending = [current]
        while pending:
            line = pending.pop()
            classified.add(line)
            for ch in np.flatnonzero(m[:, line]):
                for o in range(first, nout):
                    if m[ch, o] and o not in classified and o not in pending:
                        pending.append(o)
        groups += 1
        current += 1
        while current in classified:
            current += 1
    return groups


def nb_groups_of(maps):
    """Cell::getNbGroups (src/Cell/Cell.cpp:251-300) with its fall-back: the regular count, else the hand-made one."""
    g = get_nb_groups(maps)
    return g if g >= 0 else get_nb_groups_hand_made(maps)


def group_maps(C_in, O, groups):
    """Boolean mapping [C, O] of a regular grouped connection."""
    m = np.zeros((C_in, O), dtype=np.uint8)
    cg, og = C_in // groups, O // groups
    for g in range(groups):
        m[g * cg:(g + 1) * cg, g * og:(g + 1) * og] = 1
    return m


def conv_forward(x, w, stride=(1, 1), pad=(0, 0, 0, 0), dil=(1, 1), maps=None,
                 out=None, alpha=1.0, beta=0.0, sub=(1, 1)):
    """ConvCell_Frame_Kernels::forward. x [B,C,H,W], w [O,Cw,kH,kW]; stride/dil
    are (x,y); pad is (left, top, right, bottom)."""
    dt = x.dtype
    x = np.ascontiguousarray(x)
    w = np.ascontiguousarray(w, dtype=dt)
    B, Cin, H, W = x.shape
    O, Cw, kH, kW = w.shape
    oW = int((W + pad[0] + pad[2] - dil[0] * (kW - 1) - 1 + stride[0]) / float(stride[0]))
    oH = int((H + pad[1] + pad[3] - dil[1] * (kH - 1) - 1 + stride[1]) / float(stride[1]))
    # sub-sampling: ceil(positions / subSample) outputs (src/Cell/ConvCell.cpp:1169-1195), each the sum of its positions
    oW, oH = -(-oW // sub[0]), -(-oH // sub[1])
    if out is None:
        out = np.zeros((B, O, oH, oW), dtype=dt)
    groups = 1
    m = None
    if maps is not None:
        m = np.ascontiguousarray(maps, dtype=np.uint8)
        groups = nb_groups_of(m)
        # the weights have C / G slices with several groups, C otherwise (src/Cell/ConvCell_Frame.cpp:172-177); output o reads
        # slice n for its n-th connected channel with several groups (src/Cell/ConvCell_Frame_Kernels.cpp:97).  The reference
        # does not check that this stays inside the tensor; the restatement refuses to read past it.
        if Cw != (Cin // groups if groups > 1 else Cin):
            raise ValueError("weights have %d slices, the map's %d group(s) ask for %d" % (Cw, groups, Cin // groups if groups > 1 else Cin))
        if groups > 1 and int(m.sum(axis=0).max()) > Cw:
            raise ValueError("an output is connected to more channels than the weights have slices")
    ct = _CT[np.dtype(dt)]
    a, b = ct(alpha), ct(beta)
    _fn("conv_forward", dt)(C.byref(a), _p(x), B, Cin, H, W, _p(w), kW, kH, Cw, O,
                            _ia(stride), _ia(pad), _ia(dil), _ia(sub), C.byref(b), _p(out),
                            oW, oH, _p(m), groups)
    return out


def conv_forward_bias(out, bias, alpha=1.0, beta=1.0):
    dt = out.dtype
    B, O, oH, oW = out.shape
    bias = np.ascontiguousarray(bias, dtype=dt)
    ct = _CT[np.dtype(dt)]
    a, b = ct(alpha), ct(beta)
    _fn("conv_forward_bias", dt)(C.byref(a), _p(bias), C.byref(b), _p(out), oW, oH, O, B)
    return out


def _maps_groups(maps):
    if maps is None:
        return None, 1
    m = np.ascontiguousarray(maps, dtype=np.uint8)
    groups = get_nb_groups(m)
    if groups < 0:
        raise ValueError("irregular mapping")
    return m, groups


def conv_backward_data(w, dy, x_shape, stride=(1, 1), pad=(0, 0, 0, 0), maps=None, dx=None, alpha=1.0, beta=0.0,
                       sub=(1, 1)):
    """ConvCell_Frame_Kernels::backwardData. w [O,Cw,kH,kW], dy [B,O,oH,oW]; returns dx of x_shape [B,C,H,W]."""
    dt = dy.dtype
    w = np.ascontiguousarray(w, dtype=dt)
    dy = np.ascontiguousarray(dy)
    B, Cin, H, W = x_shape
    O, Cw, kH, kW = w.shape
    assert dy.shape[:2] == (B, O)
    if dx is None:
        dx = np.zeros(x_shape, dtype=dt)
    m, groups = _maps_groups(maps)
    ct = _CT[np.dtype(dt)]
    a, b = ct(alpha), ct(beta)
    _fn("conv_backward_data", dt)(C.byref(a), _p(w), kW, kH, Cw, O, _p(dy), dy.shape[3], dy.shape[2], B,
                                  _ia(stride), _ia(pad), _ia(sub), C.byref(b), _p(dx), Cin, H, W, _p(m), groups)
    return dx


def conv_backward_filter(x, dy, w_shape, stride=(1, 1), pad=(0, 0, 0, 0), maps=None, dw=None, alpha=1.0, beta=0.0,
                         sub=(1, 1)):
    """ConvCell_Frame_Kernels::backwardFilter. x [B,C,H,W], dy [B,O,oH,oW]; returns dw of w_shape [O,Cw,kH,kW]."""
    dt = x.dtype
    x = np.ascontiguousarray(x)
    dy = np.ascontiguousarray(dy, dtype=dt)
    B, Cin, H, W = x.shape
    O, Cw, kH, kW = w_shape
    assert dy.shape[:2] == (B, O)
    if dw is None:
        dw = np.zeros(w_shape, dtype=dt)
    m, groups = _maps_groups(maps)
    ct = _CT[np.dtype(dt)]
    a, b = ct(alpha), ct(beta)
    _fn("conv_backward_filter", dt)(C.byref(a), _p(x), B, Cin, H, W, _p(dy), dy.shape[3], dy.shape[2], O,
                                    _ia(stride), _ia(pad), _ia(sub), C.byref(b), _p(dw), kW, kH, Cw, _p(m), groups)
    return dw


def conv_backward_bias(dy, db=None, alpha=1.0, beta=0.0):
    """ConvCell_Frame_Kernels::backwardBias. dy [B,O,oH,oW]; returns db [O]."""
    dt = dy.dtype
    dy = np.ascontiguousarray(dy)
    B, O, oH, oW = dy.shape
    if db is None:
        db = np.zeros(O, dtype=dt)
    ct = _CT[np.dtype(dt)]
    a, b = ct(alpha), ct(beta)
    _fn("conv_backward_bias", dt)(C.byref(a), _p(dy), oW, oH, O, B, C.byref(b), _p(db))
    return db


def softmax_forward(x):
    """SoftmaxCell_Frame::propagate over the channels of x [B,C,H,W]."""
    x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    B, Cn, H, W = x.shape
    _fn("softmax_forward", x.dtype)(_p(x), _p(out), B, Cn, H, W)
    return out


def fc_forward(x, w, bias=None, out=None, beta=0.0):
    """FcCell_Frame::propagate inner loop. x [B, ...] (CHW flattened), w [O,K]."""
    dt = x.dtype
    B = x.shape[0]
    x = np.ascontiguousarray(x).reshape(B, -1)
    K = x.shape[1]
    w = np.ascontiguousarray(w, dtype=dt).reshape(-1, K)
    O = w.shape[0]
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=dt)
    if out is None:
        out = np.zeros((B, O), dtype=dt)
    ct = _CT[np.dtype(dt)]
    _fn("fc_forward", dt)(_p(x), B, K, _p(w), _p(bias), O, ct(beta), _p(out))
    return out


def pool_forward(x, pool, stride, pad=(0, 0), kind="max", quantized=True, maps=None,
                 count_include_padding=True, argmax=False, out=None, beta=0.0):
    """PoolCell_Frame_Kernels::forwardMax / forwardAverage with a unit map by
    default (one output per channel, as PoolCell builds it).  out / beta: the
    kernel's accumulation into an existing output (cells with several inputs)."""
    dt = x.dtype
    x = np.ascontiguousarray(x)
    B, Cin, H, W = x.shape
    oW = pool_out_dim(W, pool[0], stride[0], pad[0])
    oH = pool_out_dim(H, pool[1], stride[1], pad[1])
    if maps is None:
        maps = np.eye(Cin, dtype=np.uint8)
    m = np.ascontiguousarray(maps, dtype=np.uint8)
    O = m.shape[1]
    if out is None:
        out = np.zeros((B, O, oH, oW), dtype=dt)
    assert out.shape == (B, O, oH, oW) and out.dtype == dt and out.flags["C_CONTIGUOUS"]
    ct = _CT[np.dtype(dt)]
    a, b = ct(1.0), ct(beta)
    if kind == "max":
        am = np.zeros((B, O, oH, oW, 4), dtype=np.int32) if argmax else None
        _fn("pool_forward_max", dt)(C.byref(a), _p(x), B, Cin, H, W, _ia(pool), _ia(stride), _ia(pad),
                                    C.byref(b), _p(out), oW, oH, O, _p(am), _p(m))
        return (out, am) if argmax else out
    _fn("pool_forward_average", dt)(C.byref(a), _p(x), B, Cin, H, W, _ia(pool), _ia(stride), _ia(pad),
                                    C.byref(b), _p(out), oW, oH, O, int(bool(quantized)),
                                    int(bool(count_include_padding)), _p(m))
    return out


def pool_backward_average(dy, x_shape, pool, stride, pad=(0, 0), beta=0.0, prev=None, count_include_padding=True):
    """PoolCell_Frame_Kernels::backwardAverage, float32, unit mapping; raises where the reference throws."""
    dy = np.ascontiguousarray(dy, dtype=np.float32)
    B, Cn, H, W = x_shape
    oH, oW = dy.shape[2:]
    dx = np.zeros(x_shape, dtype=np.float32) if prev is None else np.array(prev, dtype=np.float32, order="C")
    a, b = C.c_float(1.0), C.c_float(beta)
    fn = _lib.oracle_pool_backward_average_f32
    fn.restype = C.c_int
    if fn(C.byref(a), _p(dy), B, Cn, H, W, _ia(pool), _ia(stride), _ia(pad), C.byref(b), _p(dx), oW, oH,
          int(bool(count_include_padding))) != 0:
        raise RuntimeError("PoolCell_Frame_Kernels::backwardAverage() exclude padding not implemented")
    return dx


def elemwise_sum_backward(dy, weights, k, coeff_mode="PerLayer", beta=0.0, prev=None):
    """ElemWiseCell_Frame::backPropagate, Sum: the gradient towards input k."""
    dy = np.ascontiguousarray(dy, dtype=np.float32)
    B, Cc, H, W = dy.shape
    w = np.ascontiguousarray(weights, dtype=np.float32)
    dx = np.zeros(dy.shape, dtype=np.float32) if prev is None else np.array(prev, dtype=np.float32, order="C")
    fn = _lib.oracle_elemwise_sum_backward_f32
    fn.restype = None
    fn(_p(dy), B, Cc, H, W, _p(w), {"PerLayer": 0, "PerInput": 1, "PerChannel": 2}[coeff_mode], int(k), C.c_float(beta), _p(dx))
    return dx


def elemwise_sum(inputs, weights=None, shifts=None, coeff_mode="PerLayer"):
    """ElemWiseCell_Frame::propagate, Sum. inputs: list of float32 NCHW arrays."""
    xs = [np.ascontiguousarray(x, dtype=np.float32) for x in inputs]
    B, Cc, H, W = xs[0].shape
    mode = {"PerLayer": 0, "PerInput": 1, "PerChannel": 2}[coeff_mode]
    n = len(xs)
    if weights is None:
        weights = np.ones(max(n, Cc), dtype=np.float32)
    if shifts is None:
        shifts = np.zeros(max(n, Cc), dtype=np.float32)
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    shifts = np.ascontiguousarray(shifts, dtype=np.float32)
    ptrs = (C.c_void_p * n)(*[x.ctypes.data for x in xs])
    out = np.zeros_like(xs[0])
    _lib.oracle_elemwise_sum_f32(ptrs, n, B, Cc, H, W, _p(weights), _p(shifts), mode, _p(out))
    return out


# ------------------------------------------------------------------ scaling

def _bchw(x):
    if x.ndim == 2:
        return x.shape[0], x.shape[1], 1, 1
    return x.shape


def scaling_float(x, scale, nb_bits, unsigned, clip=None):
    x = np.ascontiguousarray(x)
    B, Cc, H, W = _bchw(x)
    out = np.empty_like(x)
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    cl = None if clip is None else np.ascontiguousarray(clip, dtype=np.float32)
    _fn("scaling_floating_point", x.dtype)(_p(x), _p(out), C.c_size_t(B), C.c_size_t(Cc), C.c_size_t(H),
                                           C.c_size_t(W), int(clip is not None), _p(cl), _p(scale),
                                           C.c_size_t(nb_bits), int(bool(unsigned)))
    return out


def scaling_fixed(x, mult, frac_bits, nb_bits, unsigned, clip=None):
    x = np.ascontiguousarray(x)
    B, Cc, H, W = _bchw(x)
    out = np.empty_like(x)
    mult = np.ascontiguousarray(mult, dtype=np.int32)
    cl = None if clip is None else np.ascontiguousarray(clip, dtype=np.float32)
    rc = _fn("scaling_fixed_point", x.dtype)(_p(x), _p(out), C.c_size_t(B), C.c_size_t(Cc), C.c_size_t(H),
                                             C.c_size_t(W), int(clip is not None), _p(cl), _p(mult),
                                             C.c_size_t(frac_bits), C.c_size_t(nb_bits), int(bool(unsigned)))
    if rc != 0:
        raise RuntimeError("FixedPointScaling::propagate can only be used on quantized network.")
    return out


def scaling_single_shift(x, shift, nb_bits, unsigned):
    x = np.ascontiguousarray(x)
    B, Cc, H, W = _bchw(x)
    out = np.empty_like(x)
    shift = np.ascontiguousarray(shift, dtype=np.uint8)
    rc = _fn("scaling_single_shift", x.dtype)(_p(x), _p(out), C.c_size_t(B), C.c_size_t(Cc), C.c_size_t(H),
                                              C.c_size_t(W), _p(shift), C.c_size_t(nb_bits), int(bool(unsigned)))
    if rc != 0:
        raise RuntimeError("SingleShiftScaling::propagate can only be used on quantized network.")
    return out


def scaling_double_shift(x, pairs, nb_bits, unsigned):
    """pairs: uint8 [C,2] = (first, second) per channel."""
    x = np.ascontiguousarray(x)
    B, Cc, H, W = _bchw(x)
    out = np.empty_like(x)
    pairs = np.ascontiguousarray(pairs, dtype=np.uint8).reshape(-1, 2)
    rc = _fn("scaling_double_shift", x.dtype)(_p(x), _p(out), C.c_size_t(B), C.c_size_t(Cc), C.c_size_t(H),
                                              C.c_size_t(W), _p(pairs), C.c_size_t(nb_bits), int(bool(unsigned)))
    if rc != 0:
        raise RuntimeError("DoubleShiftScaling::propagate can only be used on quantized network.")
    return out


def rectifier(x, leak=0.0, clipping=0.0, cell_quantized=True):
    x = np.ascontiguousarray(x).copy()
    _fn("rectifier_apply", x.dtype)(_p(x), C.c_size_t(x.size), C.c_double(leak), C.c_double(clipping),
                                    int(bool(cell_quantized)))
    return x


def linear(x, clipping=0.0, cell_quantized=True):
    x = np.ascontiguousarray(x).copy()
    _fn("linear_apply", x.dtype)(_p(x), C.c_size_t(x.size), C.c_double(clipping), int(bool(cell_quantized)))
    return x


# ---------------------------------------------------------------- SAT / LSQ

SAT_MODES = {"none": 0, "default": 1, "fullrange": 2, "symrange": 3, "asymrange": 4, "none_asym": 5}


def sat_weight_forward(w, rng, mode="default", apply_scaling=False, outputs_size=1):
    """Returns (wq, tanh_max, scaling). mode as in SATQuantizerCell_Frame::propagate."""
    w = np.ascontiguousarray(w)
    dt = w.dtype
    wq = np.empty_like(w)
    ct = _CT[np.dtype(dt)]
    tmax = ct(0)
    _fn("sat_weight_forward", dt)(_p(w), _p(wq), C.c_size_t(w.size), C.c_float(rng),
                                  SAT_MODES[mode], C.byref(tmax))
    scal = ct(1.0)
    if apply_scaling:
        _fn("sat_apply_scaling", dt)(_p(wq), C.c_size_t(wq.size), C.byref(scal), C.c_uint(outputs_size))
    return wq, tmax.value, scal.value


def sat_weight_backward(dwq, w, rng, factor, mode="default"):
    w = np.ascontiguousarray(w)
    dt = w.dtype
    dwq = np.ascontiguousarray(dwq, dtype=dt)
    dw = np.empty_like(w)
    m = {"default": 0, "symrange": 0, "none": 0, "fullrange": 2, "asymrange": 4}[mode]
    _fn("sat_weight_backward", dt)(_p(dwq), _p(dw), _p(w), C.c_size_t(w.size), C.c_float(rng), m,
                                   _CT[np.dtype(dt)](factor))
    return dw


def sat_act_forward(x, rng, alpha, inference=True):
    """Returns (y, saved full-precision copy or None)."""
    x = np.ascontiguousarray(x).copy()
    dt = x.dtype
    fp = None if inference else np.empty_like(x)
    _fn("sat_act_forward", dt)(_p(x), C.c_size_t(x.size), C.c_float(rng), _CT[np.dtype(dt)](alpha),
                               _p(fp), int(bool(inference)))
    return x, fp


def sat_act_backward(dy, fp, rng, alpha, beta=0.0, prev_diff_alpha=0.0):
    """Returns (dx, dalpha, per-element dalpha terms)."""
    fp = np.ascontiguousarray(fp)
    dt = fp.dtype
    dy = np.ascontiguousarray(dy, dtype=dt)
    dx = np.empty_like(fp)
    terms = np.empty_like(fp)
    ct = _CT[np.dtype(dt)]
    da = ct(prev_diff_alpha)
    _fn("sat_act_backward", dt)(_p(dy), _p(dx), _p(terms), _p(fp), C.c_size_t(fp.size), C.c_float(rng),
                                ct(alpha), ct(beta), C.byref(da))
    return dx, da.value, terms


def lsq_forward(x, step, lo, hi):
    x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    _fn("lsq_forward", x.dtype)(_p(x), _p(out), C.c_size_t(x.size), _CT[np.dtype(x.dtype)](step), int(lo), int(hi))
    return out


def lsq_backward(dq, fp, step, lo, hi):
    """Returns (dfp, un-scaled step-size gradient sum)."""
    fp = np.ascontiguousarray(fp)
    dt = fp.dtype
    dq = np.ascontiguousarray(dq, dtype=dt)
    dfp = np.empty_like(fp)
    f = _fn("lsq_backward", dt)
    f.restype = _CT[np.dtype(dt)]
    s = f(_p(dq), _p(fp), _p(dfp), C.c_size_t(fp.size), _CT[np.dtype(dt)](step), int(lo), int(hi))
    return dfp, float(s)
