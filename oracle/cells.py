"""Reference cells assembled from the CPU oracle, in the order the N2D2 Frame
cells call their kernels (ConvCell_Frame::propagate, FcCell_Frame::propagate,
Cell_Frame::propagate -> Activation::propagate -> Scaling::propagate)."""
import numpy as np

from . import oracle as orc


class ActSpec:
    """Host description of a cell's activation (kind, Scaling, bits, signedness)."""

    def __init__(self, kind="Linear", mode="None", scaling=None, frac_bits=0, clipping=None, nb_bits=8, unsigned_out=False,
                 leak_slope=0.0):
        self.kind, self.mode, self.scaling, self.frac_bits = kind, mode, scaling, frac_bits
        self.clipping, self.nb_bits, self.unsigned_out = clipping, nb_bits, unsigned_out
        self.leak_slope = leak_slope

    def kwargs(self):
        kw = dict(kind=self.kind, mode=self.mode, scaling=self.scaling, frac_bits=self.frac_bits,
                  clipping=self.clipping, nb_bits=self.nb_bits, unsigned_out=self.unsigned_out)
        if self.leak_slope:
            kw["leak_slope"] = self.leak_slope
        return kw

    def apply(self, x):
        """Scaling::propagate dispatch (include/Scaling.hpp:434-459) then the activation pass."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        if self.mode == "None":
            y = x.copy()
        elif self.mode == "FloatMult":
            y = orc.scaling_float(x, self.scaling, self.nb_bits, self.unsigned_out, self.clipping)
        elif self.mode in ("FixedMult16", "FixedMult32"):
            y = orc.scaling_fixed(x, self.scaling, self.frac_bits, self.nb_bits, self.unsigned_out, self.clipping)
        elif self.mode == "SingleShift":
            y = orc.scaling_single_shift(x, self.scaling, self.nb_bits, self.unsigned_out)
        elif self.mode == "DoubleShift":
            y = orc.scaling_double_shift(x, self.scaling, self.nb_bits, self.unsigned_out)
        else:
            raise ValueError(self.mode)
        if self.kind == "Rectifier":
            y = orc.rectifier(y, leak=self.leak_slope)
        else:
            y = orc.linear(y)
        return y


def conv_cell(x, w, bias, act, stride=(1, 1), pad=(0, 0, 0, 0), dil=(1, 1), groups=1, maps=None, sub=(1, 1)):
    """x: one input, or a list of inputs: ConvCell_Frame<T>::propagate (src/Cell/ConvCell_Frame.cpp:438-459) then walks
    them with its slice of the weights each, beta = 0 for the first and 1 afterwards.  maps: a connection map, bool
    [channels, outputs], instead of `groups` (one input).  sub: ConvCell's SubSample (x, y): the outputs of that many
    neighbouring positions are added up before the bias and the activation (src/Cell/ConvCell_Frame_Kernels.cpp:135-140)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    if isinstance(x, (list, tuple)) and len(x) > 1:
        if groups != 1:
            raise ValueError("several inputs with a grouped mapping are not restated")
        y, first = None, 0
        for k, xk in enumerate(x):
            xk = np.ascontiguousarray(xk, dtype=np.float32)
            wk = np.ascontiguousarray(w[:, first:first + xk.shape[1]])
            y = orc.conv_forward(xk, wk, stride=stride, pad=pad, dil=dil, out=y, beta=0.0 if k == 0 else 1.0, sub=sub)
            first += xk.shape[1]
        assert first == w.shape[1]
    else:
        x = np.ascontiguousarray(x[0] if isinstance(x, (list, tuple)) else x, dtype=np.float32)
        if maps is None and groups > 1:
            maps = orc.group_maps(x.shape[1], w.shape[0], groups)
        y = orc.conv_forward(x, w, stride=stride, pad=pad, dil=dil, maps=maps, sub=sub)
    if bias is not None:
        orc.conv_forward_bias(y, np.asarray(bias, dtype=np.float32))
    return act.apply(y)


def fc_cell(x, w, bias, act):
    """x: one input, or a list of inputs: FcCell_Frame<T>::propagate (src/Cell/FcCell_Frame.cpp:273-336) then forms one inner
    product per input over that input's weights, each seeded with the bias (`:309`), beta = 0 for the first and 1 afterwards."""
    xs = list(x) if isinstance(x, (list, tuple)) else [x]
    w = np.asarray(w, dtype=np.float32).reshape(np.asarray(w).shape[0], -1)
    b = None if bias is None else np.asarray(bias, dtype=np.float32)
    y, first = None, 0
    for k, xk in enumerate(xs):
        xk = np.ascontiguousarray(xk, dtype=np.float32)
        size = xk[0].size
        y = orc.fc_forward(xk, np.ascontiguousarray(w[:, first:first + size]), b, out=y, beta=0.0 if k == 0 else 1.0)
        first += size
    assert first == w.shape[1]
    return act.apply(y.reshape(y.shape[0], y.shape[1], 1, 1))


def pool_cell(x, kind, pool, stride, pad=(0, 0), maps=None):
    """x: one input, or a list of inputs: PoolCell_Frame<T>::propagate (src/Cell/PoolCell_Frame.cpp:123-174) then walks them
    with the rows of the map over all their channels that belong to each, beta = 0 for the first and 1 afterwards (an
    output pools nothing from the inputs it is not connected to: 0 is added).  maps: bool [channels, outputs], the unit map
    (one output per channel) when None."""
    if not isinstance(x, (list, tuple)) or len(x) == 1:
        x = x[0] if isinstance(x, (list, tuple)) else x
        return orc.pool_forward(np.ascontiguousarray(x, dtype=np.float32), pool, stride, pad, kind=kind, quantized=True, maps=maps)
    total = sum(xk.shape[1] for xk in x)
    unit = np.eye(total, dtype=np.uint8) if maps is None else np.ascontiguousarray(maps, dtype=np.uint8)
    y, first = None, 0
    for k, xk in enumerate(x):
        xk = np.ascontiguousarray(xk, dtype=np.float32)
        y = orc.pool_forward(xk, pool, stride, pad, kind=kind, quantized=True, maps=unit[first:first + xk.shape[1]], out=y,
                             beta=0.0 if k == 0 else 1.0)
        first += xk.shape[1]
    return y


def elemwise_cell(xs, act, weights=None, shifts=None, coeff_mode="PerLayer"):
    n = len(xs)
    Cc = xs[0].shape[1]
    size = Cc if coeff_mode == "PerChannel" else n
    w = np.ones(size, dtype=np.float32) if weights is None else np.asarray(weights, dtype=np.float32)
    s = np.zeros(size, dtype=np.float32) if shifts is None else np.asarray(shifts, dtype=np.float32)
    y = orc.elemwise_sum([np.asarray(x, dtype=np.float32) for x in xs], w, s, coeff_mode)
    return act.apply(y)


def run_net(spec, x, keep=None):
    """Layer-ordered forward of a network description (n2d2_amd.nets.NetSpec) on the CPU oracle, as
    DeepNet::propagate calls each cell (src/DeepNet.cpp:2692-2706).  x: integer-valued [B,C,H,W].
    Returns {name: float32 NCHW output} for the names in `keep` (default: the last cell)."""
    vals = {"input": np.ascontiguousarray(x, dtype=np.float32)}
    keep = set(keep) if keep is not None else {spec.output}
    out = {}
    for i, l in enumerate(spec.layers):
        ins = [vals[n] for n in l.inputs]
        if l.type in ("conv", "fc", "elemwise", "scaling"):
            a = l.act
            act = ActSpec(a.kind, a.mode, a.scaling, a.frac_bits, a.clipping, a.nb_bits, a.unsigned_out)
        if l.type == "conv":
            y = conv_cell(ins if len(ins) > 1 else ins[0], l.w, l.bias, act, l.stride, l.pad, l.dil, l.groups,
                          maps=getattr(l, "maps", None), sub=getattr(l, "sub", (1, 1)))
        elif l.type == "fc":
            y = fc_cell(ins if len(ins) > 1 else ins[0], l.w, l.bias, act)
        elif l.type == "pool":
            y = pool_cell(ins if len(ins) > 1 else ins[0], l.kind, l.pool, l.stride, l.pad)
        elif l.type == "scaling":
            y = act.apply(ins[0])           # ScalingCell_Frame::propagate: the Scaling alone
        elif l.type == "elemwise":
            y = elemwise_cell(ins, act, l.weights, l.shifts, l.coeff_mode)
        else:
            raise ValueError(l.type)
        vals[l.name] = y
        if l.name in keep:
            out[l.name] = y
        # free tensors nobody reads any more
        later = set(n for m in spec.layers[i + 1:] for n in m.inputs)
        for n in list(vals):
            if n not in later and n != l.name:
                del vals[n]
    return out
