"""Thin object layer over the C ABI for the tests and the benchmark.

torch is used for device memory and streams only; every computation goes
through libn2d2hip.so.  Handles own their C objects and keep alive the host
arrays they were built from.
"""
import ctypes as C

import numpy as np
import torch

from . import capi
from .capi import lib, check

_TORCH_DT = {capi.U8: torch.uint8, capi.I8: torch.int8, capi.U8B: torch.int8, capi.I32: torch.int32, capi.F32: torch.float32}
_NP_DT = {capi.U8: np.uint8, capi.I8: np.int8, capi.U8B: np.int8, capi.I32: np.int32, capi.F32: np.float32}


def stream_ptr():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


class DTensor:
    """A device tensor plus its n2d2hip_tensor descriptor."""

    def __init__(self, B, Cc, H, W, dtype, layout=capi.NHWC, buf=None, halo=0):
        """halo: border pixels stored around every image (NHWC byte tensors between two convolutions), holding the value 0."""
        self.B, self.C, self.H, self.W, self.dtype, self.layout, self.halo = B, Cc, H, W, dtype, layout, halo
        if layout == capi.S2D:
            # space-to-depth form of a network input: 16-byte pixels holding 2 x 2 input pixels; n2d2hip_convert writes all of it
            self.cs = 16
            n = B * ((H + 1) // 2 + 2 * halo) * ((W + 1) // 2 + 2 * halo) * 16
            self.buf = buf if buf is not None else torch.empty(n, dtype=_TORCH_DT[dtype], device="cuda")
            assert self.buf.numel() == n
            self.desc = capi.Tensor(self.buf.data_ptr(), dtype, layout, B, Cc, H, W, 16, halo)
            return
        self.cs = capi.nhwc_cs(Cc) if layout == capi.NHWC else Cc
        n = B * (H + 2 * halo) * (W + 2 * halo) * self.cs
        self.buf = buf if buf is not None else torch.empty(n, dtype=_TORCH_DT[dtype], device="cuda")
        assert self.buf.numel() == n
        self.desc = capi.Tensor(self.buf.data_ptr(), dtype, layout, B, Cc, H, W, self.cs, halo)
        if halo:
            check(lib.n2d2hip_tensor_clear(self.ref, stream_ptr()))

    @property
    def ref(self):
        return C.byref(self.desc)

    @property
    def nbytes(self):
        return self.buf.numel() * self.buf.element_size()

    @staticmethod
    def from_numpy(x, dtype, layout=capi.NHWC, halo=0):
        """x: integer-valued NCHW numpy array. Uploads it as I32/F32 NCHW and converts on the device."""
        x = np.ascontiguousarray(x)
        B, Cc, H, W = x.shape
        if x.dtype == np.float32:
            src = DTensor(B, Cc, H, W, capi.F32, capi.NCHW, torch.from_numpy(x.reshape(-1)).cuda())
        else:
            src = DTensor(B, Cc, H, W, capi.I32, capi.NCHW, torch.from_numpy(x.astype(np.int32).reshape(-1)).cuda())
        if dtype == src.dtype and layout == capi.NCHW:
            return src
        dst = DTensor(B, Cc, H, W, dtype, layout, halo=halo)
        check(lib.n2d2hip_convert(src.ref, dst.ref, stream_ptr()))
        return dst

    def convert_from(self, src):
        """Graph-edge conversion of `src` (any layout / type of the same logical shape) into this tensor."""
        check(lib.n2d2hip_convert(src.ref, self.ref, stream_ptr()))
        return self

    def with_halo(self, halo):
        """A copy of this NHWC byte tensor stored with a border of `halo` zero pixels around every image."""
        assert self.layout == capi.NHWC and self.halo == 0
        dst = DTensor(self.B, self.C, self.H, self.W, self.dtype, halo=halo)
        dst.buf.view(self.B, self.H + 2 * halo, self.W + 2 * halo, self.cs)[:, halo:self.H + halo, halo:self.W + halo, :] = \
            self.buf.view(self.B, self.H, self.W, self.cs)
        return dst

    def to_numpy(self):
        """Logical integer values as an int64 NCHW numpy array."""
        dst = DTensor(self.B, self.C, self.H, self.W, capi.I32, capi.NCHW)
        check(lib.n2d2hip_convert(self.ref, dst.ref, stream_ptr()))
        torch.cuda.synchronize()
        return dst.buf.cpu().numpy().reshape(self.B, self.C, self.H, self.W).astype(np.int64)

    def raw(self):
        torch.cuda.synchronize()
        return self.buf.cpu().numpy()


class Act:
    """n2d2hip_act_t: Scaling + Rectifier/Linear of one cell."""

    def __init__(self, nb_channels, kind="Linear", mode="None", scaling=None, frac_bits=0, clipping=None,
                 nb_bits=8, unsigned_out=False, leak_slope=0.0):
        modes = {"None": capi.SCALING_NONE, "FloatMult": capi.SCALING_FLOAT_MULT, "FixedMult16": capi.SCALING_FIXED_MULT16,
                 "FixedMult32": capi.SCALING_FIXED_MULT32, "SingleShift": capi.SCALING_SINGLE_SHIFT,
                 "DoubleShift": capi.SCALING_DOUBLE_SHIFT}
        m = modes[mode]
        self._keep = []
        sp = None
        if scaling is not None:
            np_t = {capi.SCALING_FLOAT_MULT: np.float32, capi.SCALING_FIXED_MULT16: np.int32, capi.SCALING_FIXED_MULT32: np.int32,
                    capi.SCALING_SINGLE_SHIFT: np.uint8, capi.SCALING_DOUBLE_SHIFT: np.uint8}[m]
            s = np.ascontiguousarray(scaling, dtype=np_t)
            self._keep.append(s)
            sp = s.ctypes.data
        cp = None
        if clipping is not None:
            cl = np.ascontiguousarray(clipping, dtype=np.float32)
            self._keep.append(cl)
            cp = cl.ctypes.data
        d = capi.Activation(capi.ACT_RECTIFIER if kind == "Rectifier" else capi.ACT_LINEAR, float(leak_slope), m, sp,
                            int(frac_bits), int(clipping is not None), cp, int(nb_bits), int(bool(unsigned_out)))
        self.nb_channels = nb_channels
        self.mode = mode
        self.unsigned_out = bool(unsigned_out)
        self.handle = C.c_void_p()
        check(lib.n2d2hip_act_create(C.byref(d), nb_channels, C.byref(self.handle)))

    def out_dtype(self):
        """Storage type of this cell's output between Frame_HIP cells."""
        if self.mode == "None":
            return capi.I32
        return capi.U8B if self.unsigned_out else capi.I8

    def __del__(self):
        if getattr(self, "handle", None) and lib is not None:
            lib.n2d2hip_act_destroy(self.handle)
            self.handle = None


class Bottleneck:
    """n2d2hip_bottleneck_t: reduce -> 3x3 [-> expand + sum (+ projection)] in one launch; None when the library keeps
    the cells apart."""

    def __init__(self, handle, cells):
        self.handle, self._cells = handle, cells

    @staticmethod
    def create(reduce, conv3x3, expand=None, projection=None):
        h = C.c_void_p()
        rc = lib.n2d2hip_bottleneck_create(reduce.handle, conv3x3.handle, expand.handle if expand is not None else None,
                                           projection.handle if projection is not None else None, C.byref(h))
        if rc == capi.ERR_UNSUPPORTED:
            return None
        check(rc)
        return Bottleneck(h, (reduce, conv3x3, expand, projection))

    def pays(self, batch, H, W):
        """True where the library expects the one launch to be faster than the plan the cells would otherwise run in."""
        return bool(lib.n2d2hip_bottleneck_pays(self.handle, batch, H, W))

    def forward(self, x, out):
        check(lib.n2d2hip_bottleneck_forward(self.handle, x.ref, out.ref, stream_ptr()))
        return out

    def __del__(self):
        if getattr(self, "handle", None) and lib is not None:
            lib.n2d2hip_bottleneck_destroy(self.handle)
            self.handle = None


class DwPw:
    """n2d2hip_dw_pw_t: a 3x3 depthwise convolution and the 1x1 convolution reading it in one launch; None when the library
    keeps the cells apart."""

    def __init__(self, handle, cells):
        self.handle, self._cells = handle, cells

    @staticmethod
    def create(depthwise, pointwise):
        h = C.c_void_p()
        rc = lib.n2d2hip_dw_pw_create(depthwise.handle, pointwise.handle, C.byref(h))
        if rc == capi.ERR_UNSUPPORTED:
            return None
        check(rc)
        return DwPw(h, (depthwise, pointwise))

    def forward(self, x, out):
        check(lib.n2d2hip_dw_pw_forward(self.handle, x.ref, out.ref, stream_ptr()))
        return out

    def pays(self, batch, in_h, in_w):
        """Does the library expect the one launch to be faster than the two cells' own on inputs of this size?"""
        return bool(lib.n2d2hip_dw_pw_pays(self.handle, batch, in_h, in_w))

    def __del__(self):
        if getattr(self, "handle", None) and lib is not None:
            lib.n2d2hip_dw_pw_destroy(self.handle)
            self.handle = None


def scaling_forward(act, x, out_dtype=None):
    out = DTensor(x.B, x.C, x.H, x.W, out_dtype if out_dtype is not None else act.out_dtype(), x.layout)
    check(lib.n2d2hip_scaling_forward(act.handle, x.ref, out.ref, stream_ptr()))
    return out


def pack_int4(w):
    """int array in [-8,7] -> bytes, element 2i in the low nibble."""
    f = np.ascontiguousarray(w).reshape(-1).astype(np.int64)
    if f.size % 2:
        f = np.concatenate([f, [0]])
    return ((f[0::2] & 15) | ((f[1::2] & 15) << 4)).astype(np.uint8)


class Conv:
    def __init__(self, w, bias, act, in_dtype, stride=(1, 1), pad=(0, 0, 0, 0), dil=(1, 1), groups=1, weight_bits=8,
                 kernel_choice=0, sub=(1, 1)):
        """w: integer-valued [O, C/groups, kH, kW]; stride/dil (x,y); pad (L,T,R,B); kernel_choice: capi.KERNEL_* bits;
        sub (x,y): the sums of that many neighbouring positions are added up into one output (ConvCell's SubSample)."""
        O, Cg, kH, kW = w.shape
        self.desc = capi.ConvDesc(Cg * groups, O, kW, kH, stride[0], stride[1], pad[0], pad[1], pad[2], pad[3],
                                  dil[0], dil[1], groups, weight_bits, kernel_choice, sub[0], sub[1])
        self.act = act
        hw = pack_int4(w) if weight_bits == 4 else np.ascontiguousarray(w, dtype=np.int8)
        hb = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
        self.handle = C.c_void_p()
        check(lib.n2d2hip_conv_create(C.byref(self.desc), hw.ctypes.data, None if hb is None else hb.ctypes.data,
                                      act.handle, in_dtype, C.byref(self.handle)))

    def out_shape(self, H, W):
        oh, ow = C.c_int(), C.c_int()
        check(lib.n2d2hip_conv_out_dims(C.byref(self.desc), H, W, C.byref(oh), C.byref(ow)))
        return oh.value, ow.value

    def make_output(self, x, out_dtype=None, halo=0):
        oh, ow = self.out_shape(x.H, x.W)
        return DTensor(x.B, self.desc.O, oh, ow, out_dtype if out_dtype is not None else self.act.out_dtype(), halo=halo)

    def accepts_maxpool(self, pool, H, W):
        """True when the library computes this convolution and the max pooling `pool` (a Pool) behind it in one launch."""
        return bool(lib.n2d2hip_conv_accepts_maxpool(self.handle, C.byref(pool.desc), H, W))

    def forward_maxpool(self, pool, x, out):
        check(lib.n2d2hip_conv_forward_maxpool(self.handle, C.byref(pool.desc), x.ref, out.ref, stream_ptr()))
        return out

    def s2d_halo(self, H, W, pool=None):
        """Border a space-to-depth H x W input must carry for this convolution (with the max pooling `pool` behind it in the
        same launch, if given) to read it; -1 when the library does not serve it that way."""
        return int(lib.n2d2hip_conv_s2d_halo(self.handle, C.byref(pool.desc) if pool is not None else None, H, W))

    def accepts_halo(self):
        """True when this convolution reads and writes tensors that carry their padding as a border of zeros."""
        return bool(lib.n2d2hip_conv_accepts_halo(self.handle))

    @staticmethod
    def shape_reads_halo(w_shape, stride, pad, dil, groups, weight_bits, kernel_choice=0, sub=(1, 1)):
        """What a planner can ask before the cell exists: can a convolution of this shape ([O, C/groups, kH, kW] weights) be one
        that reads a tensor with a border?  The cell's own accepts_halo() has the last word."""
        O, Cg, kH, kW = w_shape
        pad = tuple(pad) if len(pad) == 4 else (pad[0], pad[1], pad[0], pad[1])
        d = capi.ConvDesc(Cg * groups, O, kW, kH, stride[0], stride[1], pad[0], pad[1], pad[2], pad[3], dil[0], dil[1], groups, weight_bits,
                          kernel_choice, sub[0], sub[1])
        return bool(lib.n2d2hip_conv_desc_reads_halo(C.byref(d)))

    def forward(self, x, out=None, out_dtype=None):
        if out is None:
            out = self.make_output(x, out_dtype)
        check(lib.n2d2hip_conv_forward(self.handle, x.ref, out.ref, stream_ptr()))
        return out

    def fuse_sum(self, ew, conv_input_index, other_dtype):
        """Folds the ElemWise sum fed by this convolution into its epilogue; False when the library keeps them apart."""
        rc = lib.n2d2hip_conv_fuse_sum(self.handle, ew.handle if ew is not None else None, conv_input_index, other_dtype)
        if rc == capi.ERR_UNSUPPORTED:
            return False
        check(rc)
        self._sum = ew
        return True

    def forward_sum(self, x, other, out):
        check(lib.n2d2hip_conv_forward_sum(self.handle, x.ref, other.ref, out.ref, stream_ptr()))
        return out

    def chain_supported(self, conv3x3):
        """Can `conv3x3`, whose output only this 1x1 expansion (with its folded sum) reads, run in this cell's launch?"""
        return bool(lib.n2d2hip_conv_chain_supported(conv3x3.handle, self.handle))

    def forward_chain(self, conv3x3, x, other, out):
        """out = sum(self(conv3x3(x)), other) in one launch; x carries conv3x3's padding as a border."""
        check(lib.n2d2hip_conv_chain_forward(conv3x3.handle, self.handle, x.ref, other.ref, out.ref, stream_ptr()))
        return out

    def __del__(self):
        if getattr(self, "handle", None) and lib is not None:
            lib.n2d2hip_conv_destroy(self.handle)
            self.handle = None


class Fc:
    def __init__(self, w, bias, act, in_dtype, in_shape, weight_bits=8):
        """w: integer-valued [O, C*H*W] (CHW flattening); in_shape = (C, H, W)."""
        Cc, H, W = in_shape
        O = w.shape[0]
        self.O = O
        self.act = act
        hw = pack_int4(w) if weight_bits == 4 else np.ascontiguousarray(w, dtype=np.int8)
        hb = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
        self.handle = C.c_void_p()
        check(lib.n2d2hip_fc_create(Cc, H, W, O, weight_bits, hw.ctypes.data, None if hb is None else hb.ctypes.data,
                                    act.handle, in_dtype, C.byref(self.handle)))

    def make_output(self, x, out_dtype=None):
        return DTensor(x.B, self.O, 1, 1, out_dtype if out_dtype is not None else self.act.out_dtype())

    def forward(self, x, out=None, out_dtype=None):
        if out is None:
            out = self.make_output(x, out_dtype)
        check(lib.n2d2hip_fc_forward(self.handle, x.ref, out.ref, stream_ptr()))
        return out

    def __del__(self):
        if getattr(self, "handle", None) and lib is not None:
            lib.n2d2hip_fc_destroy(self.handle)
            self.handle = None


class FcChain:
    """n2d2hip_fc_chain_t: two or three Fc cells, each reading the one before, as one launch."""

    def __init__(self, handle, cells):
        self.handle, self.cells = handle, cells     # the cells' handles are borrowed: keep them alive

    @staticmethod
    def create(cells):
        """None when the library keeps the cells apart."""
        h = C.c_void_p()
        arr = (C.c_void_p * len(cells))(*[c.handle for c in cells])
        rc = lib.n2d2hip_fc_chain_create(len(cells), arr, C.byref(h))
        if rc == capi.ERR_UNSUPPORTED:
            return None
        check(rc)
        return FcChain(h, list(cells))

    def forward(self, x, out):
        check(lib.n2d2hip_fc_chain_forward(self.handle, x.ref, out.ref, stream_ptr()))
        return out

    def __del__(self):
        if getattr(self, "handle", None) and lib is not None:
            lib.n2d2hip_fc_chain_destroy(self.handle)
            self.handle = None


class Pool:
    def __init__(self, kind, pool, stride, pad=(0, 0), maps=None):
        """maps: None for one output per channel, else a bool array [channels, outputs] (maps[c, o]: output o pools channel c)."""
        self.desc = capi.PoolDesc(capi.POOL_MAX if kind == "max" else capi.POOL_AVERAGE, pool[0], pool[1],
                                  stride[0], stride[1], pad[0], pad[1])
        self.maps = None
        if maps is not None:
            m = np.ascontiguousarray(np.asarray(maps, dtype=np.uint8).T)      # one row per output
            self.nb_channels, self.nb_outputs = m.shape[1], m.shape[0]
            self.maps = torch.from_numpy(m.reshape(-1)).cuda()

    def writes_halo(self, x):
        """True when this pooling of x can store its output with a border (its readers' padding)."""
        return self.maps is None and bool(lib.n2d2hip_pool_writes_halo(C.byref(self.desc), x.H, x.W, x.cs))

    def make_output(self, x):
        oh, ow = C.c_int(), C.c_int()
        check(lib.n2d2hip_pool_out_dims(C.byref(self.desc), x.H, x.W, C.byref(oh), C.byref(ow)))
        return DTensor(x.B, x.C if self.maps is None else self.nb_outputs, oh.value, ow.value, x.dtype)

    def forward(self, x, out=None):
        if out is None:
            out = self.make_output(x)
        if self.maps is None:
            check(lib.n2d2hip_pool_forward(C.byref(self.desc), x.ref, out.ref, stream_ptr()))
        else:
            if x.C != self.nb_channels or out.C != self.nb_outputs:
                raise ValueError("Pool: the map is %d channels x %d outputs, the tensors have %d and %d"
                                 % (self.nb_channels, self.nb_outputs, x.C, out.C))
            check(lib.n2d2hip_pool_forward_mapped(C.byref(self.desc), self.maps.data_ptr(), self.nb_outputs, self.nb_channels, x.ref, out.ref,
                                                  stream_ptr()))
        return out


def concat_channels(xs, out=None, halo=0):
    """The channels of the tensors xs (one dtype, one size) one behind the other: what a cell with several inputs reads."""
    x0 = xs[0]
    if out is None:
        out = DTensor(x0.B, sum(x.C for x in xs), x0.H, x0.W, x0.dtype, halo=halo)
    arr = (C.c_void_p * len(xs))(*[C.addressof(x.desc) for x in xs])
    check(lib.n2d2hip_concat_channels(len(xs), arr, out.ref, stream_ptr()))
    return out


class ElemWiseSum:
    def __init__(self, nb_inputs, nb_channels, act, weights=None, shifts=None, coeff_mode="PerLayer"):
        mode = {"PerLayer": capi.COEFF_PER_LAYER, "PerInput": capi.COEFF_PER_INPUT, "PerChannel": capi.COEFF_PER_CHANNEL}[coeff_mode]
        self.act = act
        self.nb_inputs = nb_inputs
        w = None if weights is None else np.ascontiguousarray(weights, dtype=np.float32)
        s = None if shifts is None else np.ascontiguousarray(shifts, dtype=np.float32)
        self.handle = C.c_void_p()
        check(lib.n2d2hip_elemwise_create(nb_inputs, nb_channels, mode, None if w is None else w.ctypes.data,
                                          None if s is None else s.ctypes.data, act.handle, C.byref(self.handle)))

    def fold_input_scaling(self, input_index, act):
        """Folds the ScalingCell feeding input `input_index`; returns False when the library keeps them separate."""
        rc = lib.n2d2hip_elemwise_fold_input_scaling(self.handle, input_index, act.handle if act is not None else None)
        if rc == capi.ERR_UNSUPPORTED:
            return False
        check(rc)
        self._folded = act
        return True

    def forward(self, xs, out=None, out_dtype=None):
        x0 = xs[0]
        if out is None:
            out = DTensor(x0.B, x0.C, x0.H, x0.W, out_dtype if out_dtype is not None else self.act.out_dtype())
        arr = (C.c_void_p * len(xs))(*[C.addressof(x.desc) for x in xs])
        check(lib.n2d2hip_elemwise_forward(self.handle, arr, out.ref, stream_ptr()))
        return out

    def __del__(self):
        if getattr(self, "handle", None) and lib is not None:
            lib.n2d2hip_elemwise_destroy(self.handle)
            self.handle = None
