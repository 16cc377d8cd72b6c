"""ctypes access to the C++ Frame_HIP host cells (libn2d2_frame_hip.so): nets are built from N2D2-style INI text
through the Registrar under the model key named by DefaultModel, parameters are installed the way N2D2's
quantization pass leaves them, and outputs come back as N2D2 float tensors."""
import ctypes as C
import os

import numpy as np

from . import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libn2d2_frame_hip.so")

if not os.path.exists(LIB_PATH):
    raise ImportError("libn2d2_frame_hip.so is not built (%s): run `python -m n2d2_amd.build`" % LIB_PATH)
lib = C.CDLL(LIB_PATH)
lib.fh_last_error.restype = C.c_char_p
lib.fh_net_from_ini.restype = C.c_void_p
lib.fh_net_from_ini.argtypes = [C.c_char_p]
lib.fh_net_model.restype = C.c_char_p
lib.fh_net_set_fusion.argtypes = [C.c_void_p, C.c_int]
for _n in ("fh_net_free", "fh_net_model", "fh_net_nb_cells", "fh_net_initialize", "fh_net_propagate", "fh_net_nb_folded", "fh_net_nb_halo"):
    getattr(lib, _n).argtypes = [C.c_void_p]
lib.fh_net_set_stimuli.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int]
lib.fh_cell_info.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_char_p, C.c_int]
lib.fh_cell_outputs_halo.argtypes = [C.c_void_p, C.c_char_p]
lib.fh_cell_set_quantized.argtypes = [C.c_void_p, C.c_char_p, C.c_int, C.c_int]
lib.fh_cell_set_weights.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
lib.fh_cell_set_biases.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t]
lib.fh_net_save_quantization.argtypes = [C.c_void_p, C.c_char_p]
lib.fh_net_load_quantization.argtypes = [C.c_void_p, C.c_char_p]
lib.fh_get_nb_groups.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p]
lib.fh_cell_set_mapping.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t, C.c_size_t]
lib.fh_cell_set_scaling.argtypes = [C.c_void_p, C.c_char_p, C.c_int, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p]
lib.fh_cell_get_outputs.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t]
lib.fh_cell_get_max_output.argtypes = [C.c_void_p, C.c_char_p, C.c_uint, C.c_void_p]
lib.fh_cell_learn_step.argtypes = [C.c_void_p, C.c_char_p, C.c_int]
lib.fh_cell_replace_input.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_char_p]
lib.fh_cell_get_clipping.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
lib.fh_cell_get_quantized.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_char_p, C.c_int]
lib.fh_qat_fuse_batchnorm_with_conv.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                                                C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double,
                                                C.c_size_t, C.c_double, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
lib.fh_qat_quantize_fc.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_size_t,
                                   C.c_double, C.c_size_t, C.c_double, C.c_int, C.c_int, C.c_int]
lib.fh_qat_quantize_elemwise.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_double, C.c_size_t, C.c_double]
lib.fh_registrar_exists.argtypes = [C.c_char_p, C.c_char_p]
lib.fh_registrar_unknown_key_is_null.argtypes = [C.c_char_p]
lib.fh_set_globals.argtypes = [C.c_int, C.c_int, C.c_int]
_F, _P, _SZ, _I = C.c_float, C.c_void_p, C.c_size_t, C.c_int
lib.fh_sat_cell_run.argtypes = [C.c_char_p, _P, _P, _SZ, _SZ, _I, _I, _I, _I, _P, _P, _P]
lib.fh_sat_act_run.argtypes = [C.c_char_p, _P, _P, _SZ, _I, _F, _F, _P, _P, _P]
lib.fh_lsq_cell_run.argtypes = [C.c_char_p, _P, _P, _SZ, _I, _F, _I, _P, _P, _P]
lib.fh_lsq_act_run.argtypes = [C.c_char_p, _P, _P, _SZ, _I, _F, _I, _P, _P, _P]


lib.fh_cell_import_free_parameters.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_int]
lib.fh_cell_export_free_parameters.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p]
lib.fh_cell_get_free_parameters.argtypes = [C.c_void_p, C.c_char_p, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]
lib.fh_approximate_scaling_with_fixed_point.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p]
lib.fh_approximate_scaling_with_power_of_2_divs.argtypes = [C.c_float, C.c_int, C.c_void_p, C.c_void_p]
lib.fh_cell_approximate_activation_scaling.argtypes = [C.c_void_p, C.c_char_p, C.c_int]
lib.fh_cell_get_scaling.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]


class FrameHipError(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise FrameHipError(lib.fh_last_error().decode())


def set_globals(precision, unsigned_data, env_data_unsigned):
    """CellExport::mPrecision, DeepNetExport::mUnsignedData, DeepNetExport::mEnvDataUnsigned."""
    lib.fh_set_globals(int(precision), int(bool(unsigned_data)), int(bool(env_data_unsigned)))


_MODE = {"None": capi.SCALING_NONE, "FloatMult": capi.SCALING_FLOAT_MULT, "FixedMult16": capi.SCALING_FIXED_MULT16,
         "FixedMult32": capi.SCALING_FIXED_MULT32, "SingleShift": capi.SCALING_SINGLE_SHIFT, "DoubleShift": capi.SCALING_DOUBLE_SHIFT}
_MODE_DT = {"FloatMult": np.float32, "FixedMult16": np.int32, "FixedMult32": np.int32, "SingleShift": np.uint8, "DoubleShift": np.uint8}


_MODE_NAME = {v: k for k, v in _MODE.items()}


def approximate_scaling_with_fixed_point(mode, scaling_per_output):
    """DeepNetQuantization::approximateScalingWithFixedPoint -> (mode finally used, nbFractionalBits, int32 factors)."""
    sc = np.ascontiguousarray(scaling_per_output, dtype=np.float32)
    out = np.zeros(sc.size, dtype=np.int32)
    mode_out, bits = C.c_int(), C.c_int()
    _check(lib.fh_approximate_scaling_with_fixed_point(_MODE[mode], sc.ctypes.data, sc.size, C.byref(mode_out), C.byref(bits), out.ctypes.data))
    return _MODE_NAME[mode_out.value], bits.value, out


def approximate_scaling_with_power_of_2_divs(scaling, nb_divisions):
    """DeepNetQuantization::approximateScalingWithPowerOf2Divs -> (exponents, precision)."""
    exps = np.zeros(max(int(nb_divisions), 1), dtype=np.uint8)
    precision = C.c_double()
    _check(lib.fh_approximate_scaling_with_power_of_2_divs(float(scaling), int(nb_divisions), exps.ctypes.data, C.byref(precision)))
    return [int(e) for e in exps], precision.value


def get_nb_groups(mapping, with_regular=False):
    """Cell::getNbGroups of a connection map [nbOutputs, nbChannels] (non-zero: connected): the number of equal groups, or
    what the reference counts by hand for any other map (with_regular: also whether it was the former)."""
    m = np.asfortranarray(np.asarray(mapping) != 0, dtype=np.uint8)      # element (o, c) at o + nbOutputs * c
    groups, regular = C.c_long(), C.c_int()
    _check(lib.fh_get_nb_groups(m.ctypes.data, m.shape[0], m.shape[1], C.byref(groups), C.byref(regular)))
    return (groups.value, bool(regular.value)) if with_regular else groups.value


class Net:
    def __init__(self, ini_text):
        self.h = lib.fh_net_from_ini(ini_text.encode())
        if not self.h:
            raise FrameHipError(lib.fh_last_error().decode())

    def __del__(self):
        if getattr(self, "h", None) and lib is not None:
            lib.fh_net_free(self.h)
            self.h = None

    @property
    def model(self):
        return lib.fh_net_model(self.h).decode()

    @property
    def nb_cells(self):
        return lib.fh_net_nb_cells(self.h)

    def cell_info(self, name):
        dims = (C.c_int * 4)()
        uns = C.c_int()
        typ = C.create_string_buffer(32)
        _check(lib.fh_cell_info(self.h, name.encode(), dims, C.byref(uns), typ, 32))
        return {"W": dims[0], "H": dims[1], "C": dims[2], "B": dims[3], "unsigned": bool(uns.value), "type": typ.value.decode(),
                "halo": lib.fh_cell_outputs_halo(self.h, name.encode())}

    def set_quantized(self, name, nb_bits, act_nb_bits=0):
        _check(lib.fh_cell_set_quantized(self.h, name.encode(), int(nb_bits), int(act_nb_bits)))

    def set_weights(self, name, w, weight_bits=8):
        """w: [O, C/groups, kH, kW] (conv) or [O, K] (fc), integer-valued."""
        a = np.ascontiguousarray(w, dtype=np.float32)
        if a.ndim == 4:
            O, Cg, kH, kW = a.shape
        else:
            O, Cg, kH, kW = a.shape[0], a.shape[1], 1, 1
        _check(lib.fh_cell_set_weights(self.h, name.encode(), a.ctypes.data, a.size, kW, kH, Cg, O, int(weight_bits)))

    def set_mapping(self, name, mapping):
        """ConvCell::setMapping: the connection map [nbOutputs, nbChannels] decides the number of groups."""
        m = np.asfortranarray(np.asarray(mapping) != 0, dtype=np.uint8)
        _check(lib.fh_cell_set_mapping(self.h, name.encode(), m.ctypes.data, m.shape[0], m.shape[1]))

    def set_biases(self, name, b):
        a = np.ascontiguousarray(b, dtype=np.float32)
        _check(lib.fh_cell_set_biases(self.h, name.encode(), a.ctypes.data, a.size))

    def set_scaling(self, name, mode, scaling=None, frac_bits=0, clipping=None):
        if mode == "None":
            _check(lib.fh_cell_set_scaling(self.h, name.encode(), capi.SCALING_NONE, None, 0, 0, 0, None))
            return
        s = np.ascontiguousarray(scaling, dtype=_MODE_DT[mode])
        n = s.size // 2 if mode == "DoubleShift" else s.size
        cl = None if clipping is None else np.ascontiguousarray(clipping, dtype=np.float32)
        _check(lib.fh_cell_set_scaling(self.h, name.encode(), _MODE[mode], s.ctypes.data, n, int(frac_bits), int(cl is not None),
                                       None if cl is None else cl.ctypes.data))

    def save_quantization(self, dir_name):
        """DeepNet::saveQuantization: one "<cell>.quant" text file per cell (bit widths and Scaling)."""
        _check(lib.fh_net_save_quantization(self.h, str(dir_name).encode()))

    def load_quantization(self, dir_name):
        _check(lib.fh_net_load_quantization(self.h, str(dir_name).encode()))

    def import_free_parameters(self, name, file_name, ignore_not_exists=False):
        """Cell::importFreeParameters: "<base>_weights<.ext>" (+ "<base>_biases<.ext>"), or one file with both."""
        _check(lib.fh_cell_import_free_parameters(self.h, name.encode(), str(file_name).encode(), int(bool(ignore_not_exists))))

    def export_free_parameters(self, name, file_name):
        _check(lib.fh_cell_export_free_parameters(self.h, name.encode(), str(file_name).encode()))

    def _free_parameters(self, name, what):
        n = C.c_size_t()
        _check(lib.fh_cell_get_free_parameters(self.h, name.encode(), what, None, 0, C.byref(n)))
        out = np.zeros(n.value, dtype=np.float32)
        _check(lib.fh_cell_get_free_parameters(self.h, name.encode(), what, out.ctypes.data, out.size, C.byref(n)))
        return out

    def weights(self, name):
        """Flat float32 copy of the cell's weights, N2D2 order (conv: kernel x fastest, then y, channel, output)."""
        return self._free_parameters(name, 0)

    def biases(self, name):
        return self._free_parameters(name, 1)

    def approximate_activation_scaling(self, name, mode):
        """DeepNetQuantization::approximateActivationScaling on the cell's FLOAT_MULT activation scaling."""
        _check(lib.fh_cell_approximate_activation_scaling(self.h, name.encode(), _MODE[mode]))

    def scaling(self, name):
        """(mode, fractional bits, per-output values) of the cell's activation scaling."""
        mode, frac, n = C.c_int(), C.c_int(), C.c_size_t()
        _check(lib.fh_cell_get_scaling(self.h, name.encode(), C.byref(mode), C.byref(frac), None, 0, C.byref(n)))
        out = np.zeros(n.value, dtype=np.float64)
        _check(lib.fh_cell_get_scaling(self.h, name.encode(), C.byref(mode), C.byref(frac), out.ctypes.data, out.size, C.byref(n)))
        return _MODE_NAME[mode.value], frac.value, out

    def clipping(self, name):
        """Per-output clipping of the cell's activation scaling, or None when it does not clip."""
        flag, n = C.c_int(), C.c_size_t()
        _check(lib.fh_cell_get_clipping(self.h, name.encode(), C.byref(flag), None, 0, C.byref(n)))
        out = np.zeros(n.value, dtype=np.float32)
        _check(lib.fh_cell_get_clipping(self.h, name.encode(), C.byref(flag), out.ctypes.data, out.size, C.byref(n)))
        return out if flag.value else None

    def quantized(self, name):
        """(bits of the cell, bits of its activation, activation type)."""
        cb, ab = C.c_int(), C.c_int()
        buf = C.create_string_buffer(32)
        _check(lib.fh_cell_get_quantized(self.h, name.encode(), C.byref(cb), C.byref(ab), buf, 32))
        return cb.value, ab.value, buf.value.decode()

    def fuse_batchnorm_with_conv(self, name, ranges, alphas, quant_weights, biases, weights_range, default_mode, bn_scales, bn_biases,
                                 bn_means, bn_variances, epsilon, act_range, act_alpha, mode="FloatMult", w_round=True, b_round=True,
                                 c_round=True):
        """DeepNetQAT::QuantizeAndfuseBatchNormWithConv into the Conv cell `name`.  quant_weights [O, C/groups, kH, kW];
        biases None for NoBias; weights_range None without weight quantizer; act_range None when the BatchNorm's activation
        has no SAT quantizer.  Returns (fused, ranges, alphas) with the pairs as the call leaves them."""
        w = np.ascontiguousarray(quant_weights, dtype=np.float32)
        O, Cg, kH, kW = w.shape
        b = None if biases is None else np.ascontiguousarray(biases, dtype=np.float32)
        bn = [np.ascontiguousarray(v, dtype=np.float64) for v in (bn_scales, bn_biases, bn_means, bn_variances)]
        r = (C.c_size_t * 2)(*[int(v) for v in ranges])
        a = (C.c_double * 2)(*[float(v) for v in alphas])
        fused = C.c_int()
        _check(lib.fh_qat_fuse_batchnorm_with_conv(self.h, name.encode(), r, a, w.ctypes.data, kW, kH, Cg, O, None if b is None else b.ctypes.data,
                                                   int(weights_range or 0), int(bool(default_mode)), bn[0].ctypes.data, bn[1].ctypes.data,
                                                   bn[2].ctypes.data, bn[3].ctypes.data, float(epsilon), int(act_range or 0), float(act_alpha or 0.0),
                                                   _MODE[mode], int(w_round), int(b_round), int(c_round), C.byref(fused)))
        return bool(fused.value), (r[0], r[1]), (a[0], a[1])

    def quantize_fc(self, name, ranges, alphas, quant_weights, biases, weights_range, sat_scaling, act_range, act_alpha, w_round=True,
                    b_round=True, c_round=True):
        """DeepNetQAT::QuantizeFC into the Fc cell `name`.  quant_weights [O, K].  Returns (ranges, alphas)."""
        w = np.ascontiguousarray(quant_weights, dtype=np.float32)
        O, K = w.shape
        b = None if biases is None else np.ascontiguousarray(biases, dtype=np.float32)
        r = (C.c_size_t * 2)(*[int(v) for v in ranges])
        a = (C.c_double * 2)(*[float(v) for v in alphas])
        _check(lib.fh_qat_quantize_fc(self.h, name.encode(), r, a, w.ctypes.data, K, O, None if b is None else b.ctypes.data, int(weights_range or 0),
                                      float(sat_scaling), int(act_range or 0), float(act_alpha or 0.0), int(w_round), int(b_round), int(c_round)))
        return (r[0], r[1]), (a[0], a[1])

    def quantize_elemwise(self, name, ranges, alphas, range_parent0, alpha_parent0, act_range, act_alpha):
        """DeepNetQAT::QuantizeElemWise on the ElemWise cell `name`.  Returns (ranges, alphas)."""
        r = (C.c_size_t * 2)(*[int(v) for v in ranges])
        a = (C.c_double * 2)(*[float(v) for v in alphas])
        _check(lib.fh_qat_quantize_elemwise(self.h, name.encode(), r, a, int(range_parent0), float(alpha_parent0), int(act_range or 0),
                                            float(act_alpha or 0.0)))
        return (r[0], r[1]), (a[0], a[1])

    def initialize(self):
        _check(lib.fh_net_initialize(self.h))

    def set_fusion(self, enabled):
        """DeepNet::setFusion: cells folded into their consumer are not launched and their outputs not written."""
        _check(lib.fh_net_set_fusion(self.h, int(bool(enabled))))

    @property
    def nb_folded(self):
        return lib.fh_net_nb_folded(self.h)

    @property
    def nb_halo(self):
        """Cells whose output is stored with a border of zeros for the convolutions that read it."""
        return lib.fh_net_nb_halo(self.h)

    def set_stimuli(self, x):
        a = np.ascontiguousarray(x, dtype=np.float32)
        B, Cc, H, W = a.shape
        _check(lib.fh_net_set_stimuli(self.h, a.ctypes.data, Cc, H, W, B))

    def propagate(self):
        _check(lib.fh_net_propagate(self.h))

    def max_output(self, name, batch_pos=0):
        """Cell_Frame<T>::getMaxOutput: index of the largest output of one batch item, the first on a tie."""
        v = C.c_uint(0)
        _check(lib.fh_cell_get_max_output(self.h, name.encode(), batch_pos, C.byref(v)))
        return v.value

    def back_propagate(self, name):
        """Raises: the integer cells have no learning pass."""
        _check(lib.fh_cell_learn_step(self.h, name.encode(), 0))

    def update(self, name):
        """Raises: the integer cells have no learning pass."""
        _check(lib.fh_cell_learn_step(self.h, name.encode(), 1))

    def check_gradient(self, name):
        """Raises: the integer cells have no gradient."""
        _check(lib.fh_cell_learn_step(self.h, name.encode(), 2))

    def replace_input(self, name, old_parent, new_parent):
        """Cell_Frame<T>::replaceInput: `name` reads the output of `new_parent` where it read that of `old_parent`."""
        _check(lib.fh_cell_replace_input(self.h, name.encode(), old_parent.encode(), new_parent.encode()))

    def outputs(self, name):
        """Outputs of a cell as N2D2 exposes them: float32 [B, C, H, W] holding integer values."""
        i = self.cell_info(name)
        out = np.empty((i["B"], i["C"], i["H"], i["W"]), dtype=np.float32)
        _check(lib.fh_cell_get_outputs(self.h, name.encode(), out.ctypes.data, out.size))
        return out


def spec_to_ini(spec, batch, model="Frame_HIP"):
    """N2D2 INI text of a nets.NetSpec (the structural part; parameters are installed afterwards)."""
    C_, H, W = spec.in_shape
    lines = ["DefaultModel=%s" % model, "", "[sp]", "SizeX=%d" % W, "SizeY=%d" % H, "NbChannels=%d" % C_, "BatchSize=%d" % batch, ""]
    for l in spec.layers:
        ins = ",".join("sp" if i == "input" else i for i in l.inputs)
        lines += ["[%s]" % l.name, "Input=%s" % ins]
        if l.type == "conv":
            O, Cg, kH, kW = l.w.shape
            lines += ["Type=Conv", "KernelDims=%d %d" % (kW, kH), "NbOutputs=%d" % O, "StrideDims=%d %d" % l.stride,
                      "PaddingDims=%d %d" % (l.pad[0], l.pad[1]), "DilationDims=%d %d" % l.dil, "ActivationFunction=%s" % l.act.kind,
                      "NoBias=%d" % (l.bias is None)]
            if l.groups > 1:
                lines.append("Mapping.NbGroups=%d" % l.groups)
            if tuple(getattr(l, "sub", (1, 1))) != (1, 1):
                lines.append("SubSampleDims=%d %d" % tuple(l.sub))
        elif l.type == "fc":
            lines += ["Type=Fc", "NbOutputs=%d" % l.w.shape[0], "ActivationFunction=%s" % l.act.kind]
        elif l.type == "pool":
            lines += ["Type=Pool"]
            if len(l.inputs) == 1:
                lines += ["Mapping.ChannelsPerGroup=1"]
            else:       # one output per channel of every input: a diagonal per parent, starting at the parent's first channel
                first = 0
                for i in l.inputs:
                    n = spec.shapes[i][0]
                    lines += ["Mapping(%s).OffsetX=%d" % (i, first), "Mapping(%s).NbIterations=%d" % (i, n)]
                    first += n
            lines += ["PoolDims=%d %d" % l.pool, "NbOutputs=%d" % l.out_shape[0], "StrideDims=%d %d" % l.stride,
                      "PaddingDims=%d %d" % l.pad, "Pooling=%s" % ("Max" if l.kind == "max" else "Average")]
        elif l.type == "elemwise":
            lines += ["Type=ElemWise", "NbOutputs=%d" % l.out_shape[0], "Operation=Sum", "ActivationFunction=%s" % l.act.kind]
            if l.weights is not None:
                lines += ["CoeffMode=%s" % l.coeff_mode, "Weights=" + " ".join("%g" % v for v in l.weights),
                          "Shifts=" + " ".join("%g" % v for v in l.shifts)]
        elif l.type == "scaling":
            lines += ["Type=Scaling", "NbOutputs=%d" % l.out_shape[0]]
        lines.append("")
    return "\n".join(lines)


def build_net(spec, batch, model="Frame_HIP"):
    """Instantiates a nets.NetSpec on the C++ Frame_HIP cells: INI -> Registrar -> cells, then parameters."""
    net = Net(spec_to_ini(spec, batch, model))
    install_parameters(net, spec)
    return net


def install_parameters(net, spec):
    """Weights, biases, quantization flags and rescales of a nets.NetSpec, as N2D2's quantization pass leaves them."""
    for l in spec.layers:
        if l.type in ("conv", "fc"):
            net.set_weights(l.name, l.w, getattr(l, "weight_bits", 8))
            if l.bias is not None:
                net.set_biases(l.name, l.bias)
        if l.type in ("conv", "fc", "elemwise", "scaling"):
            a = l.act
            net.set_quantized(l.name, 8, a.nb_bits)
            if l.type == "scaling":
                net.set_quantized(l.name, a.nb_bits)
            net.set_scaling(l.name, a.mode, a.scaling, a.frac_bits, a.clipping)
        elif l.type == "pool":
            net.set_quantized(l.name, 8)
    return net


# ------------------------------------------------------------------ float cells for quantization-aware training
lib.fh_train_last_error.restype = C.c_char_p
lib.fh_train_registrar_exists.argtypes = [C.c_char_p, C.c_char_p]
lib.fh_train_net_create.argtypes = [C.c_char_p, _P, _I, _I, _I, _I, _I, _P]
lib.fh_train_net_destroy.argtypes = [_P]
lib.fh_train_net_destroy.restype = None
lib.fh_train_add_activation_cell.argtypes = [_P, C.c_char_p, _I, _I, _I, _F]
lib.fh_train_add_conv.argtypes = [_P, C.c_char_p, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _I, _I, _I, _F, _I, _I, _I, _I, _I]
lib.fh_train_add_softmax.argtypes = [_P, C.c_char_p, _I]
lib.fh_train_set_next_inputs.argtypes = [_P, C.c_char_p]
lib.fh_train_add_elemwise.argtypes = [_P, C.c_char_p, _P, _P, _I, _I, _I, _I, C.c_float]
lib.fh_train_add_batchnorm.argtypes = [_P, C.c_char_p, _P, C.c_double, C.c_double, _I, _I, _I, _F]
lib.fh_train_get_batchnorm.argtypes = [_P, C.c_char_p, _I, _P, _SZ]
lib.fh_train_add_pool.argtypes = [_P, C.c_char_p, _I, _I, _I, _I, _I, _I, _I]
lib.fh_net_deepnet.argtypes = [_P]
lib.fh_net_deepnet.restype = C.c_void_p
lib.fh_train_fuse_into.argtypes = [_P, _P, _I, _I, _I, _I, _P]
lib.fh_train_add_fc.argtypes = [_P, C.c_char_p, _I, _P, _P, _I, _I, _I, _F, _I, _I, _I]
lib.fh_train_set_solver_parameter.argtypes = [_P, C.c_char_p, C.c_char_p, C.c_double]
lib.fh_train_learn.argtypes = [_P, _P, _SZ, _I, _P]
lib.fh_train_propagate.argtypes = [_P, _I]
lib.fh_train_get.argtypes = [_P, C.c_char_p, _I, _P, _SZ]
lib.fh_train_input_gradient.argtypes = [_P, _P, _SZ]
lib.fh_train_preset_input_gradient.argtypes = [_P, _P, _SZ]
lib.fh_train_get_activation_quantizer.argtypes = [_P, C.c_char_p, _P, _P]
lib.fh_train_get_weight_quantizer.argtypes = [_P, C.c_char_p, _P, _P]

TRAIN_MODEL = "Frame_HIP_QAT"
_ACT = {None: -1, "Linear": 0, "Rectifier": 1}
_QUANT = {None: 0, "SAT": 1, "LSQ": 2}
_QUANT_MODE = {"Default": 0, "Symmetric": 1, "Asymmetric": 2, "FullRange": 3}


def _check_train(rc):
    if rc != 0:
        raise FrameHipError(lib.fh_train_last_error().decode())


class TrainNet:
    """A sequential net of the float Frame_HIP cells (ActivationCell, ConvCell, FcCell, BatchNormCell, PoolCell, SoftmaxCell) with SAT / LSQ quantizers,
    created through the Registrar under `model`. x: float32 [B,C,H,W]."""

    def __init__(self, x, model=TRAIN_MODEL, propagate_gradient=True):
        x = np.ascontiguousarray(x, dtype=np.float32)
        self._h = C.c_void_p()
        self._shapes = {}
        self._last = x.shape
        _check_train(lib.fh_train_net_create(model.encode(), x.ctypes.data, x.shape[0], x.shape[1], x.shape[2], x.shape[3],
                                             int(propagate_gradient), C.byref(self._h)))
        self.input_shape = x.shape

    def __del__(self):
        if getattr(self, "_h", None):
            lib.fh_train_net_destroy(self._h)
            self._h = None

    def add_activation_cell(self, name, act="Linear", act_quant=None, act_range=255, act_param=1.0):
        _check_train(lib.fh_train_add_activation_cell(self._h, name.encode(), _ACT[act], _QUANT[act_quant], act_range, act_param))
        self._shapes[name] = self._last

    def add_conv(self, name, weights, bias=None, stride=(1, 1), pad=(0, 0), depthwise=False, act=None, act_quant=None, act_range=255,
                 act_param=1.0, weight_quant=None, weight_range=255, apply_quantization=True, apply_scaling=False, quant_mode="Default"):
        """weights: [O, C/groups, kH, kW]; stride / pad are (x, y)."""
        w = np.ascontiguousarray(weights, dtype=np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        O, _, kH, kW = w.shape
        _check_train(lib.fh_train_add_conv(self._h, name.encode(), O, kW, kH, stride[0], stride[1], pad[0], pad[1], int(depthwise),
                                           w.ctypes.data, None if b is None else b.ctypes.data, _ACT[act], _QUANT[act_quant], act_range,
                                           act_param, _QUANT[weight_quant], weight_range, int(apply_quantization), int(apply_scaling),
                                           _QUANT_MODE[quant_mode]))
        B, _, H, W = self._last
        oH = (H + 2 * pad[1] - kH + stride[1]) // stride[1]
        oW = (W + 2 * pad[0] - kW + stride[0]) // stride[0]
        self._last = (B, O, oH, oW)
        self._shapes[name] = self._last
        self._shapes[name + "/weights"] = w.shape

    def add_fc(self, name, weights, bias=None, act=None, act_quant=None, act_range=255, act_param=1.0, weight_quant=None,
               weight_range=255, apply_scaling=False):
        """weights: [O, C*H*W] (CHW order); apply_scaling: the SAT weight quantizer's ApplyScaling."""
        w = np.ascontiguousarray(weights, dtype=np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        _check_train(lib.fh_train_add_fc(self._h, name.encode(), w.shape[0], w.ctypes.data, None if b is None else b.ctypes.data,
                                         _ACT[act], _QUANT[act_quant], act_range, act_param, _QUANT[weight_quant], weight_range,
                                         int(apply_scaling)))
        self._last = (self._last[0], w.shape[0], 1, 1)
        self._shapes[name] = self._last
        self._shapes[name + "/weights"] = w.shape

    def add_batchnorm(self, name, scales=None, biases=None, means=None, variances=None, epsilon=1.0e-5, moving_average_momentum=0.1,
                      act=None, act_quant=None, act_range=255, act_param=1.0):
        """BatchNormCell after the last cell; all four parameter vectors or none (then 1, 0, 0, 0)."""
        params = None
        if scales is not None:
            params = np.ascontiguousarray(np.stack([np.asarray(v, dtype=np.float32) for v in (scales, biases, means, variances)]))
            if params.shape != (4, self._last[1]):
                raise ValueError("one value per channel expected")
        _check_train(lib.fh_train_add_batchnorm(self._h, name.encode(), None if params is None else params.ctypes.data, float(epsilon),
                                                float(moving_average_momentum), _ACT[act], _QUANT[act_quant], int(act_range), float(act_param)))
        self._shapes[name] = self._last

    def batchnorm(self, name):
        """dict of the cell's scales, biases, running means and variances, and the last gradients of scales and biases."""
        out = {}
        for k, what in (("scales", 0), ("biases", 1), ("means", 2), ("variances", 3), ("diff_scales", 4), ("diff_biases", 5)):
            v = np.empty(self._shapes[name][1], dtype=np.float32)
            _check_train(lib.fh_train_get_batchnorm(self._h, name.encode(), what, v.ctypes.data, v.size))
            out[k] = v
        return out

    def add_pool(self, name, pool, stride, pad=(0, 0), pooling="Max"):
        """Max or Average pooling, one output per channel; pool / stride / pad as (x, y)."""
        _check_train(lib.fh_train_add_pool(self._h, name.encode(), int(pool[0]), int(pool[1]), int(stride[0]), int(stride[1]), int(pad[0]),
                                           int(pad[1]), {"Max": 0, "Average": 1}[pooling]))
        B, Cn, H, W = self._last
        oH = int((H + 2 * pad[1] - pool[1] + stride[1]) / float(stride[1]))
        oW = int((W + 2 * pad[0] - pool[0] + stride[0]) / float(stride[0]))
        self._last = (B, Cn, oH, oW)
        self._shapes[name] = self._last

    def add_softmax(self, name, with_loss=True):
        _check_train(lib.fh_train_add_softmax(self._h, name.encode(), int(with_loss)))
        self._shapes[name] = self._last

    def read_from(self, *cells):
        """The cell added next reads these cells (in this order) instead of the cell added last: branches of a learning graph.
        Cells are added in an order in which every cell follows the cells it reads."""
        _check_train(lib.fh_train_set_next_inputs(self._h, ",".join(cells).encode()))
        self._last = self._shapes[cells[0]]

    def add_elemwise(self, name, inputs, weights=None, shifts=None, act=None, act_quant=None, act_range=255, act_param=1.0):
        """ElemWise Sum of the named cells' outputs, (w0 x0 + s0) + (w1 x1 + s1) + ... (weights 1 and shifts 0 by default)."""
        self.read_from(*inputs)
        w = None if weights is None else np.ascontiguousarray(weights, dtype=np.float32)
        sh = None if shifts is None else np.ascontiguousarray(shifts, dtype=np.float32)
        n = 0 if w is None and sh is None else len(inputs)
        if w is None and sh is not None:
            w = np.ones(n, dtype=np.float32)
        if sh is None and w is not None:
            sh = np.zeros(n, dtype=np.float32)
        _check_train(lib.fh_train_add_elemwise(self._h, name.encode(), None if w is None else w.ctypes.data, None if sh is None else sh.ctypes.data,
                                               n, _ACT[act], _QUANT[act_quant], int(act_range), float(act_param)))
        self._shapes[name] = self._last

    def fuse_into(self, net, mode="FloatMult", w_round=True, b_round=True, c_round=True):
        """The chain case of DeepNetQAT::fuseQATGraph: fills the integer Conv / Fc cells of `net` (a Net of Frame_HIP cells with
        the same cell names) from this net's trained cells, each Conv with the BatchNorm that follows it.  The learning cells
        must have propagated once.  Returns the number of integer cells filled."""
        count = C.c_int(0)
        _check_train(lib.fh_train_fuse_into(self._h, lib.fh_net_deepnet(net.h), _MODE[mode], int(w_round), int(b_round), int(c_round),
                                            C.byref(count)))
        return count.value

    def set_solver_parameter(self, cell, name, value):
        _check_train(lib.fh_train_set_solver_parameter(self._h, cell.encode(), name.encode(), float(value)))

    def learn(self, targets, iterations=1):
        """Runs learning iterations (propagate, loss against `targets`, backPropagate, update); returns the last loss."""
        t = np.ascontiguousarray(targets, dtype=np.float32)
        loss = C.c_double(0.0)
        _check_train(lib.fh_train_learn(self._h, t.ctypes.data, t.size, iterations, C.byref(loss)))
        return loss.value

    def propagate(self, inference=True):
        _check_train(lib.fh_train_propagate(self._h, int(inference)))

    def _get(self, cell, what, shape):
        out = np.empty(shape, dtype=np.float32)
        _check_train(lib.fh_train_get(self._h, cell.encode(), what, out.ctypes.data, out.size))
        return out

    def outputs(self, cell):
        return self._get(cell, 0, self._shapes[cell])

    def diff_inputs(self, cell):
        return self._get(cell, 1, self._shapes[cell])

    def weights(self, cell):
        return self._get(cell, 2, self._shapes[cell + "/weights"])

    def diff_weights(self, cell):
        return self._get(cell, 3, self._shapes[cell + "/weights"])

    def quantized_weights(self, cell):
        return self._get(cell, 4, self._shapes[cell + "/weights"])

    def preset_input_gradient(self, values):
        """What another consumer of the net's input is taken to have written to its gradient before this net's first cell
        runs its backPropagate() (that cell must add to it)."""
        v = np.ascontiguousarray(values, dtype=np.float32)
        _check_train(lib.fh_train_preset_input_gradient(self._h, v.ctypes.data, v.size))

    def input_gradient(self):
        out = np.empty(self.input_shape, dtype=np.float32)
        _check_train(lib.fh_train_input_gradient(self._h, out.ctypes.data, out.size))
        return out

    def activation_quantizer(self, cell):
        """(learned parameter, its last gradient): SAT alpha or LSQ step size."""
        v, g = C.c_float(0), C.c_float(0)
        _check_train(lib.fh_train_get_activation_quantizer(self._h, cell.encode(), C.byref(v), C.byref(g)))
        return v.value, g.value

    def weight_quantizer(self, cell):
        """(LSQ step size of the cell's weight quantizer, its last gradient)."""
        v, g = C.c_float(0), C.c_float(0)
        _check_train(lib.fh_train_get_weight_quantizer(self._h, cell.encode(), C.byref(v), C.byref(g)))
        return v.value, g.value
