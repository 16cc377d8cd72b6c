"""ctypes binding of include/n2d2hip.h, one Python function per C entry point.

This is the binding the test-suite and the benchmark go through; it adds no
arithmetic of its own.  Loading fails loudly when the HIP library has not been
built (python -m n2d2_amd.build): there is no CPU fallback.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("N2D2HIP_LIB") or os.path.join(_HERE, "lib", "libn2d2hip.so")

# enums of n2d2hip.h
U8, I8, I32, F32, U8B = 0, 1, 2, 3, 4
NCHW, NHWC, S2D = 0, 1, 2
SCALING_NONE, SCALING_FLOAT_MULT, SCALING_FIXED_MULT16, SCALING_FIXED_MULT32, SCALING_SINGLE_SHIFT, SCALING_DOUBLE_SHIFT = range(6)
ACT_LINEAR, ACT_RECTIFIER = 0, 1
POOL_MAX, POOL_AVERAGE = 0, 1
COEFF_PER_LAYER, COEFF_PER_INPUT, COEFF_PER_CHANNEL = 0, 1, 2
SAT_NONE, SAT_DEFAULT, SAT_FULLRANGE, SAT_SYMRANGE, SAT_ASYMRANGE, SAT_NONE_ASYM = range(6)
OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_HIP, ERR_NOT_QUANTIZED, ERR_WORKSPACE = range(6)
# n2d2hip_conv_desc.kernel_choice bits
KERNEL_NO_PIPE, KERNEL_NO_STEM, KERNEL_NO_HI16, KERNEL_NO_SUM16, KERNEL_TILE_M64, KERNEL_TILE_M128, KERNEL_F32_DIRECT, KERNEL_F32_GEMM = (
    1, 2, 4, 8, 16, 32, 64, 128)
KERNEL_NO_PATCH, KERNEL_PATCH, KERNEL_NO_DIRECT, KERNEL_DIRECT, KERNEL_TILE_M256 = 256, 512, 1024, 2048, 4096

# every symbol include/n2d2hip.h declares
SYMBOLS = [
    "n2d2hip_strerror", "n2d2hip_last_error", "n2d2hip_version", "n2d2hip_measure_clock",
    "n2d2hip_launch_log_begin", "n2d2hip_launch_log_end", "n2d2hip_launch_log_entry", "n2d2hip_nhwc_cs", "n2d2hip_tensor_bytes", "n2d2hip_tensor_clear",
    "n2d2hip_convert", "n2d2hip_act_create", "n2d2hip_act_destroy", "n2d2hip_scaling_forward",
    "n2d2hip_conv_create", "n2d2hip_conv_destroy", "n2d2hip_conv_out_dims", "n2d2hip_conv_forward", "n2d2hip_conv_s2d_halo", "n2d2hip_conv_accepts_halo", "n2d2hip_conv_desc_reads_halo",
    "n2d2hip_conv_fuse_sum", "n2d2hip_conv_forward_sum", "n2d2hip_conv_chain_supported", "n2d2hip_conv_chain_forward", "n2d2hip_bottleneck_create", "n2d2hip_bottleneck_destroy", "n2d2hip_bottleneck_pays", "n2d2hip_bottleneck_forward",
    "n2d2hip_conv_accepts_maxpool", "n2d2hip_conv_forward_maxpool", 
    "n2d2hip_dw_pw_create", "n2d2hip_dw_pw_destroy", "n2d2hip_dw_pw_forward", "n2d2hip_dw_pw_pays",
    "n2d2hip_fc_create", "n2d2hip_fc_destroy", "n2d2hip_fc_forward", "n2d2hip_fc_chain_create", "n2d2hip_fc_chain_destroy", "n2d2hip_fc_chain_forward",
    "n2d2hip_pool_out_dims", "n2d2hip_pool_forward", "n2d2hip_pool_writes_halo", "n2d2hip_pool_forward_mapped",
    "n2d2hip_elemwise_create", "n2d2hip_elemwise_destroy", "n2d2hip_elemwise_forward", "n2d2hip_elemwise_fold_input_scaling", "n2d2hip_concat_channels",
    "n2d2hip_quantizer_workspace_bytes", "n2d2hip_sat_weight_forward", "n2d2hip_sat_weight_forward_static", "n2d2hip_sat_weight_backward",
    "n2d2hip_sat_act_forward", "n2d2hip_sat_act_backward", "n2d2hip_lsq_forward", "n2d2hip_lsq_backward",
    "n2d2hip_conv2d_f32_forward", "n2d2hip_conv2d_f32_backward_data", "n2d2hip_conv2d_f32_backward_filter", "n2d2hip_conv2d_f32_workspace_bytes",
    "n2d2hip_conv2d_f32_backward_bias", "n2d2hip_softmax_f32_forward", "n2d2hip_loss_workspace_bytes", "n2d2hip_loss_f32",
    "n2d2hip_sgd_update_f32", "n2d2hip_rectifier_f32_forward", "n2d2hip_rectifier_f32_backward",
    "n2d2hip_batchnorm_f32_workspace_bytes", "n2d2hip_batchnorm_f32_forward", "n2d2hip_batchnorm_f32_backward", "n2d2hip_pool_max_f32_forward", "n2d2hip_pool_max_f32_backward",
    "n2d2hip_pool_average_f32_forward", "n2d2hip_pool_average_f32_backward", "n2d2hip_elemwise_sum_f32_forward", "n2d2hip_elemwise_sum_f32_backward",
]


class Tensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int), ("layout", C.c_int),
                ("B", C.c_int), ("C", C.c_int), ("H", C.c_int), ("W", C.c_int), ("cs", C.c_int), ("halo", C.c_int)]


class Activation(C.Structure):
    _fields_ = [("kind", C.c_int), ("leak_slope", C.c_float), ("scaling_mode", C.c_int), ("scaling", C.c_void_p),
                ("frac_bits", C.c_int), ("is_clipped", C.c_int), ("clipping", C.c_void_p),
                ("nb_bits", C.c_int), ("unsigned_out", C.c_int)]


class ConvDesc(C.Structure):
    _fields_ = [("C", C.c_int), ("O", C.c_int), ("kW", C.c_int), ("kH", C.c_int), ("strideX", C.c_int), ("strideY", C.c_int),
                ("padL", C.c_int), ("padT", C.c_int), ("padR", C.c_int), ("padB", C.c_int), ("dilX", C.c_int), ("dilY", C.c_int),
                ("groups", C.c_int), ("weight_bits", C.c_int), ("kernel_choice", C.c_int), ("subX", C.c_int), ("subY", C.c_int)]


class PoolDesc(C.Structure):
    _fields_ = [("pooling", C.c_int), ("poolW", C.c_int), ("poolH", C.c_int), ("strideX", C.c_int), ("strideY", C.c_int),
                ("padX", C.c_int), ("padY", C.c_int)]


class N2D2HipError(RuntimeError):
    def __init__(self, status, message):
        RuntimeError.__init__(self, message)
        self.status = status


def load():
    if not os.path.exists(LIB_PATH):
        raise ImportError("libn2d2hip.so is not built (%s): run `python -m n2d2_amd.build`; "
                          "there is no CPU fallback for the Frame_HIP path" % LIB_PATH)
    # torch ships its own HIP runtime.  Loaded first, it is the one this library binds to, so that both see the same
    # device context and a torch tensor's data pointer is valid in the library's calls; the other order puts two runtimes
    # into the process and the second one then reports no device.
    import torch  # noqa: F401
    lib = C.CDLL(LIB_PATH)
    for name in ("n2d2hip_strerror", "n2d2hip_last_error", "n2d2hip_version"):
        getattr(lib, name).restype = C.c_char_p
    lib.n2d2hip_tensor_bytes.restype = C.c_size_t
    lib.n2d2hip_quantizer_workspace_bytes.restype = C.c_size_t
    lib.n2d2hip_quantizer_workspace_bytes.argtypes = [C.c_size_t]
    P, I, F, SZ, U = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_uint
    lib.n2d2hip_convert.argtypes = [P, P, P]
    lib.n2d2hip_measure_clock.argtypes = [C.c_double, P, P]
    lib.n2d2hip_launch_log_end.argtypes = [P]
    lib.n2d2hip_launch_log_entry.argtypes = [I, P, SZ, P, P, P]
    lib.n2d2hip_act_create.argtypes = [P, I, P]
    lib.n2d2hip_act_destroy.argtypes = [P]
    lib.n2d2hip_scaling_forward.argtypes = [P, P, P, P]
    lib.n2d2hip_conv_create.argtypes = [P, P, P, P, I, P]
    lib.n2d2hip_conv_destroy.argtypes = [P]
    lib.n2d2hip_conv_out_dims.argtypes = [P, I, I, P, P]
    lib.n2d2hip_conv_forward.argtypes = [P, P, P, P]
    lib.n2d2hip_conv_accepts_halo.argtypes = [P]
    lib.n2d2hip_conv_desc_reads_halo.argtypes = [P]
    lib.n2d2hip_conv_s2d_halo.argtypes = [P, P, I, I]
    lib.n2d2hip_tensor_clear.argtypes = [P, P]
    lib.n2d2hip_conv_fuse_sum.argtypes = [P, P, I, I]
    lib.n2d2hip_concat_channels.argtypes = [I, P, P, P]
    lib.n2d2hip_conv_forward_sum.argtypes = [P, P, P, P, P]
    lib.n2d2hip_conv_chain_supported.argtypes = [P, P]
    lib.n2d2hip_conv_chain_forward.argtypes = [P, P, P, P, P, P]
    lib.n2d2hip_bottleneck_create.argtypes = [P, P, P, P, P]
    lib.n2d2hip_bottleneck_destroy.argtypes = [P]
    lib.n2d2hip_bottleneck_pays.argtypes = [P, I, I, I]
    lib.n2d2hip_bottleneck_forward.argtypes = [P, P, P, P]
    lib.n2d2hip_conv_accepts_maxpool.argtypes = [P, P, C.c_int, C.c_int]
    lib.n2d2hip_conv_forward_maxpool.argtypes = [P, P, P, P, P]
    lib.n2d2hip_dw_pw_create.argtypes = [P, P, P]
    lib.n2d2hip_dw_pw_destroy.argtypes = [P]
    lib.n2d2hip_dw_pw_forward.argtypes = [P, P, P, P]
    lib.n2d2hip_dw_pw_pays.argtypes = [P, C.c_int, C.c_int, C.c_int]
    lib.n2d2hip_fc_create.argtypes = [I, I, I, I, I, P, P, P, I, P]
    lib.n2d2hip_fc_destroy.argtypes = [P]
    lib.n2d2hip_fc_forward.argtypes = [P, P, P, P]
    lib.n2d2hip_fc_chain_create.argtypes = [I, P, P]
    lib.n2d2hip_fc_chain_destroy.argtypes = [P]
    lib.n2d2hip_fc_chain_forward.argtypes = [P, P, P, P]
    lib.n2d2hip_pool_out_dims.argtypes = [P, I, I, P, P]
    lib.n2d2hip_pool_forward.argtypes = [P, P, P, P]
    lib.n2d2hip_pool_writes_halo.argtypes = [P, I, I, I]
    lib.n2d2hip_pool_forward_mapped.argtypes = [P, P, I, I, P, P, P]
    lib.n2d2hip_elemwise_create.argtypes = [I, I, I, P, P, P, P]
    lib.n2d2hip_elemwise_destroy.argtypes = [P]
    lib.n2d2hip_elemwise_fold_input_scaling.argtypes = [P, I, P]
    lib.n2d2hip_elemwise_forward.argtypes = [P, P, P, P]
    lib.n2d2hip_sat_weight_forward.argtypes = [P, P, SZ, F, I, I, U, P, P, SZ, P]
    lib.n2d2hip_sat_weight_forward_static.argtypes = [P, P, SZ, F, I, I, U, P, P]
    lib.n2d2hip_sat_weight_backward.argtypes = [P, P, P, SZ, F, I, I, P, P]
    lib.n2d2hip_sat_act_forward.argtypes = [P, P, SZ, F, P, P]
    lib.n2d2hip_sat_act_backward.argtypes = [P, P, P, SZ, F, P, F, P, P, SZ, P]
    lib.n2d2hip_lsq_forward.argtypes = [P, P, SZ, P, I, I, P]
    lib.n2d2hip_lsq_backward.argtypes = [P, P, P, SZ, P, I, I, F, F, P, P, SZ, P]
    lib.n2d2hip_conv2d_f32_forward.argtypes = [P, I, I, I, P, P, P, F, P, P, SZ, P]
    lib.n2d2hip_conv2d_f32_backward_data.argtypes = [P, I, I, I, P, P, F, P, P, SZ, P]
    lib.n2d2hip_conv2d_f32_backward_filter.argtypes = [P, I, I, I, P, P, F, P, P, SZ, P]
    lib.n2d2hip_conv2d_f32_workspace_bytes.restype = C.c_size_t
    lib.n2d2hip_conv2d_f32_workspace_bytes.argtypes = [P, I, I, I]
    lib.n2d2hip_conv2d_f32_backward_bias.argtypes = [I, I, I, I, P, F, P, P]
    lib.n2d2hip_softmax_f32_forward.argtypes = [P, P, I, I, I, I, P]
    lib.n2d2hip_loss_workspace_bytes.restype = C.c_size_t
    lib.n2d2hip_loss_workspace_bytes.argtypes = [SZ]
    lib.n2d2hip_loss_f32.argtypes = [P, P, P, SZ, I, P, P, SZ, P]
    lib.n2d2hip_sgd_update_f32.argtypes = [P, P, SZ, F, F, F, P, I, F, F, P]
    lib.n2d2hip_rectifier_f32_forward.argtypes = [P, SZ, F, F, P]
    lib.n2d2hip_rectifier_f32_backward.argtypes = [P, P, P, SZ, F, F, P]
    D = C.c_double
    lib.n2d2hip_batchnorm_f32_workspace_bytes.restype = C.c_size_t
    lib.n2d2hip_batchnorm_f32_workspace_bytes.argtypes = [I, I, I, I]
    lib.n2d2hip_batchnorm_f32_forward.argtypes = [I, I, I, I, P, P, P, P, P, P, P, D, D, I, P, P, SZ, P]
    lib.n2d2hip_batchnorm_f32_backward.argtypes = [I, I, I, I, P, P, P, P, D, P, F, P, F, P, P, P, P, P, SZ, P]
    lib.n2d2hip_pool_max_f32_forward.argtypes = [I, I, I, I, I, I, I, I, I, I, P, P, P, P]
    lib.n2d2hip_pool_max_f32_backward.argtypes = [I, I, I, I, I, I, I, I, I, I, P, P, F, P, P]
    lib.n2d2hip_pool_average_f32_forward.argtypes = [I, I, I, I, I, I, I, I, I, I, I, P, P, P]
    lib.n2d2hip_pool_average_f32_backward.argtypes = [I, I, I, I, I, I, I, I, I, I, I, P, F, P, P]
    lib.n2d2hip_elemwise_sum_f32_forward.argtypes = [I, C.POINTER(C.c_void_p), SZ, C.POINTER(C.c_float), C.POINTER(C.c_float), P, P]
    lib.n2d2hip_elemwise_sum_f32_backward.argtypes = [SZ, F, P, F, P, P]
    return lib


lib = load()


def check(status):
    if status != OK:
        msg = lib.n2d2hip_last_error().decode() or lib.n2d2hip_strerror(status).decode()
        raise N2D2HipError(status, msg)


class launch_log(object):
    """with capi.launch_log() as log: ...; log.entries is then [(kernel name, grid, block, first probe record or -1)] of
    the kernels the library launched from this thread inside the block."""

    def __enter__(self):
        self.entries = []
        check(lib.n2d2hip_launch_log_begin())
        return self

    def __exit__(self, *exc):
        n = C.c_int(0)
        check(lib.n2d2hip_launch_log_end(C.byref(n)))
        for i in range(n.value):
            name = C.create_string_buffer(256)
            grid, block, slot = C.c_int(0), C.c_int(0), C.c_longlong(-1)
            check(lib.n2d2hip_launch_log_entry(i, name, 256, C.byref(grid), C.byref(block), C.byref(slot)))
            self.entries.append((name.value.decode(), grid.value, block.value, slot.value))
        return False


def nhwc_cs(c):
    return int(lib.n2d2hip_nhwc_cs(int(c)))
