"""CPU-only checks of the drop-in boundary: the C-ABI library loads without a
GPU and exports every symbol include/n2d2hip.h declares; argument validation
that needs no device works."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "n2d2hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(n2d2hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from n2d2_amd import capi
    names = _declared()
    assert len(names) >= 25
    assert sorted(capi.SYMBOLS) == names          # the binding lists exactly the header's entry points
    for n in names:
        assert hasattr(capi.lib, n), n


def test_status_strings_and_host_only_helpers():
    from n2d2_amd import capi
    lib = capi.lib
    assert lib.n2d2hip_strerror(0) == b"success"
    assert b"quantized network" in lib.n2d2hip_strerror(capi.ERR_NOT_QUANTIZED)
    assert b"gfx950" in lib.n2d2hip_version()
    assert [capi.nhwc_cs(c) for c in (1, 3, 4, 6, 16, 17, 64, 1000)] == [4, 4, 4, 16, 16, 32, 64, 1008]
    # output-size formulas (ConvCell::setOutputsDims / PoolCell::setOutputsDims)
    oh, ow = C.c_int(), C.c_int()
    d = capi.ConvDesc(3, 64, 7, 7, 2, 2, 3, 3, 3, 3, 1, 1, 1, 8)
    assert lib.n2d2hip_conv_out_dims(C.byref(d), 224, 224, C.byref(oh), C.byref(ow)) == 0 and (oh.value, ow.value) == (112, 112)
    p = capi.PoolDesc(capi.POOL_MAX, 3, 3, 2, 2, 0, 0)
    assert lib.n2d2hip_pool_out_dims(C.byref(p), 112, 112, C.byref(oh), C.byref(ow)) == 0 and (oh.value, ow.value) == (55, 55)
    p = capi.PoolDesc(capi.POOL_MAX, 3, 3, 2, 2, 1, 1)
    assert lib.n2d2hip_pool_out_dims(C.byref(p), 112, 112, C.byref(oh), C.byref(ow)) == 0 and (oh.value, ow.value) == (56, 56)


def test_invalid_arguments_are_rejected_before_any_device_work():
    from n2d2_amd import capi
    lib = capi.lib
    h = C.c_void_p()
    assert lib.n2d2hip_act_create(None, 4, C.byref(h)) == capi.ERR_INVALID
    a = capi.Activation(capi.ACT_LINEAR, 0.0, capi.SCALING_SINGLE_SHIFT, None, 0, 0, None, 8, 0)
    assert lib.n2d2hip_act_create(C.byref(a), 4, C.byref(h)) == capi.ERR_INVALID          # null scaling vector
    assert b"null scaling" in lib.n2d2hip_last_error()
    shifts = (C.c_ubyte * 4)(1, 2, 3, 4)
    a = capi.Activation(capi.ACT_LINEAR, 0.0, capi.SCALING_SINGLE_SHIFT, C.cast(shifts, C.c_void_p), 0, 0, None, 0, 0)
    assert lib.n2d2hip_act_create(C.byref(a), 4, C.byref(h)) == capi.ERR_NOT_QUANTIZED   # the reference throws here
    assert b"SingleShiftScaling::propagate can only be used on quantized network." in lib.n2d2hip_last_error()
    a = capi.Activation(capi.ACT_LINEAR, 0.0, 9, None, 0, 0, None, 8, 0)
    assert lib.n2d2hip_act_create(C.byref(a), 4, C.byref(h)) == capi.ERR_INVALID
    assert b"Unsupported scaling propagation" in lib.n2d2hip_last_error()
    assert lib.n2d2hip_conv_forward(None, None, None, None) == capi.ERR_INVALID
    assert lib.n2d2hip_convert(None, None, None) == capi.ERR_INVALID


def test_tensors_with_a_border_are_sized_and_policed_on_the_host():
    """n2d2hip_tensor::halo: the byte count includes the border; entry points that do not take such tensors refuse them
    before any device work; malformed borders are invalid everywhere."""
    from n2d2_amd import capi
    lib = capi.lib
    fake = 0x1000                                                      # never dereferenced: validation comes first
    t = capi.Tensor(fake, capi.U8B, capi.NHWC, 2, 64, 5, 7, 64, 0)
    assert lib.n2d2hip_tensor_bytes(C.byref(t)) == 2 * 5 * 7 * 64
    th = capi.Tensor(fake, capi.U8B, capi.NHWC, 2, 64, 5, 7, 64, 2)
    assert lib.n2d2hip_tensor_bytes(C.byref(th)) == 2 * 9 * 11 * 64
    p = capi.PoolDesc(capi.POOL_MAX, 2, 2, 2, 2, 0, 0)
    out = capi.Tensor(fake, capi.U8B, capi.NHWC, 2, 64, 2, 3, 64, 0)
    assert lib.n2d2hip_pool_forward(C.byref(p), C.byref(th), C.byref(out), None) == capi.ERR_UNSUPPORTED
    assert b"halo" in lib.n2d2hip_last_error()
    assert lib.n2d2hip_convert(C.byref(t), C.byref(th), None) == capi.ERR_UNSUPPORTED          # conversion reads a border, never writes one
    bad = capi.Tensor(fake, capi.U8B, capi.NHWC, 2, 64, 5, 7, 64, -1)
    assert lib.n2d2hip_tensor_clear(C.byref(bad), None) == capi.ERR_INVALID
    nchw = capi.Tensor(fake, capi.I32, capi.NCHW, 2, 64, 5, 7, 64, 1)
    assert lib.n2d2hip_tensor_clear(C.byref(nchw), None) == capi.ERR_INVALID                   # only NHWC byte tensors have one
    assert lib.n2d2hip_conv_accepts_halo(None) == 0


def test_planning_questions_answered_from_descriptors_alone():
    """What a planner asks before any cell exists is answered on the host: which convolution shapes can read a tensor that
    carries its padding, which poolings can write one."""
    from n2d2_amd import capi
    lib = capi.lib

    def conv(C_, O, k, groups=1, bits=8, dil=1, choice=0):
        return capi.ConvDesc(C_, O, k, k, 1, 1, k // 2, k // 2, k // 2, k // 2, dil, dil, groups, bits, choice)
    ok = lambda d: lib.n2d2hip_conv_desc_reads_halo(C.byref(d))
    assert ok(conv(64, 64, 3)) == 1 and ok(conv(128, 256, 1)) == 1 and ok(conv(64, 64, 3, bits=4)) == 1 and ok(conv(64, 128, 5)) == 1
    assert ok(conv(64, 128, 3, groups=2)) == 1                              # groups other than depthwise run as a full connection
    assert ok(conv(3, 64, 7)) == 0 and ok(conv(96, 64, 3)) == 0             # input channels not a multiple of 64
    assert ok(conv(64, 64, 3, groups=64)) == 0                              # depthwise
    assert ok(conv(64, 64, 3, dil=2)) == 0 and ok(conv(64, 64, 7)) == 0     # dilation; more than 31 taps
    assert ok(conv(64, 4, 3)) == 0                                          # a pixel of at most 4 outputs
    assert ok(conv(64, 64, 3, choice=capi.KERNEL_NO_PIPE)) == 0
    sub = conv(64, 64, 3)
    sub.subX = 2
    assert ok(sub) == 0                                                     # a sub-sampled cell takes no bordered tensor
    assert lib.n2d2hip_conv_desc_reads_halo(None) == 0

    def pool(kind, k, stride, pad):
        return capi.PoolDesc(kind, k, k, stride, stride, pad, pad)
    wh = lambda d, H, W, cs: lib.n2d2hip_pool_writes_halo(C.byref(d), H, W, cs)
    assert wh(pool(capi.POOL_MAX, 3, 2, 1), 112, 112, 64) == 1 and wh(pool(capi.POOL_MAX, 2, 2, 0), 28, 28, 16) == 1
    assert wh(pool(capi.POOL_MAX, 3, 2, 1), 112, 112, 4) == 0               # channel stride of 4: the general kernel
    assert wh(pool(capi.POOL_AVERAGE, 2, 2, 0), 28, 28, 16) == 0 and wh(pool(capi.POOL_MAX, 5, 2, 0), 28, 28, 16) == 0
    assert wh(pool(capi.POOL_MAX, 3, 2, 3), 28, 28, 16) == 0                # padding as large as the window
    assert lib.n2d2hip_pool_writes_halo(None, 28, 28, 16) == 0
    assert lib.n2d2hip_bottleneck_pays(None, 128, 56, 56) == 0
