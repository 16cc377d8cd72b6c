"""GPU parity of the float32 training kernels (convolution forward / backward, rectifier, softmax, loss, SGD) against
the CPU oracle, through the C ABI.  Every convolution case runs on both device paths: the direct kernels, whose forward
and backward-data walk their sums in the reference's order and are compared to 1e-5 relative (in practice identical),
and the matrix-core implicit GEMM, which adds the same terms in another order.  Wherever the order differs (the GEMM
path, backward-filter and backward-bias on either path) the result is held to 1e-5 of the sum of the terms' magnitudes
against the float64 oracle, which is the bound the reference's own float32 running sum obeys with room to spare."""
import os

import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-5

CASES = [  # B, C, H, W, O, k, stride, pad, groups
    (2, 3, 7, 6, 4, 3, 1, 1, 1), (2, 4, 9, 9, 4, 3, 2, 1, 4), (1, 2, 5, 5, 3, 1, 1, 0, 1), (2, 3, 10, 9, 2, 5, 2, 2, 1),
    (2, 1, 5, 5, 1, 3, 1, 0, 1), (3, 5, 8, 8, 5, 3, 1, 1, 5), (1, 3, 9, 7, 2, 3, 3, 0, 1), (2, 2, 4, 4, 3, 2, 2, 0, 1),
    (4, 16, 14, 14, 32, 3, 1, 1, 1), (2, 32, 12, 12, 32, 3, 2, 1, 32), (3, 24, 10, 10, 8, 1, 1, 0, 1), (2, 8, 17, 13, 16, 7, 2, 3, 1),
    (5, 70, 19, 23, 150, 3, 1, 1, 1), (3, 130, 15, 15, 129, 3, 2, 0, 1), (9, 40, 30, 30, 200, 1, 1, 0, 1), (2, 3, 40, 40, 20, 5, 1, 2, 1),
    (6, 96, 7, 7, 160, 3, 1, 1, 1), (4, 200, 9, 9, 70, 3, 1, 1, 1)]     # small outputs, long sums: K ranges in every pass


@pytest.fixture(scope="module")
def g():
    import torch
    from n2d2_amd import capi as capi_, runtime

    class G:
        lib, check, sp, capi = capi_.lib, staticmethod(capi_.check), staticmethod(runtime.stream_ptr), capi_

        @staticmethod
        def dev(a):
            return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()

        @staticmethod
        def host(t):
            torch.cuda.synchronize()
            return t.cpu().numpy()

        @staticmethod
        def desc(C_, O, k, s, p, groups, dil=1, path=None):
            choice = {None: 0, "direct": capi_.KERNEL_F32_DIRECT, "gemm": capi_.KERNEL_F32_GEMM}[path]
            return capi_.ConvDesc(C_, O, k, k, s, s, p, p, p, p, dil, dil, groups, 0, choice)
        torch_ = torch
    return G


def _rel(got, want, scale=None):
    scale = np.maximum(np.abs(want), 1e-3) if scale is None else scale
    return float((np.abs(got.astype(np.float64) - want.astype(np.float64)) / scale).max())


@pytest.fixture(params=["direct", "gemm"])
def path(request):
    return request.param


@pytest.mark.parametrize("case", CASES)
def test_conv_forward_and_backward(g, case, path):
    from oracle import oracle as orc
    B, Cn, H, W, O, k, s, p, groups = case
    print("conv f32", path, case, flush=True)
    exact_order = path == "direct" or groups > 1
    rng = np.random.default_rng(sum(case))
    maps = None if groups == 1 else orc.group_maps(Cn, O, groups)
    kw = dict(stride=(s, s), pad=(p, p, p, p), maps=maps)
    x = rng.normal(size=(B, Cn, H, W)).astype(np.float32)
    w = rng.normal(size=(O, Cn // groups, k, k)).astype(np.float32)
    bias = rng.normal(size=O).astype(np.float32)
    want = orc.conv_forward_bias(orc.conv_forward(x, w, **kw), bias)
    d = g.desc(Cn, O, k, s, p, groups, path=path)
    dx_, dw_, db_ = g.dev(x), g.dev(w), g.dev(bias)
    y = g.torch_.empty(want.shape, dtype=g.torch_.float32, device="cuda")
    need = int(g.lib.n2d2hip_conv2d_f32_workspace_bytes(C.byref(d), B, H, W))
    assert (need > 0) == (path == "gemm" and groups == 1)
    ws = g.torch_.empty(max(need, 4), dtype=g.torch_.uint8, device="cuda")
    g.check(g.lib.n2d2hip_conv2d_f32_forward(C.byref(d), B, H, W, dx_.data_ptr(), dw_.data_ptr(), db_.data_ptr(), 0.0, y.data_ptr(),
                                             ws.data_ptr(), need, g.sp()))
    got = g.host(y)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    want64 = orc.conv_forward(x64, w64, **kw) + bias.astype(np.float64).reshape(1, -1, 1, 1)
    magy = np.maximum(orc.conv_forward(np.abs(x64), np.abs(w64), **kw) + np.abs(bias).reshape(1, -1, 1, 1), 1e-3)
    assert got.shape == want.shape
    assert _rel(got, want) <= TOL if exact_order else _rel(got, want64, magy) <= TOL
    # beta accumulates onto what the output held (second input tensor of a cell)
    # (without a workspace: one K range, same result up to the order of the sums)
    g.check(g.lib.n2d2hip_conv2d_f32_forward(C.byref(d), B, H, W, dx_.data_ptr(), dw_.data_ptr(), None, 1.0, y.data_ptr(), None, 0, g.sp()))
    want2 = orc.conv_forward(x, w, out=want.copy(), beta=1.0, **kw)
    assert _rel(g.host(y), want2) <= TOL if exact_order else _rel(g.host(y), 2 * want64 - bias.reshape(1, -1, 1, 1), 2 * magy) <= TOL

    dy = rng.normal(size=want.shape).astype(np.float32)
    ddy = g.dev(dy)
    wantdx = orc.conv_backward_data(w, dy, x.shape, **kw)
    gdx = g.torch_.empty(x.shape, dtype=g.torch_.float32, device="cuda")
    g.check(g.lib.n2d2hip_conv2d_f32_backward_data(C.byref(d), B, H, W, dw_.data_ptr(), ddy.data_ptr(), 0.0, gdx.data_ptr(), ws.data_ptr(), need, g.sp()))
    dy64 = dy.astype(np.float64)
    wantdx64 = orc.conv_backward_data(w64, dy64, x.shape, **kw)
    magdx = np.maximum(orc.conv_backward_data(np.abs(w64), np.abs(dy64), x.shape, **kw), 1e-3)
    assert _rel(g.host(gdx), wantdx) <= TOL if exact_order else _rel(g.host(gdx), wantdx64, magdx) <= TOL
    g.check(g.lib.n2d2hip_conv2d_f32_backward_data(C.byref(d), B, H, W, dw_.data_ptr(), ddy.data_ptr(), 1.0, gdx.data_ptr(), ws.data_ptr(), need, g.sp()))
    if exact_order:
        assert _rel(g.host(gdx), orc.conv_backward_data(w, dy, x.shape, dx=wantdx.copy(), beta=1.0, **kw)) <= TOL
    else:
        assert _rel(g.host(gdx), 2 * wantdx64, 2 * magdx) <= TOL

    wantdw = orc.conv_backward_filter(x64, dy64, w.shape, **kw)
    mag = orc.conv_backward_filter(np.abs(x64), np.abs(dy64), w.shape, **kw)
    gdw = g.torch_.empty(w.shape, dtype=g.torch_.float32, device="cuda")
    if need:
        assert g.lib.n2d2hip_conv2d_f32_backward_filter(C.byref(d), B, H, W, dx_.data_ptr(), ddy.data_ptr(), 0.0, gdw.data_ptr(),
                                                        ws.data_ptr(), 4, g.sp()) == g.capi.ERR_WORKSPACE
    g.check(g.lib.n2d2hip_conv2d_f32_backward_filter(C.byref(d), B, H, W, dx_.data_ptr(), ddy.data_ptr(), 0.0, gdw.data_ptr(),
                                                     ws.data_ptr(), need, g.sp()))
    got = g.host(gdw)
    assert _rel(got, wantdw, np.maximum(mag, 1e-3)) <= TOL
    # and the reference's own float32 running sum stays within the same bound of it
    assert _rel(orc.conv_backward_filter(x, dy, w.shape, **kw), wantdw, np.maximum(mag, 1e-3)) <= 5 * TOL
    g.check(g.lib.n2d2hip_conv2d_f32_backward_filter(C.byref(d), B, H, W, dx_.data_ptr(), ddy.data_ptr(), 1.0, gdw.data_ptr(),
                                                     ws.data_ptr(), need, g.sp()))
    assert _rel(g.host(gdw), 2 * wantdw, np.maximum(2 * mag, 1e-3)) <= TOL

    gdb = g.torch_.empty(O, dtype=g.torch_.float32, device="cuda")
    g.check(g.lib.n2d2hip_conv2d_f32_backward_bias(B, O, want.shape[2], want.shape[3], ddy.data_ptr(), 0.0, gdb.data_ptr(), g.sp()))
    assert _rel(g.host(gdb), orc.conv_backward_bias(dy64), np.maximum(np.abs(dy64).sum(axis=(0, 2, 3)), 1e-3)) <= TOL


def test_conv_f32_rejects_what_the_reference_cannot_do(g):
    x = g.dev(np.zeros((1, 6, 8, 8)))
    w = g.dev(np.zeros((4, 3, 3, 3)))
    y = g.dev(np.zeros((1, 4, 6, 6)))
    d = g.desc(6, 4, 3, 1, 0, 2)          # two groups of three channels: the reference's backward is not its adjoint
    assert g.lib.n2d2hip_conv2d_f32_forward(C.byref(d), 1, 8, 8, x.data_ptr(), w.data_ptr(), None, 0.0, y.data_ptr(), None, 0, g.sp()) == g.capi.ERR_UNSUPPORTED
    d = g.desc(6, 4, 3, 1, 0, 1, dil=2)    # backward with dilation: the reference does not read it
    assert g.lib.n2d2hip_conv2d_f32_backward_data(C.byref(d), 1, 8, 8, w.data_ptr(), y.data_ptr(), 0.0, x.data_ptr(), None, 0, g.sp()) == g.capi.ERR_UNSUPPORTED
    assert b"dilation" in g.lib.n2d2hip_last_error()
    d = g.desc(6, 4, 3, 1, 0, 1)
    assert g.lib.n2d2hip_conv2d_f32_forward(C.byref(d), 1, 8, 8, None, w.data_ptr(), None, 0.0, y.data_ptr(), None, 0, g.sp()) == g.capi.ERR_INVALID


def test_conv_f32_edge_shapes(g, path):
    """One pixel, one channel, batch 1; a kernel as large as the padded input (the FcCell case); a stride larger than
    the kernel; and shapes that leave no output."""
    from oracle import oracle as orc
    rng = np.random.default_rng(17)
    for (B, Cn, H, W, O, k, s, p) in [(1, 1, 1, 1, 1, 1, 1, 0), (3, 5, 4, 4, 7, 4, 1, 0), (2, 3, 6, 6, 4, 8, 1, 1), (2, 2, 11, 11, 3, 2, 4, 0)]:
        x = rng.normal(size=(B, Cn, H, W)).astype(np.float32)
        w = rng.normal(size=(O, Cn, k, k)).astype(np.float32)
        kw = dict(stride=(s, s), pad=(p, p, p, p))
        want = orc.conv_forward(x.astype(np.float64), w.astype(np.float64), **kw)
        mag = np.maximum(orc.conv_forward(np.abs(x).astype(np.float64), np.abs(w).astype(np.float64), **kw), 1e-3)
        d = g.desc(Cn, O, k, s, p, 1, path=path)
        dx_, dw_ = g.dev(x), g.dev(w)
        y = g.torch_.empty(want.shape, dtype=g.torch_.float32, device="cuda")
        need = int(g.lib.n2d2hip_conv2d_f32_workspace_bytes(C.byref(d), B, H, W))
        ws = g.torch_.empty(max(need, 4), dtype=g.torch_.uint8, device="cuda")
        g.check(g.lib.n2d2hip_conv2d_f32_forward(C.byref(d), B, H, W, dx_.data_ptr(), dw_.data_ptr(), None, 0.0, y.data_ptr(), ws.data_ptr(), need, g.sp()))
        assert _rel(g.host(y), want, mag) <= TOL, (B, Cn, H, W, O, k, s, p)
        dy = rng.normal(size=want.shape).astype(np.float32)
        ddy = g.dev(dy)
        gdx = g.torch_.empty(x.shape, dtype=g.torch_.float32, device="cuda")
        gdw = g.torch_.empty(w.shape, dtype=g.torch_.float32, device="cuda")
        g.check(g.lib.n2d2hip_conv2d_f32_backward_data(C.byref(d), B, H, W, dw_.data_ptr(), ddy.data_ptr(), 0.0, gdx.data_ptr(), ws.data_ptr(), need, g.sp()))
        g.check(g.lib.n2d2hip_conv2d_f32_backward_filter(C.byref(d), B, H, W, dx_.data_ptr(), ddy.data_ptr(), 0.0, gdw.data_ptr(), ws.data_ptr(), need, g.sp()))
        x64, w64, dy64 = x.astype(np.float64), w.astype(np.float64), dy.astype(np.float64)
        assert _rel(g.host(gdx), orc.conv_backward_data(w64, dy64, x.shape, **kw),
                    np.maximum(orc.conv_backward_data(np.abs(w64), np.abs(dy64), x.shape, **kw), 1e-3)) <= TOL
        assert _rel(g.host(gdw), orc.conv_backward_filter(x64, dy64, w.shape, **kw),
                    np.maximum(orc.conv_backward_filter(np.abs(x64), np.abs(dy64), w.shape, **kw), 1e-3)) <= TOL
    x, w, y = g.dev(np.zeros((1, 2, 3, 3))), g.dev(np.zeros((2, 2, 5, 5))), g.dev(np.zeros(8))
    d = g.desc(2, 2, 5, 1, 0, 1)           # 5x5 kernel on an unpadded 3x3 input: no output pixel
    assert g.lib.n2d2hip_conv2d_f32_forward(C.byref(d), 1, 3, 3, x.data_ptr(), w.data_ptr(), None, 0.0, y.data_ptr(), None, 0, g.sp()) == g.capi.ERR_INVALID
    d = g.desc(2, 2, 3, 0, 0, 1)           # stride 0
    assert g.lib.n2d2hip_conv2d_f32_forward(C.byref(d), 1, 3, 3, x.data_ptr(), w.data_ptr(), None, 0.0, y.data_ptr(), None, 0, g.sp()) == g.capi.ERR_INVALID
    d = g.desc(2, 2, 3, 1, 0, 1)
    assert g.lib.n2d2hip_conv2d_f32_forward(C.byref(d), 0, 3, 3, x.data_ptr(), w.data_ptr(), None, 0.0, y.data_ptr(), None, 0, g.sp()) == g.capi.ERR_INVALID


def test_conv_f32_random_rectangular_shapes(g, path):
    """Seeded random cases with different kernel extents, strides and the four paddings in x and y."""
    from oracle import oracle as orc
    rng = np.random.default_rng(2024)
    done = 0
    while done < 16:
        B, Cn, O = int(rng.integers(1, 5)), int(rng.integers(1, 40)), int(rng.integers(1, 150))
        H, W = int(rng.integers(3, 24)), int(rng.integers(3, 24))
        kW, kH = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        sx, sy = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        pl, pt, pr, pb = (int(v) for v in rng.integers(0, 3, size=4))
        oW, oH = (W + pl + pr - kW) // sx + 1, (H + pt + pb - kH) // sy + 1
        # the reference's output size uses one padding per axis on both sides; keep to shapes where the two agree, and
        # to windows that reach the input (the reference's clipped window and zero padding then coincide)
        if W + pl + pr < kW or H + pt + pb < kH or pl != pr or pt != pb or pl >= kW or pt >= kH:
            continue
        done += 1
        x = rng.normal(size=(B, Cn, H, W)).astype(np.float32)
        w = rng.normal(size=(O, Cn, kH, kW)).astype(np.float32)
        kw = dict(stride=(sx, sy), pad=(pl, pt, pr, pb))
        x64, w64 = x.astype(np.float64), w.astype(np.float64)
        want = orc.conv_forward(x64, w64, **kw)
        assert want.shape == (B, O, oH, oW)
        d = g.capi.ConvDesc(Cn, O, kW, kH, sx, sy, pl, pt, pr, pb, 1, 1, 1, 0,
                            {"direct": g.capi.KERNEL_F32_DIRECT, "gemm": g.capi.KERNEL_F32_GEMM}[path])
        print("random conv", path, (B, Cn, H, W, O, kW, kH, sx, sy, pl, pt), flush=True)
        dx_, dw_ = g.dev(x), g.dev(w)
        need = int(g.lib.n2d2hip_conv2d_f32_workspace_bytes(C.byref(d), B, H, W))
        ws = g.torch_.empty(max(need, 4), dtype=g.torch_.uint8, device="cuda")
        y = g.torch_.empty(want.shape, dtype=g.torch_.float32, device="cuda")
        g.check(g.lib.n2d2hip_conv2d_f32_forward(C.byref(d), B, H, W, dx_.data_ptr(), dw_.data_ptr(), None, 0.0, y.data_ptr(), ws.data_ptr(), need, g.sp()))
        assert _rel(g.host(y), want, np.maximum(orc.conv_forward(np.abs(x64), np.abs(w64), **kw), 1e-3)) <= TOL
        dy = rng.normal(size=want.shape).astype(np.float32)
        dy64 = dy.astype(np.float64)
        ddy = g.dev(dy)
        gdx = g.torch_.empty(x.shape, dtype=g.torch_.float32, device="cuda")
        gdw = g.torch_.empty(w.shape, dtype=g.torch_.float32, device="cuda")
        g.check(g.lib.n2d2hip_conv2d_f32_backward_data(C.byref(d), B, H, W, dw_.data_ptr(), ddy.data_ptr(), 0.0, gdx.data_ptr(), ws.data_ptr(), need, g.sp()))
        g.check(g.lib.n2d2hip_conv2d_f32_backward_filter(C.byref(d), B, H, W, dx_.data_ptr(), ddy.data_ptr(), 0.0, gdw.data_ptr(), ws.data_ptr(), need, g.sp()))
        assert _rel(g.host(gdx), orc.conv_backward_data(w64, dy64, x.shape, **kw),
                    np.maximum(orc.conv_backward_data(np.abs(w64), np.abs(dy64), x.shape, **kw), 1e-3)) <= TOL
        assert _rel(g.host(gdw), orc.conv_backward_filter(x64, dy64, w.shape, **kw),
                    np.maximum(orc.conv_backward_filter(np.abs(x64), np.abs(dy64), w.shape, **kw), 1e-3)) <= TOL


def test_dilated_forward(g):
    from oracle import oracle as orc
    rng = np.random.default_rng(3)
    x = rng.normal(size=(2, 3, 11, 11)).astype(np.float32)
    w = rng.normal(size=(4, 3, 3, 3)).astype(np.float32)
    want = orc.conv_forward(x, w, pad=(2, 2, 2, 2), dil=(2, 2))
    d = g.desc(3, 4, 3, 1, 2, 1, dil=2)
    y = g.torch_.empty(want.shape, dtype=g.torch_.float32, device="cuda")
    dx_, dw_ = g.dev(x), g.dev(w)
    g.check(g.lib.n2d2hip_conv2d_f32_forward(C.byref(d), 2, 11, 11, dx_.data_ptr(), dw_.data_ptr(), None, 0.0, y.data_ptr(), None, 0, g.sp()))
    assert _rel(g.host(y), want) <= TOL


def test_rectifier_softmax_loss_sgd(g):
    from oracle import oracle as orc
    from oracle import qat_train as qt
    rng = np.random.default_rng(8)
    x = (rng.normal(size=(4, 10, 3, 3)) * 3).astype(np.float32)
    for leak, clip in ((0.0, 0.0), (0.1, 0.0), (0.0, 2.0), (0.25, 1.5)):
        t = g.dev(x)
        g.check(g.lib.n2d2hip_rectifier_f32_forward(t.data_ptr(), x.size, leak, clip, g.sp()))
        want = orc.rectifier(x.copy(), leak=leak, clipping=clip, cell_quantized=False)
        out = g.host(t)
        assert _rel(out, want) <= TOL
        dy = rng.normal(size=x.shape).astype(np.float32)
        dd = g.dev(dy)
        g.check(g.lib.n2d2hip_rectifier_f32_backward(t.data_ptr(), dd.data_ptr(), dd.data_ptr(), x.size, leak, clip, g.sp()))
        f = np.where((clip > 0) & (want == np.float32(clip)), 0.0, np.where(want > 0, 1.0, leak)).astype(np.float32)
        assert _rel(g.host(dd), dy * f) <= TOL
    y = g.torch_.empty(x.shape, dtype=g.torch_.float32, device="cuda")
    dx_ = g.dev(x)
    g.check(g.lib.n2d2hip_softmax_f32_forward(dx_.data_ptr(), y.data_ptr(), 4, 10, 3, 3, g.sp()))
    sm = orc.softmax_forward(x)
    assert _rel(g.host(y), sm) <= TOL
    target = np.zeros_like(x)
    target[:, 2] = 1
    diff = g.torch_.empty(x.shape, dtype=g.torch_.float32, device="cuda")
    loss = g.torch_.zeros(1, dtype=g.torch_.float64, device="cuda")
    ws = g.torch_.empty(int(g.lib.n2d2hip_loss_workspace_bytes(x.size)), dtype=g.torch_.uint8, device="cuda")
    dt_ = g.dev(target)
    g.check(g.lib.n2d2hip_loss_f32(dt_.data_ptr(), y.data_ptr(), diff.data_ptr(), x.size, 4, loss.data_ptr(), ws.data_ptr(), ws.numel(), g.sp()))
    cell = qt.SoftmaxCell()
    cell.outputs = g.host(y)
    want_loss = cell.apply_loss(target)
    assert np.array_equal(g.host(diff), cell.diff_inputs)
    assert abs(float(g.host(loss)[0]) - want_loss) <= 1e-12 * max(1.0, want_loss)
    # SGD: plain, and with momentum and decay over three updates
    for kwargs in (dict(), dict(learning_rate=0.1, momentum=0.9, decay=0.01)):
        s = qt.SGDSolver(**kwargs)
        data = rng.normal(size=1000).astype(np.float32)
        dev = g.dev(data)
        mom = g.torch_.zeros(1000, dtype=g.torch_.float32, device="cuda") if kwargs else None
        for it in range(3):
            grad = rng.normal(size=1000).astype(np.float32)
            s.update(data, grad, 4)
            rate = np.float32(s.learning_rate)
            rate_diff = np.float32(rate / np.float32(4.0))
            dgrad = g.dev(grad)
            g.check(g.lib.n2d2hip_sgd_update_f32(dev.data_ptr(), dgrad.data_ptr(), 1000, float(rate_diff), float(s.momentum),
                                                 float(np.float32(np.float32(s.decay) * rate)), mom.data_ptr() if kwargs else None,
                                                 0, 0.0, 0.0, g.sp()))
            assert _rel(g.host(dev), data) <= TOL
    dev = g.dev(np.array([0.5, -0.5, 0.0]))
    dgrad = g.dev(np.array([10.0, -10.0, 1.0]))
    g.check(g.lib.n2d2hip_sgd_update_f32(dev.data_ptr(), dgrad.data_ptr(), 3, 1.0, 0.0, 0.0, None, 1, -1.0, 1.0, g.sp()))
    assert np.array_equal(g.host(dev), np.array([1.0, -1.0, 1.0], dtype=np.float32))
    assert g.lib.n2d2hip_sgd_update_f32(dev.data_ptr(), dev.data_ptr(), 3, 1.0, 0.9, 0.0, None, 0, 0.0, 0.0, g.sp()) == g.capi.ERR_INVALID


@pytest.mark.parametrize("shape,with_workspace", [((6, 5, 7, 4), True), ((2, 3, 1, 1), False), ((16, 64, 14, 14), True), ((3, 1, 33, 17), True),
                                                  ((300, 2, 3, 3), False), ((64, 8, 56, 56), True), ((64, 8, 56, 56), False), ((40, 3, 30, 31), True)])
def test_batchnorm_forward_backward(g, shape, with_workspace):
    from oracle import qat_train as qt
    print("batchnorm f32", shape, flush=True)
    B, Cn, H, W = shape
    rng = np.random.default_rng(sum(shape))
    x = rng.normal(1.5, 2.0, size=shape).astype(np.float32)
    gamma, beta = rng.normal(1, 0.3, size=Cn).astype(np.float32), rng.normal(0, 0.5, size=Cn).astype(np.float32)
    mean0, var0 = rng.normal(0, 1, size=Cn).astype(np.float32), rng.uniform(0.5, 2, size=Cn).astype(np.float32)
    cell = qt.BatchNormCell(Cn, scales=gamma, biases=beta, means=mean0, variances=var0)
    if B * H * W > 20000:
        # The reference adds a channel's values one by one into a float: over 2e5 values of magnitude 2 that running sum
        # is itself only good to a few 1e-5 of the mean.  The device adds in double; it is held to the same sums formed
        # exactly (the order of a float sum is the part of this path that no test can pin).
        monkey = pytest.MonkeyPatch()
        monkey.setattr(qt, "_seq_sum", lambda v: np.float32(np.sum(np.asarray(v, dtype=np.float64))))
        request_finalizer = monkey.undo
    else:
        request_finalizer = lambda: None
    dx_, dg, db = g.dev(x), g.dev(gamma), g.dev(beta)
    dmean, dvar = g.dev(mean0), g.dev(var0)
    z = lambda n: g.torch_.zeros(n, dtype=g.torch_.float32, device="cuda")
    smean, svar, y = z(Cn), z(Cn), z(x.size)
    # with a workspace the sums of the larger shapes are spread over several blocks per channel; without, one block adds them
    nws = int(g.lib.n2d2hip_batchnorm_f32_workspace_bytes(B, Cn, H, W))
    assert nws >= Cn * 40 and (nws > Cn * 40) == (B * H * W >= 8192)
    ws = g.torch_.empty(nws, dtype=g.torch_.uint8, device="cuda") if with_workspace else None
    wsp, wsn = (ws.data_ptr(), nws) if with_workspace else (None, 0)
    fwd = lambda running: g.check(g.lib.n2d2hip_batchnorm_f32_forward(
        B, Cn, H, W, dx_.data_ptr(), dg.data_ptr(), db.data_ptr(), dmean.data_ptr(), dvar.data_ptr(), smean.data_ptr(), svar.data_ptr(), 1e-5,
        0.1, running, y.data_ptr(), wsp, wsn, g.sp()))
    # inference: the running statistics, untouched
    fwd(1)
    want = cell.propagate(x, inference=True)
    assert _rel(g.host(y).reshape(shape), want) <= TOL
    assert np.array_equal(g.host(dmean), mean0) and np.array_equal(g.host(dvar), var0)
    # learning: batch statistics, running ones move a tenth of the way
    fwd(0)
    want = cell.propagate(x, inference=False)
    assert _rel(g.host(y).reshape(shape), want, scale=np.maximum(np.abs(want), 1.0)) <= 2e-5
    # (a mean is a sum of terms of magnitude ~2: held to 1e-5 of that, not of a result that may cancel to nearly 0)
    assert _rel(g.host(smean), cell.saved_mean, scale=2.0) <= TOL and _rel(g.host(svar), cell.saved_variance) <= TOL
    assert _rel(g.host(dmean), cell.mean, scale=2.0) <= TOL and _rel(g.host(dvar), cell.variance) <= TOL
    # backward, accumulating into the scale gradient (beta 1) and overwriting the bias gradient (beta 0)
    dy = rng.normal(0, 1, size=shape).astype(np.float32)
    cell.diff_inputs = dy
    cell.scale_solver.iteration_pass = 1            # inside an iteration: the oracle adds to diff_scale as well
    prev = rng.normal(0, 1, size=Cn).astype(np.float32)
    cell.diff_scale[:] = prev
    wdx = cell.back_propagate()
    ddy, dgs, dgb, dsm, dsv = g.dev(dy), g.dev(prev), g.dev(prev), z(Cn), z(Cn)
    g.check(g.lib.n2d2hip_batchnorm_f32_backward(B, Cn, H, W, dx_.data_ptr(), dg.data_ptr(), smean.data_ptr(), svar.data_ptr(), 1e-5, ddy.data_ptr(),
                                                 1.0, dgs.data_ptr(), 0.0, dgb.data_ptr(), dsm.data_ptr(), dsv.data_ptr(), ddy.data_ptr(), wsp, wsn, g.sp()))
    n = B * H * W
    terms = np.abs(dy).sum(axis=(0, 2, 3)) * 4 + 1.0                 # magnitude of the sums' terms (x_hat is O(1))
    assert _rel(g.host(dgs), cell.diff_scale, scale=terms) <= TOL and _rel(g.host(dgb), cell.diff_bias, scale=terms) <= TOL
    assert _rel(g.host(ddy).reshape(shape), wdx, scale=np.maximum(np.abs(wdx), 1.0) * max(1.0, float(np.abs(gamma).max()))) <= 5e-5
    assert np.isfinite(g.host(dsm)).all() and np.isfinite(g.host(dsv)).all()
    # only the parameter gradients
    ddy2 = g.dev(dy)
    g.check(g.lib.n2d2hip_batchnorm_f32_backward(B, Cn, H, W, dx_.data_ptr(), dg.data_ptr(), smean.data_ptr(), svar.data_ptr(), 1e-5, ddy2.data_ptr(),
                                                 0.0, dgs.data_ptr(), 0.0, dgb.data_ptr(), dsm.data_ptr(), dsv.data_ptr(), None, wsp, wsn, g.sp()))
    assert _rel(g.host(dgb), cell.diff_bias, scale=terms) <= TOL
    request_finalizer()
    # rejected: batch statistics of a single value, missing buffers
    assert g.lib.n2d2hip_batchnorm_f32_forward(1, Cn, 1, 1, dx_.data_ptr(), dg.data_ptr(), db.data_ptr(), dmean.data_ptr(), dvar.data_ptr(),
                                               smean.data_ptr(), svar.data_ptr(), 1e-5, 0.1, 0, y.data_ptr(), None, 0, g.sp()) == g.capi.ERR_INVALID
    assert g.lib.n2d2hip_batchnorm_f32_forward(B, Cn, H, W, dx_.data_ptr(), dg.data_ptr(), db.data_ptr(), dmean.data_ptr(), dvar.data_ptr(), None, None,
                                               1e-5, 0.1, 0, y.data_ptr(), None, 0, g.sp()) == g.capi.ERR_INVALID


@pytest.mark.parametrize("case", [(2, 3, 9, 8, 2, 2, 2, 2, 0, 0), (2, 3, 9, 8, 3, 3, 2, 2, 0, 0), (2, 3, 9, 8, 3, 3, 2, 2, 1, 1),
                                  (1, 2, 7, 10, 3, 2, 1, 2, 0, 0), (4, 16, 28, 28, 2, 2, 2, 2, 0, 0), (3, 5, 11, 11, 3, 3, 1, 1, 1, 1),
                                  (2, 2, 6, 6, 2, 2, 3, 3, 0, 0)])
def test_max_pooling_forward_backward(g, case):
    from oracle import qat_train as qt
    print("pool max f32", case, flush=True)
    B, Cn, H, W, pw, ph, sx, sy, px, py = case
    rng = np.random.default_rng(sum(case))
    x = rng.integers(-4, 5, size=(B, Cn, H, W)).astype(np.float32)          # many ties: the first maximum must win
    cell = qt.PoolCell((pw, ph), (sx, sy), (px, py))
    want = cell.propagate(x)
    oH, oW = want.shape[2:]
    y = g.torch_.empty(want.size, dtype=g.torch_.float32, device="cuda")
    am = g.torch_.empty(want.size, dtype=g.torch_.int32, device="cuda")
    dx_ = g.dev(x)
    g.check(g.lib.n2d2hip_pool_max_f32_forward(B, Cn, H, W, pw, ph, sx, sy, px, py, dx_.data_ptr(), y.data_ptr(), am.data_ptr(), g.sp()))
    assert np.array_equal(g.host(y).reshape(want.shape), want)
    ref_am = np.where(cell.argmax[..., 3] > 0, cell.argmax[..., 1] * W + cell.argmax[..., 0], -1)
    assert np.array_equal(g.host(am).reshape(want.shape), ref_am)
    dy = rng.normal(size=want.shape).astype(np.float32)
    cell.diff_inputs = dy
    wdx = cell.back_propagate()
    prev = rng.normal(size=x.shape).astype(np.float32)
    for beta in (0.0, 1.0):
        out = g.dev(prev)
        ddy = g.dev(dy)
        g.check(g.lib.n2d2hip_pool_max_f32_backward(B, Cn, H, W, pw, ph, sx, sy, px, py, ddy.data_ptr(), am.data_ptr(), beta, out.data_ptr(), g.sp()))
        assert _rel(g.host(out), wdx + np.float32(beta) * prev, scale=1.0) <= TOL
    # strides larger than the window leave inputs that no output reads: their gradient is 0
    if sx > pw:
        assert (wdx == 0).sum() >= x.size // 3
    assert g.lib.n2d2hip_pool_max_f32_forward(B, Cn, H, W, 2, 2, 2, 2, 2, 0, dx_.data_ptr(), y.data_ptr(), am.data_ptr(), g.sp()) == g.capi.ERR_INVALID
    assert g.lib.n2d2hip_pool_max_f32_forward(B, Cn, 1, 1, 3, 3, 1, 1, 0, 0, dx_.data_ptr(), y.data_ptr(), am.data_ptr(), g.sp()) == g.capi.ERR_INVALID


@pytest.mark.parametrize("case", [(2, 3, 9, 8, 2, 2, 2, 2, 0, 0), (2, 3, 9, 8, 3, 3, 2, 2, 1, 1), (1, 2, 7, 10, 3, 2, 1, 2, 0, 0),
                                  (4, 16, 28, 28, 2, 2, 2, 2, 0, 0), (3, 5, 11, 11, 3, 3, 1, 1, 1, 1), (2, 2, 6, 6, 2, 2, 3, 3, 0, 0),
                                  (8, 64, 7, 7, 7, 7, 7, 7, 0, 0)])
def test_average_pooling_forward_backward(g, case):
    from oracle import oracle as o
    print("pool average f32", case, flush=True)
    B, Cn, H, W, pw, ph, sx, sy, px, py = case
    rng = np.random.default_rng(sum(case) + 1)
    x = rng.normal(size=(B, Cn, H, W)).astype(np.float32)
    dx_ = g.dev(x)
    for include in (1, 0):
        want = o.pool_forward(x, (pw, ph), (sx, sy), (px, py), kind="average", quantized=False, count_include_padding=bool(include))
        y = g.torch_.empty(want.size, dtype=g.torch_.float32, device="cuda")
        g.check(g.lib.n2d2hip_pool_average_f32_forward(B, Cn, H, W, pw, ph, sx, sy, px, py, include, dx_.data_ptr(), y.data_ptr(), g.sp()))
        assert np.array_equal(g.host(y).reshape(want.shape), want)          # same additions in the same order, one division
    dy = rng.normal(size=want.shape).astype(np.float32)
    prev = rng.normal(size=x.shape).astype(np.float32)
    ddy = g.dev(dy)
    for beta in (0.0, 1.0):
        wdx = o.pool_backward_average(dy, x.shape, (pw, ph), (sx, sy), (px, py), beta=beta, prev=prev)
        out = g.dev(prev)
        g.check(g.lib.n2d2hip_pool_average_f32_backward(B, Cn, H, W, pw, ph, sx, sy, px, py, 1, ddy.data_ptr(), beta, out.data_ptr(), g.sp()))
        assert np.array_equal(g.host(out), wdx)
    assert g.lib.n2d2hip_pool_average_f32_backward(B, Cn, H, W, pw, ph, sx, sy, px, py, 0, ddy.data_ptr(), 0.0, out.data_ptr(),
                                                   g.sp()) == g.capi.ERR_UNSUPPORTED
    assert g.lib.n2d2hip_pool_average_f32_forward(B, Cn, H, W, 2, 2, 2, 2, 2, 0, 1, dx_.data_ptr(), y.data_ptr(), g.sp()) == g.capi.ERR_INVALID


@pytest.mark.parametrize("shape,n_in", [((2, 3, 5, 7), 2), ((4, 16, 14, 14), 2), ((1, 1, 1, 3), 3), ((2, 8, 6, 6), 8), ((3, 5, 4, 4), 1)])
def test_elemwise_sum_float_forward_backward(g, shape, n_in):
    from oracle import oracle as o
    print("elemwise sum f32", shape, n_in, flush=True)
    rng = np.random.default_rng(sum(shape) + n_in)
    xs = [rng.normal(size=shape).astype(np.float32) for _ in range(n_in)]
    w = rng.normal(size=n_in).astype(np.float32)
    sh = rng.normal(size=n_in).astype(np.float32)
    want = o.elemwise_sum(xs, w, sh, "PerInput")
    dev = [g.dev(x) for x in xs]
    n = xs[0].size
    ptrs = (C.c_void_p * n_in)(*[d.data_ptr() for d in dev])
    wa, sa = (C.c_float * n_in)(*w.tolist()), (C.c_float * n_in)(*sh.tolist())
    y = g.torch_.empty(n, dtype=g.torch_.float32, device="cuda")
    g.check(g.lib.n2d2hip_elemwise_sum_f32_forward(n_in, ptrs, n, wa, sa, y.data_ptr(), g.sp()))
    assert np.array_equal(g.host(y).reshape(shape), want)
    # a view that starts 4 bytes into a buffer takes the one-value-per-lane kernel
    if n > 1:
        odd = [g.torch_.cat([d.flatten()[:1], d.flatten()])[1:] for d in dev]
        ptrs2 = (C.c_void_p * n_in)(*[d.data_ptr() for d in odd])
        y2 = g.torch_.empty(n, dtype=g.torch_.float32, device="cuda")
        g.check(g.lib.n2d2hip_elemwise_sum_f32_forward(n_in, ptrs2, n, wa, sa, y2.data_ptr(), g.sp()))
        assert np.array_equal(g.host(y2).reshape(shape), want)
    dy = rng.normal(size=shape).astype(np.float32)
    prev = rng.normal(size=shape).astype(np.float32)
    ddy = g.dev(dy)
    for k in range(n_in):
        for beta in (0.0, 1.0):
            wdx = o.elemwise_sum_backward(dy, w, k, "PerInput", beta=beta, prev=prev)
            out = g.dev(prev)
            g.check(g.lib.n2d2hip_elemwise_sum_f32_backward(n, float(w[k]), ddy.data_ptr(), beta, out.data_ptr(), g.sp()))
            assert np.array_equal(g.host(out).reshape(shape), wdx)
    assert g.lib.n2d2hip_elemwise_sum_f32_forward(9, ptrs, n, wa, sa, y.data_ptr(), g.sp()) == g.capi.ERR_UNSUPPORTED
    assert g.lib.n2d2hip_elemwise_sum_f32_forward(0, ptrs, n, wa, sa, y.data_ptr(), g.sp()) == g.capi.ERR_INVALID
