"""Pins the training part of the CPU oracle (float conv backward, softmax, loss, SGD, the SAT quantizers' backward
and update) two ways: what the mathematics fixes (the backward kernels are the adjoints of the forward one, checked
with dot products and against a Jacobian built from unit impulses), and the reference's own known-answer test: the
three SAT alphas after 10 000 iterations on a hand-written three-convolution net, constants derived from PyTorch by
the reference's authors (tests/Cell/class_ConvCell_QuantizerSAT_Frame.cpp:68-516, delta 0.01)."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as o
from oracle import qat_train as q

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sat_three_conv", "case.json")

CASES = [  # B, C, H, W, O, k, stride, pad, groups
    (2, 3, 7, 6, 4, 3, 1, 1, 1), (2, 4, 9, 9, 4, 3, 2, 1, 4), (1, 2, 5, 5, 3, 1, 1, 0, 1), (2, 3, 10, 9, 2, 5, 2, 2, 1),
    (2, 2, 6, 6, 2, 3, 1, 0, 1), (3, 5, 8, 8, 5, 3, 1, 1, 5), (1, 3, 9, 7, 2, 3, 3, 0, 1), (2, 2, 4, 4, 3, 2, 2, 0, 1)]


@pytest.mark.parametrize("case", CASES)
def test_backward_kernels_are_the_adjoints_of_forward(case):
    B, C, H, W, O, k, s, p, groups = case
    rng = np.random.default_rng(sum(case))
    maps = None if groups == 1 else o.group_maps(C, O, groups)
    kw = dict(stride=(s, s), pad=(p, p, p, p), maps=maps)
    x = rng.normal(size=(B, C, H, W))
    w = rng.normal(size=(O, C // groups, k, k))
    y = o.conv_forward(x, w, **kw)
    dy = rng.normal(size=y.shape)
    dx = o.conv_backward_data(w, dy, x.shape, **kw)
    dw = o.conv_backward_filter(x, dy, w.shape, **kw)
    ref = (y * dy).sum()
    assert abs(ref - (x * dx).sum()) < 1e-10 * max(1.0, abs(ref))
    assert abs(ref - (w * dw).sum()) < 1e-10 * max(1.0, abs(ref))
    # alpha / beta accumulate as in the forward kernel
    old = rng.normal(size=w.shape)
    acc = o.conv_backward_filter(x, dy, w.shape, dw=old.copy(), alpha=0.5, beta=2.0, **kw)
    np.testing.assert_allclose(acc, 0.5 * dw + 2.0 * old, rtol=1e-12, atol=1e-12)
    oldx = rng.normal(size=x.shape)
    accx = o.conv_backward_data(w, dy, x.shape, dx=oldx.copy(), alpha=0.5, beta=2.0, **kw)
    np.testing.assert_allclose(accx, 0.5 * dx + 2.0 * oldx, rtol=1e-12, atol=1e-12)
    db = o.conv_backward_bias(dy)
    np.testing.assert_allclose(db, dy.sum(axis=(0, 2, 3)), rtol=1e-12, atol=1e-12)


def test_backward_data_against_the_jacobian_of_forward():
    """Column j of the (linear) forward map is forward(unit impulse j); backward data must be its transpose times dy.
    Covers the unrolled 3x3 stride-1 branch (interior pixels) and the generic one (borders) in one tensor."""
    rng = np.random.default_rng(5)
    B, C, H, W, O = 1, 2, 5, 5, 2
    w = rng.normal(size=(O, C, 3, 3))
    for pad, stride in ((1, 1), (0, 1), (1, 2)):
        kw = dict(stride=(stride, stride), pad=(pad,) * 4)
        cols = []
        for j in range(C * H * W):
            e = np.zeros(C * H * W)
            e[j] = 1.0
            cols.append(o.conv_forward(e.reshape(1, C, H, W), w, **kw).ravel())
        J = np.stack(cols, axis=1)                      # [outputs, inputs]
        dy = rng.normal(size=(J.shape[0],))
        oh = int(np.sqrt(J.shape[0] // O))
        dx = o.conv_backward_data(w, dy.reshape(1, O, oh, oh), (B, C, H, W), **kw)
        np.testing.assert_allclose(dx.ravel(), J.T @ dy, rtol=1e-12, atol=1e-12)


def test_grouped_backward_data_follows_the_reference_only_where_it_is_right():
    """backwardData indexes the weight's channel by a count of connected *outputs* (ConvCell_Frame_Kernels.cpp:233,
    :330): the adjoint for one output per group (depthwise) and without groups, not for wider groups. The restatement
    keeps that; the product accepts depthwise and ungrouped convolutions only."""
    rng = np.random.default_rng(9)
    x = rng.normal(size=(2, 6, 8, 8))
    w = rng.normal(size=(4, 3, 3, 3))
    maps = o.group_maps(6, 4, 2)
    y = o.conv_forward(x, w, maps=maps)
    dy = rng.normal(size=y.shape)
    dx = o.conv_backward_data(w, dy, x.shape, maps=maps)
    assert abs((y * dy).sum() - (x * dx).sum()) > 1e-3


def test_softmax_and_loss():
    rng = np.random.default_rng(2)
    x = rng.normal(size=(3, 5, 2, 2)).astype(np.float32) * 4
    y = o.softmax_forward(x)
    e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    np.testing.assert_allclose(y, e / e.sum(axis=1, keepdims=True), rtol=2e-6)
    np.testing.assert_allclose(y.sum(axis=1), 1.0, rtol=1e-6)
    sm = q.SoftmaxCell()
    sm.propagate(x)
    t = np.zeros_like(x)
    t[:, 1] = 1
    loss = sm.apply_loss(t)
    assert abs(loss - ((t - y.astype(np.float64)) ** 2).sum() / 3) < 1e-12
    assert np.array_equal(sm.back_propagate(), (t.astype(np.float64) - y).astype(np.float32))


def test_sgd_solver_update():
    s = q.SGDSolver()
    d = np.array([1.0, -2.0], dtype=np.float32)
    s.update(d, np.array([4.0, 4.0], dtype=np.float32), 2)
    np.testing.assert_allclose(d, [1.02, -1.98], rtol=1e-7)          # + 0.01 / 2 * diff
    assert s.nb_iterations == 1 and s.is_new_iteration()
    m = q.SGDSolver(learning_rate=0.1, momentum=0.9, decay=0.01)
    d = np.array([1.0], dtype=np.float32)
    g = np.array([2.0], dtype=np.float32)
    m.update(d, g, 1)      # v = 0.1*2 - 0.01*0.1*1 = 0.199
    m.update(d, g, 1)      # v = 0.9*0.199 + 0.2 - 0.001*1.199
    v1 = 0.199
    v2 = 0.9 * v1 + 0.2 - 0.001 * (1 + v1)
    np.testing.assert_allclose(d, [1 + v1 + v2], rtol=1e-6)
    acc = q.SGDSolver(iteration_size=2)                               # every second call applies
    d = np.array([0.0], dtype=np.float32)
    acc.update(d, g, 1)
    assert d[0] == 0.0 and not acc.is_new_iteration()
    acc.update(d, g, 1)
    np.testing.assert_allclose(d, [0.01 / 2 * 2.0], rtol=1e-6)


def sat_three_conv_net(case):
    x = (np.array(case["input_times_255"], dtype=np.float32) / np.float32(255.0)).reshape(2, 1, 5, 5)
    qa = [q.SATQuantizerActivation(case["range_activation1"], case["alpha_init"]),
          q.SATQuantizerActivation(case["range_conv"], case["alpha_init"]),
          q.SATQuantizerActivation(case["range_conv"], case["alpha_init"])]
    cells = [q.ActivationCell(q.LinearActivation(qa[0])),
             q.ConvCell(np.array(case["conv1_weights"]).reshape(1, 1, 3, 3), activation=q.LinearActivation(qa[1]),
                        quantizer=q.SATQuantizerCell(case["range_activation1"])),
             q.ConvCell(np.array(case["conv2_weights"]).reshape(4, 1, 1, 1), activation=q.LinearActivation(qa[2]),
                        quantizer=q.SATQuantizerCell(case["range_conv"])),
             q.ConvCell(np.array(case["conv3_weights"]).reshape(4, 1, 3, 3), maps=np.eye(4, dtype=np.uint8),
                        quantizer=q.SATQuantizerCell(case["range_conv"]))]
    t = np.zeros((2, 4, 1, 1), dtype=np.float32)
    for b, k in enumerate(case["target_class"]):
        t[b, k] = 1
    return x, cells, qa, t


def test_known_answer_sat_alphas_after_training():
    case = json.load(open(GOLD))
    x, cells, qa, t = sat_three_conv_net(case)
    loss = q.train_sequential(x, cells, q.SoftmaxCell(), t, case["iterations"])
    got = {"activation1": float(qa[0].alphas[0]), "conv1": float(qa[1].alphas[0]), "conv2": float(qa[2].alphas[0])}
    print("alphas", got, "loss", loss)
    for name, want in case["expected_alpha"].items():
        assert abs(got[name] - want) < case["delta"], (name, got[name], want)


LSQ_GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lsq_known_answers", "cases.json")


def lsq_three_conv_net(case, lsq):
    x = (np.array(case["input_times_255"], dtype=np.float32) / np.float32(255.0)).reshape(2, 1, 5, 5)
    qs = [q.LSQQuantizerCell(lsq["range_conv1"]), q.LSQQuantizerCell(lsq["range_conv2"]), q.LSQQuantizerCell(lsq["range_conv3"])]
    cells = [q.ActivationCell(q.LinearActivation(None)),
             q.ConvCell(np.array(case["conv1_weights"]).reshape(1, 1, 3, 3), activation=q.LinearActivation(None), quantizer=qs[0]),
             q.ConvCell(np.array(case["conv2_weights"]).reshape(4, 1, 1, 1), activation=q.LinearActivation(None), quantizer=qs[1]),
             q.ConvCell(np.array(case["conv3_weights"]).reshape(4, 1, 3, 3), maps=np.eye(4, dtype=np.uint8), quantizer=qs[2])]
    t = np.zeros((2, 4, 1, 1), dtype=np.float32)
    for b, k in enumerate(case["target_class"]):
        t[b, k] = 1
    return x, cells, qs, t


def test_known_answer_lsq_step_sizes_three_conv():
    """tests/Cell/class_ConvCell_QuantizerLSQ_Frame_CUDA.cpp: PyTorch-derived step sizes of the three weight quantizers
    after 10 000 (constants kept in a comment there) and 100 000 iterations (asserted there), delta 0.001."""
    case = json.load(open(GOLD))
    lsq = json.load(open(LSQ_GOLD))["three_conv"]
    x, cells, qs, t = lsq_three_conv_net(case, lsq)
    sm = q.SoftmaxCell()
    done = 0
    for iters, key in ((10000, "expected_step_after_10000"), (100000, "expected_step_after_100000")):
        q.train_sequential(x, cells, sm, t, iters - done)
        done = iters
        got = dict(zip(("conv1", "conv2", "conv3"), (float(s.step[0]) for s in qs)))
        print(iters, got)
        for name, want in lsq[key].items():
            assert abs(got[name] - want) < lsq["delta"], (iters, name, got[name], want)


def test_known_answer_lsq_step_size_fc():
    """tests/Cell/class_FcCell_QuantizerLSQ_Frame_CUDA.cpp: a 9 -> 2 FcCell with an LSQ weight quantizer, run here as the
    3x3 convolution over the 3x3 input that computes the same products in the same order."""
    fc = json.load(open(LSQ_GOLD))["fc"]
    x = (np.float32(0.125) * np.arange(9, dtype=np.float32)).reshape(1, 1, 3, 3)
    w = np.zeros((2, 1, 3, 3), dtype=np.float32)
    for k, v in enumerate(fc["weights_per_output"]):
        w[k] = v
    quant = q.LSQQuantizerCell(fc["range"])
    cells = [q.ActivationCell(q.LinearActivation(None)), q.ConvCell(w, quantizer=quant)]
    t = np.array(fc["target"], dtype=np.float32).reshape(1, 2, 1, 1)
    q.train_sequential(x, cells, q.SoftmaxCell(), t, fc["iterations"])
    print("step", float(quant.step[0]))
    assert abs(float(quant.step[0]) - fc["expected_step"]) < fc["delta"]


# ------------------------------------------------------------------ BatchNorm and max pooling of the learning graph
def _bn_reference(x, gamma, beta, eps):
    """Textbook batch normalisation in float64: outputs, and the gradients of sum(dy * y) as every framework derives them."""
    x = x.astype(np.float64)
    mu = x.mean(axis=(0, 2, 3), keepdims=True)
    var = x.var(axis=(0, 2, 3), keepdims=True)
    xhat = (x - mu) / np.sqrt(var + eps)
    g, b = gamma.astype(np.float64).reshape(1, -1, 1, 1), beta.astype(np.float64).reshape(1, -1, 1, 1)

    def grads(dy):
        dy = dy.astype(np.float64)
        dxhat = dy * g
        dx = (dxhat - dxhat.mean(axis=(0, 2, 3), keepdims=True) - xhat * (dxhat * xhat).mean(axis=(0, 2, 3), keepdims=True)) / np.sqrt(var + eps)
        return dx, (dy * xhat).sum(axis=(0, 2, 3)), dy.sum(axis=(0, 2, 3))
    return g * xhat + b, mu.reshape(-1), var.reshape(-1), grads


def test_batchnorm_learning_pass_is_textbook_batch_normalisation():
    from oracle import qat_train as qt
    rng = np.random.default_rng(21)
    x = rng.normal(1.5, 2.0, size=(6, 5, 7, 4)).astype(np.float32)
    gamma, beta = rng.normal(1, 0.3, size=5).astype(np.float32), rng.normal(0, 0.5, size=5).astype(np.float32)
    bn = qt.BatchNormCell(5, scales=gamma, biases=beta)
    y = bn.propagate(x, inference=False)
    want, mu, var, grads = _bn_reference(x, gamma, beta, 1e-5)
    assert np.allclose(y, want, rtol=0, atol=2e-5)
    n = 6 * 7 * 4
    # the running statistics start at 0 and take a tenth of the batch's; the variance with Bessel's factor
    assert np.allclose(bn.mean, 0.1 * mu, rtol=1e-5) and np.allclose(bn.variance, 0.1 * var * n / (n - 1), rtol=1e-5)
    dy = rng.normal(0, 1, size=x.shape).astype(np.float32)
    bn.diff_inputs = dy
    dx = bn.back_propagate()
    wdx, wdg, wdb = grads(dy)
    assert np.allclose(dx, wdx, rtol=0, atol=3e-5 * np.abs(wdx).max())
    assert np.allclose(bn.diff_scale, wdg, rtol=1e-4, atol=1e-4) and np.allclose(bn.diff_bias, wdb, rtol=1e-5, atol=1e-4)
    # update adds rate / batch * diff to scale and bias, in that order, each through its own solver
    bn.update(6)
    assert np.allclose(bn.scale, gamma + np.float32(0.01 / 6) * bn.diff_scale) and np.allclose(bn.bias, beta + np.float32(0.01 / 6) * bn.diff_bias)
    # a second propagate moves the running statistics by another tenth of the way
    m1, v1 = bn.mean.copy(), bn.variance.copy()
    bn.propagate(x, inference=False)
    assert np.allclose(bn.mean, 0.9 * m1 + 0.1 * mu, rtol=1e-5) and np.allclose(bn.variance, 0.9 * v1 + 0.1 * var * n / (n - 1), rtol=1e-5)


def test_batchnorm_inference_uses_the_running_statistics():
    from oracle import qat_train as qt, qat_fuse as qf
    rng = np.random.default_rng(22)
    x = rng.normal(0, 1, size=(3, 4, 5, 5)).astype(np.float32)
    p = [rng.normal(1, 0.2, size=4), rng.normal(0, 1, size=4), rng.normal(0, 1, size=4), rng.uniform(0.5, 2, size=4)]
    bn = qt.BatchNormCell(4, scales=p[0], biases=p[1], means=p[2], variances=p[3])
    y = bn.propagate(x, inference=True)
    want = p[0].reshape(1, -1, 1, 1) * (x.astype(np.float64) - p[2].reshape(1, -1, 1, 1)) / np.sqrt(p[3].reshape(1, -1, 1, 1) + 1e-5) + p[1].reshape(1, -1, 1, 1)
    assert np.allclose(y, want, rtol=0, atol=1e-5)
    assert np.array_equal(y, qf.batchnorm_inference(x, *[np.asarray(v, dtype=np.float32) for v in p]))
    assert np.array_equal(bn.mean, np.asarray(p[2], dtype=np.float32))          # untouched
    # MovingAverageMomentum 0 takes the same branch while learning
    bn0 = qt.BatchNormCell(4, scales=p[0], biases=p[1], means=p[2], variances=p[3], moving_average_momentum=0.0)
    assert np.array_equal(bn0.propagate(x, inference=False), y)


@pytest.mark.parametrize("pool,stride,pad", [((2, 2), (2, 2), (0, 0)), ((3, 3), (2, 2), (0, 0)), ((3, 3), (2, 2), (1, 1)), ((3, 2), (1, 2), (0, 0))])
def test_max_pooling_backward_routes_each_gradient_to_the_first_maximum(pool, stride, pad):
    from oracle import qat_train as qt
    rng = np.random.default_rng(23)
    x = (rng.permutation(2 * 3 * 9 * 8).reshape(2, 3, 9, 8) / 1000.0).astype(np.float32)      # all distinct, 1e-3 apart
    cell = qt.PoolCell(pool, stride, pad)
    y = cell.propagate(x)
    dy = rng.normal(0, 1, size=y.shape).astype(np.float32)
    cell.diff_inputs = dy
    dx = cell.back_propagate()
    # directional derivative of sum(dy * maxpool(x)) along a random direction, exact for a piecewise-linear map
    # (the step stays below half the distance between two inputs, so that no maximum moves)
    v = np.clip(rng.normal(0, 2e-4, size=x.shape), -4e-4, 4e-4).astype(np.float32)
    x2 = (x + v).astype(np.float32)
    y2 = qt.PoolCell(pool, stride, pad).propagate(x2)
    assert np.isclose(((y2.astype(np.float64) - y) * dy).sum(), (dx.astype(np.float64) * (x2.astype(np.float64) - x)).sum(), rtol=1e-3, atol=1e-7)
    assert np.isclose(dx.sum(), dy.sum(), rtol=1e-5, atol=1e-5) and (dx != 0).sum() <= dy.size
    # ties: the first element of the window in row-major order wins, forward and backward
    flat = np.zeros((1, 1, 4, 4), dtype=np.float32)
    c2 = qt.PoolCell((2, 2), (2, 2))
    c2.propagate(flat)
    c2.diff_inputs = np.ones((1, 1, 2, 2), dtype=np.float32)
    assert np.array_equal(np.argwhere(c2.back_propagate()[0, 0] == 1), [[0, 0], [0, 2], [2, 0], [2, 2]])


def test_a_net_with_batchnorm_and_pooling_learns():
    from oracle import qat_train as qt
    rng = np.random.default_rng(24)
    x = rng.uniform(0, 1, size=(4, 1, 12, 12)).astype(np.float32)
    t = np.zeros((4, 3, 1, 1), dtype=np.float32)
    t[np.arange(4), [0, 1, 2, 0]] = 1
    cells_ = [qt.ConvCell(rng.normal(0, 0.3, size=(4, 1, 3, 3)), quantizer=qt.SATQuantizerCell(15)),
              qt.BatchNormCell(4, activation=qt.LinearActivation(qt.SATQuantizerActivation(15, 4.0))),
              qt.PoolCell((2, 2), (2, 2)),
              qt.ConvCell(rng.normal(0, 0.3, size=(3, 4, 5, 5)), quantizer=qt.SATQuantizerCell(15))]
    sm = qt.SoftmaxCell()
    first = qt.train_sequential(x, cells_, sm, t, 1)
    last = qt.train_sequential(x, cells_, sm, t, 300)
    assert last < 0.6 * first and np.isfinite(last)
    assert not np.array_equal(cells_[1].scale, np.ones(4, dtype=np.float32)) and np.all(cells_[1].variance > 0)


# ---- average pooling (forward, backward) and the ElemWise sum's gradient: what pins the oracle's restatements.
# The reference holds no known answers for them; a library routine (torch's avg_pool2d and its autograd, float64)
# and the adjoint identity <dy, A x> = <A^T dy, x> of a linear map do.
AVG_CASES = [(2, 3, 9, 8, 2, 2, 2, 2, 0, 0), (2, 3, 9, 8, 3, 3, 2, 2, 1, 1), (1, 2, 7, 10, 3, 2, 1, 2, 0, 0),
             (3, 5, 11, 11, 3, 3, 1, 1, 1, 1), (2, 2, 6, 6, 2, 2, 3, 3, 0, 0), (2, 4, 7, 7, 7, 7, 7, 7, 0, 0)]


@pytest.mark.parametrize("case", AVG_CASES)
def test_average_pooling_against_library_routine_and_adjoint(case):
    import torch
    from oracle import oracle as o
    B, Cn, H, W, pw, ph, sx, sy, px, py = case
    rng = np.random.default_rng(sum(case))
    x = rng.normal(size=(B, Cn, H, W)).astype(np.float32)
    y = o.pool_forward(x, (pw, ph), (sx, sy), (px, py), kind="average", quantized=False)
    xt = torch.tensor(x.astype(np.float64), requires_grad=True)
    yt = torch.nn.functional.avg_pool2d(xt, (ph, pw), (sy, sx), (py, px), count_include_pad=True)
    assert y.shape == tuple(yt.shape)
    assert np.abs(y - yt.detach().numpy()).max() <= 1e-5
    # the other divisor: the number of values inside the input
    y2 = o.pool_forward(x, (pw, ph), (sx, sy), (px, py), kind="average", quantized=False, count_include_padding=False)
    yt2 = torch.nn.functional.avg_pool2d(xt, (ph, pw), (sy, sx), (py, px), count_include_pad=False)
    assert np.abs(y2 - yt2.detach().numpy()).max() <= 1e-5
    dy = rng.normal(size=y.shape).astype(np.float32)
    dx = o.pool_backward_average(dy, x.shape, (pw, ph), (sx, sy), (px, py))
    yt.backward(torch.tensor(dy.astype(np.float64)))
    assert np.abs(dx - xt.grad.numpy()).max() <= 1e-5
    # adjoint identity in float64 sums of the float32 results
    assert abs((dy.astype(np.float64) * y).sum() - (dx.astype(np.float64) * x).sum()) <= 1e-4 * max(1.0, np.abs(dy).sum())
    # beta keeps what the gradient tensor held
    prev = rng.normal(size=x.shape).astype(np.float32)
    assert np.abs(o.pool_backward_average(dy, x.shape, (pw, ph), (sx, sy), (px, py), beta=1.0, prev=prev) - (dx + prev)).max() <= 1e-6
    with pytest.raises(RuntimeError):
        o.pool_backward_average(dy, x.shape, (pw, ph), (sx, sy), (px, py), count_include_padding=False)


def test_elemwise_sum_gradient_is_the_weight_per_input_or_per_channel():
    from oracle import oracle as o
    rng = np.random.default_rng(11)
    xs = [rng.normal(size=(2, 3, 4, 5)).astype(np.float32) for _ in range(3)]
    w = np.array([0.5, -2.0, 3.0], dtype=np.float32)
    sh = np.array([0.25, 0.0, -1.0], dtype=np.float32)
    y = o.elemwise_sum(xs, w, sh, "PerInput")
    assert np.abs(y - (sum(w[k] * xs[k].astype(np.float64) for k in range(3)) + sh.sum())).max() <= 1e-5
    dy = rng.normal(size=y.shape).astype(np.float32)
    for k in range(3):
        dx = o.elemwise_sum_backward(dy, w, k, "PerInput")
        assert np.array_equal(dx, w[k] * dy)                              # one rounded product per value
        # directional derivative of the (affine) forward along a random direction
        d = rng.normal(size=y.shape).astype(np.float32)
        moved = [x if i != k else x + d for i, x in enumerate(xs)]
        lhs = ((o.elemwise_sum(moved, w, sh, "PerInput").astype(np.float64) - y) * dy).sum()
        assert abs(lhs - (dx.astype(np.float64) * d).sum()) <= 1e-4 * np.abs(dy).sum()
        prev = rng.normal(size=y.shape).astype(np.float32)
        assert np.array_equal(o.elemwise_sum_backward(dy, w, k, "PerInput", beta=1.0, prev=prev), w[k] * dy + prev)
    wc = np.array([2.0, -1.0, 0.5], dtype=np.float32)
    dxc = o.elemwise_sum_backward(dy, wc, 1, "PerChannel")
    assert np.array_equal(dxc, wc[None, :, None, None] * dy)


def test_a_graph_with_a_residual_sum_backpropagates_as_autograd_does():
    """train_graph over conv -> (conv, identity) -> weighted sum -> conv -> softmax with loss: a tensor read by two cells
    receives the sum of their gradients.  Against torch's autograd in float64 on the same graph (the gradient the softmax
    hands back, target - output, is minus that of the summed cross-entropy)."""
    import torch
    from oracle import qat_train as qt
    rng = np.random.default_rng(61)
    x = rng.uniform(0, 1, size=(3, 2, 6, 6)).astype(np.float32)
    w1 = rng.normal(0, 0.4, size=(4, 2, 3, 3)).astype(np.float32)
    w2 = rng.normal(0, 0.4, size=(4, 4, 3, 3)).astype(np.float32)
    w3 = rng.normal(0, 0.4, size=(3, 4, 4, 4)).astype(np.float32)
    t = np.zeros((3, 3, 1, 1), dtype=np.float32)
    t[np.arange(3), [2, 0, 1]] = 1
    zero_lr = lambda: qt.SGDSolver(learning_rate=0.0)
    c1, c2, c3 = (qt.ConvCell(w1, solver=zero_lr()), qt.ConvCell(w2, pad=(1, 1, 1, 1), solver=zero_lr()), qt.ConvCell(w3, solver=zero_lr()))
    ew = qt.ElemWiseCell(2, weights=[1.0, 0.5], shifts=[0.0, 0.25])
    nodes = [(c1, [-1]), (c2, [0]), (ew, [1, 0]), (c3, [2])]
    qt.train_graph(x, nodes, qt.SoftmaxCell(), t, 1)
    tx = torch.tensor(x, dtype=torch.float64)
    tw = [torch.tensor(w, dtype=torch.float64, requires_grad=True) for w in (w1, w2, w3)]
    a = torch.nn.functional.conv2d(tx, tw[0])
    b = torch.nn.functional.conv2d(a, tw[1], padding=1)
    s = (1.0 * b + 0.0) + (0.5 * a + 0.25)
    z = torch.nn.functional.conv2d(s, tw[2]).reshape(3, 3)
    ce = -(torch.tensor(t.reshape(3, 3), dtype=torch.float64) * torch.log_softmax(z, 1)).sum()
    ce.backward()
    for cell, g in zip((c1, c2, c3), tw):
        want = -g.grad.numpy()
        assert np.abs(cell.diff_w - want).max() <= 1e-4 * np.abs(want).max()
    assert np.abs(ew.outputs - s.detach().numpy()).max() <= 1e-5
