"""The float Frame_HIP cells for quantization-aware training (C++ host classes created through the Registrar under
"Frame_HIP_QAT"), against the CPU oracle: one learning iteration compared tensor by tensor, a few more on the learned
parameters, and the reference's own known-answer test, the three SAT alphas after 10 000 iterations
(tests/Cell/class_ConvCell_QuantizerSAT_Frame.cpp:68-516, delta 0.01)."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sat_three_conv", "case.json")


def _gpu_net(case):
    from n2d2_amd import frame_hip as fh
    x = (np.array(case["input_times_255"], dtype=np.float32) / np.float32(255.0)).reshape(2, 1, 5, 5)
    net = fh.TrainNet(x)
    r1, r2, a = case["range_activation1"], case["range_conv"], case["alpha_init"]
    net.add_activation_cell("activation1", "Linear", "SAT", r1, a)
    net.add_conv("conv1", np.array(case["conv1_weights"]).reshape(1, 1, 3, 3), act="Linear", act_quant="SAT", act_range=r2, act_param=a,
                 weight_quant="SAT", weight_range=r1)
    net.add_conv("conv2", np.array(case["conv2_weights"]).reshape(4, 1, 1, 1), act="Linear", act_quant="SAT", act_range=r2, act_param=a,
                 weight_quant="SAT", weight_range=r2)
    net.add_conv("conv3", np.array(case["conv3_weights"]).reshape(4, 1, 3, 3), depthwise=True, weight_quant="SAT", weight_range=r2)
    net.add_softmax("softmax1", with_loss=True)
    t = np.zeros((2, 4, 1, 1), dtype=np.float32)
    for b, k in enumerate(case["target_class"]):
        t[b, k] = 1
    return net, t


def _oracle_net(case):
    from test_oracle_qat_train import sat_three_conv_net
    return sat_three_conv_net(case)


def _close(got, want, tol=1e-5):
    scale = np.maximum(np.abs(want), 1e-3)
    return float((np.abs(got.astype(np.float64) - want.astype(np.float64)) / scale).max()) <= tol


def test_registrar_holds_the_float_cells():
    from n2d2_amd import frame_hip as fh
    for t in ("Conv", "Fc", "Activation", "Softmax", "BatchNorm", "Pool"):
        assert fh.lib.fh_train_registrar_exists(t.encode(), b"Frame_HIP_QAT") == 1
        assert fh.lib.fh_train_registrar_exists(t.encode(), b"Frame_XYZ") == 0
    assert fh.lib.fh_train_registrar_exists(b"Conv", b"Frame_HIP") == 1          # the integer inference cell
    with pytest.raises(fh.FrameHipError, match="is not valid"):
        net = fh.TrainNet(np.zeros((1, 1, 4, 4)), model="Frame_XYZ")
        net.add_softmax("s")


def test_one_learning_iteration_matches_the_oracle_tensor_by_tensor():
    from oracle import qat_train as q
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    case = json.load(open(GOLD))
    net, t = _gpu_net(case)
    x, cells, qa, t2 = _oracle_net(case)
    assert np.array_equal(t, t2)
    print("one iteration", flush=True)
    loss = net.learn(t, 1)
    sm = q.SoftmaxCell()
    want_loss = q.train_sequential(x, cells, sm, t, 1)
    assert abs(loss - want_loss) <= 1e-6 * want_loss
    names = ["activation1", "conv1", "conv2", "conv3"]
    for name, c in zip(names, cells):
        assert _close(net.outputs(name), c.outputs), name
    assert _close(net.outputs("softmax1"), sm.outputs)
    assert _close(net.diff_inputs("softmax1"), sm.diff_inputs)
    for name, c in zip(names[1:], cells[1:]):
        assert _close(net.quantized_weights(name), c.wq), name
        assert _close(net.diff_weights(name), c.diff_wq, 1e-4), name       # gradient of the quantized weights
        assert _close(net.weights(name), c.w), name                        # after the update
    for name, a in zip(names[:3], qa):
        got, grad = net.activation_quantizer(name)
        assert abs(got - float(a.alphas[0])) <= 1e-6 * abs(got), name
        assert abs(grad - float(a.diff_alphas)) <= 1e-5 * max(abs(float(a.diff_alphas)), 1e-3), name
    # 50 more iterations: the learned parameters stay together
    net.learn(t, 50)
    q.train_sequential(x, cells, sm, t, 50)
    for name, a in zip(names[:3], qa):
        assert abs(net.activation_quantizer(name)[0] - float(a.alphas[0])) <= 1e-4, name
    for name, c in zip(names[1:], cells[1:]):
        assert _close(net.weights(name), c.w, 1e-3), name


def test_known_answer_sat_alphas_after_training():
    case = json.load(open(GOLD))
    net, t = _gpu_net(case)
    print("10000 iterations", flush=True)
    loss = net.learn(t, case["iterations"])
    got = {n: net.activation_quantizer(n)[0] for n in ("activation1", "conv1", "conv2")}
    print("alphas", got, "loss", loss, flush=True)
    for name, want in case["expected_alpha"].items():
        assert abs(got[name] - want) < case["delta"], (name, got[name], want)


def test_rectifier_bias_and_momentum_against_the_oracle():
    """A two-convolution net with a bias, a Rectifier activation with a SAT quantizer, stride and padding, a Symmetric
    weight quantizer and a momentum solver: five iterations against the oracle."""
    from n2d2_amd import frame_hip as fh
    from oracle import qat_train as q
    rng = np.random.default_rng(21)
    x = rng.uniform(0, 1, size=(4, 3, 9, 9)).astype(np.float32)
    w1 = rng.normal(0, 0.3, size=(6, 3, 3, 3)).astype(np.float32)
    w2 = rng.normal(0, 0.3, size=(5, 6, 3, 3)).astype(np.float32)
    net = fh.TrainNet(x, propagate_gradient=False)
    net.add_conv("c1", w1, stride=(2, 2), pad=(1, 1), act="Rectifier", act_quant="SAT", act_range=15, act_param=2.0, weight_quant="SAT", weight_range=15)
    b2 = rng.normal(0, 0.1, size=5).astype(np.float32)
    net.add_conv("c2", w2, bias=b2, stride=(1, 1), pad=(0, 0), act=None, weight_quant="SAT", weight_range=15, quant_mode="Symmetric")
    net.set_solver_parameter("c1", "Momentum", 0.9)
    assert net._last == (4, 5, 3, 3)
    t = rng.uniform(0, 1, size=net._last).astype(np.float32)

    class Rect(q.LinearActivation):
        def propagate(self, v, inference):
            self.out = q.LinearActivation.propagate(self, np.maximum(v, 0).astype(np.float32), inference)
            return self.out

        def back_propagate(self, d):
            d = q.LinearActivation.back_propagate(self, d)
            return (d * (self.out > 0)).astype(np.float32)
    qa = q.SATQuantizerActivation(15, 2.0)
    c1 = q.ConvCell(w1, stride=(2, 2), pad=(1, 1, 1, 1), activation=Rect(qa), quantizer=q.SATQuantizerCell(15), solver=q.SGDSolver(momentum=0.9))
    c2 = q.ConvCell(w2, bias=b2, quantizer=q.SATQuantizerCell(15, mode="symrange"))

    class Last:                                  # loss straight on the last convolution's outputs
        def propagate(self, v):
            self.outputs = v

        def apply_loss(self, targets):
            err = targets.astype(np.float64) - self.outputs.astype(np.float64)
            self.diff_inputs = err.astype(np.float32)
            return float((err * err).sum() / self.outputs.shape[0])

        def back_propagate(self):
            return self.diff_inputs
    print("rectifier / momentum net", flush=True)
    for it in range(5):
        loss = net.learn(t, 1)
        want = q.train_sequential(x, [c1, c2], Last(), t, 1)
        assert abs(loss - want) <= 1e-4 * want, it
    assert _close(net.weights("c1"), c1.w, 1e-3) and _close(net.weights("c2"), c2.w, 1e-3)
    assert abs(net.activation_quantizer("c1")[0] - float(qa.alphas[0])) <= 1e-4


LSQ_GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lsq_known_answers", "cases.json")


def test_known_answer_lsq_step_sizes_three_conv():
    """tests/Cell/class_ConvCell_QuantizerLSQ_Frame_CUDA.cpp: the step sizes of the three LSQ weight quantizers after
    10 000 and after 100 000 iterations, delta 0.001; one iteration first, against the oracle."""
    from n2d2_amd import frame_hip as fh
    from oracle import qat_train as q
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from test_oracle_qat_train import lsq_three_conv_net
    case = json.load(open(GOLD))
    lsq = json.load(open(LSQ_GOLD))["three_conv"]
    x, cells, qs, t = lsq_three_conv_net(case, lsq)
    net = fh.TrainNet(x)
    net.add_activation_cell("activation1", "Linear")
    net.add_conv("conv1", cells[1].w, act="Linear", weight_quant="LSQ", weight_range=lsq["range_conv1"])
    net.add_conv("conv2", cells[2].w, act="Linear", weight_quant="LSQ", weight_range=lsq["range_conv2"])
    net.add_conv("conv3", cells[3].w, depthwise=True, weight_quant="LSQ", weight_range=lsq["range_conv3"])
    net.add_softmax("softmax1", with_loss=True)
    names = ("conv1", "conv2", "conv3")
    print("lsq three conv", flush=True)
    net.learn(t, 1)
    q.train_sequential(x, cells, q.SoftmaxCell(), t, 1)
    for name, s, c in zip(names, qs, cells[1:]):
        step, grad = net.weight_quantizer(name)
        assert abs(step - float(s.step[0])) <= 1e-6 * abs(step), name
        assert abs(grad - float(s.diff_step)) <= 1e-5 * max(abs(float(s.diff_step)), 1e-3), name
        assert _close(net.quantized_weights(name), c.wq), name
        assert _close(net.weights(name), c.w), name
    done = 1
    for iters, key in ((10000, "expected_step_after_10000"), (100000, "expected_step_after_100000")):
        net.learn(t, iters - done)
        done = iters
        got = {n: net.weight_quantizer(n)[0] for n in names}
        print(iters, got, flush=True)
        for name, want in lsq[key].items():
            assert abs(got[name] - want) < lsq["delta"], (iters, name, got[name], want)


def test_known_answer_lsq_step_size_fc():
    """tests/Cell/class_FcCell_QuantizerLSQ_Frame_CUDA.cpp through the FcCell class."""
    from n2d2_amd import frame_hip as fh
    fc = json.load(open(LSQ_GOLD))["fc"]
    x = (np.float32(0.125) * np.arange(9, dtype=np.float32)).reshape(1, 1, 3, 3)
    w = np.zeros((2, 9), dtype=np.float32)
    for k, v in enumerate(fc["weights_per_output"]):
        w[k] = v
    net = fh.TrainNet(x)
    net.add_activation_cell("activation1", "Linear")
    net.add_fc("fc1", w, weight_quant="LSQ", weight_range=fc["range"])
    net.add_softmax("softmax1", with_loss=True)
    print("lsq fc", flush=True)
    net.learn(np.array(fc["target"], dtype=np.float32).reshape(1, 2, 1, 1), fc["iterations"])
    step = net.weight_quantizer("fc1")[0]
    print("step", step, flush=True)
    assert abs(step - fc["expected_step"]) < fc["delta"]


def test_conv_then_fc_with_bias_against_the_oracle():
    """ConvCell (Rectifier) -> FcCell with a bias and a SAT weight quantizer -> softmax with loss: three iterations."""
    from n2d2_amd import frame_hip as fh
    from oracle import qat_train as q
    rng = np.random.default_rng(33)
    x = rng.uniform(0, 1, size=(3, 2, 6, 6)).astype(np.float32)
    w1 = rng.normal(0, 0.4, size=(4, 2, 3, 3)).astype(np.float32)
    wf = rng.normal(0, 0.2, size=(5, 4 * 4 * 4)).astype(np.float32)
    bf = rng.normal(0, 0.1, size=5).astype(np.float32)
    net = fh.TrainNet(x, propagate_gradient=False)
    net.add_conv("c1", w1, act="Rectifier")
    net.add_fc("fc", wf, bias=bf, weight_quant="SAT", weight_range=15)
    net.add_softmax("softmax", with_loss=True)
    t = np.zeros((3, 5, 1, 1), dtype=np.float32)
    t[0, 1] = t[1, 4] = t[2, 0] = 1

    class Rect(q.LinearActivation):
        def propagate(self, v, inference):
            self.out = np.maximum(v, 0).astype(np.float32)
            return self.out

        def back_propagate(self, d):
            return (d * (self.out > 0)).astype(np.float32)
    c1 = q.ConvCell(w1, activation=Rect())
    fc = q.ConvCell(wf.reshape(5, 4, 4, 4), bias=bf, quantizer=q.SATQuantizerCell(15))
    fc.quantizer_outputs_size = 5
    sm = q.SoftmaxCell()
    print("conv -> fc net", flush=True)
    for it in range(3):
        loss = net.learn(t, 1)
        want = q.train_sequential(x, [c1, fc], sm, t, 1)
        assert abs(loss - want) <= 1e-5 * want, it
    assert _close(net.outputs("softmax"), sm.outputs)
    assert _close(net.weights("fc"), fc.w.reshape(5, -1), 1e-4) and _close(net.weights("c1"), c1.w, 1e-4)


def test_batchnorm_and_pool_cells_learn_as_the_oracle_does():
    """Conv (SAT weights) -> BatchNorm (Linear, SAT activation) -> max Pool -> Conv -> Softmax: the first iteration tensor by
    tensor, then twenty more on the loss and the learned parameters."""
    from n2d2_amd import frame_hip as fh
    from oracle import qat_train as q
    rng = np.random.default_rng(31)
    x = rng.uniform(0, 1, size=(4, 1, 12, 12)).astype(np.float32)
    w1 = rng.normal(0, 0.3, size=(4, 1, 3, 3)).astype(np.float32)
    w2 = rng.normal(0, 0.3, size=(3, 4, 5, 5)).astype(np.float32)
    t = np.zeros((4, 3, 1, 1), dtype=np.float32)
    t[np.arange(4), [0, 1, 2, 0]] = 1
    net = fh.TrainNet(x, propagate_gradient=False)
    net.add_conv("c1", w1, weight_quant="SAT", weight_range=15)
    net.add_batchnorm("bn", act="Linear", act_quant="SAT", act_range=15, act_param=4.0)
    net.add_pool("pool", (2, 2), (2, 2))
    net.add_conv("c2", w2, weight_quant="SAT", weight_range=15)
    net.add_softmax("softmax", with_loss=True)
    assert net._shapes["pool"] == (4, 4, 5, 5) and net._last == (4, 3, 1, 1)
    qa = q.SATQuantizerActivation(15, 4.0)
    cells_ = [q.ConvCell(w1, quantizer=q.SATQuantizerCell(15)), q.BatchNormCell(4, activation=q.LinearActivation(qa)), q.PoolCell((2, 2), (2, 2)),
              q.ConvCell(w2, quantizer=q.SATQuantizerCell(15))]
    sm = q.SoftmaxCell()
    print("batchnorm / pool net: first iteration", flush=True)
    loss = net.learn(t, 1)
    want = q.train_sequential(x, cells_, sm, t, 1)
    assert abs(loss - want) <= 1e-5 * want
    for name, cell in zip(("c1", "bn", "pool", "c2"), cells_):
        assert _close(net.outputs(name), cell.outputs, 2e-5), name
        if name != "bn":        # (the BatchNorm's activation works on its gradient in place)
            assert _close(net.diff_inputs(name), cell.diff_inputs, 1e-4), name
    bn = net.batchnorm("bn")
    assert _close(bn["diff_scales"], cells_[1].diff_scale, 1e-4) and _close(bn["diff_biases"], cells_[1].diff_bias, 1e-4)
    assert _close(bn["scales"], cells_[1].scale) and _close(bn["biases"], cells_[1].bias, 1e-4)
    assert _close(bn["means"], cells_[1].mean, 1e-4) and _close(bn["variances"], cells_[1].variance, 1e-4)
    assert _close(net.weights("c1"), cells_[0].w, 1e-4) and _close(net.weights("c2"), cells_[3].w, 1e-4)
    print("batchnorm / pool net: twenty more", flush=True)
    for it in range(20):
        loss = net.learn(t, 1)
        want = q.train_sequential(x, cells_, sm, t, 1)
        assert abs(loss - want) <= 1e-3 * want, it
    bn = net.batchnorm("bn")
    assert _close(bn["scales"], cells_[1].scale, 1e-3) and _close(bn["variances"], cells_[1].variance, 1e-3)
    assert abs(net.activation_quantizer("bn")[0] - float(qa.alphas[0])) <= 1e-3
    assert not np.array_equal(bn["scales"], np.ones(4, dtype=np.float32))
    # inference afterwards runs on the running statistics
    net.propagate(inference=True)
    h = x
    for c in cells_:
        h = c.propagate(h, inference=True)
    assert _close(net.outputs("c2"), h, 1e-3)
    # a backPropagate without a learning propagate has nothing to differentiate
    fresh = fh.TrainNet(x, propagate_gradient=False)
    fresh.add_batchnorm("bn", moving_average_momentum=0.0)
    fresh.add_softmax("softmax", with_loss=True)
    with pytest.raises(fh.FrameHipError, match="needs the batch statistics"):
        fresh.learn(np.zeros((4, 1, 12, 12), dtype=np.float32), 1)


def test_batchnorm_adds_to_a_gradient_that_is_already_there():
    """A cell whose input another cell reads too finds that cell's gradient already in place and adds its own
    (the `isValid * diffOutputs` term of src/Cell/BatchNormCell_Frame.cpp:458-488): the net's input gradient with a
    gradient preset there equals the preset plus what the same net gives alone."""
    from n2d2_amd import frame_hip as fh
    rng = np.random.default_rng(32)
    x = rng.uniform(0, 1, size=(4, 2, 6, 6)).astype(np.float32)
    w = rng.normal(0, 0.3, size=(3, 2, 6, 6)).astype(np.float32)
    t = np.zeros((4, 3, 1, 1), dtype=np.float32)
    t[np.arange(4), [0, 1, 2, 0]] = 1
    preset = rng.normal(0, 1, size=x.shape).astype(np.float32)

    def first_gradient(with_preset):
        net = fh.TrainNet(x, propagate_gradient=True)
        net.add_batchnorm("bn", act="Linear")
        net.add_conv("c", w)
        net.add_softmax("softmax", with_loss=True)
        if with_preset:
            net.preset_input_gradient(preset)
        net.learn(t, 1)
        return net.input_gradient()
    alone = first_gradient(False)
    assert np.abs(alone).max() > 1e-4
    assert _close(first_gradient(True), alone + preset, 1e-5)


@pytest.mark.parametrize("name", ["w8a8", "w4a4"])
def test_trained_lenet_float_graph_and_its_integer_twin_agree_on_the_gpu(name):
    """The reference's test of its QAT-to-integer pass (tests/Quantizer/QAT/Optimization/class_DeepNetQAT.cpp:96-140) runs the
    trained LeNet with BatchNorm before and after the pass and compares recognition rates.  Here both graphs run on the GPU
    on the same images: the float one on the Frame_HIP_QAT cells (checked against the oracle), the integer one on the
    Frame_HIP cells after the library's pass, and the levels after each Conv + BatchNorm stage are compared."""
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import sat_lenet as sl
    from n2d2_amd import frame_hip as fh
    from oracle import oracle as o
    d = sl.load(name)
    R = sl.act_range(name)
    imgs = sl.images(32, seed=12)
    x = (imgs / np.float32(255)).astype(np.float32)
    net = fh.TrainNet(x, propagate_gradient=False)
    chain = x
    want = {}
    for (conv, bn, shape, w_range), pool in zip(sl.conv_stages(name), ("pool1", "pool2", None)):
        alpha = float(d[bn + "_QAct_SAT_Alpha"][0])
        net.add_conv(conv, d[conv + "_weights"].reshape(shape), weight_quant="SAT", weight_range=w_range, act="Linear")
        net.add_batchnorm(bn, *sl.bn_of(d, bn), epsilon=sl.EPS, act="Linear", act_quant="SAT", act_range=R, act_param=alpha)
        levels = sl.float_conv_stage(chain, sl.quantized_conv_weights(d, conv, shape, w_range), sl.bn_of(d, bn), alpha, R)
        want[bn] = (levels, alpha)
        chain = (levels * np.float32(alpha / R)).astype(np.float32)
        if pool:
            net.add_pool(pool, (2, 2), (2, 2))
            chain = o.pool_forward(chain, (2, 2), (2, 2), kind="max", quantized=False)
    fc_want = {}
    for fc, shape, w_range, a_range in sl.fc_stages(name):
        alpha = float(d[fc + "_QAct_SAT_Alpha"][0])
        net.add_fc(fc, d[fc + "_weights"].reshape(shape), act="Linear", act_quant="SAT", act_range=a_range, act_param=alpha, weight_quant="SAT",
                   weight_range=w_range, apply_scaling=True)
        wq, _ = sl.quantized_fc_weights(d, fc, shape, w_range)
        z = o.conv_forward(chain.reshape(32, -1, 1, 1), wq.reshape(shape + (1, 1)))
        chain, _ = o.sat_act_forward(z, a_range, alpha, True)
        fc_want[fc] = (np.rint(chain * np.float32(a_range / alpha)), alpha, a_range)
    print("trained LeNet", name, "float graph", flush=True)
    net.propagate(inference=True)
    for fc, (levels, alpha, a_range) in fc_want.items():
        got = np.rint(net.outputs(fc) * np.float32(a_range / alpha))
        assert (got != levels).mean() < 5e-3 and np.abs(got - levels).max() <= 1, fc
    assert np.unique(fc_want["fc2"][0]).size > 4
    fused = sl.fuse_with_library(fh, d, name, batch=32)
    try:
        fh.set_globals(8, True, True)
        fused.set_fusion(False)
        fused.initialize()
        fused.set_stimuli(imgs)
        fused.propagate()
        for (conv, bn, _, w_range) in sl.conv_stages(name):
            levels, alpha = want[bn]
            got = np.rint(net.outputs(bn) * np.float32(R / alpha))
            # the float cells against the oracle's float graph: the same levels but where a sum lands within rounding of a tie
            assert (got != levels).mean() < 2e-3 and np.abs(got - levels).max() <= 1, bn
            dev = np.abs(fused.outputs(conv) - got)
            assert dev.max() <= (6 if R == 255 else 1) and dev.mean() < (0.3 if R == 255 else 0.06), conv
            assert np.unique(got).size > 4
        # the same pass fed from the learning cells themselves (their quantizers' tensors on the device, the BatchNorm
        # cells' vectors): the same integer net but for a weight that sits within rounding of a tie
        twin = fh.Net(sl.INI % 32)
        assert net.fuse_into(twin) == 5
        for pool in ("pool1", "pool2"):
            twin.set_quantized(pool, 8)
        for cell in ("conv1", "conv2", "conv3", "fc1", "fc2"):
            a, b = twin.weights(cell), fused.weights(cell)
            assert (a != b).mean() < 2e-3 and np.abs(a - b).max() <= 1, cell
            # (the Fc cells' SAT divisor comes from a variance summed on the device in another order than the oracle's)
            assert np.allclose(twin.scaling(cell)[2], fused.scaling(cell)[2], rtol=1e-4), cell
            assert np.allclose(twin.clipping(cell), fused.clipping(cell), rtol=1e-4, atol=1.0), cell
            assert twin.quantized(cell) == fused.quantized(cell), cell
        twin.set_fusion(False)
        twin.initialize()
        twin.set_stimuli(imgs)
        twin.propagate()
        for cell in ("conv1", "conv3", "fc2"):
            assert (twin.outputs(cell) != fused.outputs(cell)).mean() < 0.02, cell
    finally:
        fh.set_globals(0, True, False)


LEARN_INI = """
DefaultModel=Frame_HIP

[sp]
SizeX=12
SizeY=12
NbChannels=1
BatchSize=8

[c1]
Input=sp
Type=Conv
KernelDims=3 3
NbOutputs=6
ActivationFunction=Linear

[pool]
Input=c1
Type=Pool
Mapping.ChannelsPerGroup=1
PoolDims=2 2
NbOutputs=6
Stride=2
Pooling=Max

[c2]
Input=pool
Type=Conv
KernelDims=3 3
NbOutputs=8
ActivationFunction=Linear

[fc]
Input=c2
Type=Fc
NbOutputs=3
ActivationFunction=Linear
"""


def test_learn_then_fuse_then_infer_without_leaving_the_gpu():
    """Quantization-aware learning on the float cells, the pass to integer cells fed from them, integer inference: the
    integer net reproduces the levels of the float net it was made from."""
    from n2d2_amd import frame_hip as fh
    rng = np.random.default_rng(41)
    imgs = rng.integers(0, 256, size=(8, 1, 12, 12)).astype(np.float32)
    x = (imgs / np.float32(255)).astype(np.float32)
    t = np.zeros((8, 3, 1, 1), dtype=np.float32)
    t[np.arange(8), rng.integers(0, 3, size=8)] = 1
    net = fh.TrainNet(x, propagate_gradient=False)
    # (8-bit weights in the first cell, as in the reference's models: the pass rescales 4-bit default-mode weights to 5 bits
    # and then takes the cell's *input* range to be 31 as well, which only fits inputs that have 15 levels)
    net.add_conv("c1", rng.normal(0, 0.4, size=(6, 1, 3, 3)), weight_quant="SAT", weight_range=255, act="Linear")
    net.add_batchnorm("bn1", act="Linear", act_quant="SAT", act_range=15, act_param=3.0)
    net.add_pool("pool", (2, 2), (2, 2))
    net.add_conv("c2", rng.normal(0, 0.3, size=(8, 6, 3, 3)), weight_quant="SAT", weight_range=15, act="Linear")
    net.add_batchnorm("bn2", act="Linear", act_quant="SAT", act_range=15, act_param=3.0)
    net.add_fc("fc", rng.normal(0, 0.2, size=(3, 8 * 3 * 3)), act="Linear", act_quant="SAT", act_range=255, act_param=4.0, weight_quant="SAT",
               weight_range=255, apply_scaling=True)
    net.add_softmax("softmax", with_loss=True)
    print("learn, fuse, infer", flush=True)
    first = net.learn(t, 1)
    last = net.learn(t, 60)
    assert np.isfinite(last) and last < first
    net.propagate(inference=True)
    levels = {bn: np.rint(net.outputs(bn) * np.float32(15 / net.activation_quantizer(bn)[0])) for bn in ("bn1", "bn2")}
    twin = fh.Net(LEARN_INI)
    assert net.fuse_into(twin) == 3
    twin.set_quantized("pool", 8)
    assert twin.quantized("c1") == (8, 4, "Rectifier") and twin.quantized("c2") == (4, 4, "Rectifier") and twin.quantized("fc") == (8, 8, "Linear")
    try:
        fh.set_globals(8, True, True)
        twin.set_fusion(False)
        twin.initialize()
        twin.set_stimuli(imgs)
        twin.propagate()
        for conv, bn in (("c1", "bn1"), ("c2", "bn2")):
            dev = np.abs(twin.outputs(conv) - levels[bn])
            # one level at most; the second stage also inherits the first one's deviations through its 54 inputs per output
            assert dev.max() <= 1 and dev.mean() < (0.05 if conv == "c1" else 0.15) and np.unique(levels[bn]).size > 4, conv
        # the Fc stage from the integer graph's own input (one input level moves an output by several of its 255): the
        # float cell's quantized weights on c2's levels, the SAT activation, and the signed saturation N2D2 applies to a
        # Linear cell (levels above 127)
        alpha, a2 = net.activation_quantizer("fc")[0], net.activation_quantizer("bn2")[0]
        z = (twin.outputs("c2").reshape(8, -1).astype(np.float64) * a2 / 15) @ net.quantized_weights("fc").astype(np.float64).T
        want = np.minimum(np.rint(np.clip(z, 0, alpha) / alpha * 255), 127).reshape(8, 3, 1, 1)
        assert np.abs(twin.outputs("fc") - want).max() <= 1 and np.unique(want).size > 2
    finally:
        fh.set_globals(0, True, False)


def test_average_pool_cell_learns_as_the_oracle_does():
    """Conv (SAT weights, Rectifier) -> Average Pool 3x3 stride 2 with padding -> Conv -> Softmax: the first iteration tensor by
    tensor, then ten more on the loss and the learned weights."""
    from n2d2_amd import frame_hip as fh
    from oracle import qat_train as q
    rng = np.random.default_rng(37)
    x = rng.uniform(0, 1, size=(4, 2, 11, 11)).astype(np.float32)
    w1 = rng.normal(0, 0.3, size=(4, 2, 3, 3)).astype(np.float32)
    w2 = rng.normal(0, 0.3, size=(3, 4, 5, 5)).astype(np.float32)
    t = np.zeros((4, 3, 1, 1), dtype=np.float32)
    t[np.arange(4), [2, 1, 0, 1]] = 1
    net = fh.TrainNet(x, propagate_gradient=False)
    net.add_conv("c1", w1, weight_quant="SAT", weight_range=15)
    net.add_pool("pool", (3, 3), (2, 2), (1, 1), pooling="Average")
    net.add_conv("c2", w2, weight_quant="SAT", weight_range=15)
    net.add_softmax("softmax", with_loss=True)
    assert net._shapes["pool"] == (4, 4, 5, 5) and net._last == (4, 3, 1, 1)
    cells_ = [q.ConvCell(w1, quantizer=q.SATQuantizerCell(15)), q.PoolCell((3, 3), (2, 2), (1, 1), pooling="Average"),
              q.ConvCell(w2, quantizer=q.SATQuantizerCell(15))]
    sm = q.SoftmaxCell()
    print("average pool net: first iteration", flush=True)
    loss = net.learn(t, 1)
    want = q.train_sequential(x, cells_, sm, t, 1)
    assert abs(loss - want) <= 1e-5 * want
    for name, cell in zip(("c1", "pool", "c2"), cells_):
        assert _close(net.outputs(name), cell.outputs, 2e-5), name
        assert _close(net.diff_inputs(name), cell.diff_inputs, 1e-4), name
    assert _close(net.weights("c1"), cells_[0].w, 1e-4) and _close(net.weights("c2"), cells_[2].w, 1e-4)
    assert not np.array_equal(net.weights("c1"), w1)          # the gradient went through the pooling
    print("average pool net: ten more", flush=True)
    for it in range(10):
        loss = net.learn(t, 1)
        want = q.train_sequential(x, cells_, sm, t, 1)
        assert abs(loss - want) <= 1e-3 * want, it
    assert _close(net.weights("c1"), cells_[0].w, 1e-3)


def test_residual_sum_cell_learns_as_the_oracle_does():
    """A learning graph with a branch: Conv (SAT weights, SAT activation) -> [Conv -> BatchNorm -> Conv] + shortcut -> ElemWise
    Sum (weights 1 and 0.5, Rectifier) -> max Pool -> Conv -> Softmax.  The tensor read by the branch and by the sum receives
    both gradients.  First iteration tensor by tensor against the oracle's train_graph, then ten more on the loss and the
    learned weights."""
    from n2d2_amd import frame_hip as fh
    from oracle import qat_train as q
    assert fh.lib.fh_train_registrar_exists(b"ElemWise", b"Frame_HIP_QAT") == 1
    rng = np.random.default_rng(71)
    x = rng.uniform(0, 1, size=(4, 2, 10, 10)).astype(np.float32)
    w0 = rng.normal(0, 0.3, size=(4, 2, 3, 3)).astype(np.float32)
    w1 = rng.normal(0, 0.3, size=(4, 4, 3, 3)).astype(np.float32)
    w2 = rng.normal(0, 0.3, size=(4, 4, 1, 1)).astype(np.float32)
    w3 = rng.normal(0, 0.3, size=(3, 4, 4, 4)).astype(np.float32)
    t = np.zeros((4, 3, 1, 1), dtype=np.float32)
    t[np.arange(4), [0, 1, 2, 1]] = 1
    net = fh.TrainNet(x, propagate_gradient=False)
    net.add_conv("stem", w0, act="Linear", act_quant="SAT", act_range=15, act_param=3.0, weight_quant="SAT", weight_range=15)
    net.add_conv("b1", w1, pad=(1, 1), weight_quant="SAT", weight_range=15)
    net.add_batchnorm("bn", act="Linear", act_quant="SAT", act_range=15, act_param=4.0)
    net.add_conv("b2", w2, weight_quant="SAT", weight_range=15)
    net.add_elemwise("sum", ["b2", "stem"], weights=[1.0, 0.5], act="Rectifier")
    net.add_pool("pool", (2, 2), (2, 2))
    net.add_conv("head", w3, weight_quant="SAT", weight_range=15)
    net.add_softmax("softmax", with_loss=True)
    assert net._shapes["sum"] == (4, 4, 8, 8) and net._last == (4, 3, 1, 1)
    qa0, qa1 = q.SATQuantizerActivation(15, 3.0), q.SATQuantizerActivation(15, 4.0)
    stem = q.ConvCell(w0, activation=q.LinearActivation(qa0), quantizer=q.SATQuantizerCell(15))
    b1 = q.ConvCell(w1, pad=(1, 1, 1, 1), quantizer=q.SATQuantizerCell(15))
    bn = q.BatchNormCell(4, activation=q.LinearActivation(qa1))
    b2 = q.ConvCell(w2, quantizer=q.SATQuantizerCell(15))

    class Rect(q.LinearActivation):         # RectifierActivation_Frame, no quantizer: max(x, 0) and its mask
        def propagate(self, v, inference):
            self.out = np.maximum(v, 0).astype(np.float32)
            return self.out

        def back_propagate(self, d):
            return (d * (self.out > 0)).astype(np.float32)
    ew = q.ElemWiseCell(2, weights=[1.0, 0.5], activation=Rect())
    pool = q.PoolCell((2, 2), (2, 2))
    head = q.ConvCell(w3, quantizer=q.SATQuantizerCell(15))
    nodes = [(stem, [-1]), (b1, [0]), (bn, [1]), (b2, [2]), (ew, [3, 0]), (pool, [4]), (head, [5])]
    sm = q.SoftmaxCell()
    print("residual net: first iteration", flush=True)
    loss = net.learn(t, 1)
    want = q.train_graph(x, nodes, sm, t, 1)
    assert abs(loss - want) <= 1e-5 * want
    for name, cell in (("stem", stem), ("b1", b1), ("b2", b2), ("sum", ew), ("pool", pool), ("head", head)):
        assert _close(net.outputs(name), cell.outputs, 2e-5), name
    # the gradient that reaches the stem's outputs: the branch's part plus the shortcut's
    assert _close(net.diff_inputs("b2"), b2.diff_inputs, 1e-4)
    assert _close(net.weights("stem"), stem.w, 1e-4) and _close(net.weights("b1"), b1.w, 1e-4) and _close(net.weights("head"), head.w, 1e-4)
    print("residual net: ten more", flush=True)
    for it in range(10):
        loss = net.learn(t, 1)
        want = q.train_graph(x, nodes, sm, t, 1)
        assert abs(loss - want) <= 1e-3 * want, it
    assert _close(net.weights("stem"), stem.w, 1e-3) and _close(net.weights("b2"), b2.w, 1e-3)
    assert abs(net.activation_quantizer("stem")[0] - float(qa0.alphas[0])) <= 1e-3
    # an ElemWise cell other than a sum, or with one coefficient per channel, is refused by name
    bad = fh.TrainNet(x, propagate_gradient=False)
    bad.add_conv("a", w0)
    with pytest.raises(fh.FrameHipError, match="name the inputs first"):
        fh._check_train(fh.lib.fh_train_add_elemwise(bad._h, b"s", None, None, 0, -1, 0, 255, 1.0))
