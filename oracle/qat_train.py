"""CPU oracle (TEST INFRASTRUCTURE, not the product) of the float cells a
quantization-aware training step runs through: restatement of the reference's
Frame classes around the kernels of oracle.py, for a sequential net of
ActivationCell / ConvCell / BatchNormCell / PoolCell / SoftmaxCell with SAT quantizers and SGD solvers.

Pinned by tests/test_oracle_qat_train.py: closed forms for the solver, softmax and loss, and the reference's own
known-answer tests (tests/Cell/class_ConvCell_QuantizerSAT_Frame.cpp, class_ConvCell_QuantizerLSQ_Frame_CUDA.cpp,
class_FcCell_QuantizerLSQ_Frame_CUDA.cpp: trained SAT alphas and LSQ step sizes derived from PyTorch by the
reference's authors), which exercise every class below in the order the reference's learning loop calls them, but
BatchNormCell and PoolCell, for which the reference's tests hold no values: textbook batch normalisation in float64
(outputs, running statistics, the three gradients by the closed form), and the directional derivative of max pooling.
Parity unpinned, by nature: the order of BatchNormCell's float sums over batch and pixels.

Data is float32 as in the `<float>` instantiations; "diff" tensors carry the
descent direction (target - output at the loss), so a solver *adds*
rate * diff.  Cited paths are relative to the N2D2 source tree.
"""
import numpy as np

from . import oracle as o

F = np.float32


class SGDSolver:
    """src/Solver/SGDSolver.cpp:26-41 (defaults), :99-189 (getLearningRate, policy None) and
    include/Solver/SGDSolver_Frame.hpp:77-146 (update)."""

    def __init__(self, learning_rate=0.01, momentum=0.0, decay=0.0, iteration_size=1):
        self.learning_rate, self.momentum, self.decay, self.iteration_size = learning_rate, momentum, decay, iteration_size
        self.iteration_pass = 0
        self.nb_iterations = 0
        self.momentum_data = None

    def is_new_iteration(self):
        return self.iteration_pass == 0

    def get_learning_rate(self):
        if self.learning_rate == 0.0:
            return 0.0
        if self.iteration_pass < self.iteration_size - 1:
            self.iteration_pass += 1
            return 0.0
        self.iteration_pass = 0
        self.nb_iterations += 1
        return self.learning_rate

    def update(self, data, diff, batch_size):
        """data (float32 array, updated in place) += rate / (batch * iterationSize) * diff."""
        rate = F(self.get_learning_rate())
        if rate == 0.0:
            return
        rate_diff = F(rate / F(F(batch_size) * F(self.iteration_size)))
        if self.momentum == 0.0 and self.decay == 0.0:
            data += rate_diff * diff.astype(F)
            return
        if self.momentum_data is None:
            self.momentum_data = np.zeros_like(data)
        m = self.momentum_data
        m *= F(self.momentum)
        m += rate_diff * diff.astype(F)
        if self.decay != 0.0:
            m += F(-F(self.decay) * rate) * data
        data += m


class SATQuantizerActivation:
    """src/Quantizer/QAT/Activation/SAT/SATQuantizerActivation_Frame.cpp:73-143: one alpha for the whole
    tensor, created at the first propagate; its gradient is the element-order sum of the per-element terms
    (+ the previous value while the solver is inside an iteration); update() hands it to the solver."""

    def __init__(self, rng, alpha, solver=None):
        self.range, self.alpha_parameter = rng, alpha
        self.alphas = None
        self.diff_alphas = F(0.0)
        self.full_precision = None
        self.solver = solver or SGDSolver()

    def propagate(self, x, inference):
        if self.alphas is None:
            self.alphas = np.full(1, self.alpha_parameter, dtype=F)
        y, fp = o.sat_act_forward(x, self.range, float(self.alphas[0]), inference=inference)
        if not inference:
            self.full_precision = fp
        return y

    def back_propagate(self, diff_input):
        beta = 0.0 if self.solver.is_new_iteration() else 1.0
        dx, da, _ = o.sat_act_backward(diff_input, self.full_precision, self.range, float(self.alphas[0]),
                                       beta=beta, prev_diff_alpha=float(self.diff_alphas))
        self.diff_alphas = F(da)
        return dx

    def update(self, batch_size):
        self.solver.update(self.alphas, np.full(1, self.diff_alphas, dtype=F), batch_size)


class LinearActivation:
    """include/Activation/LinearActivation_Frame.hpp:56-134 without Scaling and Clipping: the quantizer, if any, is all
    that acts, forward and backward."""

    def __init__(self, quantizer=None):
        self.quantizer = quantizer

    def propagate(self, x, inference):
        return self.quantizer.propagate(x, inference) if self.quantizer else x

    def back_propagate(self, diff_input):
        return self.quantizer.back_propagate(diff_input) if self.quantizer else diff_input

    def update(self, batch_size):
        if self.quantizer:
            self.quantizer.update(batch_size)


class SATQuantizerCell:
    """src/Quantizer/QAT/Cell/SAT/SATQuantizerCell_Frame.cpp:178-294: the weights are quantized again at every
    propagate; backward scales by factor = max|tanh(w)| * scaling of that propagate; nothing to update."""

    def __init__(self, rng, quantization=True, scaling=False, mode="default"):
        self.range, self.quantization, self.scaling, self.mode = rng, quantization, scaling, mode
        self.tanh_max, self.sat_scaling = 0.0, 1.0

    def propagate(self, w, outputs_size):
        mode = self.mode if self.quantization else {"asymrange": "none_asym"}.get(self.mode, "none")
        wq, self.tanh_max, self.sat_scaling = o.sat_weight_forward(w, self.range, mode, self.scaling, outputs_size)
        return wq

    def back_propagate(self, dwq, w):
        scale = self.sat_scaling if self.scaling else 1.0
        return o.sat_weight_backward(dwq, w, self.range, float(F(F(self.tanh_max) * F(scale))),
                                     self.mode if self.mode in ("fullrange", "asymrange") else "default")


class LSQQuantizerCell:
    """src/Quantizer/QAT/Cell/LSQ/LSQQuantizerCell_Frame.cpp:106-310: range [-(R+1)/2, (R-1)/2]; at the first propagate
    the step size becomes 2 * mean|w| / sqrt(hi) (SetOptInitStepSize, :166-184); the step-size gradient is the kernel's
    sum (+ the previous value inside a solver iteration) times 1/sqrt(N * hi); update() hands it to the solver."""

    def __init__(self, rng, step_size=None, solver=None):
        self.lo, self.hi = -((rng + 1) >> 1), (rng - 1) >> 1
        self.step = None if step_size is None else np.full(1, step_size, dtype=F)
        self.diff_step = F(0.0)
        self.solver = solver or SGDSolver()

    def propagate(self, w, outputs_size):
        if self.step is None:
            self.step = np.full(1, F(2.0) * F(np.abs(w.astype(np.float64)).mean() / np.sqrt(self.hi)), dtype=F)
        self.grad_scale = F(1.0 / np.sqrt(w.size * self.hi))
        return o.lsq_forward(w, float(self.step[0]), self.lo, self.hi)

    def back_propagate(self, dwq, w):
        dw, total = o.lsq_backward(dwq, w, float(self.step[0]), self.lo, self.hi)
        total = F(total)
        if not self.solver.is_new_iteration():
            total = F(total + self.diff_step)
        self.diff_step = F(total * self.grad_scale)
        return dw

    def update(self, batch_size):
        self.solver.update(self.step, np.full(1, self.diff_step, dtype=F), batch_size)


class ActivationCell:
    """src/Cell/ActivationCell_Frame.cpp:95-205, one input: copy, then the activation in place."""

    def __init__(self, activation):
        self.activation = activation
        self.outputs = None
        self.diff_inputs = None      # written by the next cell's backPropagate
        self.diff_outputs = None

    def propagate(self, x, inference=False):
        self.outputs = self.activation.propagate(np.array(x, dtype=F), inference)
        return self.outputs

    def back_propagate(self):
        self.diff_outputs = self.activation.back_propagate(self.diff_inputs)
        return self.diff_outputs

    def update(self, batch_size):
        self.activation.update(batch_size)


class ConvCell:
    """src/Cell/ConvCell_Frame.cpp:418-597 with one input: propagate = quantize the weights, convolve, then
    the activation in place; backPropagate = activation, backwardFilter on the quantized weights' gradient, backwardData
    with the quantized weights, then the weight quantizer's backward; update = solver on the full-precision weights with
    the quantizer's gradient, then the activation's quantizer."""

    def __init__(self, weights, stride=(1, 1), pad=(0, 0, 0, 0), maps=None, activation=None, quantizer=None, solver=None,
                 bias=None, bias_solver=None):
        self.w = np.array(weights, dtype=F)
        self.bias = None if bias is None else np.array(bias, dtype=F)      # None: NoBias
        self.bias_solver = bias_solver or SGDSolver()
        self.stride, self.pad, self.maps = stride, pad, maps
        self.activation, self.quantizer = activation, quantizer
        self.solver = solver or SGDSolver()
        self.diff_inputs = None

    def propagate(self, x, inference=False):
        self.x = x
        O, Cw, kH, kW = self.w.shape
        # mOutputsSize: dimB * dimY * dimX of the weight tensor {kW,kH,Cw,O} (SATQuantizerCell_Frame.cpp:80)
        self.wq = self.quantizer.propagate(self.w, O * kH * kW) if self.quantizer else self.w
        y = o.conv_forward(x, self.wq, stride=self.stride, pad=self.pad, maps=self.maps)
        if self.bias is not None:       # the SAT / LSQ cell quantizers pass the biases through
            y = o.conv_forward_bias(y, self.bias)
        self.outputs = self.activation.propagate(y, inference) if self.activation else y
        return self.outputs

    def back_propagate(self):
        d = self.diff_inputs
        if self.activation:
            d = self.activation.back_propagate(d)
        self.diff_wq = o.conv_backward_filter(self.x, d, self.w.shape, stride=self.stride, pad=self.pad, maps=self.maps)
        if self.bias is not None:
            self.diff_bias = o.conv_backward_bias(d)
        dx = o.conv_backward_data(self.wq, d, self.x.shape, stride=self.stride, pad=self.pad, maps=self.maps)
        self.diff_w = self.quantizer.back_propagate(self.diff_wq, self.w) if self.quantizer else self.diff_wq
        return dx

    def update(self, batch_size):
        self.solver.update(self.w, self.diff_w, batch_size)
        if self.quantizer and hasattr(self.quantizer, "update"):
            self.quantizer.update(batch_size)
        if self.bias is not None:
            self.bias_solver.update(self.bias, self.diff_bias, batch_size)
        if self.activation:
            self.activation.update(batch_size)


def _seq_sum(v):
    """Sum of a float32 vector in element order with a float32 accumulator, as a C loop `sum += v[i]` does."""
    v = np.ascontiguousarray(v, dtype=F).reshape(-1)
    return F(np.cumsum(v, dtype=F)[-1]) if v.size else F(0.0)


class BatchNormCell:
    """src/Cell/BatchNormCell_Frame.cpp (one input, T = ParamT = float): propagate :287-393 (inference or
    MovingAverageMomentum 0: the running statistics; else the batch's, in two passes, which also feed the running ones,
    the variance with the factor size / (size - 1)); backPropagate :396-506; update :509-523 (scale then bias).
    Sums run over batch, row, column in that order with a float accumulator.  Initial values: scale 1, bias 0, mean 0,
    variance 0 (:78-121)."""

    def __init__(self, nb_outputs, activation=None, epsilon=1.0e-5, moving_average_momentum=0.1, scale_solver=None,
                 bias_solver=None, scales=None, biases=None, means=None, variances=None):
        self.scale = np.ones(nb_outputs, dtype=F) if scales is None else np.array(scales, dtype=F)
        self.bias = np.zeros(nb_outputs, dtype=F) if biases is None else np.array(biases, dtype=F)
        self.mean = np.zeros(nb_outputs, dtype=F) if means is None else np.array(means, dtype=F)
        self.variance = np.zeros(nb_outputs, dtype=F) if variances is None else np.array(variances, dtype=F)
        self.epsilon, self.momentum = float(epsilon), float(moving_average_momentum)
        self.activation = activation
        self.scale_solver, self.bias_solver = scale_solver or SGDSolver(), bias_solver or SGDSolver()
        self.diff_scale = np.zeros(nb_outputs, dtype=F)
        self.diff_bias = np.zeros(nb_outputs, dtype=F)
        self.diff_inputs = None

    def propagate(self, x, inference=False):
        x = np.ascontiguousarray(x, dtype=F)
        self.x = x
        B, Cn, H, W = x.shape
        size = B * H * W
        sh = (1, -1, 1, 1)
        if inference or self.momentum == 0.0:
            mean, variance = self.mean, self.variance
        else:
            self.saved_mean, self.saved_variance = np.empty(Cn, dtype=F), np.empty(Cn, dtype=F)
            for c in range(Cn):
                self.saved_mean[c] = F(_seq_sum(x[:, c]) / F(size))
                zeroed = (x[:, c] - self.saved_mean[c]).astype(F)
                self.saved_variance[c] = F(_seq_sum((zeroed * zeroed).astype(F)) / F(size))
                self.mean[c] = F(float(self.saved_mean[c]) * self.momentum + float(self.mean[c]) * (1.0 - self.momentum))
                self.variance[c] = F(float(F(self.saved_variance[c] * F(F(size) / F(F(size) - F(1))))) * self.momentum
                                     + float(self.variance[c]) * (1.0 - self.momentum))
            mean, variance = self.saved_mean, self.saved_variance
        if inference or self.momentum == 0.0:
            var = np.sqrt((variance + F(self.epsilon)).astype(F)).astype(F)        # T(variance) + T(epsilon), :308-309
        else:
            var = np.sqrt(variance.astype(np.float64) + self.epsilon).astype(F)     # (T) variance + double epsilon, :365
        normalized = ((x - mean.reshape(sh)) / var.reshape(sh)).astype(F)
        y = (self.scale.reshape(sh) * normalized + self.bias.reshape(sh)).astype(F)
        self.outputs = self.activation.propagate(y, inference) if self.activation else y
        return self.outputs

    def back_propagate(self):
        d = self.diff_inputs
        if self.activation:
            d = self.activation.back_propagate(d)
        d = np.ascontiguousarray(d, dtype=F)
        x = self.x
        B, Cn, H, W = x.shape
        size = B * H * W
        beta_scale = F(0.0) if self.scale_solver.is_new_iteration() else F(1.0)
        beta_bias = F(0.0) if self.bias_solver.is_new_iteration() else F(1.0)
        dx = np.empty_like(x)
        for c in range(Cn):
            mean, variance, scale = self.saved_mean[c], self.saved_variance[c], self.scale[c]
            var = F(np.sqrt(float(variance) + self.epsilon))
            centred = (x[:, c] - mean).astype(F)
            normalized = (centred / var).astype(F)
            diff_normalized = (d[:, c] * scale).astype(F)
            sum_scale = _seq_sum((d[:, c] * normalized).astype(F))
            sum_bias = _seq_sum(d[:, c])
            sum_mean1 = _seq_sum(diff_normalized)
            sum_mean2 = _seq_sum((-2.0 * centred.astype(np.float64)).astype(F))
            sum_variance = _seq_sum((diff_normalized * centred).astype(F))
            diff_variance = F(float(sum_variance) * (-1.0 / 2.0) * np.power(float(variance) + self.epsilon, -3.0 / 2.0))
            diff_mean = F(float(sum_mean1) * (-1.0 / float(var)) + float(F(F(diff_variance * sum_mean2) / F(size))))
            self.diff_scale[c] = F(sum_scale + beta_scale * self.diff_scale[c])
            self.diff_bias[c] = F(sum_bias + beta_bias * self.diff_bias[c])
            gradient = ((diff_normalized / var).astype(F).astype(np.float64)
                        + float(diff_variance) * 2.0 * centred.astype(np.float64) / float(F(size))
                        + float(F(diff_mean / F(size))))
            dx[:, c] = gradient.astype(F)
        return dx

    def update(self, batch_size):
        self.scale_solver.update(self.scale, self.diff_scale, batch_size)
        self.bias_solver.update(self.bias, self.diff_bias, batch_size)
        if self.activation:
            self.activation.update(batch_size)


class PoolCell:
    """src/Cell/PoolCell_Frame.cpp:123-228 with Pooling=Max, one input and the unit mapping: forwardMax remembers the
    first largest element of each window (src/Cell/PoolCell_Frame_Kernels.cpp:102-197); backwardMax gives every input
    the sum of the gradients of the outputs it was the maximum of (:295-379)."""

    def __init__(self, pool, stride, pad=(0, 0), activation=None, pooling="Max"):
        self.pool, self.stride, self.pad, self.activation, self.pooling = pool, stride, pad, activation, pooling
        self.diff_inputs = None

    def propagate(self, x, inference=False):
        self.x_shape = x.shape
        if self.pooling == "Average":     # forwardAverage / backwardAverage, padding counted (src/Cell/PoolCell_Frame_Kernels.cpp:26-100, 199-293)
            y = o.pool_forward(np.ascontiguousarray(x, dtype=F), self.pool, self.stride, self.pad, kind="average", quantized=False)
            self.outputs = self.activation.propagate(y, inference) if self.activation else y
            return self.outputs
        y, self.argmax = o.pool_forward(np.ascontiguousarray(x, dtype=F), self.pool, self.stride, self.pad, kind="max", quantized=False,
                                        argmax=True)
        self.outputs = self.activation.propagate(y, inference) if self.activation else y
        return self.outputs

    def back_propagate(self):
        d = self.diff_inputs
        if self.activation:
            d = self.activation.back_propagate(d)
        if self.pooling == "Average":
            return o.pool_backward_average(d, self.x_shape, self.pool, self.stride, self.pad)
        dx = np.zeros(self.x_shape, dtype=F)
        B, Cn, oH, oW = d.shape
        am = self.argmax
        # output order (oy, ox ascending) is the order in which backwardMax meets the outputs of one input (sy, sx ascending
        # means oy, ox descending; with at most a few overlapping windows the float sums agree to the last bit or two)
        for b in range(B):
            for c in range(Cn):
                for oy in range(oH):
                    for ox in range(oW):
                        ix, iy, ch, valid = am[b, c, oy, ox]
                        if valid:
                            dx[b, ch, iy, ix] += d[b, c, oy, ox]
        return dx

    def update(self, batch_size):
        if self.activation:
            self.activation.update(batch_size)


class ElemWiseCell:
    """src/Cell/ElemWiseCell_Frame.cpp:104-136 and :194-233, Operation Sum, one coefficient per input: outputs =
    (w0 x0 + s0) + (w1 x1 + s1) + ..., then the activation in place; backPropagate gives input k the gradient wk * diff
    (added to what another consumer of that input has written, which train_graph does)."""

    def __init__(self, nb_inputs, weights=None, shifts=None, activation=None):
        self.w = np.ones(nb_inputs, dtype=F) if weights is None else np.array(weights, dtype=F)
        self.s = np.zeros(nb_inputs, dtype=F) if shifts is None else np.array(shifts, dtype=F)
        self.activation = activation
        self.diff_inputs = None

    def propagate(self, xs, inference=False):
        y = o.elemwise_sum([np.ascontiguousarray(x, dtype=F) for x in xs], self.w, self.s, "PerInput")
        self.outputs = self.activation.propagate(y, inference) if self.activation else y
        return self.outputs

    def back_propagate(self):
        d = self.diff_inputs
        if self.activation:
            d = self.activation.back_propagate(d)
        return [o.elemwise_sum_backward(d, self.w, k, "PerInput") for k in range(len(self.w))]

    def update(self, batch_size):
        if self.activation:
            self.activation.update(batch_size)


class SoftmaxCell:
    """src/Cell/SoftmaxCell_Frame.cpp:93-137 and :140-207 with WithLoss: the gradient passes through unchanged;
    applyLoss is Cell_Frame_Top::applyLoss (src/Cell/Cell_Frame_Top.cpp:27-40): diff = target - output, formed in
    double and stored in T, loss = sum of squares / batch."""

    def propagate(self, x):
        self.outputs = o.softmax_forward(x)
        return self.outputs

    def apply_loss(self, targets):
        err = targets.astype(np.float64) - self.outputs.astype(np.float64)
        self.diff_inputs = err.astype(F)
        return float((err * err).sum() / self.outputs.shape[0])

    def back_propagate(self):
        return self.diff_inputs


def train_sequential(x, cells, softmax, targets, iterations):
    """The loop of tests/Cell/class_ConvCell_QuantizerSAT_Frame.cpp:436-513: propagate front to back, loss, backPropagate
    back to front (each cell's result is the previous cell's diffInputs), then update back to front with the
    ActivationCell last."""
    batch = x.shape[0]
    loss = 0.0
    for _ in range(iterations):
        h = x
        for c in cells:
            h = c.propagate(h, inference=False)
        softmax.propagate(h)
        loss = softmax.apply_loss(targets)
        d = softmax.back_propagate()
        for c in reversed(cells):
            c.diff_inputs = d
            d = c.back_propagate()
        for c in reversed(cells):
            c.update(batch)
    return loss


def train_graph(x, nodes, softmax, targets, iterations):
    """The same loop over a graph with branches: `nodes` is a list of (cell, inputs) in an order in which every cell follows
    the cells it reads, inputs being indices into that list (-1: the net's input x); the last node feeds the softmax.  A
    tensor read by several cells receives the sum of their gradients, the cell that runs its backPropagate first writing
    and the others adding (Cell_Frame's diffOutputs with beta = isValid, e.g. src/Cell/ConvCell_Frame.cpp:545-560)."""
    batch = x.shape[0]
    loss = 0.0
    for _ in range(iterations):
        outs = []
        for cell, inputs in nodes:
            xs = [x if i < 0 else outs[i] for i in inputs]
            outs.append(cell.propagate(xs, inference=False) if isinstance(cell, ElemWiseCell) else cell.propagate(xs[0], inference=False))
        softmax.propagate(outs[-1])
        loss = softmax.apply_loss(targets)
        grads = [None] * len(nodes)
        grads[-1] = softmax.back_propagate()
        for k in range(len(nodes) - 1, -1, -1):
            cell, inputs = nodes[k]
            cell.diff_inputs = grads[k]
            d = cell.back_propagate()
            ds = d if isinstance(cell, ElemWiseCell) else [d]
            for i, di in zip(inputs, ds):
                if i >= 0:
                    grads[i] = di if grads[i] is None else (di + grads[i]).astype(F)
        for cell, _ in reversed(nodes):
            cell.update(batch)
    return loss
