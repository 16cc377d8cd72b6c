"""CPU oracle (TEST INFRASTRUCTURE, not the product) of the pass that turns a SAT-trained float graph into integer
cells: restatement of DeepNetQAT::QuantizeAndfuseBatchNormWithConv, ::QuantizeFC and ::QuantizeElemWise
(src/Quantizer/QAT/Optimization/DeepNetQAT.cpp:902-1326, :655-900, :521-653) and of the (range, alpha) pairs
fuseQATGraph threads through a sequential net (:87-520), plus the inference pass of BatchNormCell_Frame
(src/Cell/BatchNormCell_Frame.cpp:297-322) that the float side of the parity check needs.

Pinned by tests/test_oracle_qat_fuse.py on the trained parameters N2D2's own test of this pass loads
(tests/golden/sat_lenet_bn): every fused stage, fed the integer graph's own input, must reproduce what the float graph
(convolution with the quantized weights, batch normalisation, SAT activation) computes from the same input to within
one output level, for 8-bit and 4-bit weights; a dropped term, a wrong sign or a swapped (range, alpha) breaks that for
every output.  The arithmetic types follow the reference: Float_T results formed in long double where a `long double`
factor takes part.  Cited paths are relative to the N2D2 source tree."""
import numpy as np

F = np.float32
LD = np.longdouble


def _rintf(x):
    return np.rint(np.asarray(x, dtype=F)).astype(F)


def batchnorm_inference(x, scales, biases, means, variances, eps=1.0e-5):
    """BatchNormCell_Frame<float>::propagate(inference): scale * (x - mean) / sqrt(var + eps) + bias, in float."""
    sh = (1, -1, 1, 1)
    var = np.sqrt(variances.astype(F) + F(eps)).astype(F)
    normalized = ((x.astype(F) - means.astype(F).reshape(sh)) / var.reshape(sh)).astype(F)
    return (scales.astype(F).reshape(sh) * normalized + biases.astype(F).reshape(sh)).astype(F)


def _weights_scale_factor(w_range, rounding, first_range):
    """DeepNetQAT.cpp:987-1003 / :720-735: floor(range / 2) of the weight quantizer when weights are rounded, else 1."""
    wsf = LD(1.0)
    if rounding:
        wsf = LD(np.floor(first_range / 2.0))
    if w_range is not None:
        if rounding:
            wsf = LD(np.floor(w_range / 2.0)) if w_range > 1 else LD(1)
    return wsf


def quantize_and_fuse_batchnorm_with_conv(ranges, alphas, quant_weights, conv_bias, w_range, w_mode_default,
                                          bn_scales, bn_biases, bn_means, bn_variances, eps, act_range, act_alpha,
                                          w_round=True, b_round=True, c_round=True):
    """DeepNetQAT::QuantizeAndfuseBatchNormWithConv.  ranges / alphas: (input, output) pairs as the caller holds them
    before the call (only .first is read; .second is replaced by the BatchNorm's SAT activation quantizer: act_range,
    act_alpha).  quant_weights: the weight quantizer's tensor [O, C, kH, kW] (the weights themselves if w_range is
    None); conv_bias: [O] or None (NoBias).
    Returns (weights, biases, scaling, clipping, weight_bits, act_bits, ranges, alphas) with the pairs as the call
    leaves them."""
    r1, a1 = int(ranges[0]), float(alphas[0])
    r2, a2 = int(act_range), float(F(act_alpha))
    wsf = _weights_scale_factor(w_range, w_round, r1)
    corr = 1.0
    if w_range is not None and w_mode_default:
        # :1005-1017: 4-bit weights of the default mode are odd multiples of 1/15: carried on 5 bits
        if wsf == (LD(7.0) if w_round else LD(8.0)):
            wsf, corr, r1 = LD(15.0), 2.066666666666667, 31
    bsf = wsf
    O = quant_weights.shape[0]
    w_out = np.empty(quant_weights.shape, dtype=np.float64)
    bias_out, clip_out, scal_out = np.zeros(O, dtype=F), np.zeros(O, dtype=F), np.zeros(O, dtype=F)
    for o in range(O):
        var = float(bn_variances[o])
        factor = float(bn_scales[o]) / np.sqrt(eps + var) if var > 1.0e-12 else 0.0
        sign = -1.0 if factor < 0.0 else 1.0
        bias = 0.0 if conv_bias is None else float(conv_bias[o])
        k = (quant_weights[o].astype(np.float64).astype(LD) * wsf).astype(np.float64)
        if w_round:
            k = _rintf(k).astype(np.float64)
        w_out[o] = k * sign
        if factor == 0.0:
            s = b = c = F(0.0)
        else:
            s = F(LD((a1 / float(F(r1))) * (float(F(r2)) / a2) * factor) * (LD(1) / wsf) * LD(corr))
            b = F(LD((((float(bn_biases[o]) + (bias - float(bn_means[o])) * factor) / factor) * r1 / a1)) * bsf
                  * LD(1.0 / corr))
            c = F(LD((a2 * r1) / (factor * a1)) * wsf * LD(1.0 / corr))
            s, b, c = F(s * sign), F(b * sign), F(c * sign)
        if c_round:
            c = _rintf(c)
        if b_round:
            b = _rintf(b)
        scal_out[o], bias_out[o], clip_out[o] = s, b, c
    weights_range = 1 if w_range is None else (2 if w_range == 1 else w_range)
    weight_bits = int(_rintf(np.log2(weights_range)))
    act_bits = int(_rintf(np.log2(r2)))
    return w_out.astype(F), bias_out, scal_out, clip_out, weight_bits, act_bits, (r2, r2), (a2, a2)


def quantize_fc(ranges, alphas, quant_weights, fc_bias, w_range, sat_scaling, act_range, act_alpha,
                w_round=True, b_round=True, c_round=True):
    """DeepNetQAT::QuantizeFC.  quant_weights [O, K]; sat_scaling: the divisor SATQuantizerCell applied to them
    (getSAT_scaling, 1 without ApplyScaling), read only when weights are rounded; act_range / act_alpha: the SAT
    quantizer of the cell's activation, or None.
    Returns (weights, biases or None, scaling, clipping, is_clipped, weight_bits, act_bits, ranges, alphas)."""
    r1, a1 = int(ranges[0]), float(alphas[0])
    r2, a2 = (int(ranges[1]), float(alphas[1])) if act_range is None else (int(act_range), float(F(act_alpha)))
    wsf, sat = LD(1.0), LD(1.0)
    if w_range is not None and w_round:
        wsf = LD(np.floor(w_range / 2.0)) if w_range > 1 else LD(1)
        sat = LD(float(sat_scaling))
    bsf = wsf * sat if w_range is not None else wsf
    in_scale = r1 / a1
    out_scale = float(r1) if act_range is None else r2 / a2
    k = (quant_weights.astype(np.float64).astype(LD) * (wsf * sat)).astype(np.float64)
    if w_round:
        k = _rintf(k).astype(np.float64)
    O = quant_weights.shape[0]
    s = F(LD(out_scale / in_scale) * (LD(1.0) / (sat * wsf)))
    c = F(LD(a2 * in_scale) * (wsf * sat))
    if c < 0.0:
        c = F(0.0)
    if c_round:
        c = _rintf(c)
    biases = None
    if fc_bias is not None:
        biases = ((fc_bias.astype(np.float64) * in_scale).astype(LD) * bsf).astype(F)
        if b_round:
            biases = _rintf(biases)
    weights_range = 1 if w_range is None else (2 if w_range == 1 else w_range)
    weight_bits = int(_rintf(np.log2(weights_range)))
    is_clipped = act_range is not None
    act_bits = int(_rintf(np.log2(r2))) if is_clipped else int(_rintf(np.log2(float(2 ** 32 - 1))))
    return (k.astype(F), biases, np.full(O, s, dtype=F), np.full(O, c, dtype=F), is_clipped, weight_bits, act_bits,
            (r2, r2), (a2, a2))


def quantize_elemwise(ranges, alphas, range_parent0, alpha_parent0, nb_outputs, act_range, act_alpha):
    """DeepNetQAT::QuantizeElemWise: the sum takes the levels of its first parent; its SAT activation quantizer, if any,
    becomes a clip at alpha (in input levels) and a rescale to the output levels.
    Returns (scaling, clipping, act_bits or None, ranges, alphas)."""
    r1, a1 = int(range_parent0), float(alpha_parent0)
    r2, a2 = (int(ranges[1]), float(alphas[1])) if act_range is None else (int(act_range), float(F(act_alpha)))
    in_scale, out_scale = r1 / a1, r2 / a2
    s = np.full(nb_outputs, F(out_scale / in_scale), dtype=F)
    c = np.full(nb_outputs, F(a2 * in_scale), dtype=F)
    act_bits = None if act_range is None else int(_rintf(np.log2(r2)))
    return s, c, act_bits, (r2, r2), (a2, a2)
