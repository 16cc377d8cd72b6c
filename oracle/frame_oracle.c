/* TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.
 *
 * CPU restatement ("oracle") of the N2D2 Frame (CPU) cells on the quantized
 * inference path: conv / fc / pool / scaling / activations and the SAT / LSQ
 * fake-quant kernels.  Only tests, the smoke check and the CPU-baseline leg of
 * the benchmark may load this library; the shipped HIP path never does.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the N2D2 source tree).  Element type T is instantiated for float (the type
 * N2D2 registers its cells with) and double (exact for all integer sums).
 *
 * Build: make -C oracle   (gcc, -ffp-contract=off so that no a*b+c is fused:
 * the reference is built for baseline x86-64, which has no FMA).
 *
 * What pins each function (the tests named are the CPU tests of this
 * repository; none of them runs reference code):
 *   conv forward / bias, fc, pool, elemwise, the four rescales, saturate,
 *   Clip, Rectifier / Linear, getNbGroups, output sizes
 *       tests/test_oracle_int.py: integer closed forms, the brute-force loop
 *       and the shape grid of the reference's own ConvCell test, exact
 *       rational forms of the rescales, exhaustive window sums of the pools.
 *   SAT / LSQ kernels
 *       tests/test_oracle_quant.py: the formulas the reference's quantizer
 *       tests recompute, exact ties, weights exported by N2D2 itself
 *       (tests/golden/sat_lenet4b).
 *   conv backward (data, filter, bias), softmax, and with them the SAT / LSQ
 *   backward kernels and solver updates end to end
 *       tests/test_oracle_qat_train.py: adjoint identities and the Jacobian
 *       of the forward, and the reference's PyTorch-derived known-answer
 *       tests (trained SAT alphas; LSQ step sizes of a conv net and an FC).
 *   average pooling (float forward, backward), the ElemWise sum's gradient
 *       tests/test_oracle_qat_train.py: a library routine (torch's
 *       avg_pool2d and its autograd in float64, both divisors), the adjoint
 *       identity <dy, A x> = <A^T dy, x>, and for the sum the rounded
 *       product weight * dy and the directional derivative of its forward.
 * Parity unpinned, by nature: the ORDER in which float reductions add their
 * terms where the reference runs them under OpenMP or through
 * std::accumulate (the restatement adds in element order), and the last bit
 * of libm's tanh / cosh / exp against the device's.  GPU tests hold such
 * results to 1e-5 of the sum of the terms' magnitudes.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline int imax_(int a, int b) { return a > b ? a : b; }
/* Utils::clamp<int>, include/utils/Utils.hpp:1038-1042 */
static inline int iclamp_(int x, int lo, int hi) { return x < lo ? lo : (x > hi ? hi : x); }

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)

#define T float
#define FN(name) CAT(oracle_, CAT(name, _f32))
#define ROUND roundf
#define TRUNC truncf
#define TANH tanhf
#define COSH coshf
#define FABS fabsf
#define SQRT sqrtf
#define EXP expf
#include "frame_oracle_impl.inc"
#undef T
#undef FN
#undef ROUND
#undef TRUNC
#undef TANH
#undef COSH
#undef FABS
#undef SQRT
#undef EXP

#define T double
#define FN(name) CAT(oracle_, CAT(name, _f64))
#define ROUND round
#define TRUNC trunc
#define TANH tanh
#define COSH cosh
#define FABS fabs
#define SQRT sqrt
#define EXP exp
#include "frame_oracle_impl.inc"
#undef T
#undef FN

/* src/Cell/ElemWiseCell_Frame.cpp:116-136 (Sum). ElemWiseCell_Frame is
 * Float_T only. coeffMode: 0 PerLayer, 1 PerInput, 2 PerChannel.
 * inputs: nbInputs pointers to NCHW tensors of identical shape. */
void oracle_elemwise_sum_f32(const float* const* inputs, int nbInputs, int B, int C, int H, int W,
                             const float* weights, const float* shifts, int coeffMode, float* out)
{
    for (int b = 0; b < B; ++b)
        for (int ch = 0; ch < C; ++ch)
            for (int y = 0; y < H; ++y)
                for (int x = 0; x < W; ++x) {
                    const size_t i = (size_t)x + (size_t)W * ((size_t)y + (size_t)H * ((size_t)ch + (size_t)C * b));
                    const size_t c0 = (coeffMode == 2) ? (size_t)ch : 0;
                    out[i] = weights[c0] * inputs[0][i] + shifts[c0];
                    for (int k = 1; k < nbInputs; ++k) {
                        const size_t c1 = (coeffMode == 2) ? c0 : (size_t)k;
                        out[i] += weights[c1] * inputs[k][i] + shifts[c1];
                    }
                }
}

/* src/Cell/ElemWiseCell_Frame.cpp:194-233 (backPropagate, Sum): the gradient towards input k,
 * diffOutput = weights[coeffIdx] * diffInput + beta * diffOutput, coeffIdx = channel (PerChannel) or k. */
void oracle_elemwise_sum_backward_f32(const float* diffInput, int B, int C, int H, int W, const float* weights,
                                      int coeffMode, int k, float beta, float* diffOutput)
{
    for (int b = 0; b < B; ++b)
        for (int ch = 0; ch < C; ++ch)
            for (int y = 0; y < H; ++y)
                for (int x = 0; x < W; ++x) {
                    const size_t i = (size_t)x + (size_t)W * ((size_t)y + (size_t)H * ((size_t)ch + (size_t)C * b));
                    const size_t coeffIdx = (coeffMode == 2) ? (size_t)ch : (size_t)k;
                    const float product = weights[coeffIdx] * diffInput[i];
                    const float kept = (beta != 0.0f) ? beta * diffOutput[i] : 0.0f;
                    diffOutput[i] = product + kept;
                }
}

/* src/Cell/PoolCell_Frame_Kernels.cpp:199-293 (backwardAverage) with the unit mapping (every output pools its own
 * channel, poolChannelsCount = 1).  Returns -1 where the reference throws (exclude padding). */
int oracle_pool_backward_average_f32(const float* alpha, const float* diffInputs, int B, int C, int H, int W,
                                     const int pool[2], const int stride[2], const int pad[2], const float* beta,
                                     float* diffOutputs, int outW, int outH, int countIncludePadding)
{
    if (!countIncludePadding)
        return -1;
    const unsigned int oxStride = (unsigned int)stride[0] * (unsigned int)outW;
    const unsigned int oyStride = (unsigned int)stride[1] * (unsigned int)outH;
    for (int b = 0; b < B; ++b)
        for (int channel = 0; channel < C; ++channel)
            for (unsigned int iy = 0; iy < (unsigned int)H; ++iy)
                for (unsigned int ix = 0; ix < (unsigned int)W; ++ix) {
                    const unsigned int ixPad = ix + (unsigned int)pad[0], iyPad = iy + (unsigned int)pad[1];
                    const unsigned int sxMax = (unsigned int)pool[0] < ixPad + 1 ? (unsigned int)pool[0] : ixPad + 1;
                    const unsigned int syMax = (unsigned int)pool[1] < iyPad + 1 ? (unsigned int)pool[1] : iyPad + 1;
                    float poolGradient = 0.0f;
                    for (unsigned int sy = iyPad % (unsigned int)stride[1], sx0 = ixPad % (unsigned int)stride[0]; sy < syMax;
                         sy += (unsigned int)stride[1]) {
                        if (iyPad >= oyStride + sy)
                            continue;
                        for (unsigned int sx = sx0; sx < sxMax; sx += (unsigned int)stride[0]) {
                            if (ixPad >= oxStride + sx)
                                continue;
                            const unsigned int ox = (ixPad - sx) / (unsigned int)stride[0];
                            const unsigned int oy = (iyPad - sy) / (unsigned int)stride[1];
                            poolGradient += diffInputs[ox + (size_t)outW * (oy + (size_t)outH * ((size_t)channel + (size_t)C * b))] / 1u;
                        }
                    }
                    const unsigned int poolCount = (unsigned int)(pool[0] * pool[1]);
                    const size_t i = ix + (size_t)W * (iy + (size_t)H * ((size_t)channel + (size_t)C * b));
                    const float scaled = (*alpha) * (poolGradient / poolCount);
                    const float kept = (*beta != 0.0f) ? (*beta) * diffOutputs[i] : 0.0f;
                    diffOutputs[i] = scaled + kept;
                }
    return 0;
}

/* src/Cell/Cell.cpp:251-300 (getNbGroups), regular case only: returns -1 where
 * the reference falls back to getNbGroupsHandMade (irregular mappings).
 * map[o + O*c], Tensor<bool> {O,C}. */
long oracle_get_nb_groups(const unsigned char* map, size_t nbOutputs, size_t nbChannels)
{
    size_t nbChannelsPerGroup = 0;
    for (; nbChannelsPerGroup < nbChannels && map[0 + nbOutputs * nbChannelsPerGroup];
         ++nbChannelsPerGroup) {}
    if (nbChannelsPerGroup == 0)
        return 0;
    if (nbChannels % nbChannelsPerGroup != 0)
        return -1;
    const size_t nbGroups = nbChannels / nbChannelsPerGroup;
    if (nbOutputs % nbGroups != 0)
        return -1;
    const size_t nbOutputsPerGroup = nbOutputs / nbGroups;
    size_t outputGroupOffset = 0, channelGroupOffset = 0;
    for (size_t group = 0; group < nbGroups; ++group) {
        for (size_t output = outputGroupOffset; output < outputGroupOffset + nbOutputsPerGroup; ++output) {
            size_t channel = 0;
            for (; channel < channelGroupOffset; ++channel)
                if (map[output + nbOutputs * channel]) return -1;
            for (; channel < channelGroupOffset + nbChannelsPerGroup; ++channel)
                if (!map[output + nbOutputs * channel]) return -1;
            for (; channel < nbChannels; ++channel)
                if (map[output + nbOutputs * channel]) return -1;
        }
        outputGroupOffset += nbOutputsPerGroup;
        channelGroupOffset += nbChannelsPerGroup;
    }
    return (long)nbGroups;
}

/* src/Cell/ConvCell.cpp:1169-1195 (setOutputsDims, no ext padding) */
unsigned int oracle_conv_out_dim(unsigned int in, unsigned int k, unsigned int stride,
                                 unsigned int pad, unsigned int dil, unsigned int subSample)
{
    const int kernelExtent = (int)(dil * (k - 1) + 1);
    return (unsigned int)ceil(floor(((int)in + 2 * (int)pad - kernelExtent + (int)stride)
                                    / (double)stride) / (double)subSample);
}

/* src/Cell/PoolCell.cpp:219-240 (setOutputsDims, no ext padding) */
unsigned int oracle_pool_out_dim(unsigned int in, unsigned int pool, unsigned int stride, unsigned int pad)
{
    return (unsigned int)(((int)in + 2 * (int)pad - (int)pool + (int)stride) / (double)stride);
}
