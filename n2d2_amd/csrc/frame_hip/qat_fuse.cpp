// Host-side pass from a SAT-trained float graph to the integer cells: the arithmetic of
// src/Quantizer/QAT/Optimization/DeepNetQAT.cpp on plain trained values.  Plain C++, no device code.
//
// A float stage computes  y = round(clamp(z, 0, a2) / a2 * R2)  with  z = f * (sum(w_q * x) + b - mean) + beta,
// f = gamma / sqrt(var + eps), inputs x = x_int * a1 / R1 and quantized weights w_q = w_int / S.  In accumulator units
// that is  y = round(clip(sum(w_int * x_int) + B, C) * M)  with
//   M = a1 / R1 * R2 / a2 * f / S,   B = (beta / f + b - mean) * R1 / a1 * S,   C = a2 * R1 / (f * a1) * S,
// which is what each function below installs (weights, B and C optionally rounded to integers).  A negative f flips the
// sign of the weights, of B, of C and of M, so that the clip still acts on the side that the activation keeps.
// The expressions keep the reference's operand order and types (Float_T results formed in long double where a
// long double factor takes part), so that the installed values are the reference's, bit for bit.
#include "frame_hip.hpp"

#include <cmath>

namespace N2D2 {

namespace {

std::size_t bitsOf(double range)
{
    return (std::size_t)rintf((float)std::log2(range));
}

void checkSize(const std::vector<double>& v, std::size_t n, const char* what, const std::string& cell)
{
    if (v.size() != n)
        throw std::runtime_error(std::string("DeepNetQAT: BatchNorm ") + what + " do not match the outputs of " + cell);
}

// value * factor, rounded as rintf does when asked, times sign: one trained weight on its way to an integer cell
inline Float_T scaledWeight(Float_T q, long double factor, bool round, double sign)
{
    double k = (double)((double)q * factor);
    if (round)
        k = rintf((float)k);
    return (Float_T)(k * sign);
}

} // namespace

bool DeepNetQAT::QuantizeAndfuseBatchNormWithConv(std::pair<std::size_t, std::size_t>& rangeConvBN, std::pair<double, double>& alphasConvBN,
                                                  ConvCell& convCell, const QATCellParameters& trained, const BatchNormParameters& bn,
                                                  ScalingMode actScalingMode, WeightsApprox wMode, WeightsApprox bMode, WeightsApprox cMode)
{
    const std::size_t nbOutputs = convCell.getNbOutputs();
    checkSize(bn.scales, nbOutputs, "scales", convCell.getName());
    checkSize(bn.biases, nbOutputs, "biases", convCell.getName());
    checkSize(bn.means, nbOutputs, "means", convCell.getName());
    checkSize(bn.variances, nbOutputs, "variances", convCell.getName());
    if (!(bn.epsilon > 0.0))
        throw std::runtime_error("DeepNetQAT: BatchNorm Epsilon must be positive");
    if (trained.quantWeights.empty() || trained.quantWeights.size() % nbOutputs != 0)
        throw std::runtime_error("DeepNetQAT: the trained weights do not match the outputs of " + convCell.getName());
    const bool noBias = trained.biases.empty();
    if (!noBias && trained.biases.size() != nbOutputs)
        throw std::runtime_error("DeepNetQAT: the trained biases do not match the outputs of " + convCell.getName());
    // Fuse only if the convolution has a linear activation, and only a SAT-quantized BatchNorm activation (:934-983)
    if (convCell.getActivation() && std::string(convCell.getActivation()->getType()) != "Linear")
        return false;
    if (bn.actRange == 0)
        return false;
    alphasConvBN.second = (double)(Float_T)bn.actAlpha;
    rangeConvBN.second = bn.actRange;

    long double weightsScaleFactor = 1.0;
    if (wMode == WeightsApprox::RINTF)
        weightsScaleFactor = std::floor(rangeConvBN.first / 2.0);
    long double biasScaleFactor = weightsScaleFactor;
    double corrFactor = 1.0;
    if (trained.weightsRange > 0) {
        if (wMode == WeightsApprox::RINTF)
            weightsScaleFactor = trained.weightsRange > 1 ? std::floor(trained.weightsRange / 2.0) : 1;
        // 4-bit weights of the default mode are odd multiples of 1/15: kept exactly on 5 bits (:1005-1017)
        if (trained.defaultQuantMode) {
            const long double bitRangeThreshold = wMode == WeightsApprox::RINTF ? 7.0 : 8.0;
            if (weightsScaleFactor == bitRangeThreshold) {
                weightsScaleFactor = 15.0;
                corrFactor = 2.066666666666667;
                rangeConvBN.first = 31;
            }
        }
        biasScaleFactor = weightsScaleFactor;
    }

    std::shared_ptr<Activation> activation = Registrar<RectifierActivation>::create<Float_T>("Frame_HIP")();
    convCell.setActivation(activation);
    convCell.setParameter("NoBias", false);

    const std::size_t perOutput = trained.quantWeights.size() / nbOutputs;
    Tensor<Float_T> weights = trained.quantWeights;
    Tensor<Float_T> biases({nbOutputs});
    std::vector<Float_T> biasPerOutput(nbOutputs, 0.0f), clipPerOutput(nbOutputs, 0.0f), scalingPerOutput(nbOutputs, 0.0f);
    for (std::size_t output = 0; output < nbOutputs; ++output) {
        const double factor = bn.variances[output] > 1.0e-12 ? bn.scales[output] / std::sqrt(bn.epsilon + bn.variances[output]) : 0.0;
        const double factorSign = factor < 0.0 ? -1.0 : 1.0;
        const double bias = noBias ? 0.0 : (double)trained.biases(output);
        for (std::size_t index = 0; index < perOutput; ++index)
            weights(output * perOutput + index)
                = scaledWeight(trained.quantWeights(output * perOutput + index), weightsScaleFactor, wMode == WeightsApprox::RINTF, factorSign);
        if (factor != 0.0) {
            scalingPerOutput[output] = (alphasConvBN.first / (float)rangeConvBN.first) * ((float)rangeConvBN.second / alphasConvBN.second)
                                       * factor * (1 / weightsScaleFactor) * corrFactor;
            biasPerOutput[output] = ((((bn.biases[output] + (bias - bn.means[output]) * factor) / factor) * rangeConvBN.first
                                      / alphasConvBN.first) * biasScaleFactor) * (1.0 / corrFactor);
            clipPerOutput[output] = ((alphasConvBN.second * rangeConvBN.first) / (factor * alphasConvBN.first)) * weightsScaleFactor
                                    * (1.0 / corrFactor);
            scalingPerOutput[output] *= factorSign;
            biasPerOutput[output] *= factorSign;
            clipPerOutput[output] *= factorSign;
        }
        // a channel whose variance vanished (factor 0) keeps scaling, bias and clip 0: it outputs 0
        if (cMode == WeightsApprox::RINTF)
            clipPerOutput[output] = rintf(clipPerOutput[output]);
        if (bMode == WeightsApprox::RINTF)
            biasPerOutput[output] = rintf(biasPerOutput[output]);
        biases(output) = biasPerOutput[output];
    }
    convCell.setWeights(weights);
    convCell.setBiases(biases);

    std::size_t weightsRange = trained.weightsRange > 0 ? trained.weightsRange : 1;
    if (trained.weightsRange == 1)
        weightsRange = 2;                // 1-bit weights
    convCell.setQuantized(bitsOf((double)weightsRange));
    activation->setQuantized(bitsOf((double)rangeConvBN.second));

    const bool isClipped = true;
    if (actScalingMode == ScalingMode::FLOAT_MULT) {
        activation->setActivationScaling(Scaling::floatingPointScaling(scalingPerOutput, isClipped, clipPerOutput));
    } else if (actScalingMode == ScalingMode::FIXED_MULT16 || actScalingMode == ScalingMode::FIXED_MULT32) {
        const std::size_t nbFractionalBits = 16;
        std::vector<std::int32_t> scalingFixedPoint;
        for (const Float_T sc : scalingPerOutput)
            scalingFixedPoint.push_back((std::int32_t)std::round(sc * (1ull << nbFractionalBits)));
        activation->setActivationScaling(Scaling::fixedPointScaling(actScalingMode, nbFractionalBits, scalingFixedPoint, isClipped, clipPerOutput));
    } else if (actScalingMode == ScalingMode::SINGLE_SHIFT) {
        std::vector<unsigned char> shifts(nbOutputs, 0);
        for (std::size_t out = 0; out < nbOutputs; ++out)
            if (scalingPerOutput[out] > 0.0)
                shifts[out] = DeepNetQuantization::approximateScalingWithPowerOf2Divs(scalingPerOutput[out], 1).first[0];
        activation->setActivationScaling(Scaling::singleShiftScaling(shifts, isClipped, clipPerOutput));
    } else {
        // the reference leaves the activation without Scaling for the other modes
        throw std::runtime_error("DeepNetQAT: activation scaling mode must be FLOAT_MULT, FIXED_MULT16, FIXED_MULT32 or SINGLE_SHIFT");
    }
    rangeConvBN.first = rangeConvBN.second;
    alphasConvBN.first = alphasConvBN.second;
    return true;
}

bool DeepNetQAT::QuantizeFC(std::pair<std::size_t, std::size_t>& rangeOpFc, std::pair<double, double>& alphaOpFC, FcCell& fcCell,
                            const QATCellParameters& trained, std::size_t actRange, double actAlpha, WeightsApprox wMode,
                            WeightsApprox bMode, WeightsApprox cMode)
{
    const std::size_t nbOutputs = fcCell.getNbOutputs();
    if (trained.quantWeights.empty() || trained.quantWeights.size() % nbOutputs != 0)
        throw std::runtime_error("DeepNetQAT: the trained weights do not match the outputs of " + fcCell.getName());
    const bool noBias = trained.biases.empty();
    if (!noBias && trained.biases.size() != nbOutputs)
        throw std::runtime_error("DeepNetQAT: the trained biases do not match the outputs of " + fcCell.getName());
    std::shared_ptr<Activation> activation = fcCell.getActivation();
    if (!activation)
        throw std::runtime_error("DeepNetQAT: " + fcCell.getName() + " needs an activation to carry the Scaling");
    if (actRange > 0) {
        alphaOpFC.second = (double)(Float_T)actAlpha;
        rangeOpFc.second = actRange;
    }
    long double weightsScaleFactor = 1.0;
    long double biasScaleFactor = weightsScaleFactor;
    long double SAT_scaling = 1.0;
    if (trained.weightsRange > 0) {
        if (wMode == WeightsApprox::RINTF) {
            weightsScaleFactor = trained.weightsRange > 1 ? std::floor(trained.weightsRange / 2.0) : 1;
            SAT_scaling = trained.satScaling;
        }
        biasScaleFactor = weightsScaleFactor * SAT_scaling;
    }
    const double scaleFactorInput = rangeOpFc.first / alphaOpFC.first;
    double scaleFactorOutput = rangeOpFc.first;
    if (actRange > 0)
        scaleFactorOutput = rangeOpFc.second / alphaOpFC.second;

    const std::size_t perOutput = trained.quantWeights.size() / nbOutputs;
    Tensor<Float_T> weights = trained.quantWeights;
    Tensor<Float_T> biases({nbOutputs});
    std::vector<Float_T> biasPerOutput(nbOutputs, 0.0f), clipPerOutput(nbOutputs, 0.0f), scalingPerOutput(nbOutputs, 0.0f);
    for (std::size_t output = 0; output < nbOutputs; ++output) {
        for (std::size_t index = 0; index < perOutput; ++index)
            weights(output * perOutput + index) = scaledWeight(trained.quantWeights(output * perOutput + index),
                                                               weightsScaleFactor * SAT_scaling, wMode == WeightsApprox::RINTF, 1.0);
        scalingPerOutput[output] = (scaleFactorOutput / scaleFactorInput) * (1.0 / (SAT_scaling * weightsScaleFactor));
        clipPerOutput[output] = alphaOpFC.second * scaleFactorInput * (weightsScaleFactor * SAT_scaling);
        if (!noBias)
            biasPerOutput[output] = (double)trained.biases(output) * scaleFactorInput * biasScaleFactor;
        if (clipPerOutput[output] < 0.0)
            clipPerOutput[output] = 0.0;
        if (cMode == WeightsApprox::RINTF)
            clipPerOutput[output] = rintf(clipPerOutput[output]);
        if (bMode == WeightsApprox::RINTF && !noBias)
            biasPerOutput[output] = rintf(biasPerOutput[output]);
        biases(output) = biasPerOutput[output];
    }
    fcCell.setWeights(weights);
    fcCell.setParameter("NoBias", noBias);       // the integer cell takes over the trained cell's NoBias
    if (!noBias)
        fcCell.setBiases(biases);

    std::size_t weightsRange = trained.weightsRange > 0 ? trained.weightsRange : 1;
    if (trained.weightsRange == 1)
        weightsRange = 2;
    fcCell.setQuantized(bitsOf((double)weightsRange));
    const bool isClipped = actRange > 0;
    const std::size_t activationsRange = isClipped ? rangeOpFc.second : (std::size_t)(std::pow(2, 32) - 1);
    activation->setActivationScaling(Scaling::floatingPointScaling(scalingPerOutput, isClipped, clipPerOutput));
    activation->setQuantized(bitsOf((double)activationsRange));
    rangeOpFc.first = rangeOpFc.second;
    alphaOpFC.first = alphaOpFC.second;
    return true;
}

bool DeepNetQAT::QuantizeElemWise(std::pair<std::size_t, std::size_t>& rangeElWise, std::pair<double, double>& alphaElWise,
                                  std::size_t rangeParent0, double alphaParent0, ElemWiseCell& elemWiseCell, std::size_t actRange,
                                  double actAlpha)
{
    rangeElWise.first = rangeParent0;
    alphaElWise.first = alphaParent0;
    if (actRange > 0) {
        alphaElWise.second = (double)(Float_T)actAlpha;
        rangeElWise.second = actRange;
    }
    const std::size_t nbOutputs = elemWiseCell.getNbOutputs();
    const double scaleFactorInput = (double)rangeElWise.first / alphaElWise.first;
    const double scaleFactorOutput = (double)rangeElWise.second / alphaElWise.second;
    std::vector<Float_T> clipPerOutput(nbOutputs, (Float_T)(alphaElWise.second * scaleFactorInput));
    std::vector<Float_T> scalingPerOutput(nbOutputs, (Float_T)(scaleFactorOutput / scaleFactorInput));
    if (elemWiseCell.getActivation()) {
        if (actRange > 0)
            elemWiseCell.setQuantized(bitsOf((double)rangeElWise.second));
        std::shared_ptr<Activation> activation = Registrar<RectifierActivation>::create<Float_T>("Frame_HIP")();
        activation->setParameter("Clipping", (double)rangeElWise.second);
        activation->setActivationScaling(Scaling::floatingPointScaling(scalingPerOutput, true, clipPerOutput));
        elemWiseCell.setActivation(activation);
    }
    rangeElWise.first = rangeElWise.second;
    alphaElWise.first = alphaElWise.second;
    return true;
}

} // namespace N2D2
