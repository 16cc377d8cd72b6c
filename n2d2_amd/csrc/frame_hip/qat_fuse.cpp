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

// How a cell's trained weights land on integers.
struct WeightGrid {
    long double levels = 1.0;        // integer steps per unit of trained weight (1: the weights stay as trained)
    long double biasLevels = 1.0;    // the same for a bias expressed in accumulator units
    double stretch = 1.0;            // 31 / 15 once a 4-bit grid has been widened to 5 bits
    bool widened = false;            // the stage must then count its input on 31 levels
};

// Convolutions: `half` levels on either side of zero when the weights are rounded.  Default-mode 4-bit weights are odd
// multiples of 1/15, which no 7- or 8-level grid holds: they go on 15 levels, i.e. 5 bits, and every quantity counted in
// accumulator units is stretched by 31/15 (ref: src/Quantizer/QAT/Optimization/DeepNetQAT.cpp:988-1023).
WeightGrid convGrid(const QATCellParameters& trained, bool rounded, std::size_t inputRange)
{
    WeightGrid g;
    if (rounded)
        g.levels = std::floor(inputRange / 2.0);
    g.biasLevels = g.levels;
    if (trained.weightsRange == 0)
        return g;
    if (rounded)
        g.levels = trained.weightsRange > 1 ? std::floor(trained.weightsRange / 2.0) : 1;
    const long double fourBitLevels = rounded ? 7.0 : 8.0;
    if (trained.defaultQuantMode && g.levels == fourBitLevels) {
        g.levels = 15.0;
        g.stretch = 2.066666666666667;
        g.widened = true;
    }
    g.biasLevels = g.levels;
    return g;
}

// Fully-connected cells: the SAT scaling of the trained weights joins the grid when they are rounded
// (ref: src/Quantizer/QAT/Optimization/DeepNetQAT.cpp:1130-1151).
struct FcGrid {
    long double levels = 1.0, satScaling = 1.0, biasLevels = 1.0;
};
FcGrid fcGrid(const QATCellParameters& trained, bool rounded)
{
    FcGrid g;
    if (trained.weightsRange == 0)
        return g;
    if (rounded) {
        g.levels = trained.weightsRange > 1 ? std::floor(trained.weightsRange / 2.0) : 1;
        g.satScaling = trained.satScaling;
    }
    g.biasLevels = g.levels * g.satScaling;
    return g;
}

// Bits of an integer cell whose trained weights had `trainedRange` levels (0: not quantized, 1: binary weights)
std::size_t weightBits(std::size_t trainedRange)
{
    return bitsOf((double)(trainedRange == 0 ? 1 : (trainedRange == 1 ? 2 : trainedRange)));
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

    const bool roundWeights = wMode == WeightsApprox::RINTF;
    const WeightGrid grid = convGrid(trained, roundWeights, rangeConvBN.first);
    if (grid.widened)
        rangeConvBN.first = 31;

    std::shared_ptr<Activation> activation = Registrar<RectifierActivation>::create<Float_T>("Frame_HIP")();
    convCell.setActivation(activation);
    convCell.setParameter("NoBias", false);

    // Per output channel: the integer weights, then M, B and C of the head comment.  The three expressions keep the
    // reference's operands, order and types (ref: DeepNetQAT.cpp:718-806): they decide the last bit of what is installed.
    const double inAlpha = alphasConvBN.first, outAlpha = alphasConvBN.second;
    const std::size_t inRange = rangeConvBN.first, outRange = rangeConvBN.second;
    const std::size_t fanIn = trained.quantWeights.size() / nbOutputs;
    Tensor<Float_T> weights = trained.quantWeights;
    Tensor<Float_T> biases({nbOutputs});
    std::vector<Float_T> clipPerOutput(nbOutputs, 0.0f), scalingPerOutput(nbOutputs, 0.0f);
    for (std::size_t o = 0; o < nbOutputs; ++o) {
        // gain of the BatchNorm channel; a vanished variance leaves multiplier, bias and clip at 0: the channel outputs 0
        const double gain = bn.variances[o] > 1.0e-12 ? bn.scales[o] / std::sqrt(bn.epsilon + bn.variances[o]) : 0.0;
        const double side = gain < 0.0 ? -1.0 : 1.0;
        for (std::size_t k = 0; k < fanIn; ++k)
            weights(o * fanIn + k) = scaledWeight(trained.quantWeights(o * fanIn + k), grid.levels, roundWeights, side);
        Float_T multiplier = 0.0f, offset = 0.0f, ceiling = 0.0f;
        if (gain != 0.0) {
            const double trainedBias = noBias ? 0.0 : (double)trained.biases(o);
            multiplier = (inAlpha / (float)inRange) * ((float)outRange / outAlpha) * gain * (1 / grid.levels) * grid.stretch;
            offset = ((((bn.biases[o] + (trainedBias - bn.means[o]) * gain) / gain) * inRange / inAlpha) * grid.biasLevels) * (1.0 / grid.stretch);
            ceiling = ((outAlpha * inRange) / (gain * inAlpha)) * grid.levels * (1.0 / grid.stretch);
            multiplier *= side;
            offset *= side;
            ceiling *= side;
        }
        if (cMode == WeightsApprox::RINTF)
            ceiling = rintf(ceiling);
        if (bMode == WeightsApprox::RINTF)
            offset = rintf(offset);
        scalingPerOutput[o] = multiplier;
        clipPerOutput[o] = ceiling;
        biases(o) = offset;
    }
    convCell.setWeights(weights);
    convCell.setBiases(biases);
    convCell.setQuantized(weightBits(trained.weightsRange));
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
    const bool roundWeights = wMode == WeightsApprox::RINTF;
    const FcGrid grid = fcGrid(trained, roundWeights);
    // levels per unit of the input and of the output activation (an unquantized output counts in the input's levels)
    const double inLevelsPerUnit = rangeOpFc.first / alphaOpFC.first;
    double outLevelsPerUnit = rangeOpFc.first;
    if (actRange > 0)
        outLevelsPerUnit = rangeOpFc.second / alphaOpFC.second;

    // One multiplier and one ceiling for the whole cell, a bias per output; operands, order and types are the reference's
    // (ref: DeepNetQAT.cpp:1152-1215).
    const std::size_t fanIn = trained.quantWeights.size() / nbOutputs;
    Tensor<Float_T> weights = trained.quantWeights;
    Tensor<Float_T> biases({nbOutputs});
    std::vector<Float_T> clipPerOutput(nbOutputs, 0.0f), scalingPerOutput(nbOutputs, 0.0f);
    for (std::size_t o = 0; o < nbOutputs; ++o) {
        for (std::size_t k = 0; k < fanIn; ++k)
            weights(o * fanIn + k) = scaledWeight(trained.quantWeights(o * fanIn + k), grid.levels * grid.satScaling, roundWeights, 1.0);
        Float_T multiplier = (outLevelsPerUnit / inLevelsPerUnit) * (1.0 / (grid.satScaling * grid.levels));
        Float_T ceiling = alphaOpFC.second * inLevelsPerUnit * (grid.levels * grid.satScaling);
        Float_T offset = 0.0f;
        if (!noBias)
            offset = (double)trained.biases(o) * inLevelsPerUnit * grid.biasLevels;
        if (ceiling < 0.0)
            ceiling = 0.0;
        if (cMode == WeightsApprox::RINTF)
            ceiling = rintf(ceiling);
        if (bMode == WeightsApprox::RINTF && !noBias)
            offset = rintf(offset);
        scalingPerOutput[o] = multiplier;
        clipPerOutput[o] = ceiling;
        biases(o) = offset;
    }
    fcCell.setWeights(weights);
    fcCell.setParameter("NoBias", noBias);       // the integer cell takes over the trained cell's NoBias
    if (!noBias)
        fcCell.setBiases(biases);
    fcCell.setQuantized(weightBits(trained.weightsRange));
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
