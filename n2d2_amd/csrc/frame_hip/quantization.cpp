// Host-side ingestion of a network N2D2 has trained or calibrated: free parameters from its text exports, and the
// approximation of floating-point rescales by the integer Scaling modes.  Plain C++, no device code.
#include "frame_hip.hpp"

#include <algorithm>
#include <cassert>
#include <cctype>
#include <fstream>
#include <iomanip>
#include <limits>
#include <map>
#include <sstream>

namespace N2D2 {

namespace {

// Utils::fileBaseName / Utils::fileExtension (src/utils/Utils.cpp): the part before / after the last dot of the last
// path component
std::string fileBaseName(const std::string& fileName)
{
    const size_t slash = fileName.find_last_of("/\\");
    const size_t dot = fileName.find_last_of('.');
    return (dot == std::string::npos || (slash != std::string::npos && dot < slash)) ? fileName : fileName.substr(0, dot);
}
std::string fileExtension(const std::string& fileName)
{
    const size_t slash = fileName.find_last_of("/\\");
    const size_t dot = fileName.find_last_of('.');
    return (dot == std::string::npos || (slash != std::string::npos && dot < slash)) ? "" : fileName.substr(dot + 1);
}

struct SynapticFiles {
    std::string weightsFile, biasesFile;
    bool singleFile;
    std::ifstream weights, biasesOwn;
    bool opened;
    std::istream& biases(bool noBias) { return (!singleFile && !noBias) ? biasesOwn : weights; }
};

// The file naming and opening rules shared by ConvCell and FcCell (src/Cell/ConvCell.cpp:511-549)
void openSynapticFiles(SynapticFiles& f, const std::string& fileName, bool ignoreNotExists, bool noBias)
{
    const std::string fileBase = fileBaseName(fileName);
    std::string fileExt = fileExtension(fileName);
    if (!fileExt.empty())
        fileExt = "." + fileExt;
    f.singleFile = std::ifstream(fileName.c_str()).good();
    f.weightsFile = f.singleFile ? fileName : fileBase + "_weights" + fileExt;
    f.biasesFile = f.singleFile ? fileName : fileBase + "_biases" + fileExt;
    f.opened = false;
    f.weights.open(f.weightsFile.c_str());
    if (!f.weights.good()) {
        if (ignoreNotExists) {
            std::cout << "Notice: Could not open synaptic file: " << f.weightsFile << std::endl;
            return;
        }
        throw std::runtime_error("Could not open synaptic file: " + f.weightsFile);
    }
    if (!f.singleFile && !noBias) {
        f.biasesOwn.open(f.biasesFile.c_str());
        if (!f.biasesOwn.good())
            throw std::runtime_error("Could not open synaptic file: " + f.biasesFile);
    }
    f.opened = true;
}

void expectEnd(std::istream& in, const std::string& name)
{
    while (std::isspace(in.peek()))
        in.ignore();
    if (in.get() != std::istream::traits_type::eof())
        throw std::runtime_error("Synaptic file size larger than expected: " + name);
}

} // namespace

// ------------------------------------------------------------------- ConvCell
void ConvCell::importFreeParameters(const std::string& fileName, bool ignoreNotExists)
{
    if (mNbChannels == 0)
        throw std::runtime_error("ConvCell::importFreeParameters(): connect cell " + mName + " before importing its parameters");
    SynapticFiles f;
    openSynapticFiles(f, fileName, ignoreNotExists, mNoBias);
    if (!f.opened)
        return;
    std::istream& biases = f.biases(mNoBias);
    const size_t cg = weightSlices();
    const size_t kernelSize = (size_t)mKernelDims[0] * mKernelDims[1];
    Tensor<Float_T> w({mKernelDims[0], mKernelDims[1], cg, mNbOutputs}, Float_T(0));
    Tensor<Float_T> b({mNbOutputs});
    double value;
    for (size_t output = 0; output < mNbOutputs; ++output) {
        // the channels of the output's group are its connections, in channel order; with an irregular map the file holds
        // the kernels of the connected channels only (`:559-561`), each stored in the slice the forward pass reads it from
        for (size_t slice : connectedSlices(output)) {
            for (size_t index = 0; index < kernelSize; ++index) {
                if (!(f.weights >> value))
                    throw std::runtime_error("Error while reading synaptic file: " + f.weightsFile);
                w(index + kernelSize * (slice + cg * output)) = (Float_T)value;
            }
        }
        if (!mNoBias) {
            if (!(biases >> value))
                throw std::runtime_error("Error while reading synaptic file: " + f.biasesFile);
            b(output) = (Float_T)value;
        }
    }
    expectEnd(f.weights, f.weightsFile);
    if (!f.singleFile && !mNoBias)
        expectEnd(biases, f.biasesFile);
    mWeights = w;
    if (!mNoBias)
        mBias = b;
    mDirty = true;
}

// The slices of the weights tensor that hold an output's kernels, in channel order: all of them, or with an irregular map
// one per connected channel (src/Cell/ConvCell_Frame_Kernels.cpp:93-97)
std::vector<std::size_t> ConvCell::connectedSlices(std::size_t output) const
{
    std::vector<std::size_t> slices;
    if (!hasIrregularMapping()) {
        for (std::size_t k = 0; k < weightSlices(); ++k) slices.push_back(k);
        return slices;
    }
    for (std::size_t ch = 0; ch < mNbChannels; ++ch) {
        if (!mIrregularMap.at(output, ch)) continue;
        const std::size_t slice = mNbGroups > 1 ? slices.size() : ch;
        if (slice >= weightSlices())
            throw std::runtime_error("ConvCell " + mName + ": output " + std::to_string(output) + " is connected to more channels than "
                                     "the weights have slices (the reference would read past them)");
        slices.push_back(slice);
    }
    return slices;
}

void ConvCell::exportFreeParameters(const std::string& fileName) const
{
    const std::string fileBase = fileBaseName(fileName);
    std::string fileExt = fileExtension(fileName);
    if (!fileExt.empty())
        fileExt = "." + fileExt;
    const std::string weightsFile = fileBase + "_weights" + fileExt, biasesFile = fileBase + "_biases" + fileExt;
    std::ofstream weights(weightsFile.c_str());
    if (!weights.good())
        throw std::runtime_error("Could not create synaptic file: " + weightsFile);
    const size_t kernelSize = (size_t)mKernelDims[0] * mKernelDims[1], cg = weightSlices();
    for (size_t output = 0; output < mNbOutputs; ++output) {
        for (size_t slice : connectedSlices(output))
            for (size_t i = 0; i < kernelSize; ++i)
                weights << std::setprecision(10) << mWeights(i + kernelSize * (slice + cg * output)) << " ";
        weights << "\n";
    }
    if (!mNoBias) {
        std::ofstream biases(biasesFile.c_str());
        if (!biases.good())
            throw std::runtime_error("Could not create synaptic file: " + biasesFile);
        for (size_t output = 0; output < mNbOutputs; ++output)
            biases << std::setprecision(10) << mBias(output) << "\n";
    }
}

void ConvCell::processFreeParametersPerOutput(const std::function<Float_T(Float_T)>& func, std::size_t output)
{
    const size_t perOutput = mWeights.size() / std::max<size_t>(mNbOutputs, 1);
    for (size_t i = 0; i < perOutput; ++i)
        mWeights(i + perOutput * output) = func(mWeights(i + perOutput * output));
    if (!mNoBias && output < mBias.size())
        mBias(output) = func(mBias(output));
    mDirty = true;
}

// --------------------------------------------------------------------- FcCell
void FcCell::importFreeParameters(const std::string& fileName, bool ignoreNotExists)
{
    const size_t channelsSize = (size_t)mNbChannels * mInW * mInH;
    if (channelsSize == 0)
        throw std::runtime_error("FcCell::importFreeParameters(): connect cell " + mName + " before importing its parameters");
    SynapticFiles f;
    openSynapticFiles(f, fileName, ignoreNotExists, mNoBias);
    if (!f.opened)
        return;
    std::istream& biases = f.biases(mNoBias);
    Tensor<Float_T> w({channelsSize, mNbOutputs});
    Tensor<Float_T> b({mNbOutputs});
    double value;
    for (size_t output = 0; output < mNbOutputs; ++output) {
        for (size_t channel = 0; channel < channelsSize; ++channel) {
            if (!(f.weights >> value))
                throw std::runtime_error("Error while reading synaptic file: " + fileName);
            w(channel + channelsSize * output) = (Float_T)value;
        }
        if (!mNoBias) {
            if (!(biases >> value))
                throw std::runtime_error("Error while reading synaptic file: " + fileName);
            b(output) = (Float_T)value;
        }
    }
    expectEnd(f.weights, f.weightsFile);
    if (!f.singleFile && !mNoBias)
        expectEnd(biases, f.biasesFile);
    mWeights = w;
    if (!mNoBias)
        mBias = b;
    mDirty = true;
}

void FcCell::exportFreeParameters(const std::string& fileName) const
{
    const std::string fileBase = fileBaseName(fileName);
    std::string fileExt = fileExtension(fileName);
    if (!fileExt.empty())
        fileExt = "." + fileExt;
    const std::string weightsFile = fileBase + "_weights" + fileExt, biasesFile = fileBase + "_biases" + fileExt;
    std::ofstream weights(weightsFile.c_str());
    if (!weights.good())
        throw std::runtime_error("Could not create synaptic file: " + weightsFile);
    const size_t perOutput = mWeights.size() / std::max<size_t>(mNbOutputs, 1);
    for (size_t output = 0; output < mNbOutputs; ++output) {
        for (size_t i = 0; i < perOutput; ++i)
            weights << std::setprecision(10) << mWeights(i + perOutput * output) << " ";
        weights << "\n";
    }
    if (!mNoBias) {
        std::ofstream biases(biasesFile.c_str());
        if (!biases.good())
            throw std::runtime_error("Could not create synaptic file: " + biasesFile);
        for (size_t output = 0; output < mNbOutputs; ++output)
            biases << std::setprecision(10) << mBias(output) << "\n";
    }
}

void FcCell::processFreeParametersPerOutput(const std::function<Float_T(Float_T)>& func, std::size_t output)
{
    const size_t perOutput = mWeights.size() / std::max<size_t>(mNbOutputs, 1);
    for (size_t i = 0; i < perOutput; ++i)
        mWeights(i + perOutput * output) = func(mWeights(i + perOutput * output));
    if (!mNoBias && output < mBias.size())
        mBias(output) = func(mBias(output));
    mDirty = true;
}

// -------------------------------------------------------- DeepNetQuantization
// ------------------------------------------------------------------ Scaling and bit widths as text
namespace {
const char* scalingModeName(ScalingMode mode)
{
    switch (mode) {
    case ScalingMode::NONE: return "None";
    case ScalingMode::FLOAT_MULT: return "Floating-point";
    case ScalingMode::FIXED_MULT16: return "Fixed-point16";
    case ScalingMode::FIXED_MULT32: return "Fixed-point32";
    case ScalingMode::SINGLE_SHIFT: return "Single-shift";
    default: return "Double-shift";
    }
}

// "Key=value" lines of a stream, in any order; a key given twice or a line without '=' is an error
std::map<std::string, std::string> readKeyValues(std::istream& is, const std::string& what)
{
    std::map<std::string, std::string> kv;
    std::string line;
    while (std::getline(is, line)) {
        if (line.find_first_not_of(" \t\r") == std::string::npos)
            continue;
        const size_t eq = line.find('=');
        if (eq == std::string::npos)
            throw std::runtime_error("Malformed line \"" + line + "\" in " + what);
        const std::string key = line.substr(0, eq);
        if (!kv.insert(std::make_pair(key, line.substr(eq + 1))).second)
            throw std::runtime_error("Key " + key + " given twice in " + what);
    }
    return kv;
}

const std::string& need(const std::map<std::string, std::string>& kv, const std::string& key, const std::string& what)
{
    auto it = kv.find(key);
    if (it == kv.end())
        throw std::runtime_error("Missing key " + key + " in " + what);
    return it->second;
}

// "<count> v0 v1 ..." -> values; the count must match what follows
template <class T, class Parse>
std::vector<T> readVector(const std::string& text, const std::string& key, const std::string& what, Parse parse)
{
    std::istringstream in(text);
    size_t n = 0;
    if (!(in >> n))
        throw std::runtime_error("Key " + key + " in " + what + " does not start with a count");
    std::vector<T> v;
    std::string tok;
    while (in >> tok)
        v.push_back(parse(tok));
    if (v.size() != n)
        throw std::runtime_error("Key " + key + " in " + what + " announces " + std::to_string(n) + " values and holds " + std::to_string(v.size()));
    return v;
}

Scaling scalingFromKeyValues(const std::map<std::string, std::string>& kv, const std::string& what)
{
    const ScalingMode mode = parseScalingMode(need(kv, "ScalingMode", what));
    if (mode == ScalingMode::NONE)
        return Scaling();
    const bool isClipped = std::stoi(need(kv, "IsClipped", what)) != 0;
    const std::vector<Float_T> clipping = readVector<Float_T>(need(kv, "Clipping", what), "Clipping", what,
                                                              [](const std::string& t) { return (Float_T)std::stof(t); });
    const std::string& text = need(kv, "Scaling", what);
    auto asInt = [&](const std::string& t, long long lo, long long hi) {
        size_t used = 0;
        const long long v = std::stoll(t, &used);
        if (used != t.size() || v < lo || v > hi)
            throw std::runtime_error("Value " + t + " of key Scaling in " + what + " is not an integer in [" + std::to_string(lo) + ", "
                                     + std::to_string(hi) + "]");
        return v;
    };
    switch (mode) {
    case ScalingMode::FLOAT_MULT:
        return Scaling::floatingPointScaling(readVector<Float_T>(text, "Scaling", what, [](const std::string& t) { return (Float_T)std::stof(t); }),
                                             isClipped, clipping);
    case ScalingMode::FIXED_MULT16:
    case ScalingMode::FIXED_MULT32:
        return Scaling::fixedPointScaling(mode, (std::size_t)std::stoul(need(kv, "NbFractionalBits", what)),
                                          readVector<std::int32_t>(text, "Scaling", what, [&](const std::string& t) {
                                              return (std::int32_t)asInt(t, std::numeric_limits<std::int32_t>::min(), std::numeric_limits<std::int32_t>::max());
                                          }),
                                          isClipped, clipping);
    case ScalingMode::SINGLE_SHIFT:
        return Scaling::singleShiftScaling(readVector<unsigned char>(text, "Scaling", what, [&](const std::string& t) { return (unsigned char)asInt(t, 0, 255); }),
                                           isClipped, clipping);
    default: {
        const std::vector<unsigned char> flat = readVector<unsigned char>(text, "Scaling", what, [&](const std::string& t) { return (unsigned char)asInt(t, 0, 255); });
        if (flat.size() % 2 != 0)
            throw std::runtime_error("Key Scaling in " + what + ": a double shift holds two exponents per output");
        std::vector<std::pair<unsigned char, unsigned char> > pairs;
        for (size_t i = 0; i < flat.size(); i += 2)
            pairs.push_back(std::make_pair(flat[i], flat[i + 1]));
        return Scaling::doubleShiftScaling(pairs, isClipped, {});
    }
    }
}
} // namespace

void Scaling::save(std::ostream& os) const
{
    os << "ScalingMode=" << scalingModeName(mMode) << "\n";
    if (mMode == ScalingMode::NONE)
        return;
    os << "NbFractionalBits=" << mNbFractionalBits << "\n";
    os << "IsClipped=" << (mIsClipped ? 1 : 0) << "\n";
    os << "Scaling=";
    if (mMode == ScalingMode::FLOAT_MULT) {
        os << mFloat.size() << std::setprecision(9);
        for (Float_T v : mFloat) os << " " << v;
    } else if (mMode == ScalingMode::FIXED_MULT16 || mMode == ScalingMode::FIXED_MULT32) {
        os << mFixed.size();
        for (std::int32_t v : mFixed) os << " " << v;
    } else {
        os << mShift.size();
        for (unsigned char v : mShift) os << " " << (int)v;
    }
    os << "\nClipping=" << mClipping.size() << std::setprecision(9);
    for (Float_T v : mClipping) os << " " << v;
    os << "\n";
}

Scaling Scaling::load(std::istream& is, const std::string& what)
{
    return scalingFromKeyValues(readKeyValues(is, what), what);
}

void DeepNet::saveQuantization(const std::string& dirName) const
{
    for (const std::shared_ptr<Cell>& cell : mOrder) {
        const std::string fileName = dirName + "/" + cell->getName() + ".quant";
        std::ofstream os(fileName.c_str());
        if (!os.good())
            throw std::runtime_error("Could not create quantization file: " + fileName);
        os << "CellQuantizedNbBits=" << cell->getQuantizedNbBits() << "\n";
        os << "ActivationQuantizedNbBits=" << (cell->getActivation() ? cell->getActivation()->getQuantizedNbBits() : 0) << "\n";
        if (auto sc = std::dynamic_pointer_cast<ScalingCell>(cell))
            sc->getScaling().save(os);
        else if (cell->getActivation())
            cell->getActivation()->getActivationScaling().save(os);
        else
            Scaling().save(os);
        if (!os.good())
            throw std::runtime_error("Error writing quantization file: " + fileName);
    }
}

void DeepNet::loadQuantization(const std::string& dirName)
{
    for (const std::shared_ptr<Cell>& cell : mOrder) {
        const std::string fileName = dirName + "/" + cell->getName() + ".quant";
        std::ifstream is(fileName.c_str());
        if (!is.good())
            throw std::runtime_error("Could not open quantization file: " + fileName);
        const std::map<std::string, std::string> kv = readKeyValues(is, fileName);
        Scaling scaling = scalingFromKeyValues(kv, fileName);
        const std::size_t nb = scaling.nbOutputs();
        if (scaling.getMode() != ScalingMode::NONE && nb != cell->getNbOutputs() && nb != 1)
            throw std::runtime_error("Quantization file " + fileName + " holds a scaling for " + std::to_string(nb) + " outputs, cell "
                                     + cell->getName() + " has " + std::to_string(cell->getNbOutputs()));
        cell->setQuantized((std::size_t)std::stoul(need(kv, "CellQuantizedNbBits", fileName)));
        const std::size_t actBits = (std::size_t)std::stoul(need(kv, "ActivationQuantizedNbBits", fileName));
        if (auto sc = std::dynamic_pointer_cast<ScalingCell>(cell)) {
            sc->setScaling(scaling);
        } else if (cell->getActivation()) {
            cell->getActivation()->setActivationScaling(scaling);
            cell->getActivation()->setQuantized(actBits);
        } else if (scaling.getMode() != ScalingMode::NONE) {
            throw std::runtime_error("Quantization file " + fileName + " holds a scaling, cell " + cell->getName() + " has no activation");
        }
    }
}

namespace {

// Largest multiplier a fixed-point mode can hold.
std::uint64_t multiplierCeiling(ScalingMode mode)
{
    return mode == ScalingMode::FIXED_MULT16 ? (std::uint64_t)std::numeric_limits<std::int16_t>::max()
                                             : (std::uint64_t)std::numeric_limits<std::int32_t>::max();
}

// How much of `scaling` a term 2^-shift covers, as a fraction of it.
double shareOf(double scaling, std::size_t shift) { return 1.0 / (scaling * std::pow(2, shift)); }

} // namespace

// Per-output float factors -> (fractional bits, integer multipliers): the widest fractional part, 50 bits at most, with which
// the largest factor still fits the mode's multiplier; a 16-bit request whose largest factor does not fit at all is served
// in 32 bits and `mode` says so (ref: src/DeepNetQuantization.cpp:1043-1093; the expressions are the reference's, so that
// the multipliers come out identical).
std::pair<std::size_t, std::vector<std::int32_t> > DeepNetQuantization::approximateScalingWithFixedPoint(
    ScalingMode& mode, const std::vector<Float_T>& scalingPerOutput)
{
    if (scalingPerOutput.empty())
        throw std::runtime_error("approximateScalingWithFixedPoint(): no scaling");
    const double largest = *std::max_element(scalingPerOutput.begin(), scalingPerOutput.end());
    if (mode == ScalingMode::FIXED_MULT16 && largest >= multiplierCeiling(mode)) {
        std::cout << "Notice: a scaling of " << largest << " needs more than 16 bits; FIXED_MULT32 is used instead of FIXED_MULT16."
                  << std::endl;
        mode = ScalingMode::FIXED_MULT32;
    }
    const std::uint64_t ceiling = multiplierCeiling(mode);
    if (largest >= ceiling) {
        std::ostringstream msg;
        msg << "approximateScalingWithFixedPoint(): a scaling of " << largest << " does not fit a 32-bit multiplier";
        throw std::runtime_error(msg.str());
    }
    const std::size_t fractionalBits = std::min<std::size_t>((std::size_t)std::floor(std::log(ceiling / largest) / std::log(2.0)), 50);
    std::pair<std::size_t, std::vector<std::int32_t> > result(fractionalBits, std::vector<std::int32_t>(scalingPerOutput.size()));
    std::transform(scalingPerOutput.begin(), scalingPerOutput.end(), result.second.begin(),
                   [fractionalBits](Float_T factor) { return (std::int32_t)std::round(factor * (1ull << fractionalBits)); });
    return result;
}

// A factor in (0, 1] as a sum of `nbDivisions` terms 2^-shift, greedily: every term is the largest power of two that does not
// overshoot what is still uncovered.  Returns the shifts and the fraction of the factor their sum amounts to, which the
// caller folds into the cell's parameters.  Three corrections, as in the reference (src/DeepNetQuantization.cpp:1095-1134):
// once the sum is exact, a further term is made by splitting the last one in two; a sum within 2 % of the factor counts as
// exact; one further away has its last term doubled, which takes it above the factor.
std::pair<std::vector<unsigned char>, double> DeepNetQuantization::approximateScalingWithPowerOf2Divs(Float_T scaling, std::size_t nbDivisions)
{
    if (nbDivisions == 0 || !(scaling > 0.0) || scaling > 1.0)
        throw std::runtime_error("approximateScalingWithPowerOf2Divs(): needs 0 < scaling <= 1 and at least one division");
    std::vector<unsigned char> shifts;
    shifts.reserve(nbDivisions);
    double covered = 0.0;
    while (shifts.size() < nbDivisions) {
        if (covered == 1.0) {
            const unsigned char halved = (unsigned char)(shifts.back() + 1);
            shifts.back() = halved;
            shifts.push_back(halved);
            continue;
        }
        const std::size_t shift = (std::size_t)std::ceil(std::log2(1.0 / (scaling * (1.0 - covered))));
        covered += shareOf(scaling, shift);
        shifts.push_back(static_cast<unsigned char>(shift));
    }
    if (covered >= 0.98)
        return std::make_pair(shifts, 1.0);
    covered += shareOf(scaling, shifts.back());
    shifts.back() = (unsigned char)(shifts.back() - 1);
    return std::make_pair(shifts, covered);
}

void DeepNetQuantization::approximateActivationScaling(Cell& cell, Activation& activation, ScalingMode actScalingMode)
{
    if (activation.getActivationScaling().getMode() != ScalingMode::FLOAT_MULT)
        throw std::runtime_error("approximateActivationScaling(): the activation of cell " + cell.getName() + " has no floating-point scaling");
    const std::vector<Float_T> scalingPerOutput = activation.getActivationScaling().getFloatScalingPerOutput();
    if ((actScalingMode == ScalingMode::SINGLE_SHIFT || actScalingMode == ScalingMode::DOUBLE_SHIFT)
        && std::any_of(scalingPerOutput.begin(), scalingPerOutput.end(), [](Float_T s) { return s > 1.0; })) {
        std::cout << "Warning: Scaling (" << scalingPerOutput[0] << ") > 1 for layer \"" << cell.getName()
                  << "\" is not supported with Single/Double-shift scaling. Falling back to Fixed-point scaling for this layer." << std::endl;
        actScalingMode = ScalingMode::FIXED_MULT16;
    }
    if (actScalingMode == ScalingMode::FLOAT_MULT) {
        // nothing to do
    } else if (actScalingMode == ScalingMode::FIXED_MULT32 || actScalingMode == ScalingMode::FIXED_MULT16) {
        auto scalingFixedPoint = approximateScalingWithFixedPoint(actScalingMode, scalingPerOutput);
        activation.setActivationScaling(Scaling::fixedPointScaling(actScalingMode, scalingFixedPoint.first, scalingFixedPoint.second, false,
                                                                   std::vector<Float_T>(0)));
    } else if (actScalingMode == ScalingMode::SINGLE_SHIFT || actScalingMode == ScalingMode::DOUBLE_SHIFT) {
        const std::size_t nbDivisions = actScalingMode == ScalingMode::SINGLE_SHIFT ? 1 : 2;
        std::vector<unsigned char> single;
        std::vector<std::pair<unsigned char, unsigned char> > pairs;
        for (std::size_t output = 0; output < scalingPerOutput.size(); ++output) {
            const auto approx = approximateScalingWithPowerOf2Divs(scalingPerOutput[output], nbDivisions);
            // the shifts scale by approx.second times too much: the cell's parameters take the difference
            const Float_T rescaleOutputsBy = (Float_T)(1 / approx.second);
            cell.processFreeParametersPerOutput([&](Float_T d) { return rescaleOutputsBy * d; }, output);
            if (nbDivisions == 1)
                single.push_back(approx.first[0]);
            else
                pairs.push_back({(unsigned char)(approx.first[1] - approx.first[0]), approx.first[1]});
        }
        if (nbDivisions == 1)
            activation.setActivationScaling(Scaling::singleShiftScaling(single, false, std::vector<Float_T>(0)));
        else
            activation.setActivationScaling(Scaling::doubleShiftScaling(pairs, false, {std::make_pair((unsigned char)0, (unsigned char)0)}));
    } else {
        throw std::runtime_error("Unsupported scaling mode.");
    }
}

} // namespace N2D2
